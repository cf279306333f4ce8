"""A plain, slow implementation of the Nipulorn decoder: whole sequences, no cache, NumPy
float64, one function for each mechanism.  It shares no code with the package under test:
config.json is read with ``json``, the weights with the ``safetensors`` library.

The design in short (x is the residual stream [T, width], positions count from 0):

    x = E[token] * embedding.scale
    per layer:  x += N1b(mixer(C1(N1(x))));  x += N2b(ff(C2(N2(x))))   (the second line only with a feed-forward)
    logits = E . N(x) * logit_scale

N* are RMS norms whose stored weight is an offset from one, C* add a short causal convolution over
time to their input, a mixer is either a recurrence with a matrix state per head ('wkv') or
attention through a low-rank latent ('latent_attention'), and the feed-forward is two matrices
around a piecewise activation with two learned numbers.
"""
from __future__ import annotations

import json
import math
import os

import numpy as np


# --------------------------------------------------------------------------
# mechanisms
# --------------------------------------------------------------------------

def root_mean_square_scale(x: np.ndarray, eps: float) -> np.ndarray:
    """x / sqrt(mean(x^2) + eps) over the last axis; eps inside the root."""
    x = np.asarray(x, dtype=np.float64)
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def offset_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """RMS norm whose stored weight w is an offset: the scale is 1 + w."""
    return root_mean_square_scale(x, eps) * (1.0 + np.asarray(w, dtype=np.float64))


def plain_weight_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """RMS norm whose weight multiplies as it is stored."""
    return root_mean_square_scale(x, eps) * np.asarray(w, dtype=np.float64)


def input_convolution(h: np.ndarray, w: np.ndarray) -> np.ndarray:
    """h + conv(h): per channel, conv(h)_t = sum_j w[:, j] h_(t - taps + 1 + j), with zeros before
    the sequence's start.  w is [width, taps]; its last tap multiplies the present token."""
    h = np.asarray(h, dtype=np.float64)
    w = np.asarray(w, dtype=np.float64)
    T, taps = h.shape[0], w.shape[1]
    out = h.copy()
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(z):
    return np.log1p(np.exp(-np.abs(z))) + np.maximum(z, 0.0)


def silu(z):
    return z / (1.0 + np.exp(-z))


def xielu(z: np.ndarray, p: float, q: float) -> np.ndarray:
    """z > 0: softplus(p) z^2 + z / 2;  z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2."""
    z = np.asarray(z, dtype=np.float64)
    ap, an = softplus(np.float64(p)), 0.5 + softplus(np.float64(q))
    neg = np.minimum(z, 0.0)
    return np.where(z > 0, ap * z * z + 0.5 * z, an * (np.expm1(neg) - neg) + 0.5 * z)


def dense_feed_forward(h: np.ndarray, w_up: np.ndarray, w_down: np.ndarray, act) -> np.ndarray:
    a = xielu(h @ np.asarray(w_up, dtype=np.float64).T, float(act[0]), float(act[1]))
    return a @ np.asarray(w_down, dtype=np.float64).T


def token_shift(h: np.ndarray, mu: np.ndarray, before: np.ndarray | None = None) -> np.ndarray:
    """h_t + (h_(t-1) - h_t) mu, with zeros (or `before`) as the row before the first."""
    h = np.asarray(h, dtype=np.float64)
    prev = np.zeros_like(h)
    prev[1:] = h[:-1]
    if before is not None:
        prev[0] = before
    return h + (prev - h) * np.asarray(mu, dtype=np.float64)


def wkv_recurrence(r, k, v, w, u, state=None):
    """Per head with state S [key channel, value channel], starting at zero:
        o_t = (S + diag(u) k_t v_t^T)^T r_t      (the bonus u for the present token only)
        S  <- diag(w_t) S + k_t v_t^T
    r, k, v, w are [T, heads, dim]; u is [heads, dim].  Returns (o [T, heads, dim], S)."""
    T, H, D = r.shape
    S = np.zeros((H, D, D)) if state is None else np.array(state, dtype=np.float64)
    o = np.zeros((T, H, D))
    for t in range(T):
        for h in range(H):
            kv = np.outer(k[t, h], v[t, h])
            o[t, h] = (S[h] + u[h][:, None] * kv).T @ r[t, h]
            S[h] = w[t, h][:, None] * S[h] + kv
    return o, S


def wkv_mixer(h: np.ndarray, p: dict, heads: int, dim: int, eps: float) -> np.ndarray:
    """p holds the mixer's tensors by their short names ('mu.r', 'r', 'w1', ...)."""
    f = lambda n: np.asarray(p[n], dtype=np.float64)
    T = h.shape[0]
    mix = {s: token_shift(h, f("mu." + s)) for s in "rkvgw"}
    r = (mix["r"] @ f("r").T).reshape(T, heads, dim)
    k = (mix["k"] @ f("k").T).reshape(T, heads, dim)
    v = (mix["v"] @ f("v").T).reshape(T, heads, dim)
    gate = silu(mix["g"] @ f("g").T)
    decay = np.exp(-np.exp(np.tanh(mix["w"] @ f("w1").T) @ f("w2").T + f("w0"))).reshape(T, heads, dim)
    o, _ = wkv_recurrence(r, k, v, decay, f("u"))
    o = root_mean_square_scale(o, eps).reshape(T, heads * dim) * f("norm") * gate
    return o @ f("o").T


def yarn_frequencies(dims: int, base: float, scaling: dict | None):
    """(frequencies [dims / 2], amplitude of cos and sin)."""
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=np.float64)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def at(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(at(float(scaling["fast"]))), 0)
    hi = min(math.ceil(at(float(scaling["slow"]))), dims - 1)
    ramp = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_pairs(x: np.ndarray, positions, freqs: np.ndarray, amplitude: float) -> np.ndarray:
    """x [T, ..., n]: dimensions 2i and 2i+1 of the first 2 len(freqs) are a pair turned by
    position * freqs[i]; the rest pass unchanged."""
    x = np.array(x, dtype=np.float64)
    pos = np.asarray(list(positions), dtype=np.float64)
    ang = pos[:, None] * freqs[None, :]
    shape = (len(pos),) + (1,) * (x.ndim - 2) + (len(freqs),)
    c, s = (np.cos(ang) * amplitude).reshape(shape), (np.sin(ang) * amplitude).reshape(shape)
    n = 2 * len(freqs)
    a, b = x[..., 0:n:2].copy(), x[..., 1:n:2].copy()
    x[..., 0:n:2] = a * c - b * s
    x[..., 1:n:2] = b * c + a * s
    return x


def sink_softmax_attention(scores: np.ndarray, values: np.ndarray, sink: float) -> np.ndarray:
    """Causal softmax over keys whose denominator also holds exp(sink): scores [T, T] (already
    scaled), values [T, d]."""
    T = scores.shape[0]
    s = np.where(np.tril(np.ones((T, T), dtype=bool)), scores, -np.inf)
    m = np.maximum(s.max(axis=1, keepdims=True), sink)
    e = np.exp(s - m)
    return (e @ values) / (e.sum(axis=1, keepdims=True) + np.exp(sink - m))


def latent_attention_mixer(h: np.ndarray, p: dict, m: dict, eps: float, positions=None) -> np.ndarray:
    """m is the layer's 'mixer' entry of config.json."""
    f = lambda n: np.asarray(p[n], dtype=np.float64)
    T = h.shape[0]
    H, dim, rot, vdim, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    positions = range(T) if positions is None else positions
    freqs, amp = yarn_frequencies(m["rot"]["dims"], float(m["rot"]["base"]), m["rot"].get("scaling"))
    cq = plain_weight_norm(h @ f("dq").T, f("dq.norm"), eps)
    q = (cq @ f("uq").T).reshape(T, H, dim + rot)
    q_plain, q_rot = q[..., :dim], rotate_pairs(q[..., dim:], positions, freqs, amp)
    kv = h @ f("dkv").T
    c = plain_weight_norm(kv[:, :rank], f("dkv.norm"), eps)
    k_rot = rotate_pairs(kv[:, rank:], positions, freqs, amp)            # one for all heads
    k_plain = (c @ f("uk").T).reshape(T, H, dim)
    v = (c @ f("uv").T).reshape(T, H, vdim)
    out = np.zeros((T, H, vdim))
    sink = f("sink")
    for hd in range(H):
        s = (q_plain[:, hd] @ k_plain[:, hd].T + q_rot[:, hd] @ k_rot.T) * float(m["scale"])
        out[:, hd] = sink_softmax_attention(s, v[:, hd], float(sink[hd]))
    return out.reshape(T, H * vdim) @ f("o").T


# --------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------

def load_folder(folder: str):
    from safetensors import safe_open
    import torch
    with open(os.path.join(folder, "config.json")) as fh:
        cfg = json.load(fh)
    w = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as fh:
        for name in fh.keys():
            w[name] = fh.get_tensor(name).to(torch.float64).numpy()
    return cfg, w


def _sub(w: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}


def layer(cfg: dict, w: dict, i: int, x: np.ndarray) -> np.ndarray:
    L, eps, p = cfg["layers"][i], float(cfg["norm"]["eps"]), f"l{i}."
    h = input_convolution(offset_norm(x, w[p + "norm1"], eps), w[p + "canon1"])
    if L["type"] == "wkv":
        a = wkv_mixer(h, _sub(w, p + "mix."), L["mixer"]["heads"], L["mixer"]["dim"], eps)
    elif L["type"] == "latent_attention":
        a = latent_attention_mixer(h, _sub(w, p + "mix."), L["mixer"], eps)
    else:
        raise ValueError(L["type"])
    x = x + offset_norm(a, w[p + "norm1b"], eps)
    if L["mlp"] is not None:
        h = input_convolution(offset_norm(x, w[p + "norm2"], eps), w[p + "canon2"])
        d = dense_feed_forward(h, w[p + "mlp.up"], w[p + "mlp.down"], w[p + "mlp.act"])
        x = x + offset_norm(d, w[p + "norm2b"], eps)
    return x


def forward(cfg: dict, w: dict, tokens, streams: list | None = None) -> np.ndarray:
    """Logits [T, vocab] of one sequence; `streams` collects the residual stream after every layer."""
    x = w["embed"][np.asarray(tokens, dtype=np.int64)] * float(cfg["embedding"]["scale"])
    for i in range(len(cfg["layers"])):
        x = layer(cfg, w, i, x)
        if streams is not None:
            streams.append(x.copy())
    x = offset_norm(x, w["final.norm"], float(cfg["norm"]["eps"]))
    return (x @ w["embed"].T) * float(cfg["logit_scale"])


def generate_greedy(cfg: dict, w: dict, prompt, n: int) -> list:
    toks, out = list(prompt), []
    for _ in range(n):
        t = int(np.argmax(forward(cfg, w, toks)[-1]))
        out.append(t)
        toks.append(t)
    return out
