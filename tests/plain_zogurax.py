"""A plain, slow implementation of the Zogurax decoder: whole sequences, no cache, NumPy float64,
one function for each mechanism.  It shares no code with the package under test: config.json is
read with ``json``, the weights with the ``safetensors`` library.

The design in short (x is the residual stream [T, width], positions p count from 0):

    x = E[token] + S(p)                       S: sines and cosines of p at width / 2 frequencies
    per layer:  h = LN(x);  x += mixer(h) + ff(h)        one norm, both sublayers read it
    logits = W_head LN_final(x)

A run of layers [start, stop) is gone through `times` times with the same weights; at the head of
every pass x = W_in [x ; x0] + step[pass], where x0 is the embedding output.  A mixer is softmax
attention without a rotation in one of two forms (plain projections with a short convolution over
time, a norm over the whole of q and of k and a gate on every head's output; or projections with
biases and a unit in the softmax's denominator); both bend the scores through a tanh and scale the
query with the logarithm of its position's block number.  The feed-forward is a mixture of experts
chosen by a table over token ids, with a gated shared expert.
"""
from __future__ import annotations

import json
import math
import os

import numpy as np


# --------------------------------------------------------------------------
# mechanisms
# --------------------------------------------------------------------------

def position_vector(positions, width: int) -> np.ndarray:
    """[T, width]: entry 2i is sin(p * 10000^(-2i / width)), entry 2i + 1 the cosine of the same angle."""
    p = np.asarray(positions, dtype=np.float64).reshape(-1, 1)
    out = np.zeros((p.shape[0], width))
    for i in range((width + 1) // 2):
        angle = p[:, 0] * 10000.0 ** (-2.0 * i / width)
        out[:, 2 * i] = np.sin(angle)
        if 2 * i + 1 < width:
            out[:, 2 * i + 1] = np.cos(angle)
    return out


def layer_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """(x - mean) / sqrt(variance + eps) * w over the last axis, variance = mean squared deviation."""
    x = np.asarray(x, dtype=np.float64)
    mean = x.mean(axis=-1, keepdims=True)
    var = ((x - mean) ** 2).mean(axis=-1, keepdims=True)
    return (x - mean) / np.sqrt(var + eps) * np.asarray(w, dtype=np.float64)


def root_mean_square_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """x / sqrt(mean(x^2) + eps) * w over the last axis; eps inside the root."""
    x = np.asarray(x, dtype=np.float64)
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps) * np.asarray(w, dtype=np.float64)


def time_convolution(u: np.ndarray, w: np.ndarray, before: np.ndarray = None) -> np.ndarray:
    """y_t = sum_j w[:, j] u_(t - taps + 1 + j) per channel; rows before the first are `before`
    ([taps - 1, channels], oldest first) or zeros.  w is [channels, taps]."""
    u = np.asarray(u, dtype=np.float64)
    w = np.asarray(w, dtype=np.float64)
    T, taps = u.shape[0], w.shape[1]
    pad = np.zeros((taps - 1, u.shape[1])) if before is None else np.asarray(before, dtype=np.float64)
    full = np.concatenate([pad, u], axis=0)
    out = np.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            out[t] += w[:, j] * full[t + j]
    return out


def query_temperature(positions, coef: float, every: int) -> np.ndarray:
    """1 + coef * ln(floor((p + 1) / every) + 1) for each position."""
    p = np.asarray(positions, dtype=np.int64)
    return 1.0 + coef * np.log((p + 1) // every + 1.0)


def bend(score: np.ndarray, cap: float) -> np.ndarray:
    """cap * tanh(score / cap); cap 0 or None leaves the score alone."""
    return cap * np.tanh(score / cap) if cap else score


def causal_attention(q, k, v, scale: float, cap: float, unit_sink: bool, q_positions=None, k_positions=None) -> np.ndarray:
    """q [T, H, d], k [S, G, d], v [S, G, dv] -> [T, H, dv].  Query head h reads key/value head
    h // (H / G); position i sees every j <= i; weights exp(s) / (sum exp(s) [+ 1 with unit_sink])."""
    T, H, _ = q.shape
    S, G, dv = v.shape
    qp = np.arange(T) if q_positions is None else np.asarray(q_positions)
    kp = np.arange(S) if k_positions is None else np.asarray(k_positions)
    out = np.zeros((T, H, dv))
    for h in range(H):
        g = h // (H // G)
        s = bend((q[:, h] @ k[:, g].T) * scale, cap)                      # [T, S]
        s = np.where(kp[None, :] <= qp[:, None], s, -np.inf)
        m = np.maximum(s.max(axis=1, keepdims=True), 0.0 if unit_sink else -np.inf)
        e = np.exp(s - m)
        den = e.sum(axis=1, keepdims=True) + (np.exp(-m) if unit_sink else 0.0)
        out[:, h] = (e / den) @ v[:, g]
    return out


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-np.asarray(z, dtype=np.float64)))


def squared_relu(z):
    return np.maximum(z, 0.0) ** 2


def expert(h: np.ndarray, up: np.ndarray, down: np.ndarray) -> np.ndarray:
    """W_down relu(W_up h)^2 for rows h."""
    return squared_relu(h @ up.T) @ down.T


def table_mixture(h: np.ndarray, tokens, table: np.ndarray, ups, downs) -> np.ndarray:
    """Each row goes through the experts that table[token] names, each weighted 1 / top."""
    top = table.shape[1]
    out = np.zeros((h.shape[0], downs[0].shape[0]))
    for t, tok in enumerate(tokens):
        for e in table[tok]:
            out[t] += expert(h[t:t + 1], ups[e], downs[e])[0] / top
    return out


def gated_shared_expert(h: np.ndarray, up, down, gate) -> np.ndarray:
    """expert(h) * sigmoid(gate . h), one number a row."""
    return expert(h, up, down) * sigmoid(h @ gate.T)


def loop_entry(x: np.ndarray, x0: np.ndarray, w_in: np.ndarray, step_row: np.ndarray) -> np.ndarray:
    """W_in [x ; x0] + step_row."""
    return np.concatenate([x, x0], axis=1) @ w_in.T + step_row


# --------------------------------------------------------------------------
# the two mixers
# --------------------------------------------------------------------------

def mixer(kind: str, m: dict, w: dict, p: str, h: np.ndarray, eps: float, positions=None) -> np.ndarray:
    """kind 'attention': convolution, whole-projection norms, head gates; 'attention_2': biases and
    the unit in the denominator.  m is the layer's 'mixer' entry, p the tensor prefix 'l<i>.mix.'."""
    T = h.shape[0]
    pos = np.arange(T) if positions is None else np.asarray(positions)
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = h @ w[p + "q"].T, h @ w[p + "k"].T, h @ w[p + "v"].T
    if kind == "attention_2":
        q, k, v = q + w[p + "q.b"], k + w[p + "k.b"], v + w[p + "v.b"]
    else:
        q, k, v = (time_convolution(u, w[p + n + ".conv"]) for u, n in ((q, "q"), (k, "k"), (v, "v")))
        q = root_mean_square_norm(q, w[p + "q.norm"], eps)
        k = root_mean_square_norm(k, w[p + "k.norm"], eps)
    if m.get("q_temp"):
        q = q * query_temperature(pos, m["q_temp"]["coef"], m["q_temp"]["every"])[:, None]
    a = causal_attention(q.reshape(T, H, d), k.reshape(T, G, d), v.reshape(T, G, dv), m["scale"], m.get("softcap"),
                         unit_sink=(kind == "attention_2"), q_positions=pos, k_positions=pos)
    if kind == "attention":
        a = a * sigmoid(h @ w[p + "g"].T)[:, :, None]
    out = a.reshape(T, H * dv) @ w[p + "o"].T
    if kind == "attention_2":
        out = out + w[p + "o.b"]
    return out


def feed_forward(f: dict, w: dict, p: str, h: np.ndarray, tokens) -> np.ndarray:
    n = f["router"]["experts"]
    out = table_mixture(h, tokens, w[p + "table"].astype(np.int64), [w[f"{p}e{e}.up"] for e in range(n)],
                        [w[f"{p}e{e}.down"] for e in range(n)])
    if f.get("shared"):
        out = out + gated_shared_expert(h, w[p + "shared.up"], w[p + "shared.down"], w[p + "shared.sg"])
    return out


# --------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------

def layer_runs(cfg: dict):
    """[(layer, pass number or None when the run does not open a pass)] in the order of running."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or loop["stop"] <= loop["start"]:
        return [(i, None) for i in range(n)]
    runs = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        runs += [(i, t if i == loop["start"] else None) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, None) for i in range(loop["stop"], n)]


def forward(cfg: dict, w: dict, tokens, streams: list = None) -> np.ndarray:
    """Logits [T, vocab] of one sequence; `streams` collects the residual stream after every layer run."""
    eps, W = cfg["norm"]["eps"], cfg["width"]
    x = w["embed"][list(tokens)] + position_vector(range(len(tokens)), W)
    x0 = x.copy()
    for i, opens in layer_runs(cfg):
        L, p = cfg["layers"][i], f"l{i}."
        if opens is not None:
            x = loop_entry(x, x0, w["loop.in"], w["loop.step"][opens])
        h = layer_norm(x, w[p + "norm1"], eps)
        delta = mixer(L["type"], L["mixer"], w, p + "mix.", h, eps)
        if L.get("mlp"):
            delta = delta + feed_forward(L["mlp"], w, p + "mlp.", h, tokens)
        x = x + delta
        if streams is not None:
            streams.append(x.copy())
    return layer_norm(x, w["final.norm"], eps) @ w["head"].T


def load_folder(path: str):
    """(config dict, {tensor name: float64 array, integer tables as they are})."""
    import torch
    from safetensors.torch import load_file
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    w = {}
    for k, t in load_file(os.path.join(path, "model.safetensors")).items():
        w[k] = t.numpy() if t.dtype in (torch.int32, torch.int64) else t.to(torch.float64).numpy()
    return cfg, w


def generate_greedy(cfg: dict, w: dict, prompt, n: int) -> list:
    """n tokens, each the first largest logit after everything before it (the whole sequence is run again each time)."""
    seq, out = list(prompt), []
    for _ in range(n):
        tok = int(np.argmax(forward(cfg, w, seq)[-1]))
        out.append(tok)
        seq.append(tok)
    return out
