"""The Nipulorn design on the GPU against the plain implementation: every mechanism alone, whole
prompts, prompts cut into portions, token-by-token decoding, unequal batches with slots and pages
used again, long decoding over page borders, sensitivity to a far key and to the sink, greedy
generation through the library's entry point, and the trace runner as a program."""
import copy
import importlib
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import nipulorn_configs as nc
import nipulorn_helpers as H
import plain_nipulorn as pn

pytestmark = pytest.mark.gpu
L = H.llogos
P = importlib.import_module("daisi-llogos_amd.parts")
K = importlib.import_module("daisi-llogos_amd.ops.kernels")
DEV = torch.device("cuda:0")
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
PART_TOL = {"float32": 3e-5, "bfloat16": 3e-2}
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _np(t):
    return t.detach().cpu().double().numpy()


def _ctx(rt, lens, new, slots):
    """A step that brings new[i] tokens to sequence i, which is lens[i] long afterwards."""
    B, T = len(lens), sum(new)
    tok_seq = np.repeat(np.arange(B), new).astype(np.int32)
    tok_pos = np.concatenate([np.arange(l - n, l) for l, n in zip(lens, new)]).astype(np.int32)
    i32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=DEV)
    cu = np.concatenate([[0], np.cumsum(new)])
    return P.StepContext(runtime=rt, n_tokens=T, batch=B, ids=i32(np.zeros(T)), tok_seq=i32(tok_seq), tok_pos=i32(tok_pos),
                         slots=i32(slots), cu_seqlens=cu.tolist(), starts=[l - n for l, n in zip(lens, new)],
                         slot_ids=list(slots), is_decode=max(new) == 1, max_context=max(lens),
                         cu_dev=None if max(new) == 1 else i32(cu))


def _steps(lengths, cuts):
    """Cut sequences of `lengths` into steps: cuts[s][i] tokens of sequence i in step s (0: not in the step)."""
    done = [0] * len(lengths)
    for cut in cuts:
        seqs = [i for i, c in enumerate(cut) if c]
        lo = [done[i] for i in seqs]
        for i in seqs:
            done[i] += cut[i]
        yield seqs, lo, [done[i] for i in seqs]
    assert done == list(lengths), "the cuts do not cover the sequences"


def _bind(part, rng, dtype, scale=0.3):
    tensors, plain = {}, {}
    lim = {"norm": (0.7, 1.3), "offset": (-0.3, 0.3), "unit": (0.0, 0.9), "decay": (-5.0, 0.3), "sink": (-1.0, 3.0),
           "shape": (-1.5, 0.8), "taps": (-0.8, 0.8), "bonus": (-0.5, 1.5)}
    for spec in part.tensor_specs():
        if spec.kind in lim:
            t = torch.tensor(rng.uniform(*lim[spec.kind], size=spec.shape), dtype=torch.bfloat16)
        else:
            t = torch.tensor(rng.standard_normal(spec.shape) * scale, dtype=torch.bfloat16)
        tensors[spec.name], plain[spec.name] = t, t.double().numpy()
    part.bind(tensors.get, P.Runtime(DEV, DT[dtype]))
    return plain


# ---------------------------------------------------------------------------
# mechanisms alone
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("taps", [1, 2, 4, 7])
@pytest.mark.parametrize("out", ["float32", "bfloat16"])
def test_the_input_convolution_continues_over_steps_of_any_size(taps, out):
    rng = np.random.default_rng(taps)
    W, lengths = 70, (19, 6, 1)
    conv = P.CausalConv("c", W, taps)
    plain = _bind(conv, rng, "float32")
    h = [rng.standard_normal((n, W)).astype(np.float32) for n in lengths]
    want = [pn.input_convolution(x, plain["c"]) for x in h]
    slots = [2, 0, 3]
    state = torch.zeros((5,) + conv.state_spec().shape, dtype=torch.float32, device=DEV)
    state[1].fill_(7.0)                                       # a slot nobody uses: stays as it is
    cache = P.LayerCache(state=state)
    got = [np.zeros((n, W)) for n in lengths]
    cuts = [(5, 2, 1), (1, 1, 0), (1, 1, 0), (2, 2, 0), (1, 0, 0), (9, 0, 0)]
    for seqs, lo, hi in _steps(lengths, cuts):
        ctx = _ctx(conv.rt, hi, [b - a for a, b in zip(lo, hi)], [slots[i] for i in seqs])
        rows = torch.tensor(np.concatenate([h[i][a:b] for i, a, b in zip(seqs, lo, hi)]), device=DEV)
        o = _np(conv.forward(ctx, rows, cache, out_dtype=DT[out]))
        at = 0
        for i, a, b in zip(seqs, lo, hi):
            got[i][a:b] = o[at:at + b - a]
            at += b - a
    for g, w_ in zip(got, want):
        assert np.abs(g - w_).max() <= (1e-5 if out == "float32" else 2e-2) * max(1.0, np.abs(w_).max())
    if taps > 1:
        assert float(state[1].min()) == 7.0 and float(state[1].max()) == 7.0                                              # the state is the last taps - 1 inputs, oldest first
        assert np.allclose(_np(state[2])[-1], h[0][-1]) and np.allclose(_np(state[3])[-1], h[2][-1])
        assert np.allclose(_np(state[3])[:-1], 0.0)           # a sequence of one token: zeros before its start


@pytest.mark.parametrize("kind", ["tanh", "silu", "gelu_tanh", "xielu"])
def test_activations(kind):
    z = torch.linspace(-9.0, 9.0, 2001, device=DEV).reshape(3, 667)
    want = {"tanh": np.tanh, "silu": pn.silu, "gelu_tanh": pn.gelu_tanh, "xielu": lambda v: pn.xielu(v, 0.4, -0.9)}[kind](_np(z))
    a, b = float(pn.softplus(np.float64(0.4))), 0.5 + float(pn.softplus(np.float64(-0.9)))
    assert np.abs(_np(K.activation(z, kind, torch.float32, a, b)) - want).max() <= 2e-6 * max(1.0, np.abs(want).max())
    parts = torch.stack([z * 0.25, z * 0.75])                 # partial sums are added first
    assert np.abs(_np(K.activation(parts, kind, torch.bfloat16, a, b)) - want).max() <= 1e-2 * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("heads,dim,hidden,rank,blocks", [(2, 40, 56, 6, 0), (1, 64, 64, 16, 0), (3, 24, 100, 5, 0), (2, 72, 48, 8, 0),
                                                          (5, 8, 64, 3, 0), (1, 128, 96, 4, 0), (1, 64, 64, 16, 4), (2, 40, 56, 6, 2),
                                                          (1, 128, 96, 4, 8), (3, 24, 100, 5, 3), (1, 64, 64, 16, -2), (2, 40, 56, 6, -3),
                                                          (5, 8, 64, 3, -5), (1, 128, 96, 4, -2), (1, 64, 64, 16, 16), (2, 48, 56, 6, 16),
                                                          (3, 24, 100, 5, 16), (5, 8, 64, 3, 16), (1, 128, 96, 4, 16), (2, 40, 56, 6, -16)])
def test_the_recurrent_mixer_alone_in_pieces(dtype, heads, dim, hidden, rank, blocks, monkeypatch):
    """blocks > 0: a head's state columns shared out over that many blocks in steps of several tokens, as
    long prompts of few sequences run, with the head norm in a kernel of its own.  blocks < 0: the steps of
    several tokens cut into that many segments that run side by side (more segments than some steps have
    chunks: segments beyond a sequence's end), their states chained afterwards.
    blocks 16 and -16: 16 rows of the state a thread, as steps of many sequences run, whole and in 3 segments."""
    if abs(blocks) == 16:
        monkeypatch.setattr(K, "SCAN_ROWS", 16)
        blocks = 0 if blocks > 0 else -3
    monkeypatch.setattr(K, "SCAN_COLUMN_BLOCKS", max(blocks, 0))
    monkeypatch.setattr(K, "SCAN_SEGMENTS", max(-blocks, 0))
    rng = np.random.default_rng(heads * dim)
    mixer = P.WKV("m.", hidden, heads, dim, rank, eps=1e-5)
    plain = _bind(mixer, rng, dtype, scale=0.25)
    sub = {k[2:]: v for k, v in plain.items()}
    lengths, slots = (37, 4), [1, 3]
    h = [rng.standard_normal((n, hidden)).astype(np.float32) for n in lengths]
    want = [pn.wkv_mixer(x.astype(np.float64), sub, heads, dim, 1e-5) for x in h]
    state = torch.zeros((4,) + mixer.state_spec().shape, dtype=torch.float32, device=DEV)
    cache = P.LayerCache(state=state)
    got = [np.zeros((n, hidden)) for n in lengths]
    cuts = [(17, 2), (1, 1), (1, 1), (2, 0), (16, 0)]          # a chunk of the kernel and a token more; single tokens; two
    for seqs, lo, hi in _steps(lengths, cuts):
        ctx = _ctx(mixer.rt, hi, [b - a for a, b in zip(lo, hi)], [slots[i] for i in seqs])
        rows = torch.tensor(np.concatenate([h[i][a:b] for i, a, b in zip(seqs, lo, hi)]), device=DEV)
        o = _np(K.sum_parts(mixer.forward(ctx, rows, cache), None, torch.float32))      # (a mixer may hand on partial sums)
        at = 0
        for i, a, b in zip(seqs, lo, hi):
            got[i][a:b] = o[at:at + b - a]
            at += b - a
    for g, w_ in zip(got, want):
        assert np.abs(g - w_).max() <= PART_TOL[dtype] * max(1.0, np.abs(w_).max())
    # the state holds what the plain recurrence ends with, and the last input row
    x = h[0].astype(np.float64)
    f = lambda n: plain["m." + n]
    T = lengths[0]
    mix = {s: pn.token_shift(x, f("mu." + s)) for s in "rkvw"}
    r, k, v = ((mix[s] @ f(s).T).reshape(T, heads, dim) for s in "rkv")
    decay = np.exp(-np.exp(np.tanh(mix["w"] @ f("w1").T) @ f("w2").T + f("w0"))).reshape(T, heads, dim)
    _, S = pn.wkv_recurrence(r, k, v, decay, f("u"))
    row = _np(state[1])
    kept = row[:heads * dim * dim].reshape(heads, dim, dim).transpose(0, 2, 1)       # stored [head][value][key]
    assert np.abs(kept - S).max() <= (1e-4 if dtype == "float32" else 5e-2) * max(1.0, np.abs(S).max())
    assert np.allclose(row[heads * dim * dim:], h[0][-1])
    assert float(state[0].abs().max()) == 0.0 and float(state[2].abs().max()) == 0.0


LATENT = [dict(n_heads=3, dim=32, rot_dim=8, v_dim=24, q_rank=40, kv_rank=48, scale=0.3, dims=8, yarn=True),
          dict(n_heads=1, dim=24, rot_dim=16, v_dim=40, q_rank=12, kv_rank=20, scale=0.5, dims=6, yarn=False),
          dict(n_heads=6, dim=8, rot_dim=4, v_dim=8, q_rank=64, kv_rank=60, scale=1.0, dims=0, yarn=False),
          dict(n_heads=2, dim=64, rot_dim=32, v_dim=64, q_rank=96, kv_rank=128, scale=0.11, dims=32, yarn=True),
          dict(n_heads=20, dim=16, rot_dim=64, v_dim=16, q_rank=32, kv_rank=512, scale=0.04, dims=64, yarn=True)]


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("shape", LATENT)
def test_the_latent_attention_alone_in_pieces(dtype, shape):
    rng = np.random.default_rng(shape["kv_rank"])
    hidden, eps = 72, 1e-5
    s = dict(shape)
    dims, yarn = s.pop("dims"), s.pop("yarn")
    scaling = dict(type="yarn", factor=3.0, original=40, fast=6.0, slow=1.0) if yarn else None
    pos = P.Rotary(s["rot_dim"], dims, 3000.0, pairing="interleaved", scaling=scaling) if dims else None
    mixer = P.LatentAttention("m.", hidden, eps=eps, position=pos, **s)
    plain = _bind(mixer, rng, dtype, scale=0.2)
    sub = {k[2:]: v for k, v in plain.items()}
    m = {"heads": s["n_heads"], "dim": s["dim"], "rot_dim": s["rot_dim"], "vdim": s["v_dim"], "kv_rank": s["kv_rank"],
         "scale": s["scale"], "rot": {"dims": dims, "base": 3000.0,
                                      "scaling": dict(factor=3.0, original=40, fast=6.0, slow=1.0) if yarn else None}}
    lengths = (150, 66)
    h = [rng.standard_normal((n, hidden)).astype(np.float32) for n in lengths]
    want = [pn.latent_attention_mixer(x.astype(np.float64), sub, m, eps) for x in h]
    # (in bfloat16 the latent is cached a second time, in the order the matrix cores take values in)
    assert mixer.kv_spec() == P.KVSpec(1, mixer.row, values=dtype == "bfloat16")
    assert mixer.row % 16 == 0 and mixer.row >= s["kv_rank"] + s["rot_dim"]
    pool = torch.zeros((8, 1, 64 * mixer.row), dtype=DT[dtype], device=DEV)
    pool[7].fill_(float("nan"))                                # a page of neither sequence: never read
    values = pool.clone() if dtype == "bfloat16" else None
    table = torch.tensor([[5, 0, 3], [2, 6, -1]], dtype=torch.int32, device=DEV)
    got = [np.zeros((n, hidden)) for n in lengths]
    cuts = [(63, 2), (1, 0), (1, 62), (2, 1), (64, 1), (19, 0)]   # up to a page's last place; over the border alone; in a portion
    for seqs, lo, hi in _steps(lengths, cuts):
        ctx = _ctx(mixer.rt, hi, [b - a for a, b in zip(lo, hi)], seqs)
        cache = P.LayerCache(k_pool=pool, v_pool=values, table=table[seqs].contiguous())
        rows = torch.tensor(np.concatenate([h[i][a:b] for i, a, b in zip(seqs, lo, hi)]), device=DEV).to(DT[dtype])
        o = _np(K.sum_parts(mixer.forward(ctx, rows, cache), None, torch.float32))      # (a mixer may hand on partial sums)
        at = 0
        for i, a, b in zip(seqs, lo, hi):
            got[i][a:b] = o[at:at + b - a]
            at += b - a
    for g, w_ in zip(got, want):
        assert np.abs(g - w_).max() <= PART_TOL[dtype] * max(1.0, np.abs(w_).max())
    # without its sink the plain mixer is far away: the comparison above would see a sink that is left out
    far = pn.latent_attention_mixer(h[1].astype(np.float64), dict(sub, sink=np.full(s["n_heads"], -60.0)), m, eps)
    assert np.abs(far - want[1]).max() > 5 * PART_TOL[dtype] * max(1.0, np.abs(want[1]).max())


@pytest.mark.parametrize("dtype", H.DTYPES)
def test_the_feed_forward_alone(dtype):
    rng = np.random.default_rng(4)
    ff = P.ActivatedMLP("f.", 56, 136, "xielu")
    plain = _bind(ff, rng, dtype)
    x = torch.tensor(rng.standard_normal((70, 56)), dtype=DT[dtype])
    want = pn.dense_feed_forward(x.double().numpy(), plain["f.up"], plain["f.down"], plain["f.act"])
    for n in (70, 3):
        got = _np(K.sum_parts(ff.forward(None, x[:n].to(DEV)), None, torch.float32))
        assert np.abs(got - want[:n]).max() <= PART_TOL[dtype] * max(1.0, np.abs(want).max())


def test_a_norm_whose_stored_weight_is_an_offset_from_one():
    rng = np.random.default_rng(8)
    norm = P.RMSNorm("n", 50, 1e-5, offset=1.0, suffix="")
    plain = _bind(norm, rng, "float32")
    x = torch.tensor(rng.standard_normal((9, 50)) * 3, dtype=torch.float32, device=DEV)
    assert np.abs(_np(norm.forward(x, out_dtype=torch.float32)) - pn.offset_norm(_np(x), plain["n"], 1e-5)).max() < 1e-5


# ---------------------------------------------------------------------------
# whole models
# ---------------------------------------------------------------------------
def _run(eng, slot, toks, lo, hi, want="all"):
    return eng.step([(slot, list(toks[lo:hi]))], want=want)


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("name", list(nc.ALL))
def test_a_whole_prompt_then_the_rest_token_by_token(name, dtype):
    toks = H.tokens(name, 150, 1)
    want = H.plain_logits(name, toks)
    eng = H.engine(name, dtype)
    s = eng.alloc_slot()
    got = [_np(_run(eng, s, toks, 0, 100))]
    for t in range(100, 150):                                   # over the border of the second page
        got.append(_np(_run(eng, s, toks, t, t + 1)))
    H.close(np.concatenate(got), want, dtype, f"{name} prompt and decoding")


@pytest.mark.parametrize("dtype", H.DTYPES)
def test_the_first_tokens_one_by_one_and_portions_down_to_two_tokens(dtype):
    name = "nip_a"
    toks = H.tokens(name, 140, 2)
    want = H.plain_logits(name, toks)
    eng = H.engine(name, dtype, n_slots=2)
    a, b = eng.alloc_slot(), eng.alloc_slot()
    one = np.concatenate([_np(_run(eng, a, toks, t, t + 1)) for t in range(70)])          # from the very first token on
    H.close(one, want[:70], dtype, "token by token from the start")
    cuts, at, got = [2, 3, 59, 1, 2, 64, 7, 2], 0, []
    for c in cuts:
        got.append(_np(_run(eng, b, toks, at, at + c)))
        at += c
    H.close(np.concatenate(got), want, dtype, "portions")
    if dtype == "float32":                                      # in 32-bit a row's arithmetic does not depend on the cut
        assert np.abs(np.concatenate(got)[:70] - one).max() <= 2e-5 * np.abs(want).max()


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("name", ["nip_a", "nip_c"])
def test_unequal_batches_against_each_alone_with_slots_and_pages_used_again(name, dtype):
    eng = H.engine(name, dtype, max_tokens=448, n_slots=3)              # 7 pages: the second batch needs the first one's
    for round_, lens in enumerate([(130, 9, 70), (200, 3, 66)]):
        seqs = [H.tokens(name, n + 6, 10 * round_ + i) for i, n in enumerate(lens)]
        slots = [eng.alloc_slot() for _ in seqs]
        assert slots == [0, 1, 2]
        got = [[] for _ in seqs]
        out = _np(eng.step([(s, list(t[:n])) for s, t, n in zip(slots, seqs, lens)], want="all"))
        at = 0
        for i, n in enumerate(lens):
            got[i].append(out[at:at + n])
            at += n
        live = [0, 1, 2]
        for step in range(6):
            if step == 3:                                       # the shortest request ends earlier
                eng.free_slot(slots[1])
                live = [0, 2]
            out = _np(eng.step([(slots[i], [seqs[i][lens[i] + step]]) for i in live], want="all"))
            for j, i in enumerate(live):
                got[i].append(out[j:j + 1])
        for i in live:
            eng.free_slot(slots[i])
        for i, t in enumerate(seqs):
            g = np.concatenate(got[i])
            H.close(g, H.plain_logits(name, t)[:len(g)], dtype, f"{name} round {round_} sequence {i}")
    assert eng.cache.free_pages() == [7] * len(eng.cache.groups)


@pytest.mark.parametrize("dtype", H.DTYPES)
def test_long_decoding_replayed_and_launched(dtype):
    name = "nip_b"
    toks = H.tokens(name, 210, 3)
    want = H.plain_logits(name, toks)
    outs = {}
    for graphs in (True, False):
        eng = H.engine(name, dtype, use_graphs=graphs)
        assert (eng.graphs is not None) == graphs
        s = eng.alloc_slot()
        got = [_np(_run(eng, s, toks, 0, 5))] + [_np(_run(eng, s, toks, t, t + 1)) for t in range(5, 210)]
        outs[graphs] = np.concatenate(got)
        H.close(outs[graphs], want, dtype, f"long decoding, graphs {graphs}")
    assert np.array_equal(outs[True], outs[False])              # a replayed step is the launched step


def test_a_far_key_and_the_sink_decide_and_are_there():
    """On a sharpened model the logits of late positions depend on keys hundreds of positions back and
    on the sink by many times the bound; the engine agrees with the plain implementation that has them."""
    name, dtype = "nip_c", "float32"
    cfg, w = H.plain(name)
    toks = H.tokens(name, 420, 4)
    want = H.plain_logits(name, toks)
    attend = pn.sink_softmax_attention
    try:
        def without_far_keys(scores, values, sink):
            s = scores.copy()
            s[330:, :64] = -1e30                                # the first page, for the late queries
            return attend(s, values, sink)
        pn.sink_softmax_attention = without_far_keys
        no_far = pn.forward(cfg, w, list(toks))
        pn.sink_softmax_attention = lambda s, v, sink: attend(s, v, -1e30)
        no_sink = pn.forward(cfg, w, list(toks))
    finally:
        pn.sink_softmax_attention = attend
    assert H.distance(no_far[330:], want[330:]) > 20 * H.TOL[dtype]
    assert H.distance(no_sink, want) > 20 * H.TOL[dtype]
    eng = H.engine(name, dtype)
    s = eng.alloc_slot()
    got = [_np(_run(eng, s, toks, 0, 400))] + [_np(_run(eng, s, toks, t, t + 1)) for t in range(400, 420)]
    H.close(np.concatenate(got), want, dtype, "far keys and sink")


def test_greedy_generation_through_the_entry_point():
    name = "nip_a"
    cfg, w = H.plain(name)
    prompts = [list(H.tokens(name, 9, 7)), list(H.tokens(name, 30, 8)), list(H.tokens(name, 2, 9))]
    llm = L.Llogos(H.folder(name), dtype="float32", max_context=128, max_batch=2)        # three requests, two at a time
    out = llm.generate(prompts, L.GenerationParams.greedy(max_tokens=10, stop_tokens=()))
    for p, got in zip(prompts, out.tokens):
        assert got == pn.generate_greedy(cfg, w, p, 10)
    assert out.finish_reasons == ["length"] * 3


@pytest.mark.parametrize("dtype", H.DTYPES)
def test_the_trace_runner_on_a_model_of_the_design(tmp_path, dtype):
    name = "nip_c"
    vocab = nc.ALL[name]["vocab"]
    a, b = H.tokens(name, 75, 11), H.tokens(name, 12, 12)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:70], "want": [0, 63, 64, 69]}, {"id": "b", "tokens": b[:9], "want": [8]}], "end": []}]
    for i in range(3):
        steps.append({"step": 1 + i, "entries": [{"id": "a", "tokens": [a[70 + i]], "want": [0]}, {"id": "b", "tokens": [b[9 + i]], "want": [0]}],
                      "end": ["b"] if i == 2 else []})
    steps.append({"step": 4, "entries": [{"id": "a", "tokens": list(a[73:75]), "want": [1]}], "end": ["a"]})
    out = str(tmp_path / "out")
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", H.folder(name), "--dtype", dtype, "--out", out,
           "--max-tokens", "192"]
    p = subprocess.run(cmd, input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.split("\n") if l] == [f"done {i}" for i in range(5)]
    read = lambda i: np.fromfile(os.path.join(out, f"{i}.f32"), dtype="<f4").reshape(-1, vocab)
    pa, pb = H.plain_logits(name, a), H.plain_logits(name, b)
    H.close(read(0), np.concatenate([pa[[0, 63, 64, 69]], pb[8:9]]), dtype, "step 0")
    for i in range(3):
        H.close(read(1 + i), np.concatenate([pa[70 + i:71 + i], pb[9 + i:10 + i]]), dtype, f"step {1 + i}")
    H.close(read(4), pa[74:75], dtype, "step 4")


def test_the_command_line_on_a_model_of_the_design(tmp_path):
    """`random` writes a model folder from a configuration file; generation from token ids prints what the
    plain loop generates; --bench prints its block."""
    name = "nip_b"
    cfg_file = tmp_path / "config.json"
    cfg_file.write_text(json.dumps(nc.ALL[name]))
    out = tmp_path / "model"
    run = lambda *args: subprocess.run([sys.executable, "-m", "daisi-llogos_amd", *args], capture_output=True, text=True, timeout=600, cwd=ROOT)
    p = run("random", "--config", str(cfg_file), "--output-dir", str(out), "--seed", "4")
    assert p.returncode == 0, p.stderr[-2000:]
    cfg, w = pn.load_folder(str(out))
    prompt = list(H.tokens(name, 11, 21))
    p = run("--model", str(out), "--prompt", " ".join(map(str, prompt)), "-n", "6", "-t", "0", "--repeat-penalty", "1.0",
            "--dtype", "float32", "--max-context", "64")
    assert p.returncode == 0, p.stderr[-2000:]
    assert [int(t) for t in p.stdout.split()] == pn.generate_greedy(cfg, w, prompt, 6)
    p = run("--model", str(out), "--bench", "--batch", "2", "-n", "8", "--prompt-len", "20", "--max-context", "64")
    assert p.returncode == 0, p.stderr[-2000:]
    assert "decode" in (p.stdout + p.stderr)
