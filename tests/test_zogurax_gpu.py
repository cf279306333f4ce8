"""The Zogurax design on the GPU against the plain implementation: every mechanism alone, whole
prompts, prompts cut into portions, token-by-token decoding, unequal batches with slots and pages
used again, long decoding over page borders, sensitivity to a far key, to the unit in the softmax's
denominator and to the query's factor, greedy generation through the library's entry point, and the
trace runner and the command line as programs."""
import importlib
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_zogurax as pz
import zogurax_configs as zc
import zogurax_helpers as H

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


def _i32(a):
    return torch.tensor(np.asarray(a), dtype=torch.int32, device=DEV)


def _ctx(rt, lens, new, slots, ids=None):
    """A step that brings new[i] tokens to sequence i, which is lens[i] long afterwards."""
    B, T = len(lens), sum(new)
    tok_seq = np.repeat(np.arange(B), new).astype(np.int32)
    tok_pos = np.concatenate([np.arange(l - n, l) for l, n in zip(lens, new)]).astype(np.int32)
    cu = np.concatenate([[0], np.cumsum(new)])
    return P.StepContext(runtime=rt, n_tokens=T, batch=B, ids=_i32(np.zeros(T) if ids is None else ids), tok_seq=_i32(tok_seq),
                         tok_pos=_i32(tok_pos), slots=_i32(slots), cu_seqlens=cu.tolist(), starts=[l - n for l, n in zip(lens, new)],
                         slot_ids=list(slots), is_decode=max(new) == 1, max_context=max(lens),
                         cu_dev=None if max(new) == 1 else _i32(cu))


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


def _bind(part, rng, dtype, scale=0.3, scaled=None):
    """Random tensors for a part (stored in bfloat16, as a model folder holds them); returns them as float64."""
    tensors, plain = {}, {}
    lim = {"norm": (0.7, 1.3), "taps": (-0.8, 0.8)}
    for spec in part.tensor_specs():
        if spec.kind.startswith("choices:"):
            n = int(spec.kind.split(":")[1])
            rows = np.stack([rng.permutation(n)[:spec.shape[1]] for _ in range(spec.shape[0])])
            tensors[spec.name], plain[spec.name] = torch.tensor(rows, dtype=torch.int32), rows
            continue
        if spec.kind in lim:
            t = torch.tensor(rng.uniform(*lim[spec.kind], size=spec.shape), dtype=torch.bfloat16)
        else:
            t = torch.tensor(rng.standard_normal(spec.shape) * scale * (scaled or {}).get(spec.name, 1.0), dtype=torch.bfloat16)
        tensors[spec.name], plain[spec.name] = t, t.double().numpy()
    part.bind(tensors.get, P.Runtime(DEV, DT[dtype]))
    return plain


def _run(eng, slot, toks, lo, hi):
    return eng.step([(slot, list(toks[lo:hi]))], want="all")


# ---------------------------------------------------------------------------
# mechanisms alone
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("width", [6, 70, 256, 1000, 5000, 20000])
@pytest.mark.parametrize("out", ["float32", "bfloat16"])
def test_the_layer_norm_with_the_residual_sum(width, out):
    rng = np.random.default_rng(width)
    T = 5
    x = rng.standard_normal((T, width)) * 3 + 1.5
    d = rng.standard_normal((3, T, width))
    w = rng.uniform(0.5, 1.5, size=width)
    xt = torch.tensor(x, dtype=torch.float32, device=DEV)
    dt = torch.tensor(d, dtype=torch.float32, device=DEV)
    wt = torch.tensor(w, dtype=torch.float32, device=DEV)
    tol = 2e-5 if out == "float32" else 2e-2
    got = _np(K.layernorm(xt.clone(), wt, 1e-5, DT[out]))
    assert np.abs(got - pz.layer_norm(x, w, 1e-5)).max() <= tol * 5
    x2 = xt.clone()
    got = _np(K.layernorm(x2, wt, 1e-5, DT[out], delta=dt))
    full = _np(xt) + _np(dt).sum(0)
    assert np.abs(got - pz.layer_norm(full, w, 1e-5)).max() <= tol * 5
    assert np.abs(_np(x2) - full).max() <= 1e-5                                # the sum went back to the stream
    x3 = xt.clone()
    got = _np(K.layernorm(x3, wt, 1e-5, DT[out], delta=dt[0], rows=_i32([3, 1]), write_back=False))
    assert np.abs(got - pz.layer_norm((_np(xt) + _np(dt[0]))[[3, 1]], w, 1e-5)).max() <= tol * 5
    assert torch.equal(x3, xt)


@pytest.mark.parametrize("width", [6, 7, 96, 1024])
def test_the_position_vector_is_added(width):
    pos = [0, 1, 63, 64, 1000, 4095]
    x = torch.zeros((len(pos), width), dtype=torch.float32, device=DEV) + 2.0
    K.add_sinusoid(x, _i32(pos), 10000.0)
    assert np.abs(_np(x) - 2.0 - pz.position_vector(pos, width)).max() <= 2e-7


@pytest.mark.parametrize("lengths,cuts", [((19, 6, 1), [(5, 2, 1), (1, 1, 0), (1, 1, 0), (2, 2, 0), (1, 0, 0), (9, 0, 0)]),
                                          ((700, 30, 2), [(640, 29, 1), (1, 1, 1), (59, 0, 0)])])
@pytest.mark.parametrize("taps", [1, 2, 4])
def test_the_convolution_behind_a_projection_over_steps_of_any_size(taps, lengths, cuts):
    """Without its input added, on the first columns of wider rows, with the projected rows as state; a long
    step's blocks take several tokens each."""
    rng = np.random.default_rng(taps)
    W, wide = 70, 77
    w = rng.uniform(-0.8, 0.8, size=(W, taps))
    h = [rng.standard_normal((n, wide)).astype(np.float32) for n in lengths]
    want = [pz.time_convolution(x[:, :W], w) for x in h]
    slots = [2, 0, 3]
    state = torch.zeros((5, taps - 1, W), dtype=torch.float32, device=DEV)
    got = [np.zeros((n, W)) for n in lengths]
    rt = P.Runtime(DEV, torch.float32)
    for seqs, lo, hi in _steps(lengths, cuts):
        ctx = _ctx(rt, hi, [b - a for a, b in zip(lo, hi)], [slots[i] for i in seqs])
        rows = torch.tensor(np.concatenate([h[i][a:b] for i, a, b in zip(seqs, lo, hi)]), device=DEV)
        o = _np(K.causal_conv(ctx, rows[:, :W], torch.tensor(w, dtype=torch.float32, device=DEV), state, torch.float32, add_input=False))
        at = 0
        for i, a, b in zip(seqs, lo, hi):
            got[i][a:b] = o[at:at + b - a]
            at += b - a
    for g, w_ in zip(got, want):
        assert np.abs(g - w_).max() <= 1e-5 * max(1.0, np.abs(w_).max())


def test_the_square_of_relu_on_the_first_columns_of_a_product_in_parts():
    rng = np.random.default_rng(0)
    z = rng.standard_normal((3, 7, 21)).astype(np.float32)
    got = _np(K.activation(torch.tensor(z, device=DEV), "relu2", torch.float32, cols=20))
    assert np.abs(got - pz.squared_relu(z.astype(np.float64).sum(0)[:, :20])).max() <= 1e-5


# (heads, kv heads, key width, value width, hidden, form); the forms are the design's two mixers
MIXERS = [(4, 2, 32, 48, 56, "second"), (3, 3, 16, 40, 64, "first"), (5, 1, 24, 8, 40, "first"), (2, 1, 64, 80, 64, "first"),
          (4, 2, 96, 64, 96, "second"), (2, 2, 128, 128, 64, "second"), (16, 1, 64, 64, 32, "first"), (2, 1, 40, 24, 48, "second")]


def _capped(heads, kv, dk, dv, hidden, form, cap=3.0, temp=(0.6, 5), taps=3):
    second = form == "second"
    return P.CappedAttention(prefix="m.", hidden=hidden, n_heads=heads, n_kv_heads=kv, head_dim=dk, v_dim=dv, scale=0.2, softcap=cap,
                             temp_coef=temp[0], temp_every=temp[1], eps=1e-5, bias=second, unit_sink=second,
                             conv_taps=0 if second else taps, whole_norm=not second, head_gate=not second)


def _plain_mixer(mix, plain, h, form):
    m = {"heads": mix.n_heads, "kv_heads": mix.n_kv_heads, "dim": mix.head_dim, "vdim": mix.v_dim, "scale": mix.scale,
         "softcap": mix.softcap, "q_temp": {"coef": mix.temp_coef, "every": mix.temp_every}}
    return pz.mixer("attention_2" if form == "second" else "attention", m, plain, "m.", h, mix.eps)


@pytest.mark.parametrize("dtype,tile_rows,halves", [("float32", 0, 0), ("bfloat16", 0, 0), ("bfloat16", 64, 1), ("bfloat16", 128, 1),
                                                    ("bfloat16", 128, 2)])
@pytest.mark.parametrize("shape", MIXERS)
def test_the_attention_alone_in_pieces(dtype, tile_rows, halves, shape, monkeypatch):
    """Three sequences cut into steps of several sizes, their pages in any order, a page of NaN that nobody
    may read; queries and keys scaled so that single keys decide.  Shapes that the matrix-core kernels
    take must run there in bfloat16."""
    heads, kv, dk, dv, hidden, form = shape
    monkeypatch.setattr(K, "CAPPED_PREFILL_TILE_ROWS", tile_rows)        # every prompt kernel of the matrix cores in turn
    monkeypatch.setattr(K, "CAPPED_PREFILL_HALVES", halves)
    rng = np.random.default_rng(heads * 100 + dk)
    mix = _capped(*shape)
    plain = _bind(mix, rng, dtype, scaled={"m.q": 2.0, "m.k": 2.0})
    lengths = (150, 70, 3)
    h = [np.asarray(torch.tensor(rng.standard_normal((n, hidden))).to(DT[dtype]).double()) for n in lengths]
    want = [_plain_mixer(mix, plain, x, form) for x in h]
    spec = mix.kv_spec()
    n_pages = 9
    k_pool = torch.zeros((n_pages, kv, 64 * spec.head_dim), dtype=DT[dtype], device=DEV)
    v_pool = torch.zeros((n_pages, kv, 64 * spec.value_dim), dtype=DT[dtype], device=DEV)
    k_pool[4] = float("nan"); v_pool[4] = float("nan")
    pages = {0: [7, 2, 5], 1: [0, 8], 2: [3]}
    slots = [1, 3, 0]
    st = mix.state_spec()
    state = torch.zeros((4,) + st.shape, dtype=torch.float32, device=DEV) if st is not None else None
    fast = dtype == "bfloat16" and dk in (64, 96, 128) and dv in (64, 80, 96, 128)
    if fast:
        monkeypatch.setattr(K, "attention_generic", lambda *a, **k: pytest.fail("the kernel for any shape ran"))
    got = [np.zeros((n, hidden)) for n in lengths]
    cuts = [(60, 9, 1), (1, 1, 1), (1, 1, 1), (3, 58, 0), (1, 1, 0), (2, 0, 0), (64, 0, 0), (1, 0, 0), (17, 0, 0)]
    for seqs, lo, hi in _steps(lengths, cuts):
        ctx = _ctx(mix.rt, hi, [b - a for a, b in zip(lo, hi)], [slots[i] for i in seqs])
        table = np.full((len(seqs), 3), -1, dtype=np.int32)
        for r, i in enumerate(seqs):
            table[r, :len(pages[i])] = pages[i]
        cache = P.LayerCache(k_pool=k_pool, v_pool=v_pool, table=_i32(table), state=state)
        rows = torch.tensor(np.concatenate([h[i][a:b] for i, a, b in zip(seqs, lo, hi)]), dtype=DT[dtype], device=DEV)
        o = _np(K.sum_parts(mix.forward(ctx, rows, cache), None, torch.float32))
        at = 0
        for i, a, b in zip(seqs, lo, hi):
            got[i][a:b] = o[at:at + b - a]
            at += b - a
    for i, (g, w_) in enumerate(zip(got, want)):
        assert np.isfinite(g).all()
        # (bfloat16 queries and keys move a sharp score by a hundredth of its size, and the bend is steep around zero)
        assert np.abs(g - w_).max() <= (2 if dtype == "bfloat16" else 1) * PART_TOL[dtype] * max(1.0, np.abs(w_).max()), f"sequence {i}"


def test_a_far_key_the_unit_and_the_bend_decide_in_the_attention_alone():
    """One key far back is made to stand out; without it, without the unit in the denominator or with the
    scores left unbent the plain result moves by many times the bound, and the kernels agree with the full one."""
    rng = np.random.default_rng(5)
    shape = (2, 1, 64, 80, 64, "second")
    mix = _capped(*shape, cap=6.0, temp=(0.5, 100))
    plain = _bind(mix, rng, "float32", scaled={"m.q": 3.0, "m.k": 3.0})
    n = 330
    h = rng.standard_normal((n, 64))
    h[3] *= 4.0                                                               # a loud early token: its key stands out for many queries
    want = _plain_mixer(mix, plain, h, "second")
    keep = pz.causal_attention
    try:
        def lost(q, k, v, scale, cap, unit_sink, **kw):
            k = k.copy(); k[3] = 0.0
            return keep(q, k, v, scale, cap, unit_sink, **kw)
        pz.causal_attention = lost
        no_key = _plain_mixer(mix, plain, h, "second")
        pz.causal_attention = lambda q, k, v, scale, cap, unit_sink, **kw: keep(q, k, v, scale, cap, False, **kw)
        no_unit = _plain_mixer(mix, plain, h, "second")
        pz.causal_attention = lambda q, k, v, scale, cap, unit_sink, **kw: keep(q, k, v, scale, None, unit_sink, **kw)
        no_bend = _plain_mixer(mix, plain, h, "second")
    finally:
        pz.causal_attention = keep
    size = np.abs(want).max()
    for other in (no_key[300:], no_bend[300:]):
        assert np.abs(other - want[300:]).max() > 100 * PART_TOL["float32"] * size
    assert np.abs(no_unit - want).max() > 100 * PART_TOL["float32"] * size
    for dtype in H.DTYPES:
        mix = _capped(*shape, cap=6.0, temp=(0.5, 100))
        mix.bind({k: torch.tensor(v, dtype=torch.int32 if v.dtype.kind == "i" else torch.bfloat16) for k, v in plain.items()}.get,
                 P.Runtime(DEV, DT[dtype]))
        k_pool = torch.zeros((6, 1, 64 * 64), dtype=DT[dtype], device=DEV)
        v_pool = torch.zeros((6, 1, 64 * 80), dtype=DT[dtype], device=DEV)
        table = _i32([[4, 1, 0, 5, 2, 3]])
        got = []
        for lo, hi in [(0, 257)] + [(t, t + 1) for t in range(257, n)]:
            ctx = _ctx(mix.rt, [hi], [hi - lo], [0])
            cache = P.LayerCache(k_pool=k_pool, v_pool=v_pool, table=table, state=None)
            got.append(_np(K.sum_parts(mix.forward(ctx, torch.tensor(h[lo:hi], dtype=DT[dtype], device=DEV), cache), None, torch.float32)))
        assert np.abs(np.concatenate(got) - want).max() <= PART_TOL[dtype] * size * (1 if dtype == "float32" else 2)


@pytest.mark.parametrize("dtype,form", [("float32", "auto"), ("bfloat16", "auto"), ("bfloat16", "plain"), ("bfloat16", "few"),
                                        ("bfloat16", "tiles64"), ("bfloat16", "tiles128")])
@pytest.mark.parametrize("experts,top,ff,shared,hidden,T", [(5, 2, 40, 24, 96, 9), (1, 1, 16, 8, 32, 3), (4, 4, 24, 0, 48, 70),
                                                           (7, 3, 72, 136, 64, 300), (16, 1, 96, 96, 128, 1), (3, 2, 132, 20, 200, 150),
                                                           (2, 1, 30, 6, 36, 40)])
def test_the_experts_by_table(dtype, form, experts, top, ff, shared, hidden, T, monkeypatch):
    """Every form of the experts' product (chosen by the step, or forced: plain multiply-adds, and on the matrix
    cores tiles of 16, 64 and 128 sorted rows); the last shape has a width that only the plain form takes."""
    monkeypatch.setattr(K, "MOE_PRODUCT", form)
    rng = np.random.default_rng(experts * 10 + top)
    vocab = 37
    moe = P.TableMoE(prefix="f.", hidden=hidden, vocab=vocab, n_experts=experts, top=top, intermediate=ff, shared_intermediate=shared)
    plain = _bind(moe, rng, dtype)
    ids = rng.integers(0, vocab, size=T)
    ids[: min(T, 3)] = [5, 5, 6][: min(T, 3)]                                  # one token twice in a step
    h = np.asarray(torch.tensor(rng.standard_normal((T, hidden))).to(DT[dtype]).double())
    f = {"router": {"experts": experts, "top": top}, "shared": {"ff": shared} if shared else None}
    want = pz.feed_forward(f, plain, "f.", h, ids)
    ctx = _ctx(moe.rt, [T], [T], [0], ids=ids)
    got = _np(moe.forward(ctx, torch.tensor(h, dtype=DT[dtype], device=DEV)))
    assert np.abs(got - want).max() <= PART_TOL[dtype] * max(1.0, np.abs(want).max())
    again = _np(moe.forward(ctx, torch.tensor(h, dtype=DT[dtype], device=DEV)))
    assert np.array_equal(got, again)                                         # a row's sums do not depend on its place in a segment
    with pytest.raises(ValueError):                                            # a table that names an expert that is not there
        bad = P.TableMoE(prefix="f.", hidden=hidden, vocab=vocab, n_experts=experts, top=top, intermediate=ff, shared_intermediate=shared)
        tensors = {k: torch.tensor(v, dtype=torch.int32 if v.dtype.kind == "i" else torch.bfloat16) for k, v in plain.items()}
        tensors["f.table"] = tensors["f.table"] + experts
        bad.bind(tensors.get, P.Runtime(DEV, DT[dtype]))


@pytest.mark.parametrize("dtype", H.DTYPES)
def test_the_loop_entry_alone(dtype):
    rng = np.random.default_rng(2)
    W, T = 40, 6
    part = P.LoopEntry(matrix="loop.in", steps="loop.step", width=W, times=3)
    plain = _bind(part, rng, dtype)
    x, x0, d = (np.asarray(torch.tensor(rng.standard_normal((T, W))).to(DT[dtype]).double()) for _ in range(3))
    f = lambda a: torch.tensor(a, dtype=torch.float32, device=DEV)
    for number, delta in ((0, None), (2, d)):
        got, pending = part.forward(None, f(x), None if delta is None else f(delta), f(x0), number)
        want = pz.loop_entry(x + (0 if delta is None else delta), x0, plain["loop.in"], plain["loop.step"][number])
        assert pending is None and np.abs(_np(got) - want).max() <= PART_TOL[dtype] * np.abs(want).max()
    with pytest.raises(ValueError):
        part.forward(None, f(x), None, f(x0), 3)


# ---------------------------------------------------------------------------
# whole models
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("name", list(zc.ALL))
def test_a_whole_prompt_then_the_rest_token_by_token(name, dtype):
    toks = H.tokens(name, 150, 1)
    want = H.plain_logits(name, toks)
    eng = H.engine(name, dtype)
    s = eng.alloc_slot()
    got = [_np(_run(eng, s, toks, 0, 100))]
    for t in range(100, 150):                                   # over the border of the second page
        got.append(_np(_run(eng, s, toks, t, t + 1)))
    H.close(np.concatenate(got), want, dtype, f"{name} prompt and decoding")


def test_the_residual_stream_after_every_run_of_a_layer():
    name = "zog_a"
    toks = H.tokens(name, 40, 6)
    cfg, w = H.plain(name)
    want = []
    pz.forward(cfg, w, list(toks), want)
    eng = H.engine(name, "float32", use_graphs=False)
    got = []
    for blk in eng.model.layers:
        def wrapped(ctx, x, pending, caches, _o=blk.forward, **kw):
            x, p = _o(ctx, x, pending, caches, **kw)
            got.append(_np(x) + (0 if p is None else _np(K.sum_parts(p, None, torch.float32))))
            return x, p
        blk.forward = wrapped
    _run(eng, eng.alloc_slot(), toks, 0, 40)
    assert len(got) == len(want) == 8
    for i, (g, w_) in enumerate(zip(got, want)):
        assert np.abs(g - w_).max() <= 2e-5 * np.abs(w_).max(), f"run {i}"


@pytest.mark.parametrize("dtype", H.DTYPES)
@pytest.mark.parametrize("name", ["zog_a", "zog_c"])
def test_the_first_tokens_one_by_one_and_portions_down_to_two_tokens(name, dtype):
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
@pytest.mark.parametrize("name", ["zog_a", "zog_c"])
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
@pytest.mark.parametrize("name", ["zog_b", "zog_c"])
def test_long_decoding_replayed_and_launched(name, dtype):
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


@pytest.mark.parametrize("dtype", H.DTYPES)
def test_the_feed_forward_on_a_second_stream_changes_no_bit(dtype, monkeypatch):
    """Steps of few rows queue the feed-forward beside the mixer; with everything on one stream the same kernels
    run one after the other.  Unequal batches, prompts of few rows and single tokens, replayed and launched."""
    name = "zog_a"
    seqs = [H.tokens(name, 40, 30 + i) for i in range(3)]
    outs = {}
    for rows in (64, 0):
        monkeypatch.setattr(P.ParallelBlock, "side_rows", rows)
        for graphs in (True, False):
            eng = H.engine(name, dtype, use_graphs=graphs)
            slots = [eng.alloc_slot() for _ in seqs]
            got = [_np(eng.step([(s, list(t[:n])) for s, t, n in zip(slots, seqs, (20, 3, 9))], want="all"))]
            for step in range(12):
                got.append(_np(eng.step([(s, [t[n + step]]) for s, t, n in zip(slots, seqs, (20, 3, 9))], want="all")))
            outs[(rows, graphs)] = np.concatenate(got)
    first = outs[(64, True)]
    assert all(np.array_equal(first, o) for o in outs.values())
    want = np.concatenate([H.plain_logits(name, t)[:n] for t, n in zip(seqs, (20, 3, 9))])
    H.close(first[:32], want, dtype, "two streams")


def test_far_keys_the_unit_and_the_query_factor_decide_and_are_there():
    """On a sharpened model the logits of late positions depend on keys hundreds of positions back, on the
    unit in the denominator and on the query's factor by many times the bound; the engine agrees with the
    plain implementation that has them."""
    name, dtype = "zog_c", "float32"
    cfg, w = H.plain(name)
    toks = H.tokens(name, 420, 4)
    want = H.plain_logits(name, toks)
    attend, factor = pz.causal_attention, pz.query_temperature
    try:
        def without_far_keys(q, k, v, scale, cap, unit_sink, **kw):
            out = attend(q, k, v, scale, cap, unit_sink, **kw)
            out[330:] = attend(q[330:], k[64:], v[64:], scale, cap, unit_sink, q_positions=np.arange(330, len(q)),
                               k_positions=np.arange(64, len(k)))       # the first page, for the late queries
            return out
        pz.causal_attention = without_far_keys
        no_far = pz.forward(cfg, w, list(toks))
        pz.causal_attention = lambda q, k, v, scale, cap, unit_sink, **kw: attend(q, k, v, scale, cap, False, **kw)
        no_unit = pz.forward(cfg, w, list(toks))
        pz.causal_attention = attend
        pz.query_temperature = lambda pos, coef, every: factor(np.asarray(pos) + 1, coef, every)     # the blocks one position early
        moved = pz.forward(cfg, w, list(toks))
    finally:
        pz.causal_attention, pz.query_temperature = attend, factor
    assert H.distance(no_far[330:], want[330:]) > 20 * H.TOL[dtype]
    assert H.distance(no_unit, want) > 20 * H.TOL[dtype]
    assert H.distance(moved, want) > 20 * H.TOL[dtype]
    for dt in H.DTYPES:
        eng = H.engine(name, dt)
        s = eng.alloc_slot()
        got = [_np(_run(eng, s, toks, 0, 400))] + [_np(_run(eng, s, toks, t, t + 1)) for t in range(400, 420)]
        H.close(np.concatenate(got), want, dt, "far keys, unit and factor")


def test_greedy_generation_through_the_entry_point():
    name = "zog_a"
    cfg, w = H.plain(name)
    prompts = [list(H.tokens(name, 9, 7)), list(H.tokens(name, 30, 8)), list(H.tokens(name, 2, 9))]
    llm = L.Llogos(H.folder(name), dtype="float32", max_context=128, max_batch=2)        # three requests, two at a time
    out = llm.generate(prompts, L.GenerationParams.greedy(max_tokens=10, stop_tokens=()))
    for p, got in zip(prompts, out.tokens):
        assert got == pz.generate_greedy(cfg, w, p, 10)
    assert out.finish_reasons == ["length"] * 3


@pytest.mark.parametrize("dtype", H.DTYPES)
def test_the_trace_runner_on_a_model_of_the_design(tmp_path, dtype):
    name = "zog_a"
    vocab = zc.ALL[name]["vocab"]
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
    name = "zog_d"
    cfg_file = tmp_path / "config.json"
    cfg_file.write_text(json.dumps(zc.ALL[name]))
    out = tmp_path / "model"
    run = lambda *args: subprocess.run([sys.executable, "-m", "daisi-llogos_amd", *args], capture_output=True, text=True, timeout=600, cwd=ROOT)
    p = run("random", "--config", str(cfg_file), "--output-dir", str(out), "--seed", "4")
    assert p.returncode == 0, p.stderr[-2000:]
    cfg, w = pz.load_folder(str(out))
    prompt = list(H.tokens(name, 11, 21))
    p = run("--model", str(out), "--prompt", " ".join(map(str, prompt)), "-n", "6", "-t", "0", "--repeat-penalty", "1.0",
            "--dtype", "float32", "--max-context", "64")
    assert p.returncode == 0, p.stderr[-2000:]
    assert [int(t) for t in p.stdout.split()] == pz.generate_greedy(cfg, w, prompt, 6)
    p = run("--model", str(out), "--bench", "--batch", "2", "-n", "8", "--prompt-len", "20", "--max-context", "64")
    assert p.returncode == 0, p.stderr[-2000:]
    assert "decode" in (p.stdout + p.stderr)
