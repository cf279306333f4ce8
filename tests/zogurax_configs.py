"""Small configurations of the Zogurax design for tests.  Between them every size differs from layer
to layer and from the others of its layer (heads, key/value heads equal to the heads, half of them
and one; key and value widths that differ either way; widths that are no multiple of 16), the two
layer types come in several orders, with and without a feed-forward, the looped run starts at the
first layer, later, covers one layer or is absent and is gone through once, twice and three times,
and the constants take small values that matter within a test's length (a query factor that changes
every 3 or 7 positions, scores bent at 2 or 4), are absent, or make a mechanism trivial (one tap,
one expert, top equal to the experts)."""


def _mixer(heads, kv_heads, dim, vdim, scale, softcap=None, temp=None, conv=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if softcap is not None:
        m["softcap"] = softcap
    if temp is not None:
        m["q_temp"] = {"coef": temp[0], "every": temp[1]}
    if conv is not None:
        m["conv"] = conv
    return m


def _moe(experts, top, ff, shared_ff):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}, "shared": {"ff": shared_ff}}


def first(heads, kv_heads, dim, vdim, scale, softcap, temp, conv, mlp=None):
    return {"type": "attention", "mixer": _mixer(heads, kv_heads, dim, vdim, scale, softcap, temp, conv), "mlp": mlp}


def second(heads, kv_heads, dim, vdim, scale, softcap, temp, mlp=None):
    return {"type": "attention_2", "mixer": _mixer(heads, kv_heads, dim, vdim, scale, softcap, temp), "mlp": mlp}


ZOG_A = {   # the loop starts behind the first layer and is gone through three times; top 2 and 3; a layer without a feed-forward
    "architecture": "Zogurax", "vocab": 211, "width": 96, "norm": {"eps": 1e-5},
    "layers": [second(4, 2, 32, 48, 0.3, 4.0, (0.7, 3), _moe(5, 2, 40, 24)),
               first(3, 3, 16, 40, 0.4, 2.0, (0.4, 7), 3, _moe(4, 3, 24, 56)),
               second(6, 1, 24, 16, 0.25, 3.0, (1.1, 5)),
               first(2, 1, 48, 32, 0.2, 6.0, (0.2, 2), 5, _moe(3, 1, 32, 8))],
    "loop": {"start": 1, "stop": 3, "times": 3},
    "torch_dtype": "bfloat16",
}

ZOG_B = {   # no loop; one tap (no history); one expert; top = experts; a width that is no multiple of 16; 5 query heads a kv head
    "architecture": "Zogurax", "vocab": 130, "width": 72, "norm": {"eps": 1e-6},
    "layers": [first(5, 1, 24, 8, 0.5, 5.0, (0.9, 4), 1, _moe(1, 1, 48, 16)),
               first(2, 2, 40, 56, 0.3, 2.5, (0.5, 64), 2, _moe(2, 2, 16, 32)),
               second(1, 1, 16, 24, 0.6, 8.0, (0.3, 1))],
    "loop": None,
    "torch_dtype": "bfloat16",
}

ZOG_C = {   # head shapes that the matrix-core kernels take (64/80, 96/64, 128/128, 64/64); the loop is the whole model, twice
    "architecture": "Zogurax", "vocab": 190, "width": 128, "norm": {"eps": 1e-5},
    "layers": [first(4, 2, 64, 80, 0.15, 6.0, (0.6, 50), 4, _moe(6, 2, 64, 32)),
               second(2, 1, 96, 64, 0.12, 5.0, (0.5, 33), _moe(4, 1, 48, 64)),
               second(2, 2, 128, 128, 0.1, 7.0, (0.4, 90)),
               first(3, 1, 64, 64, 0.15, 4.0, (0.8, 20), 2, _moe(3, 3, 32, 16))],
    "loop": {"start": 0, "stop": 4, "times": 2},
    "torch_dtype": "bfloat16",
}

ZOG_D = {   # one looped layer, once; the loop's last layer is the model's last
    "architecture": "Zogurax", "vocab": 67, "width": 48, "norm": {"eps": 1e-5},
    "layers": [second(2, 2, 16, 16, 0.4, 3.0, (0.5, 6), _moe(2, 1, 24, 24)),
               first(4, 2, 8, 24, 0.5, 2.0, (0.6, 9), 3, _moe(7, 4, 8, 40))],
    "loop": {"start": 1, "stop": 2, "times": 1},
    "torch_dtype": "bfloat16",
}

ALL = {"zog_a": ZOG_A, "zog_b": ZOG_B, "zog_c": ZOG_C, "zog_d": ZOG_D}
