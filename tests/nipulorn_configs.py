"""Small configurations of the Nipulorn design for tests.  Between them every size differs from
layer to layer and from the others of its layer (heads, unrotated, rotated and value dimensions,
ranks, widths that are no multiple of 16), the layer kinds come in several orders, with and without a
feed-forward behind either kind, and the constants take values that are 1, absent or unequal
(embedding and logit scale, taps, rotated dimensions fewer than the rotated part, no scaling rule)."""


def _latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, dims=None, base=10000.0, scaling=None, ff=None):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                      "scale": scale, "rot": {"base": base, "dims": rot_dim if dims is None else dims, "scaling": scaling}},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _wkv(heads, dim, ff=None, decay_rank=None):
    mixer = {"heads": heads, "dim": dim}
    if decay_rank is not None:
        mixer["decay_rank"] = decay_rank
    return {"type": "wkv", "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


YARN = {"factor": 4.0, "original": 48, "fast": 8.0, "slow": 1.5}

NIP_A = {   # latent first; a feed-forward behind both kinds and behind neither; yarn; a row that needs padding
    "architecture": "Nipulorn", "vocab": 211, "width": 96, "embedding": {"scale": 4.0}, "logit_scale": 0.25,
    "norm": {"eps": 1e-6}, "canon": {"taps": 3},
    "layers": [_latent(3, 32, 8, 24, 40, 48, 0.35, scaling=YARN, ff=160), _wkv(2, 40, ff=128, decay_rank=12),
               _latent(2, 16, 16, 48, 24, 20, 0.5, dims=8), _wkv(5, 16, decay_rank=8)],
    "torch_dtype": "bfloat16",
}

NIP_B = {   # one tap (no history), scales of one, a single head, two latent layers with the same cache row
    "architecture": "Nipulorn", "vocab": 130, "width": 64, "embedding": {"scale": 1.0}, "logit_scale": 1.0,
    "norm": {"eps": 1e-5}, "canon": {"taps": 1},
    "layers": [_wkv(1, 32, decay_rank=4), _latent(1, 24, 4, 16, 16, 28, 0.6, base=500.0, scaling={"factor": 1.0, "original": 32, "fast": 4.0, "slow": 1.0}),
               _latent(4, 8, 4, 8, 32, 28, 1.0, dims=0)],
    "torch_dtype": "bfloat16",
}

NIP_C = {   # five taps, recurrent layers only but one, head sizes that are no multiple of 16 or of the wave
    "architecture": "Nipulorn", "vocab": 97, "width": 80, "embedding": {"scale": 9.0}, "logit_scale": 2.0,
    "norm": {"eps": 1e-5}, "canon": {"taps": 5},
    "layers": [_wkv(3, 24, ff=96, decay_rank=16), _wkv(2, 72, decay_rank=6), _latent(5, 16, 32, 16, 48, 64, 0.25, scaling=YARN, ff=72),
               _wkv(7, 8, ff=40, decay_rank=5)],
    "torch_dtype": "bfloat16",
}

ALL = {"nip_a": NIP_A, "nip_b": NIP_B, "nip_c": NIP_C}
