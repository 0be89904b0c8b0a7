"""Small Lusolix configurations for the tests: sizes that are no powers of two and differ from each other, every
option on and off.

P: three taps; layers with experts (2 of 5), a dense feed-forward, and none; a rotation over all and over part of the
   rotated channels; windows of 24 and 50 and a layer without one; a residual multiplier below one.
Q: one tap (a convolution without state); experts used all at once (3 of 3) and one at a time (1 of 4); a latent
   wider than the model; five taps in R.
"""
from __future__ import annotations


def _mixer(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, rot=None, mask=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale}
    if rot is not None:
        m["rot"] = {"base": rot[0], "dims": rot[1]}
    if mask is not None:
        m["mask"] = {"size": mask}
    return m


def _layer(mixer, dense=None, moe=None):
    mlp = None
    if dense:
        mlp = {"kind": "dense", "ff": dense}
    if moe:
        mlp = {"kind": "moe", "expert": {"ff": moe[0]}, "router": {"experts": moe[1], "top": moe[2]}}
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


P = {
    "architecture": "Lusolix", "vocab": 211, "width": 96, "max_positions": 320, "norm": {"eps": 3e-5}, "residual_mult": 0.5,
    "canon": {"taps": 3},
    "layers": [
        _layer(_mixer(3, 20, 12, 24, 40, 36, 0.2, rot=(1e4, 12), mask=24), moe=(40, 5, 2)),
        _layer(_mixer(2, 16, 8, 8, 24, 72, 0.25, rot=(5e5, 4), mask=50), dense=136),
        _layer(_mixer(5, 8, 4, 12, 56, 20, 0.3, rot=(100.0, 4))),
        _layer(_mixer(1, 28, 6, 40, 16, 44, 0.18, rot=(1e6, 6), mask=7), moe=(24, 7, 3)),
    ],
}

Q = {
    "architecture": "Lusolix", "vocab": 150, "width": 80, "max_positions": 200, "norm": {"eps": 1e-6}, "residual_mult": 1.0,
    "canon": {"taps": 1},
    "layers": [
        _layer(_mixer(4, 12, 20, 10, 32, 100, 0.3, rot=(1e3, 20), mask=33), moe=(16, 3, 3)),
        _layer(_mixer(2, 36, 2, 36, 20, 12, 0.15, rot=(50.0, 2), mask=64), moe=(52, 4, 1)),
        _layer(_mixer(3, 24, 16, 16, 48, 40, 0.22, mask=5), dense=60),
    ],
}

R = {
    "architecture": "Lusolix", "vocab": 97, "width": 72, "max_positions": 160, "norm": {"eps": 1e-5}, "residual_mult": 1.7,
    "canon": {"taps": 5},
    "layers": [
        _layer(_mixer(2, 24, 8, 20, 28, 24, 0.2, rot=(1e4, 8), mask=16), dense=100),
        _layer(_mixer(6, 4, 4, 4, 12, 8, 0.5, rot=(10.0, 4), mask=40), moe=(32, 9, 2)),
    ],
}

CASES = {"P": (P, 21, 0.1, 0.15), "Q": (Q, 22, 0.12, 0.1), "R": (R, 23, 0.1, 0.2)}      # config, seed, std of matrices, std of norm weights around 1
