"""Small Modinex configurations for the tests: sizes that are no powers of two, every option on and off.

X: norm in 3 groups; a gla layer first (with a feed-forward), attention with grouped kv heads, a rotation over part
   of the head and a short chunk (no feed-forward), attention with as many kv heads as heads and the whole head
   rotated, a gla layer without feed-forward last.
Y: one norm group; attention without chunks, without rotation and without a 'kv_heads' entry; two gla layers in a row;
   values wider than keys.
"""
from __future__ import annotations


def _attention(heads, dim, vdim, scale, kv_heads=None, rot=None, mask=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "scale": scale}
    if kv_heads is not None:
        m["kv_heads"] = kv_heads
    if rot is not None:
        m["rot"] = {"base": rot[0], "dims": rot[1]}
    if mask is not None:
        m["mask"] = {"size": mask}
    return m


def _layer(kind, mixer, ff=None):
    return {"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}


X = {
    "architecture": "Modinex", "vocab": 211, "width": 96, "max_positions": 256, "norm": {"eps": 3e-5, "groups": 3},
    "layers": [
        _layer("gla", {"heads": 2, "dim": 20, "vdim": 24, "tau": 7.0}, ff=136),
        _layer("attention", _attention(6, 24, 16, 0.3, kv_heads=2, rot=(1e4, 12), mask=24)),
        _layer("attention", _attention(4, 32, 40, 0.2, kv_heads=4, rot=(5e5, 32), mask=50), ff=72),
        _layer("gla", {"heads": 3, "dim": 36, "vdim": 16, "tau": 3.0}),
    ],
}

Y = {
    "architecture": "Modinex", "vocab": 150, "width": 80, "max_positions": 200, "norm": {"eps": 1e-6, "groups": 1},
    "layers": [
        _layer("attention", _attention(5, 16, 28, 0.25), ff=100),
        _layer("gla", {"heads": 1, "dim": 68, "vdim": 12, "tau": 1.5}),
        _layer("gla", {"heads": 4, "dim": 8, "vdim": 72, "tau": 20.0}, ff=64),
        _layer("attention", _attention(2, 40, 8, 0.15, kv_heads=1, rot=(100.0, 40), mask=17)),
    ],
}

CASES = {"X": (X, 11, 0.09, 0.15), "Y": (Y, 12, 0.12, 0.1)}      # config, seed, std of matrices, std of norm weights around 1
