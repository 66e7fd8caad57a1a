"""Small Gaborax configurations for the tests: sizes that are no powers of two and differ from each other, every option
on and off.

A: both kinds of attention; three query heads a key/value head and one; a rotation over part of a head and over all of it;
   scaled frequencies and a score cap; a layer that reads another layer's keys and values; experts with and without
   identity experts and a shared expert; a layer without a feed-forward.
B: head sizes the matrix-unit attention kernels take (32, 64), as many key/value heads as query heads, values
   wider and narrower than keys, one expert a token and all at once, a feed-forward of identity experts only.
C: a wide head (96) beside a narrow one, a cap so low that every score bends, frequencies scaled by a large factor.
"""
from __future__ import annotations


def _rot(base, dims, scaling=None):
    r = {"base": base, "dims": dims}
    if scaling:
        r["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return r


def _mix(heads, kv_heads, dim, vdim, scale, rot=None, softcap=None, kv_from=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "scale": scale}
    if kv_heads is not None:
        m["kv_heads"] = kv_heads
    if rot is not None:
        m["rot"] = rot
    if softcap is not None:
        m["softcap"] = softcap
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _moe(ff, experts, identity, top, shared=None):
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "identity": identity, "top": top}}
    if shared:
        mlp["shared"] = {"ff": shared}
    return mlp


def _layer(kind, mixer, mlp=None):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


A = {
    "architecture": "Gaborax", "vocab": 211, "width": 88, "norm": {"eps": 3e-5},
    "layers": [
        _layer("attention", _mix(6, 2, 20, 20, 0.25, _rot(1e4, 12)), _moe(40, 5, 2, 2, shared=24)),
        _layer("attention_2", _mix(3, 1, 24, 24, 0.2, _rot(5e3, 24, (4.0, 64, 8.0, 1.0)), softcap=6.0), _moe(16, 3, 0, 3)),
        _layer("attention", _mix(6, 2, 20, 20, 0.3, _rot(1e4, 12), kv_from=0)),
        _layer("attention_2", _mix(2, 2, 16, 12, 0.3, _rot(100.0, 8)), _moe(32, 7, 1, 1, shared=48)),
    ],
}

B = {
    "architecture": "Gaborax", "vocab": 150, "width": 128, "norm": {"eps": 1e-6},
    "layers": [
        _layer("attention_2", _mix(4, 2, 64, 64, 0.125, _rot(1e5, 64, (8.0, 32, 4.0, 0.5)), softcap=4.0), _moe(48, 4, 0, 1, shared=32)),
        _layer("attention", _mix(4, 4, 32, 32, 0.18, _rot(50.0, 32)), _moe(24, 6, 3, 4)),
        _layer("attention", _mix(4, 4, 32, 32, 0.2, _rot(50.0, 32), kv_from=1), _moe(0, 0, 2, 1, shared=40)),
        _layer("attention", _mix(2, 1, 32, 40, 0.2), _moe(56, 2, 1, 3)),
        _layer("attention_2", _mix(8, 2, 32, 32, 0.17, _rot(2e4, 16)), None),
    ],
}

C = {
    "architecture": "Gaborax", "vocab": 97, "width": 72, "norm": {"eps": 1e-5},
    "layers": [
        _layer("attention", _mix(3, 3, 96, 96, 0.1, _rot(2e4, 96)), _moe(20, 9, 4, 2, shared=20)),
        _layer("attention_2", _mix(5, 1, 8, 8, 0.5, _rot(10.0, 8, (16.0, 16, 2.0, 0.25)), softcap=0.75), _moe(12, 2, 0, 2)),
    ],
}

CASES = {"A": (A, 31, 0.1, 0.15), "B": (B, 32, 0.12, 0.1), "C": (C, 33, 0.1, 0.2)}      # config, seed, std of matrices, std of norm weights
