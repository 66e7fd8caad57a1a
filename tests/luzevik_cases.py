"""Small Luzevik configurations for the tests: sizes that are no powers of two and differ from each other, every option on
and off.

A: both kinds of layer; a latent layer whose rows two later layers read; a second latent of other sizes whose cached row
   does not come in whole 16-byte pieces; three query heads a key/value head in the attention beside the recurrence, two
   value heads a query/key head in the recurrence, four taps; a rotation over part of a head with scaled frequencies; dense
   and routed feed-forwards and a layer without one.
B: sizes the matrix-unit kernels take; keys and values of one size in the softmax attention (the kernel library's own
   attention operation); as many key/value heads as heads; two taps; one expert a token, and all experts at once; the
   parallel layer first.
C: recurrence keys of 160 channels (eight lanes a column), one tap (no convolution state), an unscaled rotation over the
   whole head, an embedding scale of 1, a latent without rotated channels.
"""
from __future__ import annotations


def _rot(base, dims, factor=None):
    r = {"base": base, "dims": dims}
    if factor:
        r["scaling"] = {"factor": factor}
    return r


def _latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base=1e4, kv_from=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale,
         "rot": _rot(base, rot_dim)}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m}


def _parallel(left, right):
    return {"type": "parallel", "mixer": {"left": left, "right": right}}


def _left(heads, kv_heads, dim, vdim, scale, rot=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rot:
        m["rot"] = rot
    return m


def _right(heads, kv_heads, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def _with(layer, mlp):
    return {**layer, "mlp": mlp}


A = {
    "architecture": "Luzevik", "vocab": 211, "width": 88, "norm": {"eps": 3e-5}, "embedding": {"scale": 2.5},
    "layers": [
        _with(_latent(3, 12, 8, 20, 24, 40, 0.3), _dense(56)),
        _with(_parallel(_left(6, 2, 20, 12, 0.25, _rot(1e4, 8, 4.0)), _right(4, 2, 12, 20, 4)), _moe(24, 5, 2)),
        _with(_latent(3, 12, 8, 20, 32, 40, 0.2, kv_from=0), _moe(40, 3, 3)),
        _with(_latent(2, 10, 6, 14, 16, 36, 0.35, base=500.0), None),
        _with(_latent(5, 4, 8, 8, 24, 40, 0.4, kv_from=0), _dense(30)),
    ],
}

B = {
    "architecture": "Luzevik", "vocab": 150, "width": 128, "norm": {"eps": 1e-6}, "embedding": {"scale": 0.7},
    "layers": [
        _with(_parallel(_left(4, 4, 64, 64, 0.125, _rot(1e5, 32, 2.0)), _right(2, 2, 32, 48, 2)), _moe(48, 4, 1)),
        _with(_latent(4, 32, 16, 32, 64, 64, 0.15), _moe(16, 3, 3)),
        _with(_latent(20, 16, 16, 16, 48, 64, 0.18, kv_from=1), _dense(96)),
        _with(_parallel(_left(8, 2, 32, 32, 0.2, _rot(50.0, 16)), _right(6, 3, 64, 16, 3)), _dense(64)),
    ],
}

C = {
    "architecture": "Luzevik", "vocab": 97, "width": 72, "norm": {"eps": 1e-5}, "embedding": {"scale": 1.0},
    "layers": [
        _with(_parallel(_left(2, 1, 24, 40, 0.2, _rot(1e3, 24)), _right(2, 1, 160, 24, 1)), _dense(100)),
        _with({"type": "latent_attention", "mixer": {"heads": 2, "dim": 24, "rot_dim": 0, "vdim": 12, "q_rank": 20, "kv_rank": 48,
                                                      "scale": 0.25}}, _moe(20, 7, 2)),
        _with(_parallel(_left(3, 3, 16, 8, 0.3), _right(3, 1, 20, 12, 5)), None),
    ],
}

CASES = {"A": (A, 31, 0.1, 0.15), "B": (B, 32, 0.08, 0.1), "C": (C, 33, 0.1, 0.2)}      # config, seed, std of matrices, std of norm weights around 1
