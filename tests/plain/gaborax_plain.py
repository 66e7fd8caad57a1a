"""A plain, slow implementation of the Gaborax decoder on the CPU, one function per mechanism.

It shares no code with the engine: it reads a config dictionary and a dictionary of tensors and computes with ordinary
tensor expressions. ``dtype`` says what the engine's storage type is; the places where the engine rounds to it are the
places where ``rnd`` is applied here (the inputs and results of matrix products, cached keys and values, the attention's
result), everything else is 32-bit.

Notation: x is the 32-bit residual stream [T, W]; a layer is
    x += ls1 * unit(mixer(x)) * (1 + w1);   x += ls2 * unit(ff(x)) * (1 + w2)
with unit(v) = v / sqrt(mean(v^2) + eps). H query heads on G key/value heads, D channels a key, Dv a value.
"""
from __future__ import annotations

import math

import torch


def rnd(t: torch.Tensor, dtype) -> torch.Tensor:
    return t.to(dtype).float()


def linear(x, w, b=None, dtype=torch.float32):
    y = rnd(x, dtype) @ w.float().T
    if b is not None:
        y = y + b.float()
    return y


def unit(v, eps):
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def norm_one_plus(v, w, eps):
    """RMS norm whose stored weight lies around zero."""
    return unit(v, eps) * (1.0 + w.float())


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def frequencies(rot: dict):
    """(f [dims/2], magnitude): the angle of pair i at position p is p * f[i]; cos and sin are multiplied by the magnitude.
    With ``scaling`` the frequencies of slowly turning pairs are divided by ``factor``, fast ones stay, and those between
    are blended by a ramp over the pair index."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f.float(), 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def where(turns):       # the pair index whose wavelength fits `turns` times into the original length
        return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(where(float(sc["fast"]))), 0)
    hi = min(math.ceil(where(float(sc["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
    f = f / factor * ramp + f * (1 - ramp)
    return f.float(), 0.1 * math.log(factor) + 1.0


def rotate(v, positions, rot: dict, interleaved: bool):
    """v [T, heads, D]: the first rot.dims channels of every head turn by the token's position; pairs are (i, i + dims/2),
    or neighbours (2i, 2i + 1) if ``interleaved``."""
    dims = int(rot["dims"])
    f, mag = frequencies(rot)
    a = positions.float()[:, None] * f[None, :]
    c, s = (a.cos() * mag)[:, None, :], (a.sin() * mag)[:, None, :]
    out = v.clone()
    if interleaved:
        x, y = v[..., 0:dims:2], v[..., 1:dims:2]
        out[..., 0:dims:2] = x * c - y * s
        out[..., 1:dims:2] = y * c + x * s
    else:
        h = dims // 2
        x, y = v[..., :h], v[..., h:dims]
        out[..., :h] = x * c - y * s
        out[..., h:dims] = y * c + x * s
    return out


def project_kv(h, positions, kind: str, m: dict, t: dict, pre: str, eps, dtype):
    """Keys [T, G, D] (normed over the whole projection, rotated, rounded as the cache holds them) and values [T, G, Dv]."""
    G, D, Dv = int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    biased = kind == "attention_2"
    k = linear(h, t[pre + "k"], t[pre + "k.b"] if biased else None, dtype)
    v = linear(h, t[pre + "v"], t[pre + "v.b"] if biased else None, dtype)
    k = unit(k, eps) * t[pre + "k.norm"].float()
    k = k.view(-1, G, D)
    rot = m.get("rot")
    if rot and int(rot.get("dims", 0)):
        k = rotate(k, positions, rot, interleaved=biased)
    return rnd(k, dtype), rnd(v, dtype).view(-1, G, Dv)


def attend(q, keys, values, positions, key_positions, scale, softcap=None, gate=None):
    """q [T, H, D] at ``positions`` over keys [J, G, D] / values [J, G, Dv] at ``key_positions``: softmax over the keys at or
    before a query of scale * q.k, capped to softcap * tanh(. / softcap) if ``softcap``; head h times sigmoid(gate[t, h])."""
    H, G = q.shape[1], keys.shape[1]
    kk = keys.repeat_interleave(H // G, dim=1)
    vv = values.repeat_interleave(H // G, dim=1)
    score = torch.einsum("thd,jhd->htj", q, kk) * float(scale)
    if softcap:
        score = float(softcap) * torch.tanh(score / float(softcap))
    seen = key_positions[None, :] <= positions[:, None]
    score = score.masked_fill(~seen[None], float("-inf"))
    o = torch.einsum("htj,jhd->thd", torch.softmax(score, -1), vv)
    if gate is not None:
        o = o * torch.sigmoid(gate)[:, :, None]
    return o


def project_q(h, positions, kind: str, m: dict, t: dict, pre: str, eps, dtype):
    """Queries [T, H, D]: normed over the whole projection, rotated, rounded."""
    H, D = int(m["heads"]), int(m["dim"])
    biased = kind == "attention_2"
    q = linear(h, t[pre + "q"], t[pre + "q.b"] if biased else None, dtype)
    q = (unit(q, eps) * t[pre + "q.norm"].float()).view(-1, H, D)
    rot = m.get("rot")
    if rot and int(rot.get("dims", 0)):
        q = rotate(q, positions, rot, interleaved=biased)
    return rnd(q, dtype)


def attention(h, positions, kind: str, m: dict, t: dict, pre: str, eps, dtype, keys, values, key_positions):
    """h [T, W]: the mixer's input at ``positions``; keys [J, G, D] / values [J, G, Dv] at ``key_positions`` (this call's
    tokens included). ``attention_2`` has biases, neighbouring rotation pairs and capped scores; ``attention`` has a gate
    per head."""
    H, Dv = int(m["heads"]), int(m["vdim"])
    T = h.shape[0]
    q = project_q(h, positions, kind, m, t, pre, eps, dtype)
    gate = linear(h, t[pre + "g"], None, dtype) if pre + "g" in t else None
    o = attend(q, keys, values, positions, key_positions, m["scale"], m.get("softcap"), gate)
    return linear(rnd(o, dtype).reshape(T, H * Dv), t[pre + "o"], None, dtype)


def expert(h, t, pre, dtype):
    a = torch.relu(linear(h, t[pre + "up"], None, dtype)) ** 2
    return linear(a, t[pre + "down"], None, dtype)


def route(h, mlp: dict, t: dict, pre: str, dtype):
    """(chosen [T, top], weights [T, top]): softmax over all router outputs; the choice adds the correction, the weights
    do not, and are divided by their sum."""
    top = int(mlp["router"]["top"])
    z = linear(h, t[pre + "router"], None, dtype)
    s = torch.softmax(z, -1)
    chosen = torch.topk(s + t[pre + "correction"].float(), top, dim=-1).indices
    w = torch.gather(s, 1, chosen)
    return chosen, w / (w.sum(-1, keepdim=True) + 1e-20)


def experts(h, mlp: dict, t: dict, pre: str, dtype):
    """Routed experts (the last ``identity`` router outputs stand for the input itself), plus the shared expert times a
    sigmoid of one number a token."""
    E = int(mlp["router"]["experts"])             # router outputs E .. E + identity - 1 stand for the input itself
    chosen, w = route(h, mlp, t, pre, dtype)
    hr = rnd(h, dtype)
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        for k in range(chosen.shape[1]):
            e = int(chosen[i, k])
            y = hr[i] if e >= E else expert(h[i:i + 1], t, f"{pre}e{e}.", dtype)[0]
            out[i] += w[i, k] * y
    if pre + "shared.up" in t:
        gate = torch.sigmoid(linear(h, t[pre + "shared.sg"], None, dtype))
        out = out + gate * expert(h, t, pre + "shared.", dtype)
    return out


def forward(cfg: dict, t: dict, token_ids, dtype=torch.float32, start: int = 0, state: dict | None = None,
            trace: list | None = None):
    """Logits [T, vocab] of the tokens at positions start .. start + T - 1; ``state`` carries a sequence's keys and values
    from one call to the next (pass the same dictionary again). ``trace`` collects the residual stream after every layer."""
    ids = torch.as_tensor(token_ids, dtype=torch.long)
    T = ids.numel()
    pos = torch.arange(start, start + T)
    eps = float(cfg["norm"]["eps"])
    x = t["embed"].float()[ids]
    state = state if state is not None else {}
    now = {}
    for i, layer in enumerate(cfg["layers"]):
        L, m, kind = f"l{i}.", layer["mixer"], layer["type"]
        src = m.get("kv_from")
        if src is None:
            k, v = project_kv(x, pos, kind, m, t, L + "mix.", eps, dtype)
            old = state.get(i)
            now[i] = (k, v, pos) if old is None else (torch.cat([old[0], k]), torch.cat([old[1], v]), torch.cat([old[2], pos]))
            state[i] = now[i]
        kv = now[i if src is None else int(src)]
        y = attention(x, pos, kind, m, t, L + "mix.", eps, dtype, *kv)
        x = x + t[L + "ls1"].float() * norm_one_plus(rnd(y, dtype), t[L + "norm1"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            y = experts(x, mlp, t, L + "mlp.", dtype)
            x = x + t[L + "ls2"].float() * norm_one_plus(rnd(y, dtype), t[L + "norm2"], eps)
        if trace is not None:
            trace.append(x.clone())
    n = rnd(norm_one_plus(x, t["final.norm"], eps), dtype)
    return linear(n, t["embed"], None, dtype)
