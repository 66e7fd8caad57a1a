"""A plain, slow implementation of the Luzevik decoder on the CPU, one function per mechanism.

It shares no code with the engine: it reads a config dictionary and a dictionary of tensors and computes with ordinary
tensor expressions. ``dtype`` says what the engine's storage type is; the places where the engine rounds to it are the
places where ``rnd`` is applied here (inputs of matrix products and those of their results that the engine stores, cached
rows, rotated queries, each sublayer's result), and everything else is 32-bit.

Notation: x is the 32-bit residual stream [T, W]; a layer is
    x += unit(mixer(x)) * w1;   x += unit(ff(x)) * w2          (the second only with a feed-forward)
with unit(v) = v / sqrt(mean(v^2) + eps): the sublayers read the stream itself and only their results are normed.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def rnd(t: torch.Tensor, dtype) -> torch.Tensor:
    return t.to(dtype).float()


def linear(x, w, b=None, dtype=torch.float32):
    y = rnd(x, dtype) @ w.float().T
    if b is not None:
        y = y + b.float()
    return y


def unit(v, eps):
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def rms(v, w, eps):
    return unit(v, eps) * w.float()


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def frequencies(rot: dict):
    """f [dims/2]: pair i turns by p * f[i] at position p; with linear scaling every f is divided by the factor."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if sc:
        f = f / float(sc["factor"])
    return f.float()


def rotate_half(v, positions, rot: dict | None):
    """v [T, heads, D]: of every head's first rot.dims channels, channel i and channel i + dims/2 turn as a pair."""
    dims = int(rot["dims"]) if rot else 0
    if dims == 0:
        return v
    a = positions.float()[:, None] * frequencies(rot)[None, :]
    c, s = a.cos()[:, None, :], a.sin()[:, None, :]
    h = dims // 2
    x, y = v[..., :h], v[..., h:dims]
    out = v.clone()
    out[..., :h] = x * c - y * s
    out[..., h:dims] = y * c + x * s
    return out


def softmax_attention(q, k, v, scale, sink=None):
    """q [T, H, D], k [T, H, D], v [T, H, Dv] of one sequence (keys already spread over the query heads), causal.
    ``sink`` [H]: one more term exp(sink) in each row's denominator, with no key and no value."""
    T = q.shape[0]
    s = torch.einsum("thd,jhd->htj", q, k) * scale
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    s = s.masked_fill(~mask, float("-inf"))
    if sink is None:
        p = torch.softmax(s, dim=-1)
    else:
        z = sink.float()[:, None, None].expand(-1, T, 1)
        p = torch.softmax(torch.cat([s, z], dim=-1), dim=-1)[..., :T]
    return torch.einsum("htj,jhd->thd", p, v)


def latent_rows(h, m, t, pre, eps, positions, dtype):
    """What a latent layer caches per token: (c [T, kv_rank], rotated shared key part [T, rot_dim])."""
    R, Dr = int(m["kv_rank"]), int(m["rot_dim"])
    low = linear(h, t[pre + "dkv"], dtype=dtype)
    c = rnd(rms(low[:, :R], t[pre + "dkv.norm"], eps), dtype)
    kr = rotate_half(low[:, None, R:R + Dr], positions, m.get("rot"))[:, 0]
    return c, rnd(kr, dtype)


def latent_attention(h, m, t, pre, eps, positions, rows, dtype):
    """``rows``: (c, k_rot) of this layer or of the layer whose cache it reads."""
    T = h.shape[0]
    H, D, Dr, Dv = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"])
    c, kr = rows
    cq = rnd(rms(linear(h, t[pre + "dq"], dtype=dtype), t[pre + "dq.norm"], eps), dtype)
    q = rnd(linear(cq, t[pre + "uq"], dtype=dtype), dtype).view(T, H, D + Dr)
    qn, qr = q[..., :D], rnd(rotate_half(q[..., D:], positions, m.get("rot")), dtype)
    kn = (c @ t[pre + "uk"].float().T).view(T, H, D)
    v = (c @ t[pre + "uv"].float().T).view(T, H, Dv)
    k = torch.cat([kn, kr[:, None, :].expand(T, H, Dr)], dim=-1)
    o = softmax_attention(torch.cat([qn, qr], dim=-1), k, v, float(m["scale"]), sink=t[pre + "sink"])
    return rnd(linear(o.reshape(T, H * Dv), t[pre + "o"], dtype=dtype), dtype)


def grouped_attention(h, m, t, pre, eps, positions, dtype):
    """Query heads on fewer key/value heads, biases, per-head norm of q and k before the rotation, ordinary softmax."""
    T = h.shape[0]
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = linear(h, t[pre + "q"], t[pre + "q.b"], dtype).view(T, H, D)
    k = linear(h, t[pre + "k"], t[pre + "k.b"], dtype).view(T, G, D)
    v = rnd(linear(h, t[pre + "v"], t[pre + "v.b"], dtype), dtype).view(T, G, Dv)
    q = rnd(rotate_half(rms(q, t[pre + "q.norm"], eps), positions, m.get("rot")), dtype)
    k = rnd(rotate_half(rms(k, t[pre + "k.norm"], eps), positions, m.get("rot")), dtype)
    k, v = k.repeat_interleave(H // G, dim=1), v.repeat_interleave(H // G, dim=1)
    o = softmax_attention(q, k, v, float(m["scale"]))
    return rnd(linear(o.reshape(T, H * Dv), t[pre + "o"], dtype=dtype), dtype)


def conv_silu(u, w, dtype, before=None):
    """u [T, C], w [C, taps]: y_t = silu(sum_j w[:, j] u_(t - taps + 1 + j)); ``before`` [taps - 1, C]: the rows in front of
    the first (zeros at the start of a sequence). The projection's result is rounded; what follows is 32-bit."""
    taps = w.shape[1]
    front = torch.zeros(taps - 1, u.shape[1]) if before is None else before
    padded = torch.cat([front, rnd(u, dtype)])
    y = sum(padded[j:j + u.shape[0]] * w[:, j].float() for j in range(taps))
    return silu(y)


def delta_rule(q, k, v, beta, g, state=None):
    """One sequence. q, k [T, H, D], v [T, H, Dv], beta, g [T, H]; the state S [H, D, Dv] starts at zero.
    Per token: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T, H, D = q.shape
    S = torch.zeros(H, D, v.shape[-1]) if state is None else state.clone()
    out = []
    for i in range(T):
        S = S * g[i][:, None, None]
        u = beta[i][:, None] * (v[i] - torch.einsum("hdv,hd->hv", S, k[i]))
        S = S + k[i][:, :, None] * u[:, None, :]
        out.append(torch.einsum("hdv,hd->hv", S, q[i]))
    return torch.stack(out), S


def gated_delta(h, m, t, pre, eps, dtype):
    T = h.shape[0]
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = conv_silu(linear(h, t[pre + "q"], dtype=dtype), t[pre + "q.conv"], dtype).view(T, G, D)
    k = conv_silu(linear(h, t[pre + "k"], dtype=dtype), t[pre + "k.conv"], dtype).view(T, G, D)
    v = conv_silu(linear(h, t[pre + "v"], dtype=dtype), t[pre + "v.conv"], dtype).view(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    q, k = q.repeat_interleave(H // G, dim=1), k.repeat_interleave(H // G, dim=1)
    hb = rnd(h, dtype)
    beta = torch.sigmoid(hb @ t[pre + "b"].float().T)
    g = torch.exp(-torch.exp(t[pre + "A_log"].float()) * F.softplus(hb @ t[pre + "a"].float().T + t[pre + "dt_bias"].float()))
    o, _ = delta_rule(q, k, v, beta, g)
    gate = silu(rnd(linear(h, t[pre + "g"], dtype=dtype), dtype)).view(T, H, Dv)
    y = rms(o, t[pre + "norm"], eps) * gate
    return rnd(linear(y.reshape(T, H * Dv), t[pre + "o"], dtype=dtype), dtype)


def parallel_mixer(h, m, t, pre, eps, positions, dtype):
    a = grouped_attention(h, m["left"], t, pre + "left.", eps, positions, dtype)
    b = gated_delta(h, m["right"], t, pre + "right.", eps, dtype)
    return rnd(0.5 * (rms(a, t[pre + "left.out"], eps) + rms(b, t[pre + "right.out"], eps)), dtype)


def dense_ff(h, t, pre, dtype):
    a = rnd(gelu_tanh(rnd(linear(h, t[pre + "gate"], dtype=dtype), dtype)) * rnd(linear(h, t[pre + "up"], dtype=dtype), dtype), dtype)
    return rnd(linear(a, t[pre + "down"], dtype=dtype), dtype)


def route(h, mlp, t, pre, dtype):
    """(chosen [T, top], weights [T, top]): the largest router logits, softmax over the chosen logits only."""
    z = rnd(h, dtype) @ t[pre + "router"].float().T + t[pre + "router.b"].float()
    top = z.topk(int(mlp["router"]["top"]), dim=-1)
    return top.indices, torch.softmax(top.values, dim=-1)


def expert_ff(h, mlp, t, pre, dtype):
    chosen, weight = route(h, mlp, t, pre, dtype)
    out = torch.zeros_like(h)
    for e in range(int(mlp["router"]["experts"])):
        p = f"{pre}e{e}."
        a = rnd(silu(linear(h, t[p + "gate"], dtype=dtype)) * linear(h, t[p + "up"], dtype=dtype), dtype)
        y = a @ t[p + "down"].float().T
        out = out + y * (weight * (chosen == e)).sum(-1, keepdim=True)
    return rnd(out, dtype)


def feed_forward(h, mlp, t, pre, dtype):
    return dense_ff(h, t, pre, dtype) if mlp["kind"] == "dense" else expert_ff(h, mlp, t, pre, dtype)


def forward(cfg: dict, t: dict, ids, dtype=torch.float32, trace: list | None = None):
    """Logits [T, vocab] of one sequence from position 0. ``trace`` collects the stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    ids = torch.as_tensor(ids, dtype=torch.long)
    positions = torch.arange(ids.numel())
    x = t["embed"].float()[ids] * float(cfg["embedding"]["scale"])
    cached = {}
    for i, layer in enumerate(cfg["layers"]):
        m, pre = layer["mixer"], f"l{i}.mix."
        h = x
        if layer["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                cached[i] = latent_rows(h, m, t, pre, eps, positions, dtype)
            y = latent_attention(h, m, t, pre, eps, positions, cached[i if src is None else int(src)], dtype)
        elif layer["type"] == "parallel":
            y = parallel_mixer(h, m, t, pre, eps, positions, dtype)
        else:
            raise ValueError(layer["type"])
        x = x + rms(y, t[f"l{i}.norm1"], eps)
        if layer.get("mlp"):
            x = x + rms(feed_forward(x, layer["mlp"], t, f"l{i}.mlp.", dtype), t[f"l{i}.norm2"], eps)
        if trace is not None:
            trace.append(x.clone())
    return rnd(rms(x, t["final.norm"], eps), dtype) @ t["embed"].float().T
