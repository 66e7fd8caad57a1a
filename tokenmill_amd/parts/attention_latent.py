"""Attention through a shared latent.

Queries come from a narrow latent (down projection, RMS norm, up projection) and are laid out head by head as
[Dn channels without rotation | Dr rotated channels]. Keys and values come from one latent of Lk channels per token
(down projection, RMS norm) plus Dr rotated key channels that all heads share; head h's key is W_uk[h] c, its value
W_uv[h] c. Only the latent and the shared rotated channels are cached: one row of Lk + Dr numbers per token,
whatever the number of heads. The per-head matrices move to the other side of the two sums,

    score(t, j, h) = scale * ((W_uk[h]^T q_n[t, h]) . c_j + q_r[t, h] . k_r[j])
    out(t, h)      = W_uv[h] (sum_j softmax_j(score) c_j)

so that every head reads the same cached rows (a query of Lk + Dr channels, a result of Lk channels), in a prompt and
in decoding alike. Softmax over the visible rows: the token's own and the ``window - 1`` before it (None: all).
What a model may add, each a constructor parameter: a sigmoid gate per head computed from the mixer's input; a sink per
head (a learned number whose exponential joins the softmax's denominator, with no row behind it); a rotation of
neighbouring pairs or of pairs half the rotated width apart; no latent of its own (``own_kv`` False: the mixer reads
the rows that another layer caches, with its own queries and per-head matrices).
"""
from __future__ import annotations

import torch

from tokenmill_amd import profiling
from tokenmill_amd.hip import ops
from tokenmill_amd.parts.base import KVCacheSpec, KVCacheView, Mixer, StepContext, as_tensor
from tokenmill_amd.parts.linear import Linear
from tokenmill_amd.parts.position import RotaryEmbedding
from tokenmill_amd.weights.loader import TensorSpec


class LatentAttention(Mixer):
    def __init__(self, hidden: int, num_heads: int, head_dim: int, rot_dim: int, v_head_dim: int, q_rank: int, kv_rank: int,
                 scale: float, norm_eps: float, rotary: RotaryEmbedding | None = None, window: int | None = None,
                 output_gate: bool = True, sink: bool = False, own_kv: bool = True,
                 names: tuple[str, ...] = ("dq", "uq", "dkv", "uk", "uv", "g", "o"),
                 norm_names: tuple[str, str] = ("dq.norm", "dkv.norm"), suffixes: tuple[str, str] = ("", ".b"),
                 sink_name: str = "sink"):
        """``head_dim``: channels of a head's query and key that are not rotated; ``rot_dim``: the rotated ones (the key's are
        shared by the heads). ``rotary``: a ``RotaryEmbedding`` over ``rot_dim`` channels, of which it may rotate fewer, in
        either pairing; None: none. ``output_gate``: whether a per-head sigmoid gate (a projection of the input) multiplies the
        result. ``sink``: whether the checkpoint holds a number per head that joins the softmax's denominator. ``own_kv``
        False: no down projection to the key/value latent; the cache is another layer's."""
        if min(num_heads, head_dim, v_head_dim, q_rank, kv_rank) <= 0 or rot_dim < 0:
            raise ValueError("the sizes of a latent attention are positive")
        if kv_rank > ops.LATENT_MAX_RANK or kv_rank + rot_dim > ops.LATENT_MAX_ROW:
            raise ValueError(f"a latent of {kv_rank} + {rot_dim} channels: the kernels take {ops.LATENT_MAX_RANK} and rows of {ops.LATENT_MAX_ROW}")
        if rotary is not None and rotary.rotary_dim > rot_dim:
            raise ValueError("the rotation fits the rotated part of a head")
        if window is not None and window < 1:
            raise ValueError("a window holds at least one position")
        self.hidden, self.num_heads, self.head_dim, self.rot_dim, self.v_head_dim = hidden, num_heads, head_dim, rot_dim, v_head_dim
        self.q_rank, self.kv_rank, self.scale, self.norm_eps = q_rank, kv_rank, float(scale), float(norm_eps)
        self.rotary, self.window, self.output_gate = rotary, window, output_gate
        self.has_sink, self.own_kv, self.sink_name = sink, own_kv, sink_name
        self.half_pairs = rotary is not None and not rotary.interleaved
        self.row = kv_rank + rot_dim                                       # what a token caches
        n = dict(zip(("dq", "uq", "dkv", "uk", "uv", "g", "o"), names))
        self.names, self.norm_names, self.suffixes = n, norm_names, suffixes
        # the projections that read the mixer's input are one product: [query latent | latent | shared key | gates]
        outs, stacked = [q_rank], [n["dq"]]
        if own_kv:
            outs.append(kv_rank + rot_dim)
            stacked.append(n["dkv"])
        self.gate_at = sum(outs)
        if output_gate:
            outs.append(num_heads)
            stacked.append(n["g"])
        self.down = Linear(hidden, outs, stacked, bias=False, suffixes=suffixes)
        self.uq = Linear(q_rank, num_heads * (head_dim + rot_dim), n["uq"], bias=False, suffixes=suffixes)
        self.o = Linear(num_heads * v_head_dim, hidden, n["o"], bias=False, suffixes=suffixes)
        self.q_norm: torch.Tensor | None = None
        self.kv_norm: torch.Tensor | None = None
        self.sink: torch.Tensor | None = None           # float32 [H]
        self.uk: torch.Tensor | None = None             # [H, Dn, Lk]: a head's query channels onto the latent
        self.uv: torch.Tensor | None = None             # [H, Lk, Dv]: the latent onto a head's value channels
        self.uk_nt: torch.Tensor | None = None          # the same two as [H, N, K], the order the matrix-unit products read
        self.uv_nt: torch.Tensor | None = None

    def tensor_specs(self, prefix: str):
        H, Dn, Dv, Lk = self.num_heads, self.head_dim, self.v_head_dim, self.kv_rank
        sw = self.suffixes[0]
        specs = {**self.down.tensor_specs(prefix), **self.uq.tensor_specs(prefix), **self.o.tensor_specs(prefix)}
        specs[prefix + self.names["uk"] + sw] = TensorSpec((H * Dn, Lk))
        specs[prefix + self.names["uv"] + sw] = TensorSpec((H * Dv, Lk))
        specs[prefix + self.norm_names[0]] = TensorSpec((self.q_rank,), init="ones")
        if self.own_kv:
            specs[prefix + self.norm_names[1]] = TensorSpec((Lk,), init="ones")
        if self.has_sink:
            specs[prefix + self.sink_name] = TensorSpec((H,))
        return specs

    def load(self, tensors, prefix: str) -> None:
        H, Dn, Dv, Lk = self.num_heads, self.head_dim, self.v_head_dim, self.kv_rank
        sw = self.suffixes[0]
        self.down.load(tensors, prefix)
        self.uq.load(tensors, prefix)
        self.o.load(tensors, prefix)
        self.uk = tensors[prefix + self.names["uk"] + sw].view(H, Dn, Lk).contiguous()
        self.uv_nt = tensors[prefix + self.names["uv"] + sw].view(H, Dv, Lk)
        self.uv = self.uv_nt.transpose(1, 2).contiguous()
        self.uk_nt = self.uk.transpose(1, 2).contiguous() if self.uk.dtype == torch.bfloat16 else None
        # the norm weights meet 32-bit statistics and are kept in 32-bit
        self.q_norm = tensors[prefix + self.norm_names[0]].float().contiguous()
        self.kv_norm = tensors[prefix + self.norm_names[1]].float().contiguous() if self.own_kv else None
        self.sink = tensors[prefix + self.sink_name].float().contiguous() if self.has_sink else None
        if self.rotary is not None:
            self.rotary.load(tensors, prefix)

    def prepare(self, pack_weights: bool) -> None:
        for lin in (self.down, self.uq, self.o):
            lin.prepare(pack_weights)

    def cache_spec(self):
        return KVCacheSpec(1, self.row, self.window, values=False)

    def other_matrices(self) -> list[torch.Tensor]:
        """The matrices kept outside ``Linear`` parts (for a count of parameters)."""
        return [self.uk, self.uv]

    def visible_pairs(self, step: StepContext) -> tuple[int, int]:
        """(rows read, (query, row) pairs) of a step, for a profile's floor."""
        rows = pairs = 0
        for start, n in zip(step.start_positions, step.q_lens):
            first = max(0, start - self.window + 1) if self.window else 0
            rows += start + n - first
            for p in range(start, start + n):
                pairs += min(p + 1, self.window) if self.window else p + 1
        return rows, pairs

    def cost(self, label: str, step: StepContext | None, rows: int) -> tuple[int, int]:
        e = self.uq.weight.element_size()
        H, Dn, Dr, Dv, Lk = self.num_heads, self.head_dim, self.rot_dim, self.v_head_dim, self.kv_rank
        if label == "qkv":          # both down projections, the queries' up projection and their move onto the latent
            a, b = self.down.cost(rows, out_bytes=4), self.uq.cost(rows)
            return a[0] + b[0] + self.uk.numel() * e + rows * H * self.row * e, a[1] + b[1] + 2 * rows * H * Dn * Lk
        if label == "o_proj":       # the latent results onto the heads' values, and the output projection
            a = self.o.cost(rows)
            return a[0] + self.uv.numel() * e + rows * H * Lk * e, a[1] + 2 * rows * H * Lk * Dv
        seen, pairs = self.visible_pairs(step)
        return seen * self.row * e + step.num_tokens * H * (self.row + Lk) * e, 2 * pairs * H * (self.row + Lk)

    def _attend(self, qa, latent, step: StepContext, cache: KVCacheView, group) -> None:
        """Prompt portions and single tokens (the step's last ``num_decode`` rows) on the matrix unit where its kernel takes
        the sizes; the 32-bit path and every other size through the kernel that takes a token and a head a wavefront."""
        H, Lk, row, T = self.num_heads, self.kv_rank, self.row, qa.shape[0]
        tiles, first_single = step.prefill_tiles, T - step.num_decode
        if not ops.attn_latent_mfma_takes(qa.dtype, Lk, row, H) or (first_single > 0 and (tiles is None or not tiles.shape[0])):
            ops.attn_latent(qa, latent, cache.k, group.block_tables, step.seq_of_token, step.positions, H, Lk, row, self.scale,
                            self.window or 0, sink=self.sink)
            return
        if first_single > 0:
            ops.attn_latent_mfma(qa, latent, cache.k, group.block_tables, tiles, step.seq_of_token, step.positions, 0, 0, H, Lk, row,
                                 self.scale, self.window or 0, sink=self.sink)
        if step.num_decode > 0:
            ops.attn_latent_mfma(qa, latent, cache.k, group.block_tables, None, step.seq_of_token, step.positions, first_single,
                                 step.num_decode, H, Lk, row, self.scale, self.window or 0, most_context=step.max_decode_context,
                                 bound=self.rotary.max_positions if self.rotary is not None else 1 << 20, sink=self.sink)

    def forward(self, x, step: StepContext, cache: KVCacheView, residual: torch.Tensor | None = None):
        x = as_tensor(x)
        T = x.shape[0]
        H, Dn, Dr, Dv, Lq, Lk, row = self.num_heads, self.head_dim, self.rot_dim, self.v_head_dim, self.q_rank, self.kv_rank, self.row
        rot = self.rotary
        if rot is not None and step.max_context_len > rot.max_positions:
            raise ValueError(f"position {step.max_context_len - 1} is beyond the rotary table ({rot.max_positions} positions)")
        cos, sin = (rot.cos, rot.sin) if rot is not None else (None, None)
        if cache.write != self.own_kv:
            raise ValueError("a mixer with a latent of its own writes its cache, one without reads another's: the model's run list disagrees")
        group = step.groups[cache.group]
        half = self.half_pairs
        with profiling.label("qkv", lambda: self.cost("qkv", step, T)):
            low = self.down.forward(x, out_dtype=torch.float32)                         # 32-bit: it feeds norms and the rotation
            cq = torch.empty((T, Lq), dtype=x.dtype, device=x.device)
            if self.own_kv:
                ops.latent_prepare(low, Lq, Lk, Dr, self.q_norm, self.kv_norm, self.norm_eps, cos, sin, step.positions,
                                   group.slot_mapping, cq, cache.k, half_pairs=half)
            else:
                ops.latent_prepare(low, Lq, 0, 0, self.q_norm, None, self.norm_eps, None, None, None, None, cq, None)
            q = self.uq.forward(cq)
            qa = torch.empty((T, H * row), dtype=x.dtype, device=x.device)
            if self.uk_nt is not None and ops.heads_matmul_mfma_takes(q, Dn + Dr, self.uk_nt):
                # the heads' rotated channels go beside their part on the latent in the same launch
                ops.heads_matmul_mfma(q, Dn + Dr, self.uk_nt, qa, row, tail=Dr, cos=cos, sin=sin, positions=step.positions,
                                      half_pairs=half)
            else:
                ops.heads_matmul(q, Dn + Dr, self.uk, qa, row)
                if Dr:
                    ops.rotate_heads(q[:, Dn:], Dn + Dr, qa[:, Lk:], row, H, Dr, cos, sin, step.positions, half_pairs=half)
        latent = torch.empty((T, H * Lk), dtype=x.dtype, device=x.device)
        with profiling.label("attention", lambda: self.cost("attention", step, T)):
            self._attend(qa, latent, step, cache, group)
        with profiling.label("o_proj", lambda: self.cost("o_proj", step, T)):
            out = torch.empty((T, H * Dv), dtype=x.dtype, device=x.device)
            gate = low[:, self.gate_at:] if self.output_gate else None
            if ops.heads_matmul_mfma_takes(latent, Lk, self.uv_nt):
                ops.heads_matmul_mfma(latent, Lk, self.uv_nt, out, Dv, gate=gate)
            else:
                ops.heads_matmul(latent, Lk, self.uv, out, Dv, gate=gate)
            return self.o.forward(out)
