"""Softmax attention with the extras a model may ask for, each a constructor parameter:

  * grouped key/value heads and values of another size than keys;
  * biases on q, k and v;
  * an RMS norm of q and of k over the WHOLE projection (all heads of a token at once, one weight per channel of the
    projection), before the rotation; or instead an RMS norm of every head of q and of k by itself, with one weight per
    channel of a head that the heads share;
  * a rotation of the first channels of each head, pairs a half apart or neighbouring, with whatever frequencies the
    ``RotaryEmbedding`` was built with;
  * scores capped smoothly: s <- cap * tanh(s / cap);
  * a gate per head: head h of a token is multiplied by sigmoid((W_g x)_h), x the mixer's input;
  * a sliding window;
  * no keys and values of its own (``own_kv`` False): the mixer reads the cache that another layer writes, with its
    own queries.

One product gives q|k|v (and the gate, when there are no biases) in 32-bit; one kernel norms, rotates, rounds and stores;
the attention reads keys and values in place through the block tables, prompt portions and single tokens alike.
"""
from __future__ import annotations

import torch

from tokenmill_amd import profiling
from tokenmill_amd.hip import ops
from tokenmill_amd.hip.program import StepProgram
from tokenmill_amd.parts.base import KVCacheSpec, KVCacheView, Mixer, StepContext, as_tensor
from tokenmill_amd.parts.linear import Linear
from tokenmill_amd.parts.position import RotaryEmbedding
from tokenmill_amd.weights.loader import TensorSpec

MAX_HEAD_DIM = 256


class SoftmaxAttention(Mixer):
    def __init__(self, hidden: int, num_heads: int, num_kv_heads: int, head_dim: int, v_head_dim: int, scale: float,
                 rotary: RotaryEmbedding | None = None, whole_norm_eps: float | None = None, qkv_bias: bool = False,
                 softcap: float | None = None, head_gate: bool = False, window: int | None = None, own_kv: bool = True,
                 head_norm_eps: float | None = None,
                 names: tuple[str, str, str, str] = ("q", "k", "v", "o"),
                 extra_names: tuple[str, str, str] = ("q.norm", "k.norm", "g"),
                 suffixes: tuple[str, str] = ("", ".b")):
        """``whole_norm_eps``: None for no norm of q and k over the whole projection; ``head_norm_eps``: None for no norm head
        by head (one of the two at most). ``softcap``: None or 0 for none. ``extra_names``: the checkpoint's names of the two
        norm weights and of the gate's matrix, under the mixer's prefix."""
        if whole_norm_eps is not None and head_norm_eps is not None:
            raise ValueError("q and k are normed over the whole projection or head by head, not both")
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads do not divide into {num_kv_heads} kv heads")
        if head_dim % 4 or not 0 < head_dim <= MAX_HEAD_DIM or not 0 < v_head_dim <= MAX_HEAD_DIM:
            raise ValueError(f"head sizes {head_dim} / {v_head_dim}: keys in multiples of 4, both up to {MAX_HEAD_DIM}")
        if window is not None and window < 1:
            raise ValueError("a window holds at least one position")
        if rotary is not None and rotary.rotary_dim > head_dim:
            raise ValueError(f"{rotary.rotary_dim} rotated channels in a head of {head_dim}")
        if softcap is not None and softcap < 0:
            raise ValueError("a score cap is positive (or 0 / None for none)")
        self.hidden, self.num_heads, self.num_kv_heads = hidden, num_heads, num_kv_heads
        self.head_dim, self.v_head_dim = head_dim, v_head_dim
        self.scale, self.rotary, self.whole_norm_eps = float(scale), rotary, whole_norm_eps
        self.head_norm_eps = head_norm_eps
        self.norm_eps = whole_norm_eps if whole_norm_eps is not None else head_norm_eps     # None: q and k are not normed
        self.softcap, self.window, self.own_kv = float(softcap or 0.0), window, own_kv
        self.q_size, self.k_size, self.v_size = num_heads * head_dim, num_kv_heads * head_dim, num_kv_heads * v_head_dim
        sizes, stacked = [self.q_size], [names[0]]
        if own_kv:
            sizes += [self.k_size, self.v_size]
            stacked += [names[1], names[2]]
        # the gate's rows ride behind q|k|v in the one product where that product has no biases (the gate has none)
        self.gate_stacked = head_gate and not qkv_bias
        self.gate_at = sum(sizes)
        if self.gate_stacked:
            sizes.append(num_heads)
            stacked.append(extra_names[2])
        self.proj = Linear(hidden, sizes, stacked, bias=qkv_bias, suffixes=suffixes, wide_bias=True)     # its result is taken in 32-bit
        self.gate = Linear(hidden, num_heads, extra_names[2], bias=False, suffixes=suffixes) if head_gate and not self.gate_stacked else None
        self.has_gate = head_gate
        self.o = Linear(num_heads * v_head_dim, hidden, names[3], bias=False, suffixes=suffixes)
        self.extra_names = extra_names
        self.q_norm: torch.Tensor | None = None
        self.k_norm: torch.Tensor | None = None
        self._own: dict = {}                    # per cache: the library's attention operation as a program of its own

    def _linears(self):
        return [p for p in (self.proj, self.gate, self.o) if p is not None]

    def tensor_specs(self, prefix: str):
        specs = {}
        for lin in self._linears():
            specs.update(lin.tensor_specs(prefix))
        qn, kn, _ = self.extra_names
        if self.norm_eps is not None:
            per_head = self.head_norm_eps is not None
            specs[prefix + qn] = TensorSpec((self.head_dim if per_head else self.q_size,), init="ones")
            if self.own_kv:
                specs[prefix + kn] = TensorSpec((self.head_dim if per_head else self.k_size,), init="ones")
        return specs

    def load(self, tensors, prefix: str) -> None:
        for lin in self._linears():
            lin.load(tensors, prefix)
        qn, kn, _ = self.extra_names
        if self.norm_eps is not None:               # the vectors that meet 32-bit statistics are kept in 32-bit
            self.q_norm = tensors[prefix + qn].float().contiguous()
            self.k_norm = tensors[prefix + kn].float().contiguous() if self.own_kv else None
        if self.rotary is not None:
            self.rotary.load(tensors, prefix)

    def prepare(self, pack_weights: bool) -> None:
        for lin in self._linears():
            lin.prepare(pack_weights)

    def cache_spec(self):
        return KVCacheSpec(self.num_kv_heads, self.head_dim, self.window, v_head_dim=self.v_head_dim)

    def visible_pairs(self, step: StepContext) -> tuple[int, int]:
        """(keys read, (query, key) pairs) of a step, for a profile's floor."""
        keys = pairs = 0
        for start, n in zip(step.start_positions, step.q_lens):
            if self.window:
                keys += min(start + n, self.window + n - 1)
                pairs += sum(min(start + i + 1, self.window) for i in range(n))
            else:
                keys += start + n
                pairs += n * start + n * (n + 1) // 2
        return keys, pairs

    def cost(self, label: str, step: StepContext | None, rows: int) -> tuple[int, int]:
        if label == "qkv":
            moved, flops = self.proj.cost(rows, out_bytes=4)
            if self.gate is not None:
                m2, f2 = self.gate.cost(rows, out_bytes=4)
                moved, flops = moved + m2, flops + f2
            return moved, flops
        if label == "o_proj":
            return self.o.cost(rows)
        elem = self.o.weight.element_size()
        keys, pairs = self.visible_pairs(step)
        moved = keys * (self.k_size + self.v_size) * elem + step.num_tokens * (self.q_size + self.num_heads * self.v_head_dim) * elem
        return moved, 2 * pairs * self.num_heads * (self.head_dim + self.v_head_dim)

    def forward(self, x, step: StepContext, cache: KVCacheView, residual: torch.Tensor | None = None):
        x = as_tensor(x)
        T = x.shape[0]
        H, G, D, Dv = self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim
        rot = self.rotary
        if rot is not None and step.max_context_len > rot.max_positions:
            raise ValueError(f"position {step.max_context_len - 1} is beyond the rotary table ({rot.max_positions} positions)")
        if cache.write != self.own_kv:
            raise ValueError("a mixer with keys of its own writes its cache, one without reads another's: the model's run list disagrees")
        group = step.groups[cache.group]
        with profiling.label("qkv", lambda: self.cost("qkv", step, T)):
            proj = self.proj.forward(x, out_dtype=torch.float32)
            gate = None
            if self.gate_stacked:
                gate = proj[:, self.gate_at:self.gate_at + H]
            elif self.gate is not None:
                gate = self.gate.forward(x, out_dtype=torch.float32)
            q = torch.empty((T, self.q_size), dtype=x.dtype, device=x.device)
            ops.whole_norm_rope_store(proj, q, H, G, D, Dv, self.q_norm, self.k_norm, self.norm_eps or 1.0,
                                      rot.cos if rot is not None else None, rot.sin if rot is not None else None,
                                      bool(rot is not None and rot.interleaved), step.positions, group.slot_mapping,
                                      cache.k if self.own_kv else None, cache.v if self.own_kv else None, has_kv=self.own_kv,
                                      per_head=self.head_norm_eps is not None)
        if D == Dv:
            # keys and values of one size: the kernel library's own attention operation, which is handed q and chooses the
            # kernels of a step (prompt portions and single tokens on the matrix unit where it takes the sizes), then
            # gates the heads and projects
            entry = self._library_op(cache, x.dtype)
            if entry is not None:
                program, op = entry
                return program.run_one(op, step, qkv=q, gate=gate)
        out = torch.empty((T, H * Dv), dtype=x.dtype, device=x.device)
        with profiling.label("attention", lambda: self.cost("attention", step, T)):
            self._attend(q, out, gate, step, cache, group)
        with profiling.label("o_proj", lambda: self.o.cost(T)):
            return self.o.forward(out)

    def _library_op(self, cache: KVCacheView, dtype):
        key = (id(cache.k), dtype)
        if key not in self._own:
            program = StepProgram(dtype, self.hidden, cache.k.device)
            op = program.attention(self, None, None, self.o, (), cache, self.num_heads, self.num_kv_heads, self.head_dim, self.scale,
                                   self.window, self.softcap)
            self._own[key] = (program, op, cache) if op is not None else None
        entry = self._own[key]
        return entry[:2] if entry is not None else None

    def _attend(self, q, out, gate, step: StepContext, cache: KVCacheView, group) -> None:
        """Keys and values of different sizes: a token and a head a wavefront."""
        H, G, D, Dv = self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim
        ops.attn_paged_softmax(q, out, cache.k, cache.v, group.block_tables, step.seq_of_token, step.positions, H, G, D, Dv,
                               self.scale, self.window or 0, self.softcap, gate)
