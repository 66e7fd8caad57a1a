"""The gated delta rule: a recurrent mixer with a matrix of state per request and head.

    q_t, k_t = unit(silu(conv(W_q h))), unit(silu(conv(W_k h)))      [kv_heads, D]   unit(x) = x / sqrt(sum(x^2) + 1e-6); q also / sqrt(D)
    v_t      = silu(conv(W_v h))                                      [heads, Dv]
    beta_t   = sigmoid(W_b h)                                         [heads]         how much of the correction is written
    g_t      = exp(-exp(A_log) * softplus(W_a h + dt_bias))           [heads]         one decay per head, in (0, 1)
    S <- g_t S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t        S [D, Dv] per head, 32-bit, zero at a request's first token
    y_t      = W_o (concat over heads of rms_norm(o_t; w) * silu(W_g h))

``conv`` is a short causal convolution over time, channel by channel (zeros before a request's first token); value head h
reads q/k head h // (heads / kv_heads). The state is the mixer's cache: the matrices S and the convolution's last
``taps - 1`` input rows, a slot of each per request, advanced in token order inside a step's portion and carried from
step to step. Everything that enters the recurrence behind the projections and the convolution is 32-bit. A step of
single tokens works on the step's device tensors alone, so it can be recorded into a HIP graph.
"""
from __future__ import annotations

import torch

from tokenmill_amd import profiling
from tokenmill_amd.hip import ops
from tokenmill_amd.parts.base import LayerCacheSpec, Mixer, StateSpec, StateView, StepContext, as_tensor, step_segments
from tokenmill_amd.parts.linear import Linear
from tokenmill_amd.weights.loader import TensorSpec

UNIT_EPS = 1e-6         # inside the root of the unit norms of q and k: the mechanism's own constant


class GatedDeltaRule(Mixer):
    def __init__(self, hidden: int, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int, taps: int, norm_eps: float,
                 names: tuple[str, ...] = ("q", "k", "v", "g", "b", "a", "o"), conv_suffix: str = ".conv",
                 other_names: tuple[str, str, str] = ("A_log", "dt_bias", "norm"), suffixes: tuple[str, str] = ("", ".b")):
        if num_heads <= 0 or num_kv_heads <= 0 or num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads do not divide into {num_kv_heads} query/key heads")
        if not 0 < key_dim <= ops.DELTA_MAX_KEY_DIM or value_dim <= 0:
            raise ValueError(f"key size {key_dim}: the recurrence kernel takes up to {ops.DELTA_MAX_KEY_DIM}")
        if not 1 <= taps <= 16:
            raise ValueError(f"a convolution of {taps} taps: the kernel takes 1 to 16")
        self.hidden, self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim = hidden, num_heads, num_kv_heads, key_dim, value_dim
        self.taps, self.norm_eps = taps, float(norm_eps)
        self.k_size, self.v_size = num_kv_heads * key_dim, num_heads * value_dim
        self.channels = 2 * self.k_size + self.v_size                        # what the convolution runs over: q | k | v
        if self.channels > ops.DELTA_MAX_CHANNELS:
            raise ValueError(f"{self.channels} convolved channels: the kernel takes up to {ops.DELTA_MAX_CHANNELS}")
        n = dict(zip(("q", "k", "v", "g", "b", "a", "o"), names))
        self.names, self.conv_suffix, self.other_names = n, conv_suffix, other_names
        self.proj = Linear(hidden, [self.k_size, self.k_size, self.v_size, self.v_size], [n["q"], n["k"], n["v"], n["g"]], bias=False,
                           suffixes=suffixes)
        self.steps = Linear(hidden, [num_heads, num_heads], [n["b"], n["a"]], bias=False, suffixes=suffixes)     # taken in 32-bit
        self.o = Linear(self.v_size, hidden, n["o"], bias=False, suffixes=suffixes)
        self.conv_w: torch.Tensor | None = None          # [channels, taps]
        self.a_log: torch.Tensor | None = None
        self.dt_bias: torch.Tensor | None = None
        self.norm_w: torch.Tensor | None = None

    def _linears(self):
        return (self.proj, self.steps, self.o)

    def tensor_specs(self, prefix: str):
        specs = {}
        for lin in self._linears():
            specs.update(lin.tensor_specs(prefix))
        for key, size in (("q", self.k_size), ("k", self.k_size), ("v", self.v_size)):
            specs[prefix + self.names[key] + self.conv_suffix] = TensorSpec((size, self.taps))
        a_log, dt_bias, norm = self.other_names
        specs[prefix + a_log] = TensorSpec((self.num_heads,))
        specs[prefix + dt_bias] = TensorSpec((self.num_heads,))
        specs[prefix + norm] = TensorSpec((self.value_dim,), init="ones")
        return specs

    def load(self, tensors, prefix: str) -> None:
        for lin in self._linears():
            lin.load(tensors, prefix)
        self.conv_w = torch.cat([tensors[prefix + self.names[key] + self.conv_suffix] for key in ("q", "k", "v")]).contiguous()
        a_log, dt_bias, norm = self.other_names
        # what meets 32-bit arithmetic is kept in 32-bit
        self.a_log = tensors[prefix + a_log].float().contiguous()
        self.dt_bias = tensors[prefix + dt_bias].float().contiguous()
        self.norm_w = tensors[prefix + norm].float().contiguous()

    def prepare(self, pack_weights: bool) -> None:
        for lin in self._linears():
            lin.prepare(pack_weights)

    def state_specs(self) -> tuple[StateSpec, ...]:
        """The recurrence's matrices in 32-bit and, with more than one tap, the convolution's last rows in the model's type."""
        specs = [StateSpec((self.num_heads, self.key_dim, self.value_dim), torch.float32)]
        if self.taps > 1:
            specs.append(StateSpec((self.taps - 1, self.channels), None))
        return tuple(specs)

    def cache_spec(self):
        return LayerCacheSpec(None, self.state_specs())

    def cost(self, label: str, step: StepContext | None, rows: int) -> tuple[int, int]:
        if label == "qkv":
            a, b = self.proj.cost(rows), self.steps.cost(rows, out_bytes=4)
            return a[0] + b[0], a[1] + b[1]
        if label == "o_proj":
            return self.o.cost(rows)
        # the recurrence: a prepared row read once per head's columns, the result once; the state read and written once per
        # request; per token and head D * Dv multiply-adds each for the two sums and for the state
        seqs = step.num_seqs if step is not None else 1
        moved = rows * (ops.delta_row_width(self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim) + self.v_size) * 4 + \
            2 * seqs * self.num_heads * self.key_dim * self.value_dim * 4
        return moved, 6 * rows * self.num_heads * self.key_dim * self.value_dim

    def forward(self, x, step: StepContext, cache: StateView, residual: torch.Tensor | None = None):
        x = as_tensor(x)
        T = x.shape[0]
        H, G, D, Dv = self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim
        states = cache.state if isinstance(cache.state, tuple) else (cache.state,)
        matrices, conv_state = states[0], states[1] if len(states) > 1 else None
        with profiling.label("qkv", lambda: self.cost("qkv", step, T)):
            proj = self.proj.forward(x)                                          # [T, q | k | v | g]
            steps = self.steps.forward(x, out_dtype=torch.float32)               # [T, b | a]
        o = torch.empty((T, self.v_size), dtype=torch.float32, device=x.device)
        y = torch.empty((T, self.v_size), dtype=x.dtype, device=x.device)
        with profiling.label("recurrence", lambda: self.cost("attention", step, T)):
            rows = torch.empty((T, ops.delta_row_width(H, G, D, Dv)), dtype=torch.float32, device=x.device)
            ops.delta_prepare(proj, self.conv_w, conv_state, steps, self.a_log, self.dt_bias, step.cu_q_lens, step.state_slots,
                              step.seq_of_token, step.num_seqs, rows, H, G, D, Dv, UNIT_EPS)
            if conv_state is not None:
                ops.delta_conv_state(proj, self.channels, conv_state, step.cu_q_lens, step.state_slots, step.num_seqs)
            self._scan(rows, o, matrices, step)
            ops.gla_out_gate(o, proj[:, self.channels:], self.norm_w, y, H, Dv, self.norm_eps)
        with profiling.label("o_proj", lambda: self.o.cost(T)):
            return self.o.forward(y)

    # Rows of a request's portion from which the recurrence runs in segments of this many rows (see ``_scan``)
    SEGMENT = 128

    def _scan(self, rows, o, matrices, step: StepContext) -> None:
        """The recurrence over the step's rows. A step whose longest portion is short (single tokens, small portions) is one
        scan from the requests' states. A long portion is cut into segments of ``SEGMENT`` rows: the recurrence is linear in
        the state, S_end = M S_start + B over any run of tokens, so every segment is first scanned twice side by side with all
        others, from a zero state (B: what its own rows build) and, without values, from the identity (M: the product of its
        tokens' transitions g (I - beta k k^T)); a chain over the segments gives each segment's true start state and the
        request's new state; and a third scan of all segments from those gives the results. Three scans that fill the chip and
        a short chain of small products, instead of one chain over every token. The sums of a token's result are then ordered
        otherwise than in the plain chain: the two agree up to 32-bit rounding."""
        H, G, D, Dv = self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim
        if step.max_q_len < 2 * self.SEGMENT:
            ops.delta_scan(rows, o, matrices, step.cu_q_lens, step.state_slots, step.num_seqs, H, G, D, Dv)
            return
        cu_seg, ids, first, n_seg = step_segments(step, self.SEGMENT, rows.device)
        local = torch.zeros((n_seg, H, D, Dv), dtype=torch.float32, device=rows.device)
        ops.delta_scan(rows, None, local, cu_seg, ids, n_seg, H, G, D, Dv)
        trans = torch.eye(D, dtype=torch.float32, device=rows.device).expand(n_seg, H, D, D).contiguous()
        ops.delta_scan(rows, None, trans, cu_seg, ids, n_seg, H, G, D, D, transitions_of=Dv)
        start = torch.empty_like(local)
        ops.delta_combine(trans, local, start, matrices, step.state_slots, first, step.num_seqs)
        ops.delta_scan(rows, o, start, cu_seg, ids, n_seg, H, G, D, Dv)
