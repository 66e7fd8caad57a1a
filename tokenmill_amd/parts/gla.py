"""Gated linear attention: a recurrent mixer with a matrix of state per request and head.

    q_t = W_q h_t / sqrt(D),  k_t = W_k h_t        [heads, D]
    v_t = W_v h_t,            g_t = W_g h_t        [heads, Dv]
    a_t = sigmoid(W_a2 (W_a1 h_t) + b)^(1/tau)     [heads, D]   a decay per key channel, through a narrow projection
    S_t = diag(a_t) S_(t-1) + k_t v_t^T            [D, Dv] per head, 32-bit, zero at a request's first token
    o_t = S_t^T q_t
    y_t = W_o (concat over heads of rms_norm(o_t; w) * silu(g_t))

The state is the mixer's cache: a ``StateSpec`` slot per request, advanced in token order inside a step's portion
and carried from step to step. Decays, their logarithms and exponentials, the state and the norm are 32-bit; the
projections are the model's products. A step of single tokens works on the step's device tensors alone, so it can
be recorded into a HIP graph.
"""
from __future__ import annotations

import torch

from tokenmill_amd import profiling
from tokenmill_amd.hip import ops
from tokenmill_amd.parts.base import Mixer, StateSpec, StateView, StepContext, as_tensor, step_segments
from tokenmill_amd.parts.linear import Linear
from tokenmill_amd.weights.loader import TensorSpec

MAX_KEY_DIM = 256


class GatedLinearAttention(Mixer):
    def __init__(self, hidden: int, num_heads: int, key_dim: int, value_dim: int, tau: float, norm_eps: float,
                 gate_rank: int | None = None, drawn_gate_rank: int = 16,
                 names: tuple[str, ...] = ("q", "k", "v", "g", "a1", "a2", "o", "norm"),
                 suffixes: tuple[str, str] = ("", ".b")):
        """``gate_rank``: the width of the narrow projection in front of the decays; None leaves it to the
        checkpoint's tensors (``drawn_gate_rank`` is what a model drawn at random gets then)."""
        if not 0 < key_dim <= MAX_KEY_DIM:
            raise ValueError(f"key size {key_dim}: the recurrence kernel takes up to {MAX_KEY_DIM}")
        if tau <= 0:
            raise ValueError("tau must be positive")
        self.hidden, self.num_heads, self.key_dim, self.value_dim = hidden, num_heads, key_dim, value_dim
        self.tau, self.norm_eps = float(tau), float(norm_eps)
        self.gate_rank, self.drawn_gate_rank = gate_rank, drawn_gate_rank
        self.names, self.suffixes = names, suffixes
        self.k_size, self.v_size = num_heads * key_dim, num_heads * value_dim
        self.proj: Linear | None = None          # q | k | v | g | a1 stacked: one product over the input
        self.gate: Linear | None = None          # a2, with its bias
        self.o = Linear(self.v_size, hidden, names[6], bias=False, suffixes=suffixes)
        self.norm_w: torch.Tensor | None = None
        if gate_rank is not None:
            self._make_projections(gate_rank)

    def _make_projections(self, rank: int) -> None:
        n = self.names
        self.proj = Linear(self.hidden, [self.k_size, self.k_size, self.v_size, self.v_size, rank], list(n[:5]), bias=False,
                           suffixes=self.suffixes)
        self.gate = Linear(rank, self.k_size, n[5], bias=True, suffixes=self.suffixes)

    def tensor_specs(self, prefix: str):
        n, (sw, sb) = self.names, self.suffixes
        if self.proj is not None:
            specs = {**self.proj.tensor_specs(prefix), **self.gate.tensor_specs(prefix)}
        else:
            free = (self.drawn_gate_rank,)
            specs = {prefix + n[0] + sw: TensorSpec((self.k_size, self.hidden)), prefix + n[1] + sw: TensorSpec((self.k_size, self.hidden)),
                     prefix + n[2] + sw: TensorSpec((self.v_size, self.hidden)), prefix + n[3] + sw: TensorSpec((self.v_size, self.hidden)),
                     prefix + n[4] + sw: TensorSpec((None, self.hidden), free=free),
                     prefix + n[5] + sw: TensorSpec((self.k_size, None), free=free),
                     prefix + n[5] + sb: TensorSpec((self.k_size,))}
        specs.update(self.o.tensor_specs(prefix))
        specs[prefix + n[7]] = TensorSpec((self.value_dim,), init="ones")
        return specs

    def load(self, tensors, prefix: str) -> None:
        n, (sw, _) = self.names, self.suffixes
        if self.proj is None:
            rank = tensors[prefix + n[4] + sw].shape[0]
            if tensors[prefix + n[5] + sw].shape[1] != rank:
                raise ValueError(f"{prefix}{n[4]} and {prefix}{n[5]} disagree on the width between them")
            self._make_projections(rank)
        self.proj.load(tensors, prefix)
        self.gate.load(tensors, prefix)
        self.o.load(tensors, prefix)
        self.norm_w = tensors[prefix + n[7]].float().contiguous()

    def cache_spec(self):
        return StateSpec((self.num_heads, self.key_dim, self.value_dim), torch.float32)

    def cost(self, label: str, step: StepContext | None, rows: int) -> tuple[int, int]:
        if label == "qkv":
            a, b = self.proj.cost(rows), self.gate.cost(rows, out_bytes=4)
            return a[0] + b[0], a[1] + b[1]
        if label == "o_proj":
            return self.o.cost(rows)
        # the recurrence: q, k, v, the decays and the result once; the state read and written once per request;
        # per token and head D * Dv multiply-adds for the state and as many for the result
        e = self.proj.weight.element_size()
        seqs = step.num_seqs if step is not None else 1
        moved = rows * ((2 * self.k_size + self.v_size) * e + self.k_size * 4 + self.v_size * 4) + \
            2 * seqs * self.num_heads * self.key_dim * self.value_dim * 4
        return moved, 4 * rows * self.num_heads * self.key_dim * self.value_dim

    # Rows of a request's portion from which the recurrence runs in segments of this many rows (see ``_scan``)
    SEGMENT = 64

    def forward(self, x, step: StepContext, cache: StateView, residual: torch.Tensor | None = None):
        x = as_tensor(x)
        T = x.shape[0]
        H, D, Dv = self.num_heads, self.key_dim, self.value_dim
        ks, vs = self.k_size, self.v_size
        with profiling.label("qkv", lambda: self.cost("qkv", step, T)):
            proj = self.proj.forward(x)                                          # [T, q | k | v | g | a1]
            narrow = proj[:, 2 * ks + 2 * vs:]
            gate = self.gate
            if gate.weight.dtype == narrow.dtype and (gate.bias is None or gate.bias.dtype == narrow.dtype):
                decay = torch.empty((T, ks), dtype=torch.float32, device=x.device)
                ops.gla_gate_decay(narrow, gate.weight, gate.bias, self.tau, decay)
            else:                                                                # a matrix kept in another type: the product rule's way
                decay = gate.forward(narrow, out_dtype=torch.float32)
                ops.gla_decay(decay, self.tau)
        o = torch.empty((T, vs), dtype=torch.float32, device=x.device)
        y = torch.empty((T, vs), dtype=x.dtype, device=x.device)
        with profiling.label("recurrence", lambda: self.cost("attention", step, T)):
            self._scan(proj, decay, o, cache.state, step)
            ops.gla_out_gate(o, proj[:, 2 * ks + vs:2 * ks + 2 * vs], self.norm_w, y, H, Dv, self.norm_eps)
        with profiling.label("o_proj", lambda: self.o.cost(T)):
            return self.o.forward(y)

    def _scan(self, proj, decay, o, state, step: StepContext) -> None:
        """The recurrence over the step's rows. A step whose longest portion is short (single tokens, small
        portions) is one scan from the requests' states. A long portion is cut into segments of ``SEGMENT`` rows:
        the recurrence is linear in the state, so every segment is first scanned from a zero state (what its own
        rows build), a chain over the segments' decay products gives each segment's true start state and the
        request's new state, and a second scan of all segments from those gives the results. Two scans that fill
        the chip and a short chain, instead of one chain over every token. The sums of a token's result are then
        ordered otherwise than in the plain chain: the two agree up to 32-bit rounding."""
        H, D, Dv = self.num_heads, self.key_dim, self.value_dim
        ks = self.k_size
        scale = D ** -0.5
        if step.max_q_len < 2 * self.SEGMENT:
            ops.gla_scan(proj, 0, ks, 2 * ks, decay, o, state, step.cu_q_lens, step.state_slots, step.num_seqs, H, D, Dv, scale)
            return
        cu_seg, ids, first, n_seg = self._segments(step, proj.device)
        local = torch.zeros((n_seg, H, D, Dv), dtype=torch.float32, device=proj.device)
        states_only = ops.gla_scan_states_only(proj, 0, ks, decay, D)                                    # else o is written and overwritten below
        ops.gla_scan(proj, 0, ks, 2 * ks, decay, None if states_only else o, local, cu_seg, ids, n_seg, H, D, Dv, scale)
        products = torch.empty((n_seg, ks), dtype=torch.float32, device=proj.device)
        ops.gla_segment_decay(decay, cu_seg, n_seg, products)
        start = torch.empty_like(local)
        ops.gla_combine(state, step.state_slots, first, products, local, start, step.num_seqs)
        ops.gla_scan(proj, 0, ks, 2 * ks, decay, o, start, cu_seg, ids, n_seg, H, D, Dv, scale)

    def _segments(self, step: StepContext, device):
        """(first row of each segment [n + 1], 0..n-1, first segment of each request [S + 1], n) on the device, made once per step
        and shared by the step's layers."""
        return step_segments(step, self.SEGMENT, device)
