"""Feed-forwards of many small experts, of which every token uses a few.

    y[t] = sum over the token's experts e of weight(t, e) * W_down[e] (silu(W_gate[e] x[t]) * (W_up[e] x[t]))

``TableRoutedExperts``: there is no router; a table with one row per token id names the token's experts (the entries of
a row differ) and every one of them weighs 1 / (entries of a row). Experts have no biases.

The step's (token, expert) pairs are sorted by expert on the device and every expert multiplies its own rows, in tiles,
from one launch per product; nothing about the routing crosses to the host, so a step of single tokens can be recorded
into a graph like any other.
"""
from __future__ import annotations

import torch

from tokenmill_amd import profiling
from tokenmill_amd.hip import ops
from tokenmill_amd.parts.base import FeedForward, StepContext, as_tensor
from tokenmill_amd.parts.linear import Linear
from tokenmill_amd.weights.loader import TensorSpec


class TableRoutedExperts(FeedForward):
    def __init__(self, hidden: int, intermediate: int, experts: int, top: int, vocab: int,
                 names: tuple[str, str, str] = ("gate", "up", "down"), expert_prefix: str = "e{e}.", table_name: str = "table",
                 suffix: str = ""):
        if not 0 < top <= experts <= ops.MOE_MAX_EXPERTS:
            raise ValueError(f"{top} of {experts} experts: a token uses at least one and at most all, of up to {ops.MOE_MAX_EXPERTS}")
        self.hidden, self.intermediate, self.experts, self.top, self.vocab = hidden, intermediate, experts, top, vocab
        self.names, self.expert_prefix, self.table_name, self.suffix = names, expert_prefix, table_name, suffix
        self.gate_up: torch.Tensor | None = None       # [E, 2 F, hidden]: an expert's gate rows, then its up rows
        self.down: torch.Tensor | None = None          # [E, hidden, F]
        self.table: torch.Tensor | None = None         # int32 [vocab, top]

    def _name(self, prefix: str, e: int, which: int) -> str:
        return prefix + self.expert_prefix.format(e=e) + self.names[which] + self.suffix

    def tensor_specs(self, prefix: str):
        F, W = self.intermediate, self.hidden
        specs = {prefix + self.table_name: TensorSpec((self.vocab, self.top), kind="int", init=f"distinct_below:{self.experts}")}
        for e in range(self.experts):
            specs[self._name(prefix, e, 0)] = TensorSpec((F, W))
            specs[self._name(prefix, e, 1)] = TensorSpec((F, W))
            specs[self._name(prefix, e, 2)] = TensorSpec((W, F))
        return specs

    def load(self, tensors, prefix: str) -> None:
        E = self.experts
        self.gate_up = torch.stack([torch.cat([tensors[self._name(prefix, e, 0)], tensors[self._name(prefix, e, 1)]]) for e in range(E)]).contiguous()
        self.down = torch.stack([tensors[self._name(prefix, e, 2)] for e in range(E)]).contiguous()
        table = tensors[prefix + self.table_name]
        # an entry outside the experts would send a kernel beyond the matrices: refused here, once
        if table.numel() and (int(table.min()) < 0 or int(table.max()) >= E):
            raise ValueError(f"{prefix}{self.table_name} names an expert outside 0..{E - 1}")
        if self.top > 1:
            rows = table.sort(dim=1).values
            if bool((rows[:, 1:] == rows[:, :-1]).any()):
                raise ValueError(f"{prefix}{self.table_name}: a row names an expert twice")
        self.table = table.to(torch.int32).contiguous()

    def other_matrices(self) -> list[torch.Tensor]:
        """The matrices kept outside ``Linear`` parts (for a count of parameters)."""
        return [self.gate_up, self.down]

    def cost(self, label: str, step: StepContext | None, rows: int) -> tuple[int, int]:
        e = self.gate_up.element_size()
        used = min(self.experts, rows * self.top)               # matrices read at least once each when every pair differs
        moved = used * 3 * self.intermediate * self.hidden * e + rows * self.hidden * 2 * e + rows * self.top * self.intermediate * 2 * e
        return moved, 6 * rows * self.top * self.intermediate * self.hidden

    def forward(self, x, step: StepContext, residual: torch.Tensor | None = None):
        x = as_tensor(x)
        T = x.shape[0]
        out = torch.empty((T, self.hidden), dtype=x.dtype, device=x.device)
        with profiling.label("experts", lambda: self.cost("experts", step, T)):
            mfma = x.dtype == torch.bfloat16 and self.hidden % 8 == 0 and self.intermediate % 8 == 0 and x.stride(0) % 8 == 0
            rows = ops.moe_tile_rows(T * self.top, self.experts, x.dtype) if mfma else ops.MOE_TILE_ROWS
            routed = ops.moe_route(step.token_ids, self.table, self.experts, rows)
            return ops.moe_experts(x, routed, self.gate_up, self.down, self.top, 1.0 / self.top, out)


class RoutedExperts(FeedForward):
    """Experts chosen by a learned router, each W_down act(W_up x) without biases (``activation``: "relu2", the square of
    relu; or "swiglu": W_down (silu(W_gate x) * (W_up x)), with ``names`` then (gate, up, down)), plus what a model may add
    around them:

      z = W_router x (32-bit);  s = softmax(z) over all router outputs;  the ``top`` largest of s + correction are chosen
      (``correction``: a stored vector that shifts the choice only);  weight = s of the chosen / (their sum + 1e-20)
      the last ``identity`` router outputs are experts without matrices: their output is x itself
      y = sum of weight * expert(x)  +  sigmoid(w_sg . x) * shared(x)      (``shared_ff``: the width of an expert of the same
      form that every token uses; None for none; ``shared_gate`` False: the shared result is added as it is)
      ``scoring`` "chosen_logits": the ``top`` largest z themselves are chosen and the weights are the softmax over the chosen z
      only (no correction); ``router_bias``: z = W_router x + b, the bias added in 32-bit

    The router's rows and the shared gate's row are one 32-bit product. The step's (token, expert) pairs are sorted by expert
    on the device and every expert multiplies its own rows in tiles; nothing about the routing crosses to the host."""

    ACTIVATIONS = ("relu2", "swiglu")
    SCORINGS = ("softmax", "chosen_logits")

    def __init__(self, hidden: int, intermediate: int, experts: int, top: int, identity: int = 0, correction: bool = True,
                 shared_ff: int | None = None, shared_gate: bool = True, activation: str = "relu2",
                 names: tuple[str, ...] | None = None, expert_prefix: str = "e{e}.", router_name: str = "router",
                 correction_name: str = "correction", shared_prefix: str = "shared.", shared_gate_name: str = "shared.sg",
                 scoring: str = "softmax", router_bias: bool = False):
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"activation '{activation}' is not one of {list(self.ACTIVATIONS)}")
        if scoring not in self.SCORINGS:
            raise ValueError(f"scoring '{scoring}' is not one of {list(self.SCORINGS)}")
        if scoring == "chosen_logits" and correction:
            raise ValueError("a correction shifts a choice among softmax scores; the chosen-logits scoring has none")
        self.gated = activation == "swiglu"
        if names is None:
            names = ("gate", "up", "down") if self.gated else ("up", "down")
        if len(names) != (3 if self.gated else 2):
            raise ValueError("an expert's tensors are (up, down), or (gate, up, down) with a gate")
        if self.gated and shared_ff:
            raise ValueError("a shared expert with a gate of its own is not arranged for")
        self.scoring = scoring
        if experts < 0 or identity < 0 or not 0 < top <= experts + identity <= ops.MOE_MAX_EXPERTS:
            raise ValueError(f"{top} of {experts} + {identity} experts: a token uses at least one and at most all, of up to {ops.MOE_MAX_EXPERTS}")
        self.hidden, self.intermediate, self.experts, self.identity, self.top = hidden, intermediate, experts, identity, top
        self.outputs = experts + identity                       # what the router has an output for
        self.names, self.expert_prefix = names, expert_prefix
        self.has_correction, self.correction_name = correction, correction_name
        self.shared_ff, self.has_shared_gate = shared_ff, bool(shared_gate and shared_ff)
        rows, stacked = [self.outputs], [router_name]
        if self.has_shared_gate:
            rows.append(1)
            stacked.append(shared_gate_name)
        if router_bias and self.has_shared_gate:
            raise ValueError("a router with a bias beside a shared gate is not arranged for")
        self.router = Linear(hidden, rows, stacked, bias=router_bias, suffixes=("", ".b"), wide_bias=True)
        self.shared_up = Linear(hidden, shared_ff, shared_prefix + names[0], bias=False, suffixes=("", ".b"), activation="relu2") if shared_ff else None
        self.shared_down = Linear(shared_ff, hidden, shared_prefix + names[1], bias=False, suffixes=("", ".b")) if shared_ff else None
        self.up: torch.Tensor | None = None             # [E, F, hidden]; with a gate [E, 2 F, hidden]: an expert's gate rows, then its up rows
        self.down: torch.Tensor | None = None           # [E, hidden, F]
        self.correction: torch.Tensor | None = None     # float32 [experts + identity]

    def _name(self, prefix: str, e: int, which: int) -> str:
        return prefix + self.expert_prefix.format(e=e) + self.names[which]

    def _linears(self):
        return [p for p in (self.router, self.shared_up, self.shared_down) if p is not None]

    def tensor_specs(self, prefix: str):
        F, W = self.intermediate, self.hidden
        specs = {}
        for lin in self._linears():
            specs.update(lin.tensor_specs(prefix))
        if self.has_correction:
            specs[prefix + self.correction_name] = TensorSpec((self.outputs,))
        for e in range(self.experts):
            for which in range(len(self.names) - 1):
                specs[self._name(prefix, e, which)] = TensorSpec((F, W))
            specs[self._name(prefix, e, len(self.names) - 1)] = TensorSpec((W, F))
        return specs

    def load(self, tensors, prefix: str) -> None:
        for lin in self._linears():
            lin.load(tensors, prefix)
        if self.experts and self.gated:
            self.up = torch.stack([torch.cat([tensors[self._name(prefix, e, 0)], tensors[self._name(prefix, e, 1)]])
                                   for e in range(self.experts)]).contiguous()
            self.down = torch.stack([tensors[self._name(prefix, e, 2)] for e in range(self.experts)]).contiguous()
        elif self.experts:
            self.up = torch.stack([tensors[self._name(prefix, e, 0)] for e in range(self.experts)]).contiguous()
            self.down = torch.stack([tensors[self._name(prefix, e, 1)] for e in range(self.experts)]).contiguous()
        if self.has_correction:
            self.correction = tensors[prefix + self.correction_name].float().contiguous()

    def prepare(self, pack_weights: bool) -> None:
        for lin in self._linears():
            lin.prepare(pack_weights)

    def other_matrices(self) -> list[torch.Tensor]:
        return [t for t in (self.up, self.down) if t is not None]

    def cost(self, label: str, step: StepContext | None, rows: int) -> tuple[int, int]:
        e = self.router.weight.element_size()
        if label == "router":
            return self.router.cost(rows, out_bytes=4)
        if label == "shared":
            m1, f1 = self.shared_up.cost(rows)
            m2, f2 = self.shared_down.cost(rows, out_bytes=4)
            return m1 + m2, f1 + f2
        used = min(self.experts, rows * self.top)
        mats = 3 if self.gated else 2
        moved = used * mats * self.intermediate * self.hidden * e + rows * self.hidden * 2 * e + rows * self.top * self.intermediate * 2 * e
        return moved, 2 * mats * rows * self.top * self.intermediate * self.hidden

    def forward(self, x, step: StepContext, residual: torch.Tensor | None = None):
        x = as_tensor(x)
        T = x.shape[0]
        out = torch.empty((T, self.hidden), dtype=x.dtype, device=x.device)
        with profiling.label("router", lambda: self.cost("router", step, T)):
            z = self.router.forward(x, out_dtype=torch.float32)
            chosen, weight = ops.moe_router(z, self.outputs, self.top, self.correction, over_chosen=self.scoring == "chosen_logits")
        shared = None
        if self.shared_up is not None:
            with profiling.label("shared", lambda: self.cost("shared", step, T)):
                a = self.shared_up.forward(x)                   # with the activation (the product's own epilogue or pass)
                shared = self.shared_down.forward(a, out_dtype=torch.float32)
        with profiling.label("experts", lambda: self.cost("experts", step, T)):
            mfma = x.dtype == torch.bfloat16 and self.hidden % 8 == 0 and self.intermediate % 8 == 0 and x.stride(0) % 8 == 0
            rows = ops.moe_tile_rows(T * self.top, max(self.experts, 1), x.dtype) if mfma else ops.MOE_TILE_ROWS
            routed = ops.moe_route_chosen(chosen, self.outputs, self.experts, rows)
            gate = z[:, self.outputs:self.outputs + 1] if self.has_shared_gate else None
            return ops.moe_experts_weighted(x, routed, weight, self.up, self.down, self.top, out, shared, gate, gated=self.gated)
