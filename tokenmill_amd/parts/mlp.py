"""SwiGLU feed-forward: down(silu(gate(x)) * up(x)), gate and up stacked into one product
(reference src/infer/model/layers.py:153-164)."""
from __future__ import annotations

import torch

from tokenmill_amd.hip import ops
from tokenmill_amd.hip.program import StepProgram
from tokenmill_amd.parts.base import FeedForward, Norm, NormedInput, StepContext, as_tensor
from tokenmill_amd.parts.linear import Linear
from tokenmill_amd.weights.loader import TensorSpec


class SwiGLU(FeedForward):
    def __init__(self, hidden: int, intermediate: int, bias: bool = False,
                 names: tuple[str, str, str] = ("gate_proj", "up_proj", "down_proj")):
        self.hidden, self.intermediate = hidden, intermediate
        self.gate_up = Linear(hidden, [intermediate, intermediate], list(names[:2]), bias=bias)
        self.down = Linear(intermediate, hidden, names[2], bias=bias)
        self._own: dict = {}                    # one-operation programs for calls of ``forward``

    def tensor_specs(self, prefix: str):
        return {**self.gate_up.tensor_specs(prefix), **self.down.tensor_specs(prefix)}

    def load(self, tensors, prefix: str) -> None:
        self.gate_up.load(tensors, prefix)
        self.down.load(tensors, prefix)

    def prepare(self, pack_weights: bool) -> None:
        if not pack_weights:
            return
        self.gate_up.pack(16, [self.intermediate, self.intermediate])
        self.down.pack(lambda: ops.skinny_strip_rows(self.hidden, self.intermediate))

    def emit(self, program, norm: Norm | None) -> int | None:
        if self.gate_up.bias is not None or self.down.bias is not None:
            return None                         # the library's operation has no biases
        return program.feed_forward(self, norm, self.gate_up, self.down, self.intermediate)

    def cost(self, label: str, step: StepContext | None, rows: int) -> tuple[int, int]:
        return self.gate_up.cost(rows) if label == "gate_up" else self.down.cost(rows)   # gate_up: with norm and SiLU*up

    def _alone(self, norm: Norm | None, dtype, device):
        key = (id(norm), dtype)
        entry = self._own.get(key)
        if entry is None:
            program = StepProgram(dtype, self.hidden, device)
            op = self.emit(program, norm)
            entry = self._own[key] = (program, op, norm)
        return entry[0], entry[1]

    def forward(self, x, step: StepContext | None = None, residual: torch.Tensor | None = None):
        """The same operation called by itself: by a block or a feed-forward that is not described to a step
        program (an expert of a routed one), or a test."""
        if isinstance(x, NormedInput) and x.lazy:
            program, op = self._alone(x.norm, x.dtype, x.resid.device)
            if op is not None:
                resid, delta = x.take()
                return program.run_one(op, None, resid=resid, delta=delta, accumulate=residual is resid, rows=resid.shape[0])
        x = as_tensor(x)
        program, op = self._alone(None, x.dtype, x.device)
        if op is None:                          # with biases: the two products and the activation one by one
            act = torch.empty((x.shape[0], self.intermediate), dtype=x.dtype, device=x.device)
            ops.silu_mul(self.gate_up.forward(x), act)
            return self.down.forward(act, accumulate_into=residual)
        if x.shape[0] == 0:
            return None if residual is not None else torch.empty_like(x)
        return program.run_one(op, None, resid=residual, x=x.contiguous(), accumulate=residual is not None, rows=x.shape[0])


class DenseFeedForward(FeedForward):
    """down(act(up(x))) with one up matrix and no gate. ``activation``: "gelu_tanh", the tanh form of GELU,
    0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))); or "poly_norm", a N(z) + b N(z^2) + c N(z^3) + e with four learned
    numbers (a, b, c, e) (the tensor ``act_name``), powers taken element by element and N(v) = v / sqrt(mean(v^2) + eps)
    over a token's row (``act_eps``). Both are computed in 32-bit. Both products may have biases."""

    ACTIVATIONS = ("gelu_tanh", "poly_norm")

    def __init__(self, hidden: int, intermediate: int, activation: str = "gelu_tanh", bias: bool = True,
                 names: tuple[str, str] = ("up", "down"), suffixes: tuple[str, str] = (".weight", ".bias"),
                 act_name: str = "act", act_eps: float = 1e-6):
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"activation '{activation}' is not one of {sorted(self.ACTIVATIONS)}")
        self.hidden, self.intermediate, self.activation = hidden, intermediate, activation
        self.up = Linear(hidden, intermediate, names[0], bias=bias, suffixes=suffixes)
        self.down = Linear(intermediate, hidden, names[1], bias=bias, suffixes=suffixes)
        self.act_name, self.act_eps = act_name, float(act_eps)
        self.act: torch.Tensor | None = None        # the activation's learned numbers, 32-bit

    def tensor_specs(self, prefix: str):
        specs = {**self.up.tensor_specs(prefix), **self.down.tensor_specs(prefix)}
        if self.activation == "poly_norm":
            specs[prefix + self.act_name] = TensorSpec((4,), init="ones")
        return specs

    def load(self, tensors, prefix: str) -> None:
        self.up.load(tensors, prefix)
        self.down.load(tensors, prefix)
        if self.activation == "poly_norm":
            self.act = tensors[prefix + self.act_name].float().contiguous()

    def prepare(self, pack_weights: bool) -> None:
        self.up.prepare(pack_weights)
        self.down.prepare(pack_weights)

    def cost(self, label: str, step: StepContext | None, rows: int) -> tuple[int, int]:
        return self.up.cost(rows) if label == "gate_up" else self.down.cost(rows)

    def forward(self, x, step: StepContext | None = None, residual: torch.Tensor | None = None):
        from tokenmill_amd import profiling
        x = as_tensor(x)
        with profiling.label("gate_up", lambda: self.up.cost(x.shape[0])):
            if self.activation == "poly_norm":          # the row's statistics want the products' sums as they are
                z = self.up.forward(x, out_dtype=torch.float32)
                a = ops.poly_norm(z, self.act, torch.empty(z.shape, dtype=x.dtype, device=x.device), self.act_eps)
            else:
                a = self.up.forward(x)
                ops.gelu_tanh(a, a)
        with profiling.label("down", lambda: self.down.cost(x.shape[0])):
            return self.down.forward(a)


class GatedFeedForward(FeedForward):
    """down(act(gate(x)) * up(x)) without biases, gate and up stacked into one product. ``activation``: "gelu_tanh", the
    tanh form of GELU, or "silu"; it is computed in 32-bit on the gate's rounded result and the product with up is rounded
    once. (``SwiGLU`` is the "silu" case as one operation of the kernel library's step program, for models whose blocks
    describe themselves to it.)"""

    ACTIVATIONS = ("gelu_tanh", "silu")

    def __init__(self, hidden: int, intermediate: int, activation: str = "gelu_tanh", names: tuple[str, str, str] = ("gate", "up", "down"),
                 suffixes: tuple[str, str] = ("", ".b")):
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"activation '{activation}' is not one of {sorted(self.ACTIVATIONS)}")
        self.hidden, self.intermediate, self.activation = hidden, intermediate, activation
        self.gate_up = Linear(hidden, [intermediate, intermediate], list(names[:2]), bias=False, suffixes=suffixes)
        self.down = Linear(intermediate, hidden, names[2], bias=False, suffixes=suffixes)

    def tensor_specs(self, prefix: str):
        return {**self.gate_up.tensor_specs(prefix), **self.down.tensor_specs(prefix)}

    def load(self, tensors, prefix: str) -> None:
        self.gate_up.load(tensors, prefix)
        self.down.load(tensors, prefix)

    def prepare(self, pack_weights: bool) -> None:
        self.gate_up.prepare(pack_weights)
        self.down.prepare(pack_weights)

    def cost(self, label: str, step: StepContext | None, rows: int) -> tuple[int, int]:
        return self.gate_up.cost(rows) if label == "gate_up" else self.down.cost(rows)

    def forward(self, x, step: StepContext | None = None, residual: torch.Tensor | None = None):
        from tokenmill_amd import profiling
        x = as_tensor(x)
        with profiling.label("gate_up", lambda: self.gate_up.cost(x.shape[0])):
            gu = self.gate_up.forward(x)
            a = torch.empty((x.shape[0], self.intermediate), dtype=x.dtype, device=x.device)
            (ops.gelu_mul if self.activation == "gelu_tanh" else ops.silu_mul)(gu, a)
        with profiling.label("down", lambda: self.down.cost(x.shape[0])):
            return self.down.forward(a)
