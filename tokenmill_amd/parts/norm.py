"""RMSNorm fused with the residual add (reference src/infer/model/layers.py:35-44,
src/infer/model/qwen2.py:22-23)."""
from __future__ import annotations

import torch

from tokenmill_amd import profiling
from tokenmill_amd.hip import ops
from tokenmill_amd.parts.base import Norm
from tokenmill_amd.weights.loader import TensorSpec


class RMSNorm(Norm):
    """out = weight * round(x * rsqrt(mean(x^2) + eps)); the weight is used as it is (not 1 + w)."""

    def __init__(self, hidden: int, eps: float):
        self.hidden = hidden
        self.eps = float(eps)
        self.weight: torch.Tensor | None = None

    def tensor_specs(self, prefix: str):
        return {f"{prefix}weight": TensorSpec((self.hidden,), init="ones")}

    def load(self, tensors, prefix: str) -> None:
        self.weight = tensors[f"{prefix}weight"]

    def add_norm(self, resid, delta, out_dtype, rows=None):
        n = resid.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.hidden), dtype=out_dtype, device=resid.device)
        with profiling.label("norm", lambda: (n * self.hidden * (4 + (0 if rows is not None else 4) + out.element_size()
                                                                 + (out.element_size() if delta is not None else 0)), 0)):
            return ops.add_rmsnorm(resid, delta, self.weight, self.eps, out, rows)

    def rms_params(self):
        return self.weight, self.eps


class GroupRMSNorm(Norm):
    """RMS norm in groups: the row is cut into ``groups`` equal consecutive parts, each part is divided by its own
    sqrt(mean(part^2) + eps), and the whole is multiplied by the weight; all of it in 32-bit, the result rounded
    once. ``groups = 1`` is the usual RMS norm (rounded after the weight, not before it as ``RMSNorm`` does).

    It can also stand behind a sublayer (``add_normed``: resid += self(y)); a ``GroupRMSNorm`` that is asked for
    the next sublayer's input while such a result is pending does both in one kernel when the two agree on
    groups and eps."""

    def __init__(self, hidden: int, eps: float, groups: int = 1, name: str = "weight", one_plus: bool = False):
        """``one_plus``: the checkpoint stores the weight around zero and the norm multiplies by 1 + w; the sum is made
        once, at load, in 32-bit."""
        if groups < 1 or hidden % groups:
            raise ValueError(f"{groups} groups do not divide a width of {hidden}")
        self.hidden, self.eps, self.groups, self.name, self.one_plus = hidden, float(eps), groups, name, one_plus
        self.weight: torch.Tensor | None = None

    def tensor_specs(self, prefix: str):
        return {f"{prefix}{self.name}": TensorSpec((self.hidden,), init="normal" if self.one_plus else "ones")}

    def load(self, tensors, prefix: str) -> None:
        self.weight = tensors[f"{prefix}{self.name}"]
        if self.one_plus:
            self.weight = (1.0 + self.weight.float()).contiguous()

    def fold(self, scale: torch.Tensor) -> None:
        """Multiply a per-channel scale that follows the norm (a layer scale) into its weight, in 32-bit: one vector where
        the model has two."""
        self.weight = (self.weight.float() * scale.float()).contiguous()

    def _cost(self, n: int, out_bytes: int, added: int):
        return n * self.hidden * (4 + out_bytes + added), 0

    def add_norm(self, resid, delta, out_dtype, rows=None, delta_norm: Norm | None = None):
        n = resid.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.hidden), dtype=out_dtype, device=resid.device)
        post = None
        if delta is not None and delta_norm is not None:
            if isinstance(delta_norm, GroupRMSNorm) and (delta_norm.groups, delta_norm.eps) == (self.groups, self.eps):
                post = delta_norm.weight
            elif rows is None:
                delta_norm.add_normed(resid, delta)
                delta = None
            else:
                # only some rows are wanted and the residual is to stay as it is: the pending result's norm on a copy
                resid = resid.index_select(0, rows.long())
                delta_norm.add_normed(resid, delta.index_select(0, rows.long()))
                delta, rows = None, None
        added = 0 if delta is None else (4 if rows is None else 0) + delta.element_size()
        with profiling.label("norm", lambda: self._cost(n, out.element_size(), added)):
            return ops.group_norm(resid, delta, post, self.weight, out, self.groups, self.eps, rows)

    def add_normed(self, resid, y) -> None:
        with profiling.label("norm", lambda: self._cost(resid.shape[0], 4, y.element_size())):
            ops.group_norm(resid, y, self.weight, None, None, self.groups, self.eps)


class PassThrough(Norm):
    """No norm in front of a sublayer: its input is the residual stream itself, rounded to the model's type. What is still
    pending on the stream (a sublayer's result and the norm it has to pass) is added by the same kernel."""

    def __init__(self, hidden: int):
        self.hidden = hidden

    def add_norm(self, resid, delta, out_dtype, rows=None, delta_norm: Norm | None = None):
        n = resid.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.hidden), dtype=out_dtype, device=resid.device)
        post, groups, eps = None, 1, 1.0
        if delta is not None and delta_norm is not None:
            if isinstance(delta_norm, GroupRMSNorm):
                post, groups, eps = delta_norm.weight, delta_norm.groups, delta_norm.eps
            elif rows is None:
                delta_norm.add_normed(resid, delta)
                delta = None
            else:
                resid = resid.index_select(0, rows.long())
                delta_norm.add_normed(resid, delta.index_select(0, rows.long()))
                delta, rows = None, None
        added = 0 if delta is None else (4 if rows is None else 0) + delta.element_size()
        with profiling.label("norm", lambda: (n * self.hidden * (4 + out.element_size() + added), 0)):
            return ops.group_norm(resid, delta, post, None, out, groups, eps, rows)

    def add_normed(self, resid, y) -> None:
        raise NotImplementedError("a pass-through stands in front of a sublayer, not behind it")


class GatedAdd:
    """What a sublayer's result passes on its way into the residual stream when the block scales and gates it:
    resid += mult * y * sigmoid(gate), with ``gate`` [T, hidden] the gate's values before the sigmoid (None: no gate).
    It stands where a norm behind a sublayer stands (``Flow.delta_norm``), so the norm in front of the next sublayer
    can do the add and its own work in one kernel."""

    def __init__(self, gate: torch.Tensor | None, mult: float = 1.0):
        self.gate, self.mult = gate, float(mult)

    def add_normed(self, resid, y) -> None:
        with profiling.label("norm", lambda: (resid.numel() * 8 + y.numel() * y.element_size() * (2 if self.gate is not None else 1), 0)):
            ops.layer_norm(resid, y, self.gate, self.mult, None, None, None, 1.0)


class LayerNorm(Norm):
    """(x - mean) / sqrt(mean((x - mean)^2) + eps) * weight + bias over a row, in 32-bit, rounded once. The weight and
    the bias are kept in 32-bit. ``names``: what the checkpoint appends to the prefix for the two."""

    def __init__(self, hidden: int, eps: float, names: tuple[str, str] = ("weight", "bias")):
        self.hidden, self.eps, self.names = hidden, float(eps), names
        self.weight: torch.Tensor | None = None
        self.bias: torch.Tensor | None = None

    def tensor_specs(self, prefix: str):
        return {prefix + self.names[0]: TensorSpec((self.hidden,), init="ones"),
                prefix + self.names[1]: TensorSpec((self.hidden,), init="zeros")}

    def load(self, tensors, prefix: str) -> None:
        self.weight = tensors[prefix + self.names[0]].float().contiguous()
        self.bias = tensors[prefix + self.names[1]].float().contiguous()

    def _cost(self, n: int, out_bytes: int, added: int):
        return n * self.hidden * (4 + out_bytes + added), 0

    def add_norm(self, resid, delta, out_dtype, rows=None, delta_norm=None):
        n = resid.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.hidden), dtype=out_dtype, device=resid.device)
        gate, mult = None, 1.0
        if delta is not None and delta_norm is not None:
            if isinstance(delta_norm, GatedAdd):
                gate, mult = delta_norm.gate, delta_norm.mult
            elif rows is None:
                delta_norm.add_normed(resid, delta)
                delta = None
            else:       # only some rows are wanted and the residual is to stay as it is: the pending result's way in on a copy
                resid = resid.index_select(0, rows.long())
                delta_norm.add_normed(resid, delta.index_select(0, rows.long()))
                delta, rows = None, None
        added = 0 if delta is None else (4 if rows is None else 0) + delta.element_size() * (2 if gate is not None else 1)
        with profiling.label("norm", lambda: self._cost(n, out.element_size(), added)):
            return ops.layer_norm(resid, delta, gate, mult, self.weight, self.bias, out, self.eps, rows)

    def add_normed(self, resid, y) -> None:
        raise NotImplementedError("a layer norm stands in front of a sublayer, not behind it")
