"""Two mixers side by side: both read the same input, each result is RMS-normed over the model's width with a weight of
its own, and the mixer's result is half their sum,

    y = (rms_norm(left(h); w_left) + rms_norm(right(h); w_right)) / 2.

The two may be any mixers of which at most one keeps pages and at most one keeps state slots (an attention beside a
recurrence): the layer's cache is then the pages of the one with the state of the other beside them.
"""
from __future__ import annotations

import torch

from tokenmill_amd import profiling
from tokenmill_amd.hip import ops
from tokenmill_amd.parts.base import KVCacheSpec, KVCacheView, LayerCacheSpec, Mixer, StateSpec, StateView, StepContext, as_tensor
from tokenmill_amd.weights.loader import TensorSpec


def _split(spec):
    """(pages, states) that a mixer's cache spec asks for."""
    if spec is None:
        return None, None
    if isinstance(spec, KVCacheSpec):
        return spec, None
    if isinstance(spec, StateSpec):
        return None, spec
    return spec.kv, spec.state


class ParallelMixer(Mixer):
    def __init__(self, hidden: int, left: Mixer, right: Mixer, norm_eps: float, prefixes: tuple[str, str] = ("left.", "right."),
                 norm_names: tuple[str, str] = ("left.out", "right.out")):
        self.hidden, self.left, self.right, self.norm_eps = hidden, left, right, float(norm_eps)
        self.prefixes, self.norm_names = prefixes, norm_names
        (lk, ls), (rk, rs) = _split(left.cache_spec()), _split(right.cache_spec())
        if (lk is not None and rk is not None) or (ls is not None and rs is not None):
            raise ValueError("of two mixers side by side, one may keep pages and one may keep state")
        self.pages_of = 0 if lk is not None else 1 if rk is not None else None
        self.state_of = 0 if ls is not None else 1 if rs is not None else None
        self._spec = LayerCacheSpec(lk or rk, ls if ls is not None else rs) if (self.pages_of is not None or self.state_of is not None) else None
        self.w_left: torch.Tensor | None = None
        self.w_right: torch.Tensor | None = None

    @property
    def capturable(self) -> bool:
        return self.left.capturable and self.right.capturable

    def tensor_specs(self, prefix: str):
        specs = {**self.left.tensor_specs(prefix + self.prefixes[0]), **self.right.tensor_specs(prefix + self.prefixes[1])}
        for name in self.norm_names:
            specs[prefix + name] = TensorSpec((self.hidden,), init="ones")
        return specs

    def load(self, tensors, prefix: str) -> None:
        self.left.load(tensors, prefix + self.prefixes[0])
        self.right.load(tensors, prefix + self.prefixes[1])
        self.w_left = tensors[prefix + self.norm_names[0]].float().contiguous()
        self.w_right = tensors[prefix + self.norm_names[1]].float().contiguous()

    def prepare(self, pack_weights: bool) -> None:
        self.left.prepare(pack_weights)
        self.right.prepare(pack_weights)

    def cache_spec(self):
        return self._spec

    def _cache_for(self, which: int, cache):
        """What mixer ``which`` is handed of the layer's cache: the pages, the state, or nothing."""
        if cache is None:
            return None
        if isinstance(cache, KVCacheView):
            if which == self.pages_of:
                return cache
            return StateView(cache.state) if which == self.state_of and cache.state is not None else None
        return cache if which == self.state_of else None

    def forward(self, x, step: StepContext, cache, residual: torch.Tensor | None = None):
        x = as_tensor(x)
        a = self.left.forward(x, step, self._cache_for(0, cache))
        b = self.right.forward(x, step, self._cache_for(1, cache))
        out = torch.empty_like(a)
        with profiling.label("norm", lambda: (3 * a.numel() * a.element_size(), 0)):
            return ops.pair_norm_mean(a, b, self.w_left, self.w_right, out, self.norm_eps)
