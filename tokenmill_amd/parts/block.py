"""The arrangement of parts in a layer.

PreNormBlock: h = x + mixer(norm_in(x)); y = h + ffn(norm_post(h))
(reference src/infer/model/qwen2.py:13-23). The residual stream is a 32-bit tensor that the
block updates in place; each add is fused into the norm that follows it, so a block takes the
not-yet-added output of the previous block (``delta``) and returns its own.
"""
from __future__ import annotations

import torch

from tokenmill_amd.parts.base import Block, FeedForward, LayerCacheSpec, Mixer, Norm, NormedInput, StepContext


class PreNormBlock(Block):
    def __init__(self, norm_in: Norm, mixer: Mixer, norm_post: Norm, ffn: FeedForward,
                 names: tuple[str, str, str, str] = ("input_layernorm.", "self_attn.",
                                                     "post_attention_layernorm.", "mlp.")):
        self.norm_in, self.mixer, self.norm_post, self.ffn = norm_in, mixer, norm_post, ffn
        self.names = names

    def _parts(self):
        return zip((self.norm_in, self.mixer, self.norm_post, self.ffn), self.names)

    def tensor_specs(self, prefix: str):
        specs = {}
        for part, name in self._parts():
            specs.update(part.tensor_specs(prefix + name))
        return specs

    def load(self, tensors, prefix: str) -> None:
        for part, name in self._parts():
            part.load(tensors, prefix + name)

    def prepare(self, pack_weights: bool) -> None:
        for part, _ in self._parts():
            part.prepare(pack_weights)

    def emit(self, program, cache) -> None:
        """The block as two operations of a step program; a mixer or feed-forward the kernel library has no
        operation for runs through its own ``forward`` between the library's operations."""
        if self.mixer.emit(program, self.norm_in, cache) is None:
            def mix(flow, step):
                flow.settle()
                x = NormedInput(self.norm_in, flow.resid, flow.delta, program.dtype)
                flow.delta = self.mixer.forward(x, step, cache, residual=flow.resid)
                assert x.delta is None, f"{type(self.mixer).__name__}.forward did not take its input"
            program.foreign(self.mixer, mix)
        if self.ffn.emit(program, self.norm_post) is None:
            def feed(flow, step):
                flow.settle()
                x = NormedInput(self.norm_post, flow.resid, flow.delta, program.dtype)
                flow.delta = self.ffn.forward(x, step, residual=flow.resid)
                assert x.delta is None, f"{type(self.ffn).__name__}.forward did not take its input"
            program.foreign(self.ffn, feed)

    def forward(self, resid: torch.Tensor, delta: torch.Tensor | None, step: StepContext, cache,
                dtype: torch.dtype) -> torch.Tensor:
        """resid float32 [T, hidden], updated in place; returns the delta still to be added (None if the
        feed-forward added its result itself)."""
        a = self.mixer.forward(NormedInput(self.norm_in, resid, delta, dtype), step, cache, residual=resid)
        return self.ffn.forward(NormedInput(self.norm_post, resid, a, dtype), step, residual=resid)


class SandwichBlock(Block):
    """A norm before and a norm behind each sublayer:

        h = x + norm_mixed(mixer(norm_in(x)));   y = h + norm_fed(ffn(norm_post(h)))

    A block without a feed-forward (``ffn`` None) has the first line only. The residual stream is the 32-bit tensor
    every block updates in place. A sublayer's result is left pending together with the norm it has to pass
    (``flow.delta``, ``flow.delta_norm``), so that the norm in front of the next sublayer, of this block or the
    next, can norm it, add it and norm the sum in one kernel."""

    def __init__(self, norm_in: Norm, mixer: Mixer, norm_mixed: Norm, norm_post: Norm | None = None,
                 ffn: FeedForward | None = None, norm_fed: Norm | None = None,
                 names: tuple[str, str, str, str, str, str] = ("norm1", "mix.", "norm1b", "norm2", "mlp.", "norm2b"),
                 scales: tuple[str, str] | None = None):
        """A norm in front may be a ``PassThrough`` (the sublayer reads the stream itself). ``scales``: names, under the
        layer's prefix, of per-channel vectors that multiply the two normed results (a layer scale); they are folded into
        the weights of the norms behind the sublayers when the tensors are loaded."""
        if (ffn is None) != (norm_post is None) or (ffn is None) != (norm_fed is None):
            raise ValueError("a feed-forward comes with the norm before it and the norm behind it, or not at all")
        self.norm_in, self.mixer, self.norm_mixed = norm_in, mixer, norm_mixed
        self.norm_post, self.ffn, self.norm_fed = norm_post, ffn, norm_fed
        self.names = names
        self.scales = scales

    def _parts(self):
        return [(p, n) for p, n in zip((self.norm_in, self.mixer, self.norm_mixed, self.norm_post, self.ffn, self.norm_fed),
                                       self.names) if p is not None]

    def _scaled(self):
        if self.scales is None:
            return []
        return [(n, name) for n, name in zip((self.norm_mixed, self.norm_fed), self.scales) if n is not None]

    def tensor_specs(self, prefix: str):
        from tokenmill_amd.weights.loader import TensorSpec
        specs = {}
        for part, name in self._parts():
            specs.update(part.tensor_specs(prefix + name))
        for norm, name in self._scaled():
            specs[prefix + name] = TensorSpec((norm.hidden,), init="ones")
        return specs

    def load(self, tensors, prefix: str) -> None:
        for part, name in self._parts():
            part.load(tensors, prefix + name)
        for norm, name in self._scaled():
            norm.fold(tensors[prefix + name])

    def prepare(self, pack_weights: bool) -> None:
        for part, _ in self._parts():
            part.prepare(pack_weights)

    def emit(self, program, cache) -> None:
        """Each sublayer runs through its part's own ``forward``, between whatever operations of the kernel library
        the model's other parts describe."""
        def mix(flow, step):
            x = NormedInput(self.norm_in, flow.resid, flow.delta, program.dtype, delta_norm=flow.delta_norm)
            flow.delta, flow.delta_norm = self.mixer.forward(x, step, cache), self.norm_mixed
            assert x.delta is None, f"{type(self.mixer).__name__}.forward did not take its input"
        program.foreign(self.mixer, mix)
        if self.ffn is not None:
            def feed(flow, step):
                x = NormedInput(self.norm_post, flow.resid, flow.delta, program.dtype, delta_norm=flow.delta_norm)
                flow.delta, flow.delta_norm = self.ffn.forward(x, step), self.norm_fed
                assert x.delta is None, f"{type(self.ffn).__name__}.forward did not take its input"
            program.foreign(self.ffn, feed)

    def forward(self, resid: torch.Tensor, delta: torch.Tensor | None, step: StepContext, cache,
                dtype: torch.dtype) -> None:
        """The block by itself: resid float32 [T, hidden] is updated in place with everything, ``delta`` (a plain
        result of the block before, still to be added) included; nothing is left pending."""
        y = self.mixer.forward(NormedInput(self.norm_in, resid, delta, dtype), step, cache)
        if self.ffn is None:
            self.norm_mixed.add_normed(resid, y)
            return None
        y = self.ffn.forward(NormedInput(self.norm_post, resid, y, dtype, delta_norm=self.norm_mixed), step)
        self.norm_fed.add_normed(resid, y)
        return None


class GatedResidualBlock(Block):
    """Pre-norm sublayers whose results are scaled and gated on their way into the residual stream:

        n = norm_in(x);    x += mult * mixer(n + conv(n)) * sigmoid(gate_mixed(n))
        n = norm_post(x);  x += mult * ffn(n) * sigmoid(gate_fed(n))             (only with a feed-forward)

    ``conv`` (a ``ShortConvolution`` in front of the mixer), the two gates (``Linear`` parts with a bias) and the
    feed-forward are each optional, and ``mult`` = 1 with no gate is the plain pre-norm block. A gate reads the normed
    input before the convolution. A sublayer's result stays pending with its gate (``GatedAdd``) so that the norm in front
    of the next sublayer, of this block or the next, adds it and norms the sum in one kernel. The convolution's state lies
    beside the mixer's pages in the layer's cache."""

    def __init__(self, norm_in: Norm, mixer: Mixer, norm_post: Norm | None = None, ffn: FeedForward | None = None,
                 gate_mixed=None, gate_fed=None, conv=None, mult: float = 1.0,
                 names: tuple[str, str, str, str] = ("norm1", "mix.", "norm2", "mlp.")):
        if (ffn is None) != (norm_post is None):
            raise ValueError("a feed-forward comes with the norm before it, or not at all")
        if ffn is None and gate_fed is not None:
            raise ValueError("a gate for a feed-forward that is not there")
        self.norm_in, self.mixer, self.norm_post, self.ffn = norm_in, mixer, norm_post, ffn
        self.gate_mixed, self.gate_fed, self.conv, self.mult = gate_mixed, gate_fed, conv, float(mult)
        self.names = names

    def _parts(self):
        # the gates and the convolution carry their own names and take the layer's prefix
        pairs = list(zip((self.norm_in, self.mixer, self.norm_post, self.ffn), self.names))
        pairs += [(self.gate_mixed, ""), (self.gate_fed, ""), (self.conv, "")]
        return [(p, n) for p, n in pairs if p is not None]

    def tensor_specs(self, prefix: str):
        specs = {}
        for part, name in self._parts():
            specs.update(part.tensor_specs(prefix + name))
        return specs

    def load(self, tensors, prefix: str) -> None:
        for part, name in self._parts():
            part.load(tensors, prefix + name)

    def prepare(self, pack_weights: bool) -> None:
        for part, _ in self._parts():
            part.prepare(pack_weights)

    def cache_spec(self):
        spec = self.mixer.cache_spec()
        state = self.conv.state_spec() if self.conv is not None else None
        if state is None:
            return spec
        if spec is not None and not hasattr(spec, "kv_heads"):
            raise ValueError("a convolution in front of a mixer that keeps state of its own is not arranged for")
        return LayerCacheSpec(spec, state)

    def _pending(self, gate):
        from tokenmill_amd.parts.norm import GatedAdd
        return GatedAdd(gate, self.mult) if gate is not None or self.mult != 1.0 else None

    def _gate(self, part, n):
        from tokenmill_amd import profiling
        if part is None:
            return None
        with profiling.label("gate", lambda: part.cost(n.shape[0])):
            return part.forward(n)

    def _mix(self, x: NormedInput, step: StepContext, cache):
        n = x.tensor()
        gate = self._gate(self.gate_mixed, n)
        u = self.conv.forward(n, step, getattr(cache, "state", None)) if self.conv is not None else n
        return self.mixer.forward(u, step, cache), self._pending(gate)

    def _feed(self, x: NormedInput, step: StepContext):
        n = x.tensor()
        gate = self._gate(self.gate_fed, n)
        return self.ffn.forward(n, step), self._pending(gate)

    def emit(self, program, cache) -> None:
        def mix(flow, step):
            x = NormedInput(self.norm_in, flow.resid, flow.delta, program.dtype, delta_norm=flow.delta_norm)
            flow.delta, flow.delta_norm = self._mix(x, step, cache)
        program.foreign(self.mixer, mix)
        if self.ffn is not None:
            def feed(flow, step):
                x = NormedInput(self.norm_post, flow.resid, flow.delta, program.dtype, delta_norm=flow.delta_norm)
                flow.delta, flow.delta_norm = self._feed(x, step)
            program.foreign(self.ffn, feed)

    def forward(self, resid: torch.Tensor, delta: torch.Tensor | None, step: StepContext, cache,
                dtype: torch.dtype) -> None:
        """The block by itself: resid float32 [T, hidden] is updated in place with everything; nothing is left pending."""
        y, way = self._mix(NormedInput(self.norm_in, resid, delta, dtype), step, cache)
        if self.ffn is not None:
            y, way = self._feed(NormedInput(self.norm_post, resid, y, dtype, delta_norm=way), step)
        if way is not None:
            way.add_normed(resid, y)
        else:
            from tokenmill_amd.parts.norm import GatedAdd
            GatedAdd(None, 1.0).add_normed(resid, y)
        return None
