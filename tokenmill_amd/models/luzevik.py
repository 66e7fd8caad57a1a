"""The Luzevik decoder assembled from parts.

    x = embed[token] * scale
    every layer:  x += N1(mixer(x));   x += N2(ff(x))        (the second only if the layer has a feed-forward)
    logits = embed . Nf(x)

with N(v) = v / sqrt(mean(v^2) + eps) * w: the sublayers read the residual stream itself, and only their results are
normed. A layer's mixer is, by its ``type``,
  * ``latent_attention``: attention through a shared latent (queries through a latent of their own; the cached row of a
    token is its latent and one rotated key part that all heads share), rotation of pairs half the rotated width apart,
    a sink per head in the softmax's denominator, and with ``kv_from: j`` no latent of its own (it reads the rows layer j
    cached);
  * ``parallel``: softmax attention over grouped heads (biases, q and k normed head by head, linearly scaled rotation of
    part of a head) beside a gated delta rule behind short convolutions; each result is normed over the width and the two
    are averaged.
The feed-forward is dense with a tanh-GELU gate, or a set of routed SwiGLU experts whose router has a bias and weighs the
chosen experts by the softmax over their logits.
Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.<name>`` (+ ``.b`` for a bias, ``.conv`` for a
convolution, ``left.`` / ``right.`` in a parallel mixer), ``l<i>.mlp.<name>``, ``final.norm``.
"""
from __future__ import annotations

from tokenmill_amd.config.model_config import LuzevikConfig, LuzevikLayer
from tokenmill_amd.config.registry import register_architecture
from tokenmill_amd.models.decoder import DecoderModel, LayerCall
from tokenmill_amd.parts import (GatedDeltaRule, GatedFeedForward, GroupRMSNorm, LatentAttention, OutputHead, ParallelMixer, PassThrough,
                                 RotaryEmbedding, RoutedExperts, SandwichBlock, SoftmaxAttention, TokenEmbedding)

DEFAULT_POSITIONS = 8192        # positions the rotation tables reach when neither the engine nor config.json says


def _rotary(rot: dict | None, width: int, n_pos: int, tables: dict):
    """The table of angles for a rotation over the first ``rot.dims`` of ``width`` channels; layers with the same rotation share one."""
    rot = rot or {}
    dims = int(rot.get("dims", 0))
    if not dims:
        return None
    sc = rot.get("scaling")
    factor = float(sc["factor"]) if sc else None
    key = (width, float(rot["base"]), dims, factor)
    if key not in tables:
        tables[key] = RotaryEmbedding(width, key[1], n_pos, rotary_dim=dims, scaling={"factor": factor} if factor else None, exact=True)
    return tables[key]


def _mixer(cfg: LuzevikConfig, layer: LuzevikLayer, n_pos: int, tables: dict):
    m = layer.mixer
    hidden, eps = cfg.hidden_size, cfg.norm_eps
    if layer.type == "latent_attention":
        rot_dim = int(m["rot_dim"])
        return LatentAttention(hidden, int(m["heads"]), int(m["dim"]), rot_dim, int(m["vdim"]), int(m["q_rank"]), int(m["kv_rank"]),
                               float(m["scale"]), eps, rotary=_rotary(m.get("rot"), rot_dim, n_pos, tables) if rot_dim else None,
                               output_gate=False, sink=True, own_kv=m.get("kv_from") is None)
    left, right = m["left"], m["right"]
    attention = SoftmaxAttention(hidden, int(left["heads"]), int(left["kv_heads"]), int(left["dim"]), int(left["vdim"]),
                                 float(left["scale"]), rotary=_rotary(left.get("rot"), int(left["dim"]), n_pos, tables),
                                 qkv_bias=True, head_norm_eps=eps)
    recurrence = GatedDeltaRule(hidden, int(right["heads"]), int(right["kv_heads"]), int(right["dim"]), int(right["vdim"]),
                                int(right["conv"]), eps)
    return ParallelMixer(hidden, attention, recurrence, eps)


def _feed_forward(cfg: LuzevikConfig, mlp: dict):
    if mlp["kind"] == "dense":
        return GatedFeedForward(cfg.hidden_size, mlp["ff"], "gelu_tanh")
    return RoutedExperts(cfg.hidden_size, mlp["ff"], mlp["experts"], mlp["top"], correction=False, activation="swiglu",
                         scoring="chosen_logits", router_bias=True)


def build_luzevik(cfg: LuzevikConfig, max_positions: int | None = None) -> DecoderModel:
    n_pos = max_positions or cfg.max_position_embeddings or DEFAULT_POSITIONS
    if cfg.max_position_embeddings:
        n_pos = min(n_pos, cfg.max_position_embeddings)
    hidden = cfg.hidden_size

    def behind():
        return GroupRMSNorm(hidden, cfg.norm_eps, name="")

    embedding = TokenEmbedding(cfg.vocab_size, hidden, name="embed", scale=cfg.embedding_scale)
    tables: dict = {}
    layers, run = [], []
    names = ("norm1", "mix.", "norm1", "norm2", "mlp.", "norm2")    # the pass-throughs in front have no tensors: the names are the norms' behind
    for i, layer in enumerate(cfg.layers):
        mixer = _mixer(cfg, layer, n_pos, tables)
        if layer.mlp is None:
            layers.append(SandwichBlock(PassThrough(hidden), mixer, behind(), names=names))
        else:
            layers.append(SandwichBlock(PassThrough(hidden), mixer, behind(), PassThrough(hidden), _feed_forward(cfg, layer.mlp), behind(),
                                        names=names))
        src = layer.mixer.get("kv_from") if layer.type == "latent_attention" else None
        run.append(LayerCall(i, cache_of=int(src) if src is not None else None))
    head = OutputHead(hidden, cfg.vocab_size, tied_to=embedding, name="head")
    return DecoderModel(cfg, embedding, layers, GroupRMSNorm(hidden, cfg.norm_eps, name=""), head, run=run,
                        names=("", "l{i}.", "final.norm", ""))


register_architecture(LuzevikConfig.architecture, LuzevikConfig.from_dict, build_luzevik, replace=True)
