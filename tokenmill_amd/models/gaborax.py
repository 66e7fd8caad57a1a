"""The Gaborax decoder assembled from parts.

    x = embed[token]
    every layer:  x += ls1 * N1(mixer(x));   x += ls2 * N2(ff(x))        (the second only if the layer has a feed-forward)
    logits = embed . Nf(x)

with N(v) = v / sqrt(mean(v^2) + eps) * (1 + w): the sublayers read the residual stream itself, and only their results are
normed. A layer's mixer is softmax attention over grouped key/value heads with q and k normed over the whole projection;
by its ``type``,
  * ``attention``: rotation of pairs half the rotated width apart, a sigmoid gate per head from the mixer's input, and with
    ``kv_from: j`` no keys and values of its own (it reads what layer j cached);
  * ``attention_2``: biases on q, k and v, rotation of neighbouring pairs with frequencies scaled over a ramp, scores
    capped by a tanh.
The feed-forward is a set of routed experts (relu squared; a router with a choice-only correction; experts that stand for
the input; a shared expert behind a sigmoid gate).
Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.ls1``, ``l<i>.mix.<name>`` (+ ``.b`` for a bias), ``l<i>.mlp.<name>``,
``final.norm``.
"""
from __future__ import annotations

from tokenmill_amd.config.model_config import GaboraxConfig, GaboraxLayer
from tokenmill_amd.config.registry import register_architecture
from tokenmill_amd.models.decoder import DecoderModel, LayerCall
from tokenmill_amd.parts import (GroupRMSNorm, OutputHead, PassThrough, RotaryEmbedding, RoutedExperts, SandwichBlock,
                                 SoftmaxAttention, TokenEmbedding)

DEFAULT_POSITIONS = 8192        # positions the rotation tables reach when neither the engine nor config.json says


def _mixer(cfg: GaboraxConfig, layer: GaboraxLayer, n_pos: int, tables: dict):
    m = layer.mixer
    second = layer.type == "attention_2"
    rot = m.get("rot") or {}
    dims = int(rot.get("dims", 0))
    rotary = None
    if dims:
        sc = rot.get("scaling") if second else None
        key = (int(m["dim"]), float(rot["base"]), dims, second, tuple(sorted(sc.items())) if sc else None)
        if key not in tables:           # layers with the same rotation share one table of angles
            tables[key] = RotaryEmbedding(key[0], key[1], n_pos, rotary_dim=dims, interleaved=second, scaling=sc, exact=True)
        rotary = tables[key]
    return SoftmaxAttention(cfg.hidden_size, int(m["heads"]), int(m.get("kv_heads") or m["heads"]), int(m["dim"]), int(m["vdim"]),
                            float(m["scale"]), rotary=rotary, whole_norm_eps=cfg.norm_eps, qkv_bias=second,
                            softcap=float(m["softcap"]) if second and m.get("softcap") else None, head_gate=not second,
                            own_kv=m.get("kv_from") is None)


def _feed_forward(cfg: GaboraxConfig, mlp: dict):
    return RoutedExperts(cfg.hidden_size, mlp["ff"], mlp["experts"], mlp["top"], identity=mlp["identity"], correction=True,
                         shared_ff=mlp["shared_ff"], shared_gate=True, activation="relu2")


def build_gaborax(cfg: GaboraxConfig, max_positions: int | None = None) -> DecoderModel:
    n_pos = max_positions or cfg.max_position_embeddings or DEFAULT_POSITIONS
    if cfg.max_position_embeddings:
        n_pos = min(n_pos, cfg.max_position_embeddings)
    hidden = cfg.hidden_size

    def behind():
        return GroupRMSNorm(hidden, cfg.norm_eps, name="", one_plus=True)

    embedding = TokenEmbedding(cfg.vocab_size, hidden, name="embed")
    tables: dict = {}
    layers, run = [], []
    names = ("norm1", "mix.", "norm1", "norm2", "mlp.", "norm2")    # the pass-throughs in front have no tensors: the names are the norms' behind
    for i, layer in enumerate(cfg.layers):
        mixer = _mixer(cfg, layer, n_pos, tables)
        if layer.mlp is None:
            layers.append(SandwichBlock(PassThrough(hidden), mixer, behind(), names=names, scales=("ls1", "ls2")))
        else:
            layers.append(SandwichBlock(PassThrough(hidden), mixer, behind(), PassThrough(hidden), _feed_forward(cfg, layer.mlp), behind(),
                                        names=names, scales=("ls1", "ls2")))
        src = layer.mixer.get("kv_from")
        run.append(LayerCall(i, cache_of=int(src) if src is not None else None))
    head = OutputHead(hidden, cfg.vocab_size, tied_to=embedding, name="head")
    return DecoderModel(cfg, embedding, layers, GroupRMSNorm(hidden, cfg.norm_eps, name="", one_plus=True), head, run=run,
                        names=("", "l{i}.", "final.norm", ""))


register_architecture(GaboraxConfig.architecture, GaboraxConfig.from_dict, build_gaborax, replace=True)
