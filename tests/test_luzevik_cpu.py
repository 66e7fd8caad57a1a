"""Luzevik without a GPU: configuration, tensor declarations, what the layers ask of the cache manager, and the plain
implementation's mechanisms pinned against special cases that reduce to something known."""
from __future__ import annotations

import copy
import math

import pytest
import torch

from luzevik_cases import A, B, C
from plain import luzevik_plain as P


# ----------------------------------------------------------------------------------------------- configuration

def test_config_reads_every_size_and_constant():
    from tokenmill_amd.config.model_config import LuzevikConfig
    from tokenmill_amd.config.registry import architecture_name, get_architecture
    assert architecture_name(A) == "Luzevik" and get_architecture("Luzevik").name == "Luzevik"
    cfg = LuzevikConfig.from_dict(A)
    assert (cfg.vocab_size, cfg.hidden_size, cfg.norm_eps, cfg.embedding_scale, cfg.max_position_embeddings) == (211, 88, 3e-5, 2.5, None)
    assert [l.type for l in cfg.layers] == ["latent_attention", "parallel", "latent_attention", "latent_attention", "latent_attention"]
    assert cfg.layers[0].mlp == {"kind": "dense", "ff": 56} and cfg.layers[1].mlp == {"kind": "moe", "ff": 24, "experts": 5, "top": 2}
    assert cfg.layers[3].mlp is None and cfg.layers[2].mixer["kv_from"] == 0 and "kv_from" not in cfg.layers[3].mixer
    assert cfg.layers[1].mixer["left"]["rot"]["scaling"] == {"factor": 4.0} and cfg.layers[1].mixer["right"]["conv"] == 4
    limited = dict(copy.deepcopy(C), max_positions=77)
    assert LuzevikConfig.from_dict(limited).max_position_embeddings == 77


@pytest.mark.parametrize("edit,match", [
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c.pop("embedding"), "embedding"),
    (lambda c: c["layers"][0].update(type="attention"), "type"),
    (lambda c: c["layers"][0]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=10), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(scaling={"factor": 2.0}), "scaling"),
    (lambda c: c["layers"][1]["mixer"].pop("right"), "left' and 'right"),
    (lambda c: c["layers"][1]["mixer"]["left"].update(kv_heads=4), "kv_heads"),
    (lambda c: c["layers"][1]["mixer"]["right"].update(kv_heads=3), "kv_heads"),
    (lambda c: c["layers"][1]["mixer"]["right"].pop("conv"), "conv"),
    (lambda c: c["layers"][1]["mixer"]["right"].update(conv=0), "conv"),
    (lambda c: c["layers"][1]["mixer"]["left"]["rot"].update(dims=22), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["left"]["rot"]["scaling"].update(factor=0.0), "factor"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=2), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=1), "kv_from"),
    (lambda c: c["layers"][4]["mixer"].update(kv_from=2), "kv_from"),
    (lambda c: c["layers"][4]["mixer"].update(kv_from=3), "equal"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=6), "experts"),
    (lambda c: c["layers"][1]["mlp"]["expert"].pop("ff"), "ff"),
    (lambda c: c["layers"][0]["mlp"].update(kind="glu"), "kind"),
])
def test_config_refuses_what_the_model_cannot_be(edit, match):
    from tokenmill_amd.config import ConfigError
    from tokenmill_amd.config.model_config import LuzevikConfig
    raw = copy.deepcopy(A)
    edit(raw)
    with pytest.raises(ConfigError, match=match):
        LuzevikConfig.from_dict(raw)


def test_tensor_names_shapes_and_caches():
    from tokenmill_amd.config.model_config import LuzevikConfig
    from tokenmill_amd.models.luzevik import build_luzevik
    from tokenmill_amd.parts import KVCacheSpec, LayerCacheSpec
    model = build_luzevik(LuzevikConfig.from_dict(A), 64)
    specs = {k: tuple(v.shape) for k, v in model.tensor_specs().items()}
    assert specs["embed"] == (211, 88) and specs["final.norm"] == (88,) and "head" not in specs and "lm_head" not in specs
    assert specs["l0.mix.dq"] == (24, 88) and specs["l0.mix.dq.norm"] == (24,) and specs["l0.mix.uq"] == (3 * 20, 24)
    assert specs["l0.mix.dkv"] == (48, 88) and specs["l0.mix.dkv.norm"] == (40,) and specs["l0.mix.sink"] == (3,)
    assert specs["l0.mix.uk"] == (36, 40) and specs["l0.mix.uv"] == (60, 40) and specs["l0.mix.o"] == (88, 60)
    assert "l2.mix.dkv" not in specs and "l2.mix.dkv.norm" not in specs and specs["l2.mix.uk"] == (36, 40)      # a layer that reads layer 0's rows
    assert specs["l1.mix.left.q"] == (120, 88) and specs["l1.mix.left.q.b"] == (120,) and specs["l1.mix.left.k.norm"] == (20,)
    assert specs["l1.mix.left.v"] == (24, 88) and specs["l1.mix.left.o"] == (88, 72) and specs["l1.mix.left.out"] == (88,)
    assert specs["l1.mix.right.q"] == (24, 88) and specs["l1.mix.right.q.conv"] == (24, 4) and specs["l1.mix.right.v.conv"] == (80, 4)
    assert specs["l1.mix.right.b"] == (4, 88) and specs["l1.mix.right.A_log"] == (4,) and specs["l1.mix.right.norm"] == (20,)
    assert specs["l1.mix.right.g"] == (80, 88) and specs["l1.mix.right.o"] == (88, 80) and "l1.mix.right.q.b" not in specs
    assert specs["l1.mlp.router"] == (5, 88) and specs["l1.mlp.router.b"] == (5,) and specs["l1.mlp.e4.gate"] == (24, 88)
    assert specs["l1.mlp.e0.down"] == (88, 24) and "l1.mlp.e5.up" not in specs and specs["l0.mlp.gate"] == (56, 88)
    assert "l3.norm2" not in specs and "l3.mlp.up" not in specs and specs["l3.norm1"] == (88,)
    caches = model.cache_specs()
    assert caches[0] == KVCacheSpec(1, 48, None, values=False) and caches[2] is None and caches[4] is None
    assert caches[3] == KVCacheSpec(1, 42, None, values=False)
    assert isinstance(caches[1], LayerCacheSpec) and caches[1].kv == KVCacheSpec(2, 20, None, v_head_dim=12)
    assert [tuple(s.shape) for s in caches[1].state] == [(4, 12, 20), (3, 128)] and caches[1].state[0].dtype == torch.float32
    assert [c.cache_of for c in model.run] == [None, None, 0, None, 0]
    one_tap = build_luzevik(LuzevikConfig.from_dict(C), 64).cache_specs()[0]
    assert len(one_tap.state) == 1                        # one tap: no rows to carry


def test_random_weights_round_trip(tmp_path):
    from safetensors.torch import load_file
    from tokenmill_amd.weights.random_init import write_random_model
    write_random_model(B, tmp_path, seed=3)
    w = load_file(str(tmp_path / "model.safetensors"))
    assert w["l0.mix.right.q.conv"].shape == (64, 2) and w["l1.mix.sink"].shape == (4,)
    assert torch.isfinite(P.forward(B, w, [3, 1, 4, 1, 5, 9, 2, 6])).all()


# ----------------------------------------------------------------------------------------------- the plain mechanisms

@pytest.mark.parametrize("rot", [{"base": 1e4, "dims": 8}, {"base": 500.0, "dims": 24, "scaling": {"factor": 3.0}}, {"base": 2.5e5, "dims": 16, "scaling": {"factor": 8.0}}])
def test_frequencies_of_the_part_are_the_plain_ones(rot):
    from tokenmill_amd.parts import RotaryEmbedding
    part = RotaryEmbedding(32, rot["base"], 16, rotary_dim=rot["dims"], scaling=rot.get("scaling"), exact=True)
    f, magnitude = part.frequencies()
    assert magnitude == 1.0 and torch.equal(f, P.frequencies(rot))
    if "scaling" in rot:
        plain = dict(rot)
        plain.pop("scaling")
        assert torch.allclose(f * rot["scaling"]["factor"], P.frequencies(plain), rtol=1e-6)


def test_rotation_pairs_channels_half_the_rotated_width_apart():
    rot = {"base": 100.0, "dims": 4}
    v = torch.zeros(1, 1, 6)
    v[0, 0, 0] = 1.0                                       # channel 0 pairs with channel 2
    v[0, 0, 5] = 7.0                                       # behind the rotated channels: untouched
    out = P.rotate_half(v, torch.tensor([3]), rot)
    a = 3.0 * 1.0
    assert torch.allclose(out[0, 0], torch.tensor([math.cos(a), 0.0, math.sin(a), 0.0, 0.0, 7.0]), atol=1e-6)
    x = torch.randn(5, 2, 6)
    pos = torch.arange(5)
    y = P.rotate_half(x, pos, rot)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), atol=1e-5)
    # scores depend on the distance only
    k = torch.randn(1, 1, 6).expand(5, 1, 6)
    a, b = P.rotate_half(k, pos, rot), P.rotate_half(k, pos + 9, rot)
    assert torch.allclose((a[1] * a[3]).sum(), (b[1] * b[3]).sum(), atol=1e-5)


def test_a_sink_joins_the_denominator_once_and_has_no_value():
    T, H, D = 4, 2, 3
    qk = torch.zeros(T, H, D)                              # every score is zero
    v = torch.arange(T, dtype=torch.float32)[:, None, None].expand(T, H, 1)
    sink = torch.tensor([0.0, math.log(3.0)])
    out = P.softmax_attention(qk, qk, v, 1.0, sink)
    for p in range(T):
        assert math.isclose(float(out[p, 0, 0]), sum(range(p + 1)) / (p + 2), rel_tol=1e-6)
        assert math.isclose(float(out[p, 1, 0]), sum(range(p + 1)) / (p + 4), rel_tol=1e-6)
    assert torch.allclose(P.softmax_attention(qk, qk, v, 1.0)[:, 0, 0], torch.tensor([0.0, 0.5, 1.0, 1.5]))
    # the sink is not scaled: another scale leaves zero scores and the sink's share as they are
    assert torch.allclose(P.softmax_attention(qk, qk, v, 0.01, sink), out)


def test_the_delta_rule_replaces_what_a_key_held_and_carries_its_state():
    H, D, Dv, T = 1, 4, 3, 9
    k = torch.eye(D)[[0, 1, 2, 3, 0, 1, 2, 3, 0]].view(T, H, D)
    q = torch.eye(D)[[0] * T].view(T, H, D)
    v = torch.randn(T, H, Dv)
    ones = torch.ones(T, H)
    o, S = P.delta_rule(q, k, v, ones, ones)
    assert torch.allclose(o[3, 0], v[0, 0]) and torch.allclose(o[4, 0], v[4, 0]) and torch.allclose(o[8, 0], v[8, 0])      # replaced, not added
    o2, _ = P.delta_rule(q, k, v, ones, ones * 0.5)
    assert torch.allclose(o2[3, 0], v[0, 0] * 0.125)
    half, _ = P.delta_rule(q, k, v, ones * 0.5, ones)
    assert torch.allclose(half[4, 0], 0.5 * v[4, 0] + 0.25 * v[0, 0])                 # beta: how far towards the new value
    # a cut anywhere: the state carries everything
    torch.manual_seed(0)
    q, k, v = torch.randn(T, 2, D), torch.randn(T, 2, D), torch.randn(T, 2, Dv)
    beta, g = torch.rand(T, 2), torch.rand(T, 2)
    whole, S = P.delta_rule(q, k, v, beta, g)
    a, Sa = P.delta_rule(q[:5], k[:5], v[:5], beta[:5], g[:5])
    b, Sb = P.delta_rule(q[5:], k[5:], v[5:], beta[5:], g[5:], Sa)
    assert torch.allclose(torch.cat([a, b]), whole, atol=1e-6) and torch.allclose(Sb, S, atol=1e-6)


def test_convolution_is_causal_and_its_last_column_is_the_current_token():
    u = torch.randn(6, 2)
    w = torch.tensor([[0.0, 0.0, 1.0], [1.0, 0.0, 0.0]])
    y = P.conv_silu(u, w, torch.float32)
    assert torch.allclose(y[:, 0], P.silu(u[:, 0]))                                   # the last tap alone: the token itself
    assert torch.allclose(y[2:, 1], P.silu(u[:-2, 1])) and float(y[:2, 1].abs().max()) == 0.0     # the first tap: two tokens back, zeros at the start
    ref = torch.nn.functional.conv1d(torch.nn.functional.pad(u.T[None], (2, 0)), w[:, None, :], groups=2)[0].T
    assert torch.allclose(y, P.silu(ref), atol=1e-6)
    # cut: the rows in front of a portion are the state
    tail = P.conv_silu(u[4:], w, torch.float32, before=u[2:4])
    assert torch.allclose(tail, y[4:], atol=1e-6)


def test_router_chooses_by_logits_and_weighs_by_the_softmax_over_the_chosen():
    mlp = {"router": {"experts": 4, "top": 2}}
    t = {"r.router": torch.eye(4), "r.router.b": torch.tensor([0.0, 0.0, 0.0, 5.0])}
    h = torch.tensor([[1.0, 3.0, 2.0, -1.0]])
    chosen, weight = P.route(h, mlp, t, "r.", torch.float32)
    assert chosen.tolist() == [[3, 1]]                                                # the bias counts for the choice and the weight
    assert torch.allclose(weight, torch.softmax(torch.tensor([[4.0, 3.0]]), dim=-1))
    assert math.isclose(float(weight.sum()), 1.0, rel_tol=1e-6)


def test_the_model_taken_apart():
    """With every sublayer's closing norm weight at zero the model is head(norm(scale * embed)); with only layer 0's mixer
    open, its latent attention on the first token is W_o W_uv c / (1 + exp(sink - score)) head by head."""
    from safetensors.torch import load_file  # noqa: F401
    from tokenmill_amd.weights.random_init import random_tensors
    from tokenmill_amd.config.model_config import LuzevikConfig
    from tokenmill_amd.models.luzevik import build_luzevik
    w = dict(random_tensors(build_luzevik(LuzevikConfig.from_dict(A), 64).tensor_specs(), seed=5, std=0.1))
    shut = {k: (torch.zeros_like(v) if k.endswith((".norm1", ".norm2")) else v) for k, v in w.items()}
    ids = [4, 9, 2]
    x = w["embed"].float()[ids] * 2.5
    want = P.rms(x, w["final.norm"], 3e-5) @ w["embed"].float().T
    assert torch.allclose(P.forward(A, shut, ids), want, atol=1e-5)
    # a single token sees itself and the sink
    m = A["layers"][0]["mixer"]
    h = x[:1]
    rows = P.latent_rows(h, m, w, "l0.mix.", 3e-5, torch.tensor([0]), torch.float32)
    got = P.latent_attention(h, m, w, "l0.mix.", 3e-5, torch.tensor([0]), rows, torch.float32)
    c, kr = rows
    cq = P.rms(h @ w["l0.mix.dq"].float().T, w["l0.mix.dq.norm"], 3e-5)
    qh = (cq @ w["l0.mix.uq"].float().T).view(3, 20)
    kh = torch.cat([(c @ w["l0.mix.uk"].float().T).view(3, 12), kr.expand(3, 8)], dim=-1)       # position 0: no rotation
    score = (qh * kh).sum(-1) * m["scale"]
    share = 1.0 / (1.0 + torch.exp(w["l0.mix.sink"].float() - score))
    v = (c @ w["l0.mix.uv"].float().T).view(3, 20) * share[:, None]
    assert torch.allclose(got, v.reshape(1, 60) @ w["l0.mix.o"].float().T, atol=1e-5)


@pytest.mark.parametrize("cfg", [A, B, C])
def test_a_later_token_never_changes_an_earlier_row(cfg):
    from tokenmill_amd.config.model_config import LuzevikConfig
    from tokenmill_amd.models.luzevik import build_luzevik
    from tokenmill_amd.weights.random_init import random_tensors
    w = dict(random_tensors(build_luzevik(LuzevikConfig.from_dict(cfg), 64).tensor_specs(), seed=6, std=0.1, norm_std=0.1))
    ids = [3, 1, 4, 1, 5, 9, 2, 6, 5, 3, 5, 8]
    whole = P.forward(cfg, w, ids)
    assert torch.allclose(P.forward(cfg, w, ids[:7]), whole[:7], atol=2e-5)
