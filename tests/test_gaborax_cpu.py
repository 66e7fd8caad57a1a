"""Gaborax without a GPU: configuration, tensor declarations, what the layers ask of the cache manager, and the plain
implementation's mechanisms pinned against special cases that reduce to something known."""
from __future__ import annotations

import copy
import math

import pytest
import torch

from gaborax_cases import A, B, C
from plain import gaborax_plain as G


# ----------------------------------------------------------------------------------------------- configuration

def test_config_reads_every_size_and_constant():
    from tokenmill_amd.config.model_config import GaboraxConfig
    from tokenmill_amd.config.registry import architecture_name, get_architecture
    assert architecture_name(A) == "Gaborax" and get_architecture("Gaborax").name == "Gaborax"
    cfg = GaboraxConfig.from_dict(A)
    assert (cfg.vocab_size, cfg.hidden_size, cfg.norm_eps, cfg.max_position_embeddings) == (211, 88, 3e-5, None)
    assert [l.type for l in cfg.layers] == ["attention", "attention_2", "attention", "attention_2"]
    assert cfg.layers[0].mlp == {"ff": 40, "experts": 5, "identity": 2, "top": 2, "shared_ff": 24}
    assert cfg.layers[1].mlp == {"ff": 16, "experts": 3, "identity": 0, "top": 3, "shared_ff": None}
    assert cfg.layers[2].mlp is None and cfg.layers[2].mixer["kv_from"] == 0
    assert cfg.layers[1].mixer["rot"]["scaling"] == {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
    assert cfg.layers[1].mixer["softcap"] == 6.0 and "softcap" not in cfg.layers[3].mixer
    limited = dict(copy.deepcopy(C), max_positions=77)
    assert GaboraxConfig.from_dict(limited).max_position_embeddings == 77


@pytest.mark.parametrize("edit,match", [
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c["layers"][0].update(type="gla"), "type"),
    (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][1]["mixer"].pop("vdim"), "vdim"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=4), "kv_heads"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=22), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["rot"]["scaling"].pop("fast"), "scaling.fast"),
    (lambda c: c["layers"][1]["mixer"].update(softcap=0.0), "softcap"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=2), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=1), "equal"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=1), "only an 'attention'"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=8), "experts"),
    (lambda c: c["layers"][0]["mlp"]["router"].pop("experts"), "experts"),
    (lambda c: c["layers"][0]["mlp"]["expert"].pop("ff"), "ff"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "kind"),
])
def test_config_refuses_what_the_model_cannot_be(edit, match):
    from tokenmill_amd.config import ConfigError
    from tokenmill_amd.config.model_config import GaboraxConfig
    raw = copy.deepcopy(A)
    edit(raw)
    with pytest.raises(ConfigError, match=match):
        GaboraxConfig.from_dict(raw)


def test_tensor_names_shapes_and_caches():
    from tokenmill_amd.config.registry import get_architecture
    from tokenmill_amd.parts.base import KVCacheSpec
    arch = get_architecture("Gaborax")
    model = arch.build_model(arch.config_from_dict(A, None), 64)
    specs = model.tensor_specs()
    shape = {k: tuple(v.shape) for k, v in specs.items()}
    assert shape["embed"] == (211, 88) and shape["final.norm"] == (88,) and "head" not in shape
    assert shape["l0.mix.q"] == (120, 88) and shape["l0.mix.k"] == (40, 88) and shape["l0.mix.v"] == (40, 88)
    assert shape["l0.mix.q.norm"] == (120,) and shape["l0.mix.k.norm"] == (40,) and shape["l0.mix.g"] == (6, 88)
    assert shape["l0.mix.o"] == (88, 120) and shape["l0.norm1"] == (88,) and shape["l0.ls2"] == (88,)
    assert "l0.mix.q.b" not in shape and shape["l1.mix.q.b"] == (72,) and shape["l1.mix.v.b"] == (24,) and "l1.mix.g" not in shape
    assert not any(k.startswith(("l2.mix.k", "l2.mix.v", "l2.mlp", "l2.norm2", "l2.ls2")) for k in shape)
    assert shape["l2.mix.q"] == (120, 88) and shape["l2.mix.g"] == (6, 88) and shape["l2.ls1"] == (88,)
    assert shape["l3.mix.v"] == (24, 88) and shape["l3.mix.o"] == (88, 24)
    assert shape["l0.mlp.router"] == (7, 88) and shape["l0.mlp.correction"] == (7,) and shape["l0.mlp.e4.up"] == (40, 88)
    assert "l0.mlp.e5.up" not in shape and shape["l0.mlp.shared.down"] == (88, 24) and shape["l0.mlp.shared.sg"] == (1, 88)
    assert "l1.mlp.shared.up" not in shape and "l1.mlp.shared.sg" not in shape and shape["l1.mlp.e2.down"] == (88, 16)
    caches = model.cache_specs()
    assert caches[2] is None and model.run[2].cache_of == 0
    assert caches[0] == KVCacheSpec(2, 20, None, v_head_dim=20) and caches[3] == KVCacheSpec(2, 16, None, v_head_dim=12)
    # a feed-forward of identity experts only has no expert matrices
    model = arch.build_model(arch.config_from_dict(B, None), 64)
    assert not any(".mlp.e" in k for k in model.tensor_specs() if k.startswith("l2.")) and "l2.mlp.router" in model.tensor_specs()


def test_random_weights_round_trip(tmp_path):
    from safetensors.torch import load_file
    from tokenmill_amd.config.registry import load_config
    from tokenmill_amd.weights.random_init import write_random_model
    write_random_model(C, tmp_path, seed=3, std=0.1, norm_std=0.1)
    arch, cfg = load_config(tmp_path)
    assert arch.name == "Gaborax" and len(cfg.layers) == 2
    w = load_file(str(tmp_path / "model.safetensors"))
    assert set(w) == set(arch.build_model(cfg).tensor_specs())
    assert G.forward(C, w, [1, 2, 3], torch.float32).shape == (3, 97)


# ----------------------------------------------------------------------------------------------- the rotation's frequencies

@pytest.mark.parametrize("rot", [A["layers"][1]["mixer"]["rot"], B["layers"][0]["mixer"]["rot"], C["layers"][1]["mixer"]["rot"],
                                 A["layers"][0]["mixer"]["rot"]])
def test_frequencies_of_the_part_are_the_plain_ones(rot):
    from tokenmill_amd.parts import RotaryEmbedding
    part = RotaryEmbedding(int(rot["dims"]) + 4, rot["base"], 50, rotary_dim=rot["dims"], interleaved=True, scaling=rot.get("scaling"), exact=True)
    f, mag = part.frequencies()
    want, want_mag = G.frequencies(rot)
    assert torch.equal(f, want) and mag == want_mag
    part.build_tables("cpu")
    a = torch.arange(50).float()[:, None] * want[None, :]
    assert torch.equal(part.cos, a.cos() * want_mag if want_mag != 1.0 else a.cos()) and part.sin.shape == (50, rot["dims"] // 2)


def test_scaled_frequencies_keep_fast_pairs_and_divide_slow_ones():
    rot = {"base": 1e4, "dims": 64, "scaling": {"factor": 8.0, "original": 512, "fast": 32.0, "slow": 1.0}}
    f, mag = G.frequencies(rot)
    plain, one = G.frequencies({"base": 1e4, "dims": 64})
    assert one == 1.0 and mag == pytest.approx(0.1 * math.log(8.0) + 1.0)
    turns = 512 * plain / (2 * math.pi)                       # how often a pair turns over the original length
    assert torch.equal(f[turns > 40], plain[turns > 40])      # well above `fast`: unchanged
    assert torch.allclose(f[turns < 0.9], plain[turns < 0.9] / 8.0, rtol=1e-6)
    mid = (turns > 1.5) & (turns < 25)
    assert bool(((f[mid] < plain[mid]) & (f[mid] > plain[mid] / 8.0)).all()) and int(mid.sum()) >= 3
    # a ramp of no width (fast == slow): the divisor keeps the expression finite and the ramp is a step
    step, _ = G.frequencies({"base": 1e4, "dims": 64, "scaling": {"factor": 2.0, "original": 512, "fast": 4.0, "slow": 4.0}})
    assert torch.isfinite(step).all() and set((plain / step).round().tolist()) <= {1.0, 2.0}


def test_rotation_pairs_and_untouched_channels():
    v = torch.randn(5, 2, 12)
    pos = torch.tensor([0, 1, 7, 30, 100])
    rot = {"base": 100.0, "dims": 8}
    for inter in (False, True):
        out = G.rotate(v, pos, rot, interleaved=inter)
        assert torch.equal(out[0], v[0]) and torch.equal(out[..., 8:], v[..., 8:])                  # position 0; channels behind the rotated
        assert torch.allclose(out[..., :8].norm(dim=-1), v[..., :8].norm(dim=-1), rtol=1e-5)
    f, _ = G.frequencies(rot)
    a = 7 * f[1]
    half = G.rotate(v, pos, rot, interleaved=False)[2, 0]
    assert half[1] == pytest.approx(float(v[2, 0, 1] * a.cos() - v[2, 0, 5] * a.sin()), abs=1e-5)
    near = G.rotate(v, pos, rot, interleaved=True)[2, 0]
    assert near[3] == pytest.approx(float(v[2, 0, 3] * a.cos() + v[2, 0, 2] * a.sin()), abs=1e-5)


# ----------------------------------------------------------------------------------------------- attention

def test_capped_scores_and_gate():
    torch.manual_seed(0)
    q, k, v = torch.randn(4, 2, 8) * 3, torch.randn(4, 1, 8) * 3, torch.randn(4, 1, 6)
    pos = torch.arange(4)
    free = G.attend(q, k, v, pos, pos, 0.5)
    assert torch.allclose(free[0], v[0].expand(2, 6))                                  # the first token sees itself only
    capped = G.attend(q, k, v, pos, pos, 0.5, softcap=1e-3)                            # every score ~0: the mean of what is seen
    assert torch.allclose(capped[3, 0], v[:, 0].mean(0), atol=2e-3)
    loose = G.attend(q, k, v, pos, pos, 0.5, softcap=1e4)
    assert torch.allclose(loose, free, atol=1e-4)
    gate = torch.tensor([[0.0, 100.0]] * 4)
    gated = G.attend(q, k, v, pos, pos, 0.5, gate=gate)
    assert torch.allclose(gated[:, 0], free[:, 0] * 0.5) and torch.allclose(gated[:, 1], free[:, 1])


# ----------------------------------------------------------------------------------------------- experts

def _mlp_weights(width, ff, experts, identity, shared, seed):
    torch.manual_seed(seed)
    t = {"m.router": torch.randn(experts + identity, width), "m.correction": torch.zeros(experts + identity)}
    for e in range(experts):
        t[f"m.e{e}.up"], t[f"m.e{e}.down"] = torch.randn(ff, width) * 0.3, torch.randn(width, ff) * 0.3
    if shared:
        t["m.shared.up"], t["m.shared.down"], t["m.shared.sg"] = torch.randn(shared, width) * 0.3, torch.randn(width, shared) * 0.3, torch.randn(1, width)
    return t


def test_router_weights_and_the_correction_that_only_chooses():
    mlp = {"router": {"experts": 4, "identity": 2, "top": 2}}
    t = _mlp_weights(16, 8, 4, 2, None, 1)
    h = torch.randn(9, 16)
    chosen, w = G.route(h, mlp, t, "m.", torch.float32)
    s = torch.softmax(h @ t["m.router"].T, -1)
    assert torch.equal(chosen, s.topk(2).indices) and torch.allclose(w.sum(-1), torch.ones(9))
    assert torch.allclose(w, s.gather(1, chosen) / s.gather(1, chosen).sum(-1, keepdim=True))
    t["m.correction"][5] = 10.0                               # expert 5 is always chosen now, with the weight its own score gives
    chosen2, w2 = G.route(h, mlp, t, "m.", torch.float32)
    assert bool((chosen2[:, 0] == 5).all())
    keep = s.gather(1, chosen2)
    assert torch.allclose(w2, keep / keep.sum(-1, keepdim=True))


def test_identity_experts_return_the_input_and_the_shared_expert_is_gated():
    mlp = {"router": {"experts": 0, "identity": 3, "top": 2}}
    t = _mlp_weights(16, 8, 0, 3, None, 2)
    h = torch.randn(5, 16)
    assert torch.allclose(G.experts(h, mlp, t, "m.", torch.float32), h, atol=1e-6)         # weights sum to one
    t = _mlp_weights(16, 8, 0, 3, 12, 3)
    y = G.experts(h, mlp, t, "m.", torch.float32)
    sh = torch.relu(h @ t["m.shared.up"].T) ** 2 @ t["m.shared.down"].T
    assert torch.allclose(y, h + torch.sigmoid(h @ t["m.shared.sg"].T) * sh, atol=1e-5)
    mlp = {"router": {"experts": 2, "identity": 0, "top": 2}}
    t = _mlp_weights(16, 8, 2, 0, None, 4)
    s = torch.softmax(h @ t["m.router"].T, -1)
    want = sum(s[:, e:e + 1] * (torch.relu(h @ t[f"m.e{e}.up"].T) ** 2 @ t[f"m.e{e}.down"].T) for e in range(2))
    assert torch.allclose(G.experts(h, mlp, t, "m.", torch.float32), want, atol=1e-5)


# ----------------------------------------------------------------------------------------------- the whole model

@pytest.mark.parametrize("cfg", [A, B, C])
def test_plain_prefill_equals_token_by_token(cfg):
    from tokenmill_amd.config.registry import get_architecture
    from tokenmill_amd.weights.random_init import random_tensors
    arch = get_architecture("Gaborax")
    model = arch.build_model(arch.config_from_dict(cfg, None))
    w = dict(random_tensors(model.tensor_specs(), 5, 0.1, 0.1))
    ids = torch.randint(0, cfg["vocab"], (19,), generator=torch.Generator().manual_seed(1)).tolist()
    whole = G.forward(cfg, w, ids, torch.float32)
    state: dict = {}
    parts = [G.forward(cfg, w, ids[:7], torch.float32, 0, state), G.forward(cfg, w, ids[7:9], torch.float32, 7, state)]
    parts += [G.forward(cfg, w, ids[p:p + 1], torch.float32, p, state) for p in range(9, 19)]
    assert torch.allclose(torch.cat(parts), whole, atol=2e-5 * float(whole.abs().max()))
    # a layer that reads another layer's keys and values sees that layer's values: with that layer's own output projection
    # zeroed, scaling its value projection changes nothing before the reading layer and something from it on
    shares = [i for i, l in enumerate(cfg["layers"]) if l["mixer"].get("kv_from") is not None]
    for i in shares:
        src = cfg["layers"][i]["mixer"]["kv_from"]
        w0 = dict(w)
        w0[f"l{src}.mix.o"] = torch.zeros_like(w[f"l{src}.mix.o"])
        w1 = dict(w0)
        w1[f"l{src}.mix.v"] = w[f"l{src}.mix.v"] * 1.5
        trace_a, trace_b = [], []
        G.forward(cfg, w0, ids, torch.float32, trace=trace_a)
        G.forward(cfg, w1, ids, torch.float32, trace=trace_b)
        assert all(torch.equal(trace_a[j], trace_b[j]) for j in range(i))
        assert not torch.allclose(trace_a[i], trace_b[i])
