"""Gaborax on the GPU against the plain implementation (``tests/plain/gaborax_plain.py``): every mechanism alone, then whole
models through the replay session and the engine: whole prompts, prefill + decoding, portions down to two tokens, mixed
batches with pages used again, far keys and page borders, the first tokens, long decoding, greedy generation through the
scheduler."""
from __future__ import annotations

import json
import math

import pytest
import torch

from conftest import random_ids
from gaborax_cases import A, B, CASES
from plain import gaborax_plain as G
from tolerances import F32_REL

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTS = [torch.float32, torch.bfloat16]


def q(x, dt):
    return x.to(dt).float()


def close(got, want, dt, what, bf16=2.0 ** -7):
    assert got.shape == want.shape and torch.isfinite(got).all(), f"{what}: shape or non-finite values"
    scale = float(want.abs().max())
    bound = (F32_REL if dt == torch.float32 else bf16) * max(scale, 1e-6)
    err = float((got - want).abs().max())
    assert err <= bound, f"{what}: max |diff| {err:.3e} > {bound:.3e} (largest value {scale:.3g})"


def ints(v):
    return torch.tensor(v, dtype=torch.int32, device=DEV)


# ----------------------------------------------------------------------------------------------- mechanisms alone

@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("hidden", [72, 88, 1000, 4096])
def test_stream_read_as_it_is_behind_a_scaled_norm(dt, hidden):
    """x += ls * unit(y) * (1 + w), then the next sublayer's input is x itself, rounded: one kernel; also for chosen rows
    only, and with a final norm in place of the pass-through."""
    from tokenmill_amd.parts import GroupRMSNorm, NormedInput, PassThrough, as_tensor
    torch.manual_seed(hidden)
    T, eps = 6, 2e-5
    w, ls, wf = q(torch.randn(hidden) * 0.2, dt), q(torch.rand(hidden) + 0.5, dt), q(torch.randn(hidden) * 0.2, dt)
    behind = GroupRMSNorm(hidden, eps, name="", one_plus=True)
    behind.load({"n": w.to(dt).to(DEV)}, "n")
    behind.fold(ls.to(dt).to(DEV))
    final = GroupRMSNorm(hidden, eps, name="", one_plus=True)
    final.load({"f": wf.to(dt).to(DEV)}, "f")
    resid = torch.randn(T, hidden) * 3 + 1.0
    y = q(torch.randn(T, hidden) * 4, dt)
    y[2] *= 1e-4                                      # a row so small that eps matters
    y = q(y, dt)
    want_sum = resid + ls * G.norm_one_plus(y, w, eps)
    r = resid.to(DEV)
    x = NormedInput(PassThrough(hidden), r, y.to(dt).to(DEV), dt, delta_norm=behind)
    got = as_tensor(x)
    close(r.cpu(), want_sum, torch.float32, "residual after the normed, scaled add")
    close(got.float().cpu(), q(want_sum, dt), dt, "the stream itself, rounded", bf16=2.0 ** -8)
    r2 = resid.to(DEV)
    got = PassThrough(hidden).add_norm(r2, None, dt)
    assert torch.equal(got.float().cpu(), q(resid, dt)) and torch.equal(r2.cpu(), resid)
    rows = ints([5, 0, 5, 3])
    got = final.add_norm(r2, y.to(dt).to(DEV), dt, rows=rows, delta_norm=behind)
    close(got.float().cpu(), q(G.norm_one_plus(want_sum, wf, eps), dt)[rows.cpu().long()], dt, "final norm of chosen rows", bf16=2.0 ** -7)
    assert torch.equal(r2.cpu(), resid)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("H,G_,D,Dv,rot,inter,own", [(6, 2, 20, 20, 12, False, True), (3, 1, 24, 24, 24, True, True), (2, 2, 16, 12, 8, True, True),
                                                      (4, 4, 32, 32, 32, False, False), (5, 1, 8, 8, 8, True, True), (3, 3, 96, 96, 0, False, True)])
def test_whole_projection_norm_rotation_and_store(dt, H, G_, D, Dv, rot, inter, own):
    """q and k normed over all their heads at once, rotated in either pairing over part of a head, rounded once; k and v in
    the tokens' cache slots; a row without k and v (a layer that reads another's cache)."""
    from tokenmill_amd.hip import ops
    from tokenmill_amd.parts import RotaryEmbedding
    torch.manual_seed(H * 100 + D)
    T, page, eps = 11, 4, 1e-5
    Q, K, V = H * D, G_ * D, G_ * Dv
    width = Q + (K + V if own else 0) + 3                     # something behind (a gate's columns)
    proj = torch.randn(T, width) * 2
    qw, kw = torch.rand(Q) + 0.5, torch.rand(K) + 0.5
    pos = torch.tensor([0, 1, 2, 3, 40, 41, 7, 99, 63, 64, 65])
    rd = {"base": 500.0, "dims": rot, "scaling": {"factor": 4.0, "original": 32, "fast": 4.0, "slow": 1.0}} if rot else None
    table = None
    if rot:
        table = RotaryEmbedding(D, 500.0, 128, rotary_dim=rot, interleaved=inter, scaling=rd["scaling"], exact=True)
        table.build_tables(DEV)
    slots = torch.randperm(T + 5)[:T].to(torch.int32)
    k_pool = torch.zeros((4, page, G_, D), dtype=dt, device=DEV)
    v_pool = torch.zeros((4, G_, Dv, page), dtype=dt, device=DEV)
    q_out = torch.empty((T, Q), dtype=dt, device=DEV)
    ops.whole_norm_rope_store(proj.to(DEV), q_out, H, G_, D, Dv, qw.to(DEV), kw.to(DEV) if own else None, eps,
                              table.cos if rot else None, table.sin if rot else None, inter, pos.to(torch.int32).to(DEV), slots.to(DEV),
                              k_pool if own else None, v_pool if own else None, has_kv=own)
    want_q = (G.unit(proj[:, :Q], eps) * qw).view(T, H, D)
    if rot:
        want_q = G.rotate(want_q, pos, rd, inter)
    close(q_out.float().cpu().view(T, H, D), q(want_q, dt), dt, "q", bf16=2.0 ** -8)
    if own:
        want_k = (G.unit(proj[:, Q:Q + K], eps) * kw).view(T, G_, D)
        if rot:
            want_k = G.rotate(want_k, pos, rd, inter)
        got_k = k_pool.float().cpu().view(-1, G_, D)[slots.long()]
        close(got_k, q(want_k, dt), dt, "cached k", bf16=2.0 ** -8)
        got_v = v_pool.float().cpu().permute(0, 3, 1, 2).reshape(-1, G_, Dv)[slots.long()]
        assert torch.equal(got_v, q(proj[:, Q + K:Q + K + V], dt).view(T, G_, Dv)), "cached v"
        unused = torch.ones(16, dtype=torch.bool)
        unused[slots.long()] = False
        assert float(k_pool.float().cpu().view(-1, G_, D)[unused].abs().max()) == 0.0, "wrote a slot of no token"


def _cache_of(keys, values, page, dt, seed):
    """Pools holding keys [n, G, D] / values [n, G, Dv] in pages scattered over the pool (the rest NaN), and the block table."""
    n, G_, D = keys.shape
    Dv = values.shape[2]
    pages = -(-n // page)
    order = torch.randperm(pages + 3, generator=torch.Generator().manual_seed(seed))[:pages]
    k_pool = torch.full((pages + 3, page, G_, D), math.nan, dtype=dt, device=DEV)
    v_pool = torch.full((pages + 3, G_, Dv, page), math.nan, dtype=dt, device=DEV)
    for j in range(pages):
        lo, hi = j * page, min(n, (j + 1) * page)
        k_pool[order[j], :hi - lo] = keys[lo:hi].to(dt).to(DEV)
        v_pool[order[j], :, :, :hi - lo] = values[lo:hi].permute(1, 2, 0).to(dt).to(DEV)
    return k_pool, v_pool, order.to(torch.int32).view(1, -1).to(DEV)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("H,G_,D,Dv,softcap,gated", [(6, 2, 20, 20, 0.0, True), (3, 1, 24, 24, 6.0, False), (2, 2, 16, 12, 2.0, True),
                                                      (4, 1, 32, 40, 0.0, False), (2, 1, 96, 64, 1.0, False)])
def test_attention_a_token_and_a_head_a_wavefront(dt, H, G_, D, Dv, softcap, gated):
    """Keys and values of different sizes, capped scores, a gate per head; 300 keys in scattered pages, one far key that
    one head asks for; queries at the first positions, at page borders and at the end."""
    from tokenmill_amd.hip import ops
    torch.manual_seed(H + D)
    n, page = 300, 8
    keys, values = q(torch.randn(n, G_, D) * 0.3, dt), q(torch.randn(n, G_, Dv), dt)
    keys[13, 0, 2] = 9.0                                    # the far key stands out in one channel
    pos = torch.tensor([0, 1, 2, 7, 8, 9, 12, 13, 14, 63, 64, 255, 256, 298, 299])
    T = len(pos)
    qs = q(torch.randn(T, H, D) * 0.3, dt)
    qs[:, 1 % H, 2] = 9.0                                   # head 1 asks for it
    gate = torch.randn(T, H + 2) if gated else None
    k_pool, v_pool, table = _cache_of(keys, values, page, dt, 1)
    out = torch.empty((T, H * Dv), dtype=dt, device=DEV)
    ops.attn_paged_softmax(qs.view(T, H * D).to(dt).to(DEV), out, k_pool, v_pool, table, ints([0] * T), pos.to(torch.int32).to(DEV), H, G_, D, Dv,
                           0.4, 0, softcap, gate.to(DEV)[:, 1:] if gated else None)
    want = G.attend(qs, keys, values, pos, torch.arange(n), 0.4, softcap, gate[:, 1:1 + H] if gated else None)
    close(out.float().cpu().view(T, H, Dv), q(want, dt), dt, "attention", bf16=2.0 ** -6)
    if not softcap and not gated:
        far = out.float().cpu().view(T, H, Dv)[-1, 1 % H]
        close(far, values[13, 0], dt, "the far key's value", bf16=2.0 ** -5)


@pytest.mark.parametrize("D,H,G_", [(32, 4, 4), (64, 4, 2), (96, 6, 2), (128, 8, 1), (64, 24, 2)])
@pytest.mark.parametrize("softcap", [0.0, 3.0])
def test_capped_scores_on_the_matrix_unit(D, H, G_, softcap):
    """The prompt kernels (keys split over wavefronts; keys shared by a kv head's query heads), the single-token kernels
    (a block a request and kv head; contexts split over blocks) and the 32-bit prompt kernel against the plain softmax with
    capped scores: 600 keys in scattered pages, a far key, tiles that start inside a page and a last one that is not full."""
    from tokenmill_amd.hip import ops
    torch.manual_seed(D + H)
    n, page, dt = 600, 16, torch.bfloat16
    keys, values = q(torch.randn(n, G_, D) * 0.3, dt), q(torch.randn(n, G_, D), dt)
    keys[13, :, 5] = 8.0
    first = n - 53                                          # a portion of 53 tokens at the end of the sequence
    pos = torch.arange(first, n)
    T = len(pos)
    qs = q(torch.randn(T, H, D) * 0.3, dt)
    qs[:, 1, 5] = 8.0
    k_pool, v_pool, table = _cache_of(keys, values, page, dt, 2)
    want = G.attend(qs, keys, values, pos, torch.arange(n), 0.35, softcap)
    qd = qs.view(T, H * D).to(dt).to(DEV)
    cuts = [(0, 16), (16, 16), (32, 5), (37, 16)]
    tiles = torch.tensor([[0, a, k, first + a] for a, k in cuts], dtype=torch.int32, device=DEV)
    for shared in (False, True):
        if shared and not ops.library().tm_attn_prefill_shared_takes(H, G_, D):
            continue
        out = torch.full((T, H * D), math.nan, dtype=dt, device=DEV)
        ops.attn_prefill_mfma(qd, out, k_pool, v_pool, table, tiles, H, G_, D, 0.35, 0, shared=shared, softcap=softcap)
        close(out.float().cpu().view(T, H, D), q(want, dt), dt, f"prompt tiles (shared keys: {shared})", bf16=2.0 ** -6)
    if H // G_ <= 16:
        # every token of the portion as a request of its own that decodes one token over the same pages
        tables = table.expand(T, -1).contiguous()
        ctx = (pos + 1).to(torch.int32).to(DEV)
        for split in (False, True):
            out = torch.full((T, H * D), math.nan, dtype=dt, device=DEV)
            ops.attn_decode_mfma(qd, out, k_pool, v_pool, tables, ctx, H, G_, D, 0.35, 0, n, split=split, softcap=softcap)
            close(out.float().cpu().view(T, H, D), q(want, dt), dt, f"single tokens (contexts split: {split})", bf16=2.0 ** -6)
    if D % 16 == 0 and D <= 128:
        k32, v32, table32 = _cache_of(keys, values, page, torch.float32, 3)
        out = torch.full((T, H * D), math.nan, dtype=torch.float32, device=DEV)
        ops.attn_prefill_f32(qs.view(T, H * D).to(DEV), out, k32, v32, table32, tiles, H, G_, D, 0.35, 0, softcap=softcap)
        close(out.cpu().view(T, H, D), want, torch.float32, "prompt tiles in 32-bit")


def test_router_choices_ties_and_correction():
    from tokenmill_amd.hip import ops
    torch.manual_seed(0)
    for E, top, T in ((7, 2, 33), (3, 3, 5), (16, 4, 64), (130, 6, 9), (1, 1, 4), (64, 64, 3)):
        z = torch.randn(T, E + 2) * 2
        corr = torch.randn(E) * 0.05
        t = {"m.router": torch.eye(E), "m.correction": corr}
        chosen, w = ops.moe_router(z.to(DEV)[:, :E + 2], E, top, corr.to(DEV))
        want_c, want_w = G.route(z[:, :E], {"router": {"top": top}}, t, "m.", torch.float32)
        assert torch.equal(chosen.cpu().long(), want_c), f"choices of {top} among {E}"
        close(w.cpu(), want_w, torch.float32, "weights")
    # equal scores: the lower index first; a correction that lifts the last expert over all others chooses it, with the
    # weight its own (small) score gives
    z = torch.zeros(2, 6)
    chosen, w = ops.moe_router(z.to(DEV), 6, 3, None)
    assert chosen.cpu().tolist() == [[0, 1, 2]] * 2 and torch.allclose(w.cpu(), torch.full((2, 3), 1 / 3))
    z = torch.tensor([[5.0, 0.0, 0.0, -5.0]])
    corr = torch.tensor([0.0, 0.0, 0.0, 3.0])
    chosen, w = ops.moe_router(z.to(DEV), 4, 2, corr.to(DEV))
    s = torch.softmax(z, -1)[0]
    assert chosen.cpu().tolist() == [[3, 0]]
    close(w.cpu()[0], torch.stack([s[3], s[0]]) / (s[3] + s[0]), torch.float32, "weights without the correction")


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("width,ff,experts,identity,top,shared,T", [(88, 40, 5, 2, 2, 24, 77), (88, 16, 3, 0, 3, None, 9), (88, 32, 7, 1, 1, 48, 1),
                                                                      (128, 48, 4, 0, 1, 32, 300), (128, 24, 6, 3, 4, None, 130), (128, 0, 0, 2, 1, 40, 20),
                                                                      (72, 20, 9, 4, 2, 20, 600), (100, 12, 2, 0, 2, None, 2)])
def test_routed_experts(dt, width, ff, experts, identity, top, shared, T):
    """Router, experts (relu squared), experts that stand for the input, the gated shared expert: the part against the plain
    sum, at tile sizes of 32, 64 and 128 rows; a row alone gives the bits it has in the batch."""
    from types import SimpleNamespace
    from tokenmill_amd.parts import RoutedExperts
    torch.manual_seed(width + T)
    part = RoutedExperts(width, ff, experts, top, identity=identity, shared_ff=shared)
    w = {name: q(torch.randn(spec.shape) * (1.0 if name.endswith(("router", "sg")) else 0.2), dt) for name, spec in part.tensor_specs("m.").items()}
    w["m.correction"] = q(torch.randn(experts + identity) * 0.3, dt)
    part.load({k: v.to(dt).to(DEV) for k, v in w.items()}, "m.")
    x = q(torch.randn(T, width), dt)
    mlp = {"router": {"experts": experts, "identity": identity, "top": top}}
    step = SimpleNamespace(num_seqs=1)
    got = part.forward(x.to(dt).to(DEV), step).float().cpu()
    want = G.experts(x, mlp, w, "m.", dt)
    # a choice that is a near-tie in the router's scores may fall the other way: such rows are left out (few)
    z = G.linear(x, w["m.router"], None, dt)
    c = (torch.softmax(z, -1) + w["m.correction"]).topk(min(top + 1, experts + identity)).values
    sure = torch.ones(T, dtype=torch.bool) if top == experts + identity else (c[:, top - 1] - c[:, top]) > 1e-4
    assert int(sure.sum()) >= T * 0.9
    close(got[sure], q(want, dt)[sure], dt, "experts", bf16=2.0 ** -6)
    i = int(sure.nonzero()[len(sure.nonzero()) // 2])
    one = part.forward(x[i:i + 1].to(dt).to(DEV), step).float().cpu()
    close(one[0], got[i], dt, "a row alone against the row in the batch", bf16=2.0 ** -7)


# ----------------------------------------------------------------------------------------------- whole models

def decisive(cfg, w, seed):
    """The same weights with every router's correction replaced by one that decides the choice alone: 2 for `top` experts
    drawn at random (identity experts among them where there are any), 0 for the others; the scores themselves stay below 1.
    Which experts a token uses then does not hang on a close call, and its weights still come from its own scores."""
    g = torch.Generator().manual_seed(seed)
    out = dict(w)
    for i, layer in enumerate(cfg["layers"]):
        if layer.get("mlp") is None:
            continue
        r = layer["mlp"]["router"]
        n = r["experts"] + r.get("identity", 0)
        corr = torch.zeros(n)
        corr[torch.randperm(n, generator=g)[:r["top"]]] = 2.0
        out[f"l{i}.mlp.correction"] = corr.to(w[f"l{i}.mlp.correction"].dtype)
    return out


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    """name -> (folder, config, plain weights); name + "!" -> the same with routers that decide by their correction alone.
    Under bfloat16 a choice of experts that is a close call falls one way in the engine and the other way in the plain run
    (their roundings differ), which moves a token's logits by much and says nothing about either; such calls cannot be kept
    out of a random model (a token in twenty has one), so the bfloat16 runs of whole models use the decisive routers. The
    32-bit runs use the random ones, where every token's choice is its own."""
    from safetensors.torch import load_file, save_file
    from tokenmill_amd.weights.random_init import write_random_model
    out = {}
    for name, (cfg, seed, std, norm_std) in CASES.items():
        d = tmp_path_factory.mktemp(f"gaborax{name}")
        write_random_model(cfg, d, seed=seed, std=std, norm_std=norm_std)
        w = load_file(str(d / "model.safetensors"))
        out[name] = (d, cfg, w)
        d2 = tmp_path_factory.mktemp(f"gaborax{name}decisive")
        w2 = decisive(cfg, w, seed)
        (d2 / "config.json").write_text(json.dumps(cfg))
        save_file(w2, str(d2 / "model.safetensors"))
        out[name + "!"] = (d2, cfg, w2)
    return out


def variant(name, dt):
    return name if dt == torch.float32 else name + "!"


_plain_cache: dict = {}


def plain_logits(models, name, ids, dt):
    key = (name, tuple(ids), dt)
    if key not in _plain_cache:
        _, cfg, w = models[name]
        _plain_cache[key] = G.forward(cfg, w, ids, dt)
    return _plain_cache[key]


def check_rows(models, name, got, reqs, dt, what):
    """float32: 5e-5 of the largest logit. bfloat16: the engine may be twice as far from the plain bfloat16 run as that run
    is from the plain float32 run (both differ from it by the same roundings, falling differently), per request."""
    assert got, "no rows"
    for (rid, p), row in sorted(got.items()):
        want = plain_logits(models, name, reqs[rid], dt)
        if dt == torch.float32:
            bound = 2.5 * F32_REL * float(want.abs().max())
        else:
            bound = max(2.0 * float((want - plain_logits(models, name, reqs[rid], torch.float32)).abs().max()),
                        2.0 ** -7 * float(want.abs().max()))
        err = float((row - want[p]).abs().max())
        assert torch.isfinite(row).all() and err <= bound, f"{what}: request {rid} position {p}: {err:.3e} > {bound:.3e}"


def make_requests(name, lengths, seed):
    vocab = CASES[name.rstrip("!")][0]["vocab"]
    return {f"r{i}": random_ids(n, vocab, seed * 100 + i) for i, n in enumerate(lengths)}


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", [("A", 16), ("B", 16), ("B", 8), ("C", 4), ("A", 64), ("C", 16)])
def test_whole_decode_portions_mixed(models, name, page, dtype_name):
    from tokenmill_amd.replay import ReplaySession
    from test_gpu_replay import assert_all_given_back, mixed, poison_freed_pages, portions, prefill_then_decode, run_trace, whole
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype_name]
    layers = CASES[name][0]["layers"]
    name = variant(name, dt)
    s = ReplaySession(models[name][0], dtype_name, 4 * 128, max_requests=4, page_size=page)
    assert sum(v is not None for v in s.pools.views) == len(layers) and not s.pools.states
    shared = [i for i, l in enumerate(layers) if l["mixer"].get("kv_from") is not None]
    for i in shared:
        src = s.pools.views[layers[i]["mixer"]["kv_from"]]
        assert s.pools.views[i].k is src.k and s.pools.views[i].v is src.v and not s.pools.views[i].write and src.write
    poison_freed_pages(s)
    lengths = [1, 9, 26, 53, 120]
    reqs = make_requests(name, lengths, 1)
    got = run_trace(s, whole(reqs))
    assert len(got) == sum(lengths)
    check_rows(models, name, got, reqs, dt, "whole")
    assert_all_given_back(s)
    check_rows(models, name, run_trace(s, prefill_then_decode(reqs, tail=60)), reqs, dt, "prefill + decode")
    assert_all_given_back(s)
    steps = portions({k: v for k, v in reqs.items() if len(v) >= 2})
    assert min(len(e["tokens"]) for st in steps for e in st["entries"]) == 2
    check_rows(models, name, run_trace(s, steps), reqs, dt, "portions")
    assert_all_given_back(s)
    many = make_requests(name, [37, 64, 21, 90, 48, 33, 75, 18, 59, 44, 96, 27, 70, 52, 85, 40, 113, 66], 2)
    steps = mixed(many, seed=5)
    assert max(len(st["entries"]) for st in steps) == 4
    got = run_trace(s, steps)
    assert len(got) == sum(len(v) for v in many.values())
    check_rows(models, name, got, many, dt, "mixed")
    assert_all_given_back(s)


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_a_far_token_decides_the_logits(models, name, dtype_name):
    """Weights made so that it shows. Hidden channel 0 is zero in every embedding row but one token's, channel 1 is the same
    constant in all; the first layer's key projection reads channel 0 into the last channel of key head 0 (which the
    rotation leaves alone, or turns by next to nothing), its query projection reads channel 1 into the same channel of that
    key head's query heads. So every query points at the ONE position that holds the token, hundreds of positions back, and
    the logits follow the plain implementation's only if that key is read, from the right page, by prompts and by decoded
    tokens alike."""
    from safetensors.torch import save_file
    from tokenmill_amd.replay import ReplaySession
    from test_gpu_replay import prefill_then_decode, run_trace, whole
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype_name]
    d, cfg, w = models[variant(name, dt)]
    w2 = {k: v.clone() for k, v in w.items()}
    far_id = 7
    m = cfg["layers"][0]["mixer"]
    H, G_, D = m["heads"], m["kv_heads"], m["dim"]
    emb = w["embed"].float().clone()
    emb[:, 0], emb[:, 1] = 0.0, 1.0
    emb[far_id, 0] = 8.0
    wk, wq = w["l0.mix.k"].float().clone(), w["l0.mix.q"].float().clone()
    wk[D - 1] = 0.0
    wk[D - 1, 0] = 4.0
    for h in range(H // G_):
        wq[h * D + D - 1] = 0.0
        wq[h * D + D - 1, 1] = 4.0
    w2["embed"], w2["l0.mix.k"], w2["l0.mix.q"] = emb.to(torch.bfloat16), wk.to(torch.bfloat16), wq.to(torch.bfloat16)
    w2["l0.mix.v"] = (w["l0.mix.v"].float() * 3).to(torch.bfloat16)
    folder = d.parent / f"far_{name}_{dtype_name}"
    folder.mkdir(exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg))
    save_file(w2, str(folder / "model.safetensors"))
    ids = [t if t != far_id else far_id + 1 for t in random_ids(420, cfg["vocab"], 9)]
    ids[5] = far_id
    local = {name: (folder, cfg, w2)}
    with_far = G.forward(cfg, w2, ids, torch.float32)
    swapped = list(ids)
    swapped[5] = far_id + 1
    without = G.forward(cfg, w2, swapped, torch.float32)
    moved = float((with_far[-40:] - without[-40:]).abs().max()) / float(with_far.abs().max())
    assert moved > 0.02, f"the far token moves the last logits by {moved:.3g} of their size only: the test would not show a lost key"
    s = ReplaySession(folder, dtype_name, 448, max_requests=4, page_size=16)
    for steps, what in ((whole({"a": ids}), "whole"), (prefill_then_decode({"a": ids}, tail=48), "decoded")):
        got = run_trace(s, steps)
        check_rows(local, name, got, {"a": ids}, dt, f"far token, {what}")


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_long_decoding_over_many_page_borders(models, dtype_name):
    """One token at a time from the third token on: every page border is passed by decoded tokens, two requests beside each
    other that start at different times."""
    from tokenmill_amd.replay import ReplaySession
    from test_gpu_replay import assert_all_given_back, poison_freed_pages, run_trace
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype_name]
    which = variant("A", dt)
    s = ReplaySession(models[which][0], dtype_name, 512, max_requests=4, page_size=8)
    poison_freed_pages(s)
    n, m = 260, 150
    a, b = random_ids(n, 211, 77), random_ids(m, 211, 78)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:3], "want": [0, 1, 2]}], "end": []}]
    for p in range(3, n):
        entries = [{"id": "a", "tokens": [a[p]], "want": [0]}]
        if p == 60:
            entries.append({"id": "b", "tokens": b[:2], "want": [0, 1]})
        elif 60 < p < 60 + m - 1:
            entries.append({"id": "b", "tokens": [b[p - 59]], "want": [0]})
        ends = (["a"] if p == n - 1 else []) + (["b"] if p == 60 + m - 2 else [])
        steps.append({"step": p - 2, "entries": entries, "end": ends})
    got = run_trace(s, steps)
    assert len(got) == n + m
    check_rows(models, which, got, {"a": a, "b": b}, dt, "long decoding")
    assert_all_given_back(s)


def test_greedy_generation_through_the_engine_and_its_graphs(models):
    """The engine's own entry point: scheduler, chunked prefill, sampling, HIP graphs for the decode steps, decode steps
    queued ahead. Every token is the plain implementation's first choice at its place (or a near-tie with it), and all
    modes agree."""
    from tokenmill_amd import EngineConfig, LLMEngine, SamplingParams
    d, cfg, w = models["A"]
    prompts = [random_ids(n, 211, 500 + i) for i, n in enumerate([12, 3, 30, 7, 21, 16, 45, 25, 5, 18])]
    params = [SamplingParams(max_tokens=8 + 5 * (i % 4), ignore_eos=True) for i in range(len(prompts))]
    outs = {}
    for mode in ("eager", "graphs", "chunked", "ahead"):
        eng = LLMEngine(EngineConfig(model=str(d), dtype="float32", block_size=8, num_blocks=48, max_model_len=96,
                                     max_num_seqs=4, max_num_batched_tokens=32 if mode == "chunked" else 64, watermark=0.0,
                                     hip_graphs=mode != "eager", enable_chunked_prefill=mode == "chunked",
                                     pipeline_decode=mode == "ahead"))
        kinds = [type(p).__name__ for p in eng.runner.program.foreign_parts]
        assert kinds.count("SoftmaxAttention") == 4 and kinds.count("RoutedExperts") == 3
        outs[mode] = eng.generate(prompts, params)
        if mode in ("graphs", "ahead"):
            assert eng.runner.graphs.replays > 10
        assert (eng.stats["steps_ahead"] > 5) == (mode == "ahead")
        assert eng.cache.num_free_pages == eng.cache.num_pages
    tokens = {m: [list(o) for o in outs[m]] for m in outs}
    assert tokens["eager"] == tokens["graphs"] == tokens["chunked"] == tokens["ahead"]
    exempt = 0
    for prompt, toks in zip(prompts, tokens["eager"]):
        rows = G.forward(cfg, w, prompt + toks[:-1], torch.float32)[len(prompt) - 1:]
        for row, tok in zip(rows, toks):
            best = int(row.argmax())
            if tok != best:
                assert float(row[best] - row[tok]) <= 4 * F32_REL * float(row.abs().max()), "a token that is no near-tie"
                exempt += 1
    assert exempt <= 2


def test_command_line_generates_with_a_random_gaborax_model(tmp_path):
    import subprocess
    import sys
    from conftest import ROOT
    (tmp_path / "config.json").write_text(json.dumps(B))
    r = subprocess.run([sys.executable, "-m", "tokenmill_amd.generate", "--random", str(tmp_path / "config.json"), "--prompt-ids",
                        "5,9,33,2;7,7", "--max-tokens", "6", "--max-model-len", "64", "--ignore-eos"], capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [json.loads(ln) for ln in r.stdout.splitlines() if ln.startswith("{")]
    assert [len(ln["output_ids"]) for ln in lines] == [6, 6] and all(0 <= t < 150 for ln in lines for t in ln["output_ids"])
