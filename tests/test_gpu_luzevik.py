"""Luzevik on the GPU against the plain implementation (``tests/plain/luzevik_plain.py``): every mechanism alone, then whole
models through the replay session and the engine: whole prompts, prefill + decoding, portions down to two tokens, mixed
batches with pages and state slots used again, a sink that shows, far rows and page borders, the first tokens, long
decoding, greedy generation through the scheduler."""
from __future__ import annotations

import json
import math

import pytest
import torch

from conftest import random_ids
from luzevik_cases import B, CASES
from plain import luzevik_plain as P
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


# ----------------------------------------------------------------------------------------------- small kernels

@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("W", [72, 88, 1000, 4096])
def test_two_normed_results_averaged(dt, W):
    from tokenmill_amd.hip import ops
    torch.manual_seed(W)
    a, b = q(torch.randn(7, W) * 3, dt), q(torch.randn(7, W) * 0.01, dt)
    b[3] *= 1e-3                                          # a row so small that eps matters
    b = q(b, dt)
    wa, wb = torch.rand(W) + 0.5, torch.randn(W)
    out = torch.empty((7, W), dtype=dt, device=DEV)
    ops.pair_norm_mean(a.to(dt).to(DEV), b.to(dt).to(DEV), wa.to(DEV), wb.to(DEV), out, 1e-5)
    close(out.float().cpu(), q(0.5 * (P.rms(a, wa, 1e-5) + P.rms(b, wb, 1e-5)), dt), dt, "mean of two normed rows", bf16=2.0 ** -8)


@pytest.mark.parametrize("dt", DTS)
def test_gated_gelu_and_scaled_embedding(dt):
    from tokenmill_amd.hip import ops
    from tokenmill_amd.parts import TokenEmbedding
    torch.manual_seed(1)
    gu = q(torch.randn(9, 2 * 52) * 3, dt)
    out = torch.empty((9, 52), dtype=dt, device=DEV)
    ops.gelu_mul(gu.to(dt).to(DEV), out)
    close(out.float().cpu(), q(P.gelu_tanh(gu[:, :52]) * gu[:, 52:], dt), dt, "gelu(gate) * up", bf16=2.0 ** -8)
    table = q(torch.randn(31, 44), dt)
    emb = TokenEmbedding(31, 44, name="e", scale=1.75)
    emb.load({"e": table.to(dt).to(DEV)}, "")
    assert emb.emit(None) is None
    ids = [30, 0, 7, 7]
    assert torch.equal(emb.forward(ints(ids)).cpu(), table[ids] * 1.75)


def test_router_ranks_logits_and_weighs_the_chosen_ones():
    from tokenmill_amd.hip import ops
    torch.manual_seed(2)
    for E, top in ((5, 2), (3, 3), (12, 4), (70, 1), (130, 6), (7, 7)):
        z = torch.randn(40, E + 3) * 2
        z[5, :E] = 0.25                                   # all equal: the lowest indices, equal weights
        z[6, :E] = -300.0                                 # far below zero: no underflow to a zero sum
        z[6, E - 1] = -299.0
        chosen, weight = ops.moe_router(z.to(DEV)[:, :E], E, top, over_chosen=True)
        want = z[:, :E].topk(top, dim=-1)
        chosen, weight = chosen.cpu(), weight.cpu()
        assert chosen[5].tolist() == list(range(top)) and chosen[6].tolist() == [E - 1] + list(range(top - 1))
        free = [t for t in range(40) if t not in (5, 6)]       # rows 5 and 6 hold equal logits: of equals the lower index
        assert torch.equal(chosen[free].long(), want.indices[free]), f"{top} of {E}: another choice"
        close(weight, torch.softmax(want.values, dim=-1), torch.float32, f"{top} of {E}: weights")
    with pytest.raises(ValueError):
        ops.moe_router(z.to(DEV)[:, :7], 7, 2, torch.zeros(7, device=DEV), over_chosen=True)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("H,G_,D,Dv,rot,own", [(6, 2, 20, 12, 8, True), (4, 4, 64, 64, 32, True), (3, 1, 24, 40, 24, True), (3, 3, 16, 8, 0, True),
                                                (5, 1, 36, 36, 12, False)])
def test_norm_head_by_head_rotation_and_store(dt, H, G_, D, Dv, rot, own):
    """Every head of q and k normed over its own channels with a weight the heads share, the first channels rotated in pairs
    half the rotated width apart with scaled frequencies, rounded once; k and v in the tokens' cache slots."""
    from tokenmill_amd.hip import ops
    from tokenmill_amd.parts import RotaryEmbedding
    torch.manual_seed(H * 100 + D)
    T, page, eps = 11, 4, 1e-5
    Q, K, V = H * D, G_ * D, G_ * Dv
    proj = torch.randn(T, Q + (K + V if own else 0) + 2) * 2
    proj[3, D:2 * D] *= 1e-3                               # one head far smaller than its neighbours
    qw, kw = torch.rand(D) + 0.5, torch.rand(D) + 0.5
    pos = torch.tensor([0, 1, 2, 3, 40, 41, 7, 99, 63, 64, 65])
    rd = {"base": 500.0, "dims": rot, "scaling": {"factor": 3.0}} if rot else None
    table = None
    if rot:
        table = RotaryEmbedding(D, 500.0, 128, rotary_dim=rot, scaling=rd["scaling"], exact=True)
        table.build_tables(DEV)
    slots = torch.randperm(T + 5)[:T].to(torch.int32)
    k_pool = torch.zeros((4, page, G_, D), dtype=dt, device=DEV)
    v_pool = torch.zeros((4, G_, Dv, page), dtype=dt, device=DEV)
    q_out = torch.empty((T, Q), dtype=dt, device=DEV)
    ops.whole_norm_rope_store(proj.to(DEV), q_out, H, G_, D, Dv, qw.to(DEV), kw.to(DEV) if own else None, eps,
                              table.cos if rot else None, table.sin if rot else None, False, pos.to(torch.int32).to(DEV), slots.to(DEV),
                              k_pool if own else None, v_pool if own else None, has_kv=own, per_head=True)
    want_q = P.rotate_half(P.rms(proj[:, :Q].view(T, H, D), qw, eps), pos, rd)
    close(q_out.float().cpu().view(T, H, D), q(want_q, dt), dt, "q", bf16=2.0 ** -8)
    if own:
        want_k = P.rotate_half(P.rms(proj[:, Q:Q + K].view(T, G_, D), kw, eps), pos, rd)
        close(k_pool.float().cpu().view(-1, G_, D)[slots.long()], q(want_k, dt), dt, "cached k", bf16=2.0 ** -8)
        got_v = v_pool.float().cpu().permute(0, 3, 1, 2).reshape(-1, G_, Dv)[slots.long()]
        assert torch.equal(got_v, q(proj[:, Q + K:Q + K + V], dt).view(T, G_, Dv)), "cached v"


# ----------------------------------------------------------------------------------------------- mixers alone

def _random_weights(part, dt, std):
    w = {}
    for name, spec in part.tensor_specs("a.").items():
        w[name] = q((torch.rand(spec.shape) + 0.5) if spec.init == "ones" else torch.randn(spec.shape) * std, dt)
    part.load({k: v.to(dt).to(DEV) for k, v in w.items()}, "a.")
    part.prepare(True)
    return w


def _alone(mixer, dt, page=8, pages=80, max_pos=640, slots=4):
    """Pools, manager and the engine's runner around one mixer."""
    from tokenmill_amd.cache import CacheManager
    from tokenmill_amd.cache.pool import CachePools
    from tokenmill_amd.engine.runner import ModelRunner
    from test_gpu_parts import OneLayer
    pools = CachePools(OneLayer(mixer), pages, page, slots, dt, DEV)
    manager = CacheManager(pools.group_specs, pages, page, slots)

    class Shell:
        device = torch.device(DEV)
        head = type("H", (), {"vocab": 10})()

        def program(self, views, tune=None):
            return None
    runner = ModelRunner.__new__(ModelRunner)
    ModelRunner.__init__(runner, Shell(), pools, max_pos)
    return pools, manager, runner


def _run_cuts(mixer, pools, manager, runner, x, cuts, dt, rid="a", beside=None):
    """The rows of x through the mixer in steps of ``cuts`` tokens; ``beside``: rows of a second request that decodes one token
    in every step next to it (its results are dropped)."""
    from tokenmill_amd.engine.runner import StepEntry
    outs, start, rc, other, at = [], 0, None, None, 0
    for n in cuts:
        if rc is None:
            rc = manager.allocate(rid, n)
        else:
            manager.append(rc, start + n)
        entries, rows = [StepEntry(rc, start, [0] * n, [])], [x[start:start + n]]
        if beside is not None and at < beside.shape[0]:
            if other is None:
                other = manager.allocate(rid + "2", 1)
            else:
                manager.append(other, at + 1)
            entries.append(StepEntry(other, at, [0], []))
            rows.append(beside[at:at + 1])
            at += 1
        for e in entries:
            if e.cache.fresh:
                pools.reset_state_slot(e.cache.state_slot)
                e.cache.fresh = False
        ctx, _ = runner.prepare(entries)
        out = mixer.forward(torch.cat(rows).to(dt).to(DEV), ctx, pools.views[0]).float().cpu()
        outs.append(out[:n])
        start += n
    manager.free(rc)
    if other is not None:
        manager.free(other)
    return torch.cat(outs)


CUTS = lambda T: ([T], [2, 5, 40, 1, 1, 64, T - 113], [3] + [1] * (T - 3))     # noqa: E731


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("H,Dn,Dr,Dv,Lq,Lk,own", [(3, 12, 8, 20, 24, 40, True), (2, 10, 6, 14, 16, 36, True), (5, 8, 0, 12, 56, 24, True),
                                                  (4, 64, 32, 64, 96, 128, True), (20, 16, 16, 16, 48, 264, True), (2, 32, 16, 24, 40, 48, False)])
def test_latent_attention_with_sinks_whole_in_portions_and_token_by_token(dt, H, Dn, Dr, Dv, Lq, Lk, own):
    """Pairs half the rotated width apart, a sink per head, no window; the cached rows written by the mixer itself, or (``own``
    False) by a second mixer of other head counts whose rows it reads."""
    from tokenmill_amd.parts import LatentAttention, RotaryEmbedding
    from tokenmill_amd.parts.base import KVCacheView
    std = 0.3 if Dn < 64 and Lk < 256 else 0.1
    rotary = RotaryEmbedding(Dr, 1e4, 640, rotary_dim=Dr, exact=True) if Dr else None
    attn = LatentAttention(64, H, Dn, Dr, Dv, Lq, Lk, 0.3, 1e-5, rotary=rotary, output_gate=False, sink=True, own_kv=own)
    torch.manual_seed(H * 10 + Dn)
    w = _random_weights(attn, dt, std)
    w["a.sink"] = q(torch.randn(H) * 2, dt)
    attn.sink = w["a.sink"].to(DEV)
    m = {"heads": H, "dim": Dn, "rot_dim": Dr, "vdim": Dv, "q_rank": Lq, "kv_rank": Lk, "scale": 0.3}
    if Dr:
        m["rot"] = {"base": 1e4, "dims": Dr}
    T = 150
    x = q(torch.randn(T, 64), dt)
    pos = torch.arange(T)
    if own:
        pools, manager, runner = _alone(attn, dt)
        rows = P.latent_rows(x, m, w, "a.", 1e-5, pos, dt)
        want = q(P.latent_attention(x, m, w, "a.", 1e-5, pos, rows, dt), dt)
        for cuts in CUTS(T):
            close(_run_cuts(attn, pools, manager, runner, x, cuts, dt), want, dt, f"cuts {cuts[:4]}..", bf16=2.0 ** -6)
        assert manager.num_free_pages == manager.num_pages
        return
    writer = LatentAttention(64, 3, 8, Dr, 8, 16, Lk, 0.2, 1e-5, rotary=rotary, output_gate=False, sink=True)
    ww = _random_weights(writer, dt, std)
    pools, manager, runner = _alone(writer, dt)
    mw = {**m, "heads": 3, "dim": 8, "vdim": 8, "q_rank": 16}
    want = q(P.latent_attention(x, m, w, "a.", 1e-5, pos, P.latent_rows(x, mw, ww, "a.", 1e-5, pos, dt), dt), dt)

    class Both:                                            # the writer, then the reader on the writer's rows, as two layers of a model do
        def forward(self, h, ctx, view):
            writer.forward(h, ctx, view)
            return attn.forward(h, ctx, KVCacheView(view.k, view.v, view.group, False))
    for cuts in CUTS(T):
        close(_run_cuts(Both(), pools, manager, runner, x, cuts, dt), want, dt, f"another layer's rows, cuts {cuts[:4]}..", bf16=2.0 ** -6)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("page,H", [(8, 5), (16, 20), (4, 70)])
def test_a_sink_counts_once_and_the_first_rows_show(dt, page, H):
    """Cached rows whose latent is one channel set to one (row j sets channel j % Lk) and whose scores are all zero: a token's
    result is, channel by channel, how many visible rows set that channel, over the number of visible rows plus exp(sink) of
    the head. A sink left out, counted twice (once a chunk of a single token's rows) or scaled, and a row too many or too few
    at the token itself or at position 0, all change it."""
    from tokenmill_amd.hip import ops
    Lk, Dr = 40, 8
    Dk = Lk + Dr
    n = 90
    pool = torch.zeros((n // page + 2, page, 1, Dk), dtype=dt, device=DEV)
    table = torch.randperm(n // page + 2)[: -(-n // page)].to(torch.int32)          # pages in no order
    flat = pool.view(-1, Dk)
    for j in range(n):
        flat[int(table[j // page]) * page + j % page, j % Lk] = 1.0
    sink = (torch.arange(H).float() % 7) - 3.0                                       # exp(sink) from 0.05 to 20
    qa = torch.zeros((n, H * Dk), dtype=dt, device=DEV)
    out = torch.empty((n, H * Lk), dtype=dt, device=DEV)
    tab, seqs, places = table.view(1, -1).to(DEV), ints([0] * n), ints(list(range(n)))
    ops.attn_latent(qa, out, pool, tab, seqs, places, H, Lk, Dk, 0.3, 0, sink=sink.to(DEV))
    results = {"a wavefront a pair": out.float().cpu().view(n, H, Lk)}
    if dt == torch.bfloat16:
        assert ops.attn_latent_mfma_takes(dt, Lk, Dk, H)
        cuts = [(0, 16), (16, 16), (32, 5), (37, 16), (53, 16), (69, 16), (85, 5)]
        tiles = torch.tensor([[0, a, k, a] for a, k in cuts], dtype=torch.int32, device=DEV)
        tiled = torch.full_like(out, math.nan)
        ops.attn_latent_mfma(qa, tiled, pool, tab, tiles, seqs, places, 0, 0, H, Lk, Dk, 0.3, 0, sink=sink.to(DEV))
        results["prompt tiles on the matrix unit"] = tiled.float().cpu().view(n, H, Lk)
        for bound in (n, 4096):                                                     # one run a chunk, and several
            alone = torch.full_like(out, math.nan)
            ops.attn_latent_mfma(qa, alone, pool, tab, None, seqs, places, 0, n, H, Lk, Dk, 0.3, 0, most_context=n, bound=bound, sink=sink.to(DEV))
            results[f"single tokens on the matrix unit, chunks for {bound}"] = alone.float().cpu().view(n, H, Lk)
    for how, got in results.items():
        for p in range(n):
            counts = torch.zeros(Lk)
            for j in range(p + 1):
                counts[j % Lk] += 1.0
            for h in range(H):
                close(got[p, h], q(counts / (p + 1 + math.exp(float(sink[h]))), dt), dt, f"{how}: position {p} head {h}", bf16=2.0 ** -7)


@pytest.mark.parametrize("dt", DTS)
def test_one_far_row_among_hundreds_dominates(dt):
    """A token near position 600 whose query points at one early row gets that row's latent back, less the sink's share."""
    from tokenmill_amd.hip import ops
    H, Lk, Dr, page = 3, 24, 8, 16
    Dk = Lk + Dr
    n = 600
    torch.manual_seed(4)
    rows = q(torch.randn(n, Dk) * 0.1, dt)
    rows[13, Lk + 2] = 8.0                       # the far row stands out in one rotated channel
    pool = torch.zeros((n // page + 1, page, 1, Dk), dtype=dt, device=DEV)
    pool.view(-1, Dk)[:n] = rows.to(dt).to(DEV)
    table = torch.arange(n // page + 1, dtype=torch.int32).view(1, -1).to(DEV)
    qa = torch.zeros((2, H * Dk), dtype=dt, device=DEV)
    qa.view(2, H, Dk)[:, 1, Lk + 2] = 8.0        # head 1 asks for it: its score is 64
    sink = torch.tensor([0.0, 64.0, -5.0])       # head 1's sink weighs as much as the far row: half of it comes back
    out = torch.empty((2, H * Lk), dtype=dt, device=DEV)
    calls = [lambda: ops.attn_latent(qa, out, pool, table, ints([0, 0]), ints([598, 599]), H, Lk, Dk, 1.0, 0, sink=sink.to(DEV))]
    if dt == torch.bfloat16:
        tile = torch.tensor([[0, 0, 2, 598]], dtype=torch.int32, device=DEV)
        for tiles in (None, tile):
            calls.append(lambda tiles=tiles: ops.attn_latent_mfma(qa, out, pool, table, tiles, ints([0, 0]), ints([598, 599]), 0, 2, H, Lk, Dk,
                                                                  1.0, 0, most_context=600, sink=sink.to(DEV)))
    for call in calls:
        out.fill_(math.nan)
        call()
        got = out.float().cpu().view(2, H, Lk)
        close(got[:, 1], 0.5 * rows[13, :Lk].expand(2, Lk), dt, "half the far row", bf16=2.0 ** -6)
        close(got[1, 0], q(rows[:600, :Lk].sum(0) / 601.0, dt), dt, "a head that asks for nothing sees the mean", bf16=2.0 ** -4)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("H,G_,D,Dv,taps", [(4, 2, 12, 20, 4), (2, 2, 32, 48, 2), (6, 3, 64, 16, 3), (2, 1, 160, 24, 1), (3, 1, 20, 12, 5),
                                             (4, 4, 128, 64, 4)])
def test_gated_delta_rule_whole_in_portions_token_by_token_and_beside_another(dt, H, G_, D, Dv, taps):
    from tokenmill_amd.parts import GatedDeltaRule
    torch.manual_seed(H * 7 + D)
    mixer = GatedDeltaRule(64, H, G_, D, Dv, taps, 1e-5)
    w = _random_weights(mixer, dt, 0.25)
    m = {"heads": H, "kv_heads": G_, "dim": D, "vdim": Dv, "conv": taps}
    T = 300                                                # whole, the portion is scanned in segments; in pieces, as one chain
    assert T >= 2 * mixer.SEGMENT > T - 113
    x = q(torch.randn(T, 64), dt)
    want = q(P.gated_delta(x, m, w, "a.", 1e-5, dt), dt)
    pools, manager, runner = _alone(mixer, dt)
    assert len(pools.states) == (2 if taps > 1 else 1) and pools.states[0].dtype == torch.float32
    other = q(torch.randn(60, 64) * 2, dt)
    for cuts in CUTS(T):
        close(_run_cuts(mixer, pools, manager, runner, x, cuts, dt), want, dt, f"cuts {cuts[:4]}..", bf16=2.0 ** -6)
        for t in pools.states.values():                    # whoever comes next into a slot finds zeros by the runner, not by luck
            t.fill_(math.nan)
        close(_run_cuts(mixer, pools, manager, runner, x, cuts, dt, beside=other), want, dt, f"beside another, cuts {cuts[:4]}..", bf16=2.0 ** -6)


@pytest.mark.parametrize("dt", DTS)
def test_the_recurrence_keeps_what_was_written_long_ago_and_forgets_by_its_decay(dt):
    """The scan alone, on rows made by hand. With g = 1, beta = 1 and orthogonal unit keys the state stores every value under
    its key: a query for the first key, 300 tokens later, returns the first value exactly; with g = 0.9 it returns it times
    0.9^299; writing a key a second time replaces its value (the delta rule) instead of adding to it."""
    from tokenmill_amd.hip import ops
    H, G_, D, Dv, T = 2, 1, 8, 6, 300
    C = 2 * G_ * D + H * Dv
    ld = ops.delta_row_width(H, G_, D, Dv)
    for g_val in (1.0, 0.9):
        rows = torch.zeros(T, ld)
        v = torch.randn(T, H, Dv)
        for t in range(T):
            rows[t, D + (t % D)] = 1.0                     # key t % D
            rows[t, 0] = 1.0                               # every query asks for key 0
            rows[t, C + 2 * H] = 1.0 if t % D == 0 else 0.0        # k . q
        rows[:, 2 * D:C] = v.reshape(T, -1)
        rows[:, C:C + H] = 1.0
        rows[:, C + H:C + 2 * H] = g_val
        o = torch.empty((T, H * Dv), dtype=torch.float32, device=DEV)
        state = torch.zeros((2, H, D, Dv), dtype=torch.float32, device=DEV)
        ops.delta_scan(rows.to(DEV), o, state, ints([0, T]), ints([1]), 1, H, G_, D, Dv)
        got = o.cpu().view(T, H, Dv)
        for t in (0, 1, 7, 8, 9, 299):
            last = t - t % D                               # when key 0 was last written
            close(got[t], v[last] * g_val ** (t - last), torch.float32, f"decay {g_val}, token {t}")
        assert float(state[0].abs().max()) == 0.0


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("H,G_,D,Dv,rot,factor", [(6, 2, 20, 12, 8, 4.0), (4, 4, 64, 64, 32, 2.0), (8, 2, 32, 32, 16, None), (3, 3, 16, 8, 0, None),
                                                   (2, 1, 24, 40, 24, None)])
def test_softmax_attention_normed_head_by_head_whole_in_portions_and_token_by_token(dt, H, G_, D, Dv, rot, factor):
    """Biases, q and k normed head by head, a linearly scaled rotation over part of a head; keys and values of one size (the
    kernel library's attention operation) and of two (a wavefront a token and head)."""
    from tokenmill_amd.parts import RotaryEmbedding, SoftmaxAttention
    torch.manual_seed(H * 3 + D)
    rotary = RotaryEmbedding(D, 1e4, 640, rotary_dim=rot, scaling={"factor": factor} if factor else None, exact=True) if rot else None
    attn = SoftmaxAttention(64, H, G_, D, Dv, 0.2, rotary=rotary, qkv_bias=True, head_norm_eps=1e-5)
    w = _random_weights(attn, dt, 0.25)
    m = {"heads": H, "kv_heads": G_, "dim": D, "vdim": Dv, "scale": 0.2}
    if rot:
        m["rot"] = {"base": 1e4, "dims": rot, **({"scaling": {"factor": factor}} if factor else {})}
    T = 150
    x = q(torch.randn(T, 64), dt)
    want = q(P.grouped_attention(x, m, w, "a.", 1e-5, torch.arange(T), dt), dt)
    pools, manager, runner = _alone(attn, dt, page=16, pages=40)
    for cuts in CUTS(T):
        close(_run_cuts(attn, pools, manager, runner, x, cuts, dt), want, dt, f"cuts {cuts[:4]}..", bf16=2.0 ** -6)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("width,ff,experts,top,T", [(88, 24, 5, 2, 77), (88, 40, 3, 3, 9), (128, 48, 4, 1, 1), (72, 20, 7, 2, 200), (64, 24, 40, 4, 3),
                                                    (128, 64, 6, 2, 700)])
def test_routed_gated_experts(dt, width, ff, experts, top, T):
    """A router with a bias that ranks its logits, SwiGLU experts, the chosen ones weighed by the softmax over their logits;
    tiles of 32, 64 and 128 rows; a row alone gives the bits of the row in a batch."""
    from tokenmill_amd.parts import RoutedExperts
    torch.manual_seed(width + experts)
    part = RoutedExperts(width, ff, experts, top, correction=False, activation="swiglu", scoring="chosen_logits", router_bias=True)
    w = _random_weights(part, dt, 0.2)
    # a bias that decides the choice alone: which experts a row uses does not hang on a close call, its weights still do on its logits
    bias = torch.zeros(experts)
    bias[torch.randperm(experts)[:top]] = 6.0
    w["a.router.b"] = q(bias, dt)
    part.router.bias = bias.to(DEV)
    part.router._desc = None
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    x = q(torch.randn(T, width), dt)
    got = part.forward(x.to(dt).to(DEV), None)
    close(got.float().cpu(), q(P.expert_ff(x, mlp, w, "a.", dt), dt), dt, "routed experts", bf16=2.0 ** -6)
    one = part.forward(x[T // 2:T // 2 + 1].to(dt).to(DEV), None)
    if dt == torch.bfloat16 or T <= 100:
        assert torch.equal(one, got[T // 2:T // 2 + 1]), "a row alone differs from the row in a batch"
    else:       # the router's 32-bit product sums a row of many in another order than a row alone: the weights' last bits
        close(one.float().cpu(), got[T // 2:T // 2 + 1].float().cpu(), dt, "a row alone against the row in a batch")


# ----------------------------------------------------------------------------------------------- whole models

def decisive(cfg, w, seed):
    """The same weights with every router's bias replaced by one that decides the choice alone: 6 for `top` experts drawn at
    random, 0 for the others. Which experts a token uses then does not hang on a close call, and its weights still come from
    its own logits."""
    g = torch.Generator().manual_seed(seed)
    out = dict(w)
    for i, layer in enumerate(cfg["layers"]):
        if not layer.get("mlp") or layer["mlp"]["kind"] != "moe":
            continue
        r = layer["mlp"]["router"]
        bias = torch.zeros(r["experts"])
        bias[torch.randperm(r["experts"], generator=g)[:r["top"]]] = 6.0
        out[f"l{i}.mlp.router.b"] = bias.to(w[f"l{i}.mlp.router.b"].dtype)
    return out


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    """name -> (folder, config, plain weights); name + "!" -> the same with routers whose bias decides the choice alone. Under
    bfloat16 a choice of experts that is a close call falls one way in the engine and the other way in the plain run (their
    roundings differ), which moves a token's logits by much and says nothing about either, so the bfloat16 runs of whole
    models use the decisive routers. The 32-bit runs use the random ones."""
    from safetensors.torch import load_file, save_file
    from tokenmill_amd.weights.random_init import write_random_model
    out = {}
    for name, (cfg, seed, std, norm_std) in CASES.items():
        d = tmp_path_factory.mktemp(f"luzevik{name}")
        write_random_model(cfg, d, seed=seed, std=std, norm_std=norm_std)
        w = load_file(str(d / "model.safetensors"))
        out[name] = (d, cfg, w)
        d2 = tmp_path_factory.mktemp(f"luzevik{name}decisive")
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
        _plain_cache[key] = P.forward(cfg, w, ids, dt)
    return _plain_cache[key]


def check_rows(models, name, got, reqs, dt, what):
    """float32: 5e-5 of the largest logit, every row. bfloat16: the model's floor is the largest distance of the plain bfloat16
    run from the plain float32 run over the requests at hand, and the engine may be twice as far from the plain bfloat16 run
    (both differ from the 32-bit run by the same roundings, falling differently). One row in a hundred may be up to four times
    further: where a recurrence's read-out happens to be next to nothing (a query that meets none of the stored keys), the
    norms behind it blow the roundings of the layers before up for that one token, in the plain run as in the engine (fed the
    plain run's own stream, the engine's recurrence gives the plain run's bits there)."""
    assert got, "no rows"
    if dt == torch.float32:
        for (rid, p), row in sorted(got.items()):
            want = plain_logits(models, name, reqs[rid], dt)
            err = float((row - want[p]).abs().max())
            bound = 2.5 * F32_REL * float(want.abs().max())
            assert torch.isfinite(row).all() and err <= bound, f"{what}: request {rid} position {p}: {err:.3e} > {bound:.3e}"
        return
    floor = max(float((plain_logits(models, name, ids, dt) - plain_logits(models, name, ids, torch.float32)).abs().max()) for ids in reqs.values())
    over = 0
    for (rid, p), row in sorted(got.items()):
        want = plain_logits(models, name, reqs[rid], dt)
        bound = max(2.0 * floor, 2.0 ** -7 * float(want.abs().max()))
        err = float((row - want[p]).abs().max())
        assert torch.isfinite(row).all() and err <= 4 * bound, f"{what}: request {rid} position {p}: {err:.3e} > 4 * {bound:.3e}"
        over += err > bound
    assert over <= max(1, len(got) // 100), f"{what}: {over} of {len(got)} rows beyond twice the model's floor"


def make_requests(name, lengths, seed):
    vocab = CASES[name.rstrip("!")][0]["vocab"]
    return {f"r{i}": random_ids(n, vocab, seed * 100 + i) for i, n in enumerate(lengths)}


def poison_freed_slots(session):
    slots, pools = session.manager.slots, session.pools
    plain_release = slots.release

    def release(slot):
        for t in pools.states.values():
            t[slot].fill_(math.nan)
        return plain_release(slot)

    slots.release = release


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", [("A", 16), ("B", 16), ("B", 8), ("C", 4), ("A", 64), ("C", 16)])
def test_whole_decode_portions_mixed(models, name, page, dtype_name):
    from tokenmill_amd.replay import ReplaySession
    from test_gpu_replay import assert_all_given_back, mixed, poison_freed_pages, portions, prefill_then_decode, run_trace, whole
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype_name]
    layers = CASES[name][0]["layers"]
    name = variant(name, dt)
    s = ReplaySession(models[name][0], dtype_name, 4 * 128, max_requests=4, page_size=page)
    assert sum(v is not None for v in s.pools.views) == len(layers)
    for i, layer in enumerate(layers):
        src = layer["mixer"].get("kv_from") if layer["type"] == "latent_attention" else None
        if src is not None:
            assert s.pools.views[i].k is s.pools.views[src].k and not s.pools.views[i].write and s.pools.views[src].write
        if layer["type"] == "parallel":
            held = s.pools.views[i].state
            assert isinstance(held, tuple) and held[0].dtype == torch.float32 and len(held) == (2 if layer["mixer"]["right"]["conv"] > 1 else 1)
    poison_freed_pages(s)
    poison_freed_slots(s)
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
def test_a_far_token_decides_the_logits(models, dtype_name):
    """Weights made so that it shows. Hidden channel 0 is zero in every embedding row but one token's, channel 1 is the same
    constant in all; the first layer's down projection reads channel 0 into the last shared key channel (which the rotation
    turns by next to nothing), and the queries' latent carries channel 1 into the last rotated channel of every head. So
    every query points at the ONE position that holds the token, hundreds of positions back, and the logits follow the plain
    implementation's only if that row is read, from the right page, by prompts and by decoded tokens alike; the layers that
    read layer 0's rows see it too."""
    from safetensors.torch import save_file
    from tokenmill_amd.replay import ReplaySession
    from test_gpu_replay import prefill_then_decode, run_trace, whole
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype_name]
    d, cfg, w = models[variant("A", dt)]
    w2 = {k: v.clone() for k, v in w.items()}
    far_id = 7
    m = cfg["layers"][0]["mixer"]
    H, Dn, Dr, Lq, Lk = m["heads"], m["dim"], m["rot_dim"], m["q_rank"], m["kv_rank"]
    emb = w["embed"].float().clone()
    emb[:, 0], emb[:, 1] = 0.0, 1.0
    emb[far_id, 0] = 8.0
    dkv, dq, uq = w["l0.mix.dkv"].float().clone(), w["l0.mix.dq"].float().clone(), w["l0.mix.uq"].float().clone()
    dkv[Lk + Dr - 1] = 0.0
    dkv[Lk + Dr - 1, 0] = 2.0
    dq[0] = 0.0
    dq[0, 1] = 4.0
    for h in range(H):
        uq[h * (Dn + Dr) + Dn + Dr - 1] = 0.0
        uq[h * (Dn + Dr) + Dn + Dr - 1, 0] = 3.0
    w2["embed"], w2["l0.mix.dkv"], w2["l0.mix.dq"], w2["l0.mix.uq"] = (t.to(torch.bfloat16) for t in (emb, dkv, dq, uq))
    w2["l0.mix.sink"] = torch.full((H,), -4.0).to(torch.bfloat16)
    w2["l0.mix.uv"] = (w["l0.mix.uv"].float() * 3).to(torch.bfloat16)
    folder = d.parent / f"far_{dtype_name}"
    folder.mkdir(exist_ok=True)
    (folder / "config.json").write_text(json.dumps(cfg))
    save_file(w2, str(folder / "model.safetensors"))
    ids = [t if t != far_id else far_id + 1 for t in random_ids(420, cfg["vocab"], 9)]
    ids[5] = far_id
    local = {"A": (folder, cfg, w2)}
    with_far = P.forward(cfg, w2, ids, torch.float32)
    swapped = list(ids)
    swapped[5] = far_id + 1
    without = P.forward(cfg, w2, swapped, torch.float32)
    moved = float((with_far[-40:] - without[-40:]).abs().max()) / float(with_far.abs().max())
    assert moved > 0.02, f"the far token moves the last logits by {moved:.3g} of their size only: the test would not show a lost row"
    s = ReplaySession(folder, dtype_name, 448, max_requests=4, page_size=16)
    for steps, what in ((whole({"a": ids}), "whole"), (prefill_then_decode({"a": ids}, tail=48), "decoded")):
        check_rows(local, "A", run_trace(s, steps), {"a": ids}, dt, f"far token, {what}")


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_long_decoding_over_many_page_borders(models, dtype_name):
    """One token at a time from the third token on: every page border is passed by decoded tokens and the recurrence's state is
    carried over 250 steps, two requests beside each other that start at different times."""
    from tokenmill_amd.replay import ReplaySession
    from test_gpu_replay import assert_all_given_back, poison_freed_pages, run_trace
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype_name]
    which = variant("A", dt)
    s = ReplaySession(models[which][0], dtype_name, 512, max_requests=4, page_size=8)
    poison_freed_pages(s)
    poison_freed_slots(s)
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
        assert kinds.count("LatentAttention") == 4 and kinds.count("ParallelMixer") == 1 and kinds.count("RoutedExperts") == 2
        outs[mode] = eng.generate(prompts, params)
        if mode in ("graphs", "ahead"):
            assert eng.runner.graphs.replays > 10
        assert (eng.stats["steps_ahead"] > 5) == (mode == "ahead")
        assert eng.cache.num_free_pages == eng.cache.num_pages
    tokens = {m: [list(o) for o in outs[m]] for m in outs}
    assert tokens["eager"] == tokens["graphs"] == tokens["chunked"] == tokens["ahead"]
    exempt = 0
    for prompt, toks in zip(prompts, tokens["eager"]):
        rows = P.forward(cfg, w, prompt + toks[:-1], torch.float32)[len(prompt) - 1:]
        for row, tok in zip(rows, toks):
            best = int(row.argmax())
            if tok != best:
                assert float(row[best] - row[tok]) <= 4 * F32_REL * float(row.abs().max()), "a token that is no near-tie"
                exempt += 1
    assert exempt <= 2


def test_command_line_generates_with_a_random_luzevik_model(tmp_path):
    import subprocess
    import sys
    from conftest import ROOT
    (tmp_path / "config.json").write_text(json.dumps(B))
    r = subprocess.run([sys.executable, "-m", "tokenmill_amd.generate", "--random", str(tmp_path / "config.json"), "--prompt-ids",
                        "5,9,33,2;7,7", "--max-tokens", "6", "--max-model-len", "64", "--ignore-eos"], capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [json.loads(ln) for ln in r.stdout.splitlines() if ln.startswith("{")]
    assert [len(ln["output_ids"]) for ln in lines] == [6, 6] and all(0 <= t < 150 for ln in lines for t in ln["output_ids"])
