"""Mafosun on the GPU against the plain implementation (plain_mafosun.py): every mechanism alone, then whole models
of small configurations through the step function, the scheduler and the replay program.

The weights are drawn here with a spread that keeps activations of order one and head norms whose weights make the
softmax rows peaked; the mechanism tests scale single queries and keys so that one score stands out: a key that is
missed, a pooled block that is seen a position too early, a window or chunk that is one token off, a sink that is left
out or a state that is lost then moves the result far beyond rounding."""

import copy
import json
import math
import os
import subprocess
import sys
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import helpers
import plain_mafosun as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from from_scratch_inference_engine_amd import ops as o

    o.load()
    return o


def rnd(shape, seed, scale=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale


def rel(got, ref):
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    return float(np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-30))


def tol(dtype, f32=2e-5, bf16=2.0 ** -6):
    return f32 if dtype == torch.float32 else bf16


def i32(values):
    return torch.tensor(values, dtype=torch.int32).cuda()


# ------------------------------------------------------------------------------------------------
# mechanisms alone
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [64, 90, 257, 4104])
def test_output_norm_sum_and_stream_in_one_pass(ops, dtype, hidden):
    """x + norm(y) written back and returned as it is (no second norm), for a delta of the activations' type, a float32
    delta beside 16-bit activations and partial sums; chosen rows without writing back."""
    t, eps = 9, 1e-3
    res, w = rnd((t, hidden), 1, 3.0), rnd((hidden,), 2) + 1.0
    for kind in ("same", "f32", "parts"):
        if kind == "parts":
            delta = rnd((3, t, hidden), 3)
            whole = delta.double().sum(0)
        else:
            delta = rnd((t, hidden), 3).to(dtype if kind == "same" else torch.float32)
            whole = delta.double()
        ref = res.double().numpy() + plain.rms_norm(whole.numpy(), w.double().numpy(), eps)
        r = res.clone().cuda()
        out = ops.sandwich_norm(r, delta.cuda(), w.cuda(), eps, None, 0.0, dtype, write_back=True)
        assert out.dtype == dtype and rel(out.float().cpu(), ref) <= tol(dtype, 2e-6, 2.0 ** -8), kind
        assert rel(r.cpu(), ref) <= 2e-6, kind
        rows = torch.tensor([7, 0, 7, 3], dtype=torch.int32)
        r = res.clone().cuda()
        out = ops.sandwich_norm(r, delta.cuda(), w.cuda(), eps, None, 0.0, dtype, rows=rows.cuda())
        assert rel(out.float().cpu(), ref[rows.long().numpy()]) <= tol(dtype, 2e-6, 2.0 ** -8) and torch.equal(r.cpu(), res)


def test_stream_reader_and_branch_norm_block(ops):
    """The block x += n1(mixer(x)); x += n2(ffn(x)) with sublayers that read the stream itself, on toy sublayers."""
    from from_scratch_inference_engine_amd.parts import BranchNormBlock, HiddenState, RMSNorm, StreamReader

    t, h, eps = 5, 48, 1e-5

    class Twice:
        def forward(self, x, ctx, cache=None):
            return (x.float() * 2.0 + 1.0).to(x.dtype)

    class Square:
        def forward(self, x, ctx):
            return (x.float() ** 2).to(x.dtype)
    n1, n2 = RMSNorm(h, eps), RMSNorm(h, eps)
    n1.weight, n2.weight = (rnd((h,), 1) + 1.0).cuda(), (rnd((h,), 2) + 1.0).cuda()
    block = BranchNormBlock(StreamReader(h), Twice(), n1, Square(), n2)
    x0 = rnd((t, h), 3)
    hidden = HiddenState(x0.clone().cuda())
    ctx = SimpleNamespace(compute_dtype=torch.float32)
    block.forward(hidden, ctx, None)
    x = x0.double().numpy()
    x = x + plain.rms_norm(2 * x + 1, n1.weight.double().cpu().numpy(), eps)
    assert rel(hidden.residual.cpu(), x) <= 1e-6  # (the first sum is made; the second is pending)
    x = x + plain.rms_norm(x * x, n2.weight.double().cpu().numpy(), eps)
    got = StreamReader(h)(hidden, torch.float32)
    assert rel(got.cpu(), x) <= 1e-6 and hidden.delta is None


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv, dim, vdim, rot", [(6, 3, 24, 40, 16), (4, 4, 64, 64, 0), (3, 1, 20, 7, 10), (8, 2, 80, 160, 0)])
def test_attention_prep_norms_values_as_they_are_cached(ops, dtype, heads, kv, dim, vdim, rot):
    """q and k heads through their weighted RMS norm and the rotation, every kv head's values divided by their root mean
    square; all of it as the cache and the queries hold it."""
    t, page, eps = 11, 4, 1e-3
    pd = dim if vdim == dim else -(-max(dim, vdim) // 16) * 16
    width = heads * dim + kv * dim + kv * vdim
    proj = rnd((t, width), 1, 2.0).to(dtype)
    qw, kw = rnd((dim,), 2) + 1.0, rnd((dim,), 3) + 1.0
    pos = np.arange(3, 3 + t)
    freqs = plain.rotary_frequencies(rot, 100.0) if rot else None
    table = None
    if rot:
        ang = pos[:, None] * freqs[None, :]
        table = torch.tensor(np.stack([np.cos(ang), np.sin(ang)], -1), dtype=torch.float32).cuda()
    units = 5
    k_pool, v_pool = torch.zeros((units, kv, page, pd), dtype=dtype).cuda(), torch.zeros((units, kv, pd, page), dtype=dtype).cuda()
    slots = i32([4 + i for i in range(t)])
    q, _ = ops.attention_prep(proj.cuda(), 0, heads * dim, heads * dim + kv * dim, 0, heads, kv, dim, vdim, pd, qw.cuda(), kw.cuda(),
                              eps, rot // 2, table, False, slots=slots, k_pool=k_pool, v_pool=v_pool, v_unit_norm_eps=eps)
    p = proj.double().numpy()
    qr = plain.rms_norm(p[:, :heads * dim].reshape(t, heads, dim), qw.double().numpy(), eps)
    kr = plain.rms_norm(p[:, heads * dim:heads * dim + kv * dim].reshape(t, kv, dim), kw.double().numpy(), eps)
    if rot:
        qr, kr = plain.rotate(qr, pos, freqs, rot, "half"), plain.rotate(kr, pos, freqs, rot, "half")
    vr = plain.unit_rms(p[:, heads * dim + kv * dim:].reshape(t, kv, vdim), eps)
    got_q = q.float().cpu().numpy().reshape(t, heads, pd)
    assert rel(got_q[..., :dim], qr) <= tol(dtype, 1e-5) and not got_q[..., dim:].any()
    kp, vp = k_pool.float().cpu().numpy(), v_pool.float().cpu().numpy()
    for i in range(t):
        unit, off = (4 + i) // page, (4 + i) % page
        assert rel(kp[unit, :, off, :dim], kr[i]) <= tol(dtype, 1e-5), i
        assert rel(vp[unit, :, :vdim, off], vr[i]) <= tol(dtype, 1e-5), i
        assert not vp[unit, :, vdim:, off].any()


def attention_case(seqs, heads, kv, hd, page, dtype, seed, planner, pool=None, pooled_page=None, edit=None):
    """Pools, tables and the planner's items for requests (past, new); with ``pool`` also the pools of pooled blocks,
    empty: the test fills them with the kernel."""
    g = torch.Generator().manual_seed(seed)
    n_pages = sum(-(-(p + n) // page) for p, n in seqs) + 2
    order = torch.randperm(n_pages, generator=g).tolist()
    k_pool, v_pool = torch.full((n_pages, kv, page, hd), 7.0), torch.full((n_pages, kv, hd, page), -9.0)
    tables = torch.full((len(seqs), max(-(-(p + n) // page) for p, n in seqs)), -1, dtype=torch.int32)
    qs, ks, vs = [], [], []
    for p, n in seqs:
        qs.append(torch.randn(p + n, heads * hd, generator=g).to(dtype).float())
        ks.append(torch.randn(p + n, kv * hd, generator=g).to(dtype).float())
        vs.append(torch.randn(p + n, kv * hd, generator=g).to(dtype).float())
    if edit is not None:
        edit(qs, ks, vs)
    for s, (p, n) in enumerate(seqs):
        total, held = p + n, -(-(p + n) // page)
        k_all, v_all = torch.full((held * page, kv, hd), 7.0), torch.full((held * page, kv, hd), -9.0)
        k_all[:total], v_all[:total] = ks[s].reshape(total, kv, hd), vs[s].reshape(total, kv, hd)
        for i in range(held):
            unit = order.pop()
            tables[s, i] = unit
            k_pool[unit] = k_all[i * page:(i + 1) * page].permute(1, 0, 2)
            v_pool[unit] = v_all[i * page:(i + 1) * page].permute(1, 2, 0)
    host = SimpleNamespace(n_seqs=len(seqs), q_lens=[n for _, n in seqs], past_lens=[p for p, _ in seqs], q_starts=[0],
                           page_size=page, compute_dtype=dtype, pad=None)
    for _, n in seqs:
        host.q_starts.append(host.q_starts[-1] + n)
    host.n_tokens = host.q_starts[-1]
    case = dict(q=torch.cat([q[p:] for q, (p, n) in zip(qs, seqs)]).to(dtype), k_pool=k_pool.to(dtype), v_pool=v_pool.to(dtype),
                tables=tables, plan=planner.plan(host), qs=qs, ks=ks, vs=vs)
    if pool:
        held = [-(-((p + n) // pool) // pooled_page) for p, n in seqs]
        units = sum(held) + 2
        order = torch.randperm(units - 1, generator=g).add(1).tolist()
        ptab = torch.full((len(seqs), max(max(held), 1)), -1, dtype=torch.int32)
        for s, h in enumerate(held):
            for i in range(h):
                ptab[s, i] = order.pop()
        case.update(pk=torch.full((units, kv, pooled_page, hd), 3.0).to(dtype), pv=torch.full((units, kv, hd, pooled_page), 3.0).to(dtype),
                    ptab=ptab)
    return case


def run_attention(case, heads, kv, hd, window, scale, cap=None, sinks=None, pooled=None, share_keys=True):
    from from_scratch_inference_engine_amd.parts.attention import paged_attention

    plan = {k: (torch.from_numpy(v).cuda() if isinstance(v, np.ndarray) else v) for k, v in case["plan"].items()}
    cache = SimpleNamespace(k_pool=case["k_pool"].cuda(), v_pool=case["v_pool"].cuda(), block_tables=case["tables"].cuda(),
                            page_size=case["k_pool"].shape[2])
    q = case["q"].cuda()
    return paged_attention(q, heads * hd, cache, SimpleNamespace(**plan), heads, kv, hd, window, scale, q.shape[0],
                           share_keys=share_keys, softcap=cap, sinks=sinks, pooled=pooled).float().cpu().numpy()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv, hd, page, chunk", [(4, 2, 64, 16, 48), (6, 1, 32, 8, 10), (2, 2, 48, 16, 7), (8, 2, 128, 16, 100),
                                                        (3, 3, 20, 5, 1), (3, 1, 16, 8, 11), (6, 2, 16, 4, 5)])
def test_chunked_attention_on_every_kernel(ops, dtype, heads, kv, hd, page, chunk):
    """A query reads the keys of its own chunk, counted from the request's start: decoded tokens at a chunk's first and
    last position, portions that start and end inside chunks and span several, first tokens.  Peaked rows: a key of
    the chunk before would take the row if it were seen."""
    from from_scratch_inference_engine_amd.parts.attention import AttentionPlanner

    seqs = [(0, 1), (chunk - 1, 1), (chunk, 1), (3 * chunk + chunk // 2, 1), (0, 3 * chunk + 2), (chunk // 2, 150), (2 * chunk - 1, 2),
            (500, 70)]
    scale = 0.6
    planner = AttentionPlanner(heads, kv, hd, None, chunk=chunk)
    case = attention_case(seqs, heads, kv, hd, page, dtype, seed=hd + chunk, planner=planner)
    outs = [run_attention(case, heads, kv, hd, None, scale)]
    if case["plan"]["mfma"] and ops.attention_mfma_lds_ok(hd, page):
        outs.append(run_attention(case, heads, kv, hd, None, scale, share_keys=False))
    if dtype == torch.bfloat16:
        assert case["plan"]["mfma"] == (hd % 16 == 0 and page % 4 == 0)
    row = 0
    for (p, n), q, k, v in zip(seqs, case["qs"], case["ks"], case["vs"]):
        total = p + n
        ref = plain.chunk_attention(q.double().numpy().reshape(total, heads, hd), k.double().numpy().reshape(total, kv, hd),
                                    v.double().numpy().reshape(total, kv, hd), scale, chunk)[p:].reshape(n, heads * hd)
        for out in outs:
            err = np.abs(out[row:row + n] - ref).max()
            assert err <= (3e-6 if dtype == torch.float32 else 2.0 ** -7) * v.abs().max().item(), f"past {p} new {n}: {err}"
        row += n


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv, hd, page, window, pool, pooled_page", [(4, 2, 64, 16, 32, 8, 16), (6, 1, 32, 8, 10, 4, 8),
                                                                            (2, 2, 48, 16, 5, 7, 3), (3, 3, 20, 4, 1, 1, 4),
                                                                            (4, 4, 64, 16, 80, 10, 16), (6, 2, 32, 8, 9, 5, 8),
                                                                            (3, 1, 16, 4, 7, 3, 2)])
def test_window_with_pooled_blocks_a_sink_and_a_cap(ops, dtype, heads, kv, hd, page, window, pool, pooled_page):
    """The pooled blocks are made by the kernel from the cached keys and values (the mean of a block's positions), then
    every query reads its window, the blocks that lie wholly before it, and a sink of score 0: decoded tokens against long
    contexts (cut into items and merged, on an idle and on a full device), short and long portions, blocks larger than
    the window, blocks and windows of one position."""
    from from_scratch_inference_engine_amd.parts.attention import AttentionPlanner

    seqs = [(0, 1), (window + pool - 2, 1), (window + pool - 1, 1), (window + pool, 1), (700, 1), (0, 150), (300, 2), (123, 70),
            (2100, 1)]
    scale, cap = 0.5, 4.0
    sinks = torch.zeros(heads).cuda()
    outs = []
    for units in (4096, 1):
        AttentionPlanner.compute_units = units
        try:
            planner = AttentionPlanner(heads, kv, hd, window, pool=pool)
            case = attention_case(seqs, heads, kv, hd, page, dtype, seed=hd + pool, planner=planner, pool=pool, pooled_page=pooled_page)
        finally:
            AttentionPlanner.compute_units = None
        assert case["plan"]["mfma"] == (dtype == torch.bfloat16 and hd % 16 == 0 and page % 4 == 0)
        # every whole block of every request, as if all its positions had come in this step
        jobs = [(s, b) for s, (p, n) in enumerate(seqs) for b in range((p + n) // pool)]
        pk, pv, ptab = case["pk"].cuda(), case["pv"].cuda(), case["ptab"].cuda()
        ops.pool_blocks(case["k_pool"].cuda(), case["v_pool"].cuda(), case["tables"].cuda(), pk, pv, ptab,
                        i32(jobs + [(-1, 0)]).reshape(-1, 2), len(jobs) + 1, pool)
        outs.append(run_attention(case, heads, kv, hd, window, scale, cap, sinks, pooled=(pk, pv, ptab, pool)))
    # the pooled entries are the blocks' means
    pkc, pvc = pk.float().cpu().numpy(), pv.float().cpu().numpy()
    for s, (p, n) in enumerate(seqs):
        for b in range((p + n) // pool):
            unit, off = int(case["ptab"][s, b // pooled_page]), b % pooled_page
            k_mean = case["ks"][s][b * pool:(b + 1) * pool].double().mean(0).reshape(kv, hd).numpy()
            v_mean = case["vs"][s][b * pool:(b + 1) * pool].double().mean(0).reshape(kv, hd).numpy()
            assert rel(pkc[unit, :, off, :], k_mean) <= tol(dtype, 1e-6, 2.0 ** -8) and rel(pvc[unit, :, :, off], v_mean) <= tol(dtype, 1e-6, 2.0 ** -8)
    row = 0
    for (p, n), q, k, v in zip(seqs, case["qs"], case["ks"], case["vs"]):
        total = p + n
        ref = plain.window_pool_attention(q.double().numpy().reshape(total, heads, hd), k.double().numpy().reshape(total, kv, hd),
                                          v.double().numpy().reshape(total, kv, hd), scale, window, pool, cap, True)[p:].reshape(n, heads * hd)
        for out in outs:
            err = np.abs(out[row:row + n] - ref).max()
            assert err <= (3e-6 if dtype == torch.float32 else 2.0 ** -6) * v.abs().max().item(), f"past {p} new {n}: {err}"
        row += n


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_finds_a_far_block_and_the_edges_of_window_and_pool(ops, dtype):
    """For every query one key carries the softmax: a position in the very first pooled block of a long context, the
    oldest key the window still holds, a position of the block that has just become visible; a louder key in the gap
    between window and the last visible block, and one after the query, must stay unseen.  And with nothing loud the
    sink takes its share."""
    from from_scratch_inference_engine_amd.parts.attention import AttentionPlanner

    heads, kv, hd, page, window, pool, scale = 4, 2, 64, 16, 24, 6, 1.0
    seqs = [(900, 1), (window + 2 * pool - 1, 3), (0, 60), (0, 3)]  # (fewer positions than dimensions: a direction each)

    def target_of(pos):
        first = pos - window + 1
        seen = max(0, first) // pool
        return ("block", 0) if pos >= 400 else (("block", seen - 1) if seen and pos % 2 else ("key", max(first, 0)))

    def edit(qs, ks, vs):
        for s, (p, n) in enumerate(seqs):
            ks[s].mul_(0.02)
            for pos in range(p, p + n):
                kind, at = target_of(pos)
                direction = torch.zeros(hd)
                direction[(5 * s + 3 * pos) % hd] = 1.0
                qs[s][pos] = (2.0 * direction).repeat(heads)
                if kind == "key":
                    ks[s][at] += (6.0 * direction).repeat(kv)
                else:  # every position of the block, so that the mean is loud
                    ks[s][at * pool:(at + 1) * pool] += (6.0 * direction).repeat(kv)
                gap = (max(0, pos - window + 1) // pool) * pool  # first position that is neither pooled nor in the window
                if gap < pos - window + 1:
                    ks[s][gap] += (40.0 * direction).repeat(kv)
                if pos + 1 < p + n:
                    ks[s][pos + 1] += (40.0 * direction).repeat(kv)
            for t in (qs[s], ks[s]):
                t.copy_(t.to(dtype).float())
    planner = AttentionPlanner(heads, kv, hd, window, pool=pool)
    case = attention_case(seqs, heads, kv, hd, page, dtype, seed=3, planner=planner, pool=pool, pooled_page=8, edit=edit)
    jobs = [(s, b) for s, (p, n) in enumerate(seqs) for b in range((p + n) // pool)]
    pk, pv, ptab = case["pk"].cuda(), case["pv"].cuda(), case["ptab"].cuda()
    ops.pool_blocks(case["k_pool"].cuda(), case["v_pool"].cuda(), case["tables"].cuda(), pk, pv, ptab, i32(jobs), len(jobs), pool)
    sinks = torch.zeros(heads).cuda()
    out = run_attention(case, heads, kv, hd, window, scale, None, sinks, pooled=(pk, pv, ptab, pool))
    no_sink = run_attention(case, heads, kv, hd, window, scale, None, None, pooled=(pk, pv, ptab, pool))
    row = 0
    for s, ((p, n), q, k, v) in enumerate(zip(seqs, case["qs"], case["ks"], case["vs"])):
        total = p + n
        shaped = (q.double().numpy().reshape(total, heads, hd), k.double().numpy().reshape(total, kv, hd),
                  v.double().numpy().reshape(total, kv, hd))
        ref = plain.window_pool_attention(*shaped, scale, window, pool, None, True)[p:].reshape(n, heads * hd)
        assert np.abs(out[row:row + n] - ref).max() <= (1e-5 if dtype == torch.float32 else 2.0 ** -6) * v.abs().max().item(), s
        for i in range(n):
            kind, at = target_of(p + i)
            chosen = v[at].double().numpy() if kind == "key" else v[at * pool:(at + 1) * pool].double().mean(0).numpy()
            chosen = chosen.reshape(kv, hd)
            for h in range(heads):
                mine = out[row + i, h * hd:(h + 1) * hd]
                assert np.abs(mine - chosen[h // (heads // kv)]).max() <= 0.05 * np.abs(chosen).max() + 0.05, (s, i, h, kind, at)
        row += n
    # quiet keys: with scores near zero the sink holds one part in (keys + 1) of every row
    quiet = attention_case([(0, 3)], heads, kv, hd, page, dtype, seed=4, planner=planner, pool=pool, pooled_page=8,
                           edit=lambda qs, ks, vs: [k.mul_(0.0) for k in ks])
    pk, pv, ptab = quiet["pk"].cuda(), quiet["pv"].cuda(), quiet["ptab"].cuda()
    with_sink = run_attention(quiet, heads, kv, hd, window, scale, None, sinks, pooled=(pk, pv, ptab, pool))
    v = quiet["vs"][0].double().numpy().reshape(3, kv, hd)
    for i in range(3):
        want = v[:i + 1].sum(0) / (i + 2)
        for h in range(heads):
            assert np.abs(with_sink[i, h * hd:(h + 1) * hd] - want[h // (heads // kv)]).max() <= tol(dtype, 1e-5, 2.0 ** -6)
    assert np.abs(no_sink - out).max() >= 0.0  # (both ran; the loud rows hardly feel the sink)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, dim, vdim, decays", [(4, 40, 56, (0.5, 0.9, 0.999, 1.0)), (1, 20, 7, (0.97,)), (3, 130, 33, (0.875, 0.99, 0.9995)),
                                                      (2, 64, 64, (0.96875, 0.99993896484375))])
def test_retention_over_portions_steps_and_slots(ops, dtype, heads, dim, vdim, decays):
    """Three requests in unequal portions (single tokens, portions below and above the length from which the walk goes
    chunk by chunk, ragged chunks) over several steps, one of them in a slot that another has used: every output is
    the recurrence over the request's own earlier tokens, with decays from one half to one."""
    lens = {"a": 330, "b": 21, "c": 47}
    width = 2 * heads * dim + heads * vdim
    proj = {r: rnd((n, width), 1 + i, 1.0).to(dtype) for i, (r, n) in enumerate(lens.items())}
    for r in proj:
        proj[r][0] *= 4.0  # a loud first token: a state that forgets it too early is far off at the end
    state = torch.full((4, heads, dim, vdim), 55.0).cuda()
    slot = {"a": 0, "b": 2, "c": 2}
    plan = [[("a", 1), ("b", 1)], [("b", 2), ("a", 2)], [("a", 15), ("b", 17)], [("a", 16), ("b", 1)], [("a", 200), ("c", 3)],
            [("c", 1), ("a", 1)], [("c", 43), ("a", 95)]]
    fed, got = {r: 0 for r in lens}, {r: [] for r in lens}
    decay = torch.tensor(decays, dtype=torch.float32).cuda()
    scale = dim ** -0.5
    rot = dim // 4 * 2  # the first channels of every q and k head turn by the position, inside the scan's first kernel
    freqs = plain.rotary_frequencies(rot, 300.0)
    for step in plan:
        rows, starts, slots, pos = [], [0], [], []
        for r, n in step:
            if fed[r] == 0:
                state[slot[r]] = 0.0  # (the engine zeroes the slots of the requests that start)
            rows.append(proj[r][fed[r]:fed[r] + n])
            pos += list(range(fed[r], fed[r] + n))
            starts.append(starts[-1] + n)
            slots.append(slot[r])
        ang = np.asarray(pos, dtype=np.float64)[:, None] * freqs[None, :]
        table = torch.tensor(np.stack([np.cos(ang), np.sin(ang)], -1), dtype=torch.float32).cuda()
        o = ops.gla_scan(torch.cat(rows).cuda(), 0, heads * dim, 2 * heads * dim, None, state, i32(starts), i32(slots), heads, dim,
                         vdim, scale, 1.0, head_decay=decay, cos_sin=table).sum(0).cpu()
        at = 0
        for r, n in step:
            got[r].append(o[at:at + n])
            at += n
            fed[r] += n
    for r, n in lens.items():
        p = proj[r].double().numpy()
        q, k = p[:, :heads * dim].reshape(n, heads, dim), p[:, heads * dim:2 * heads * dim].reshape(n, heads, dim)
        q, k = plain.rotate(q, np.arange(n), freqs, rot, "half"), plain.rotate(k, np.arange(n), freqs, rot, "half") * scale
        ref = plain.retention(q, k, p[:, 2 * heads * dim:].reshape(n, heads, vdim), decays).reshape(n, heads * vdim)
        assert rel(torch.cat(got[r]), ref) <= 2e-5, r  # (the scan is float32 whatever the inputs' type)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("t, hidden, ff, experts, top, groups, keep", [(50, 64, 96, 8, 2, 2, 1), (7, 90, 34, 6, 3, 3, 2), (300, 40, 18, 4, 1, 1, 1),
                                                                      (1, 32, 32, 1, 1, 1, 1), (130, 72, 50, 12, 4, 4, 4), (33, 48, 16, 9, 3, 3, 1)])
def test_grouped_softmax_routing_and_gated_experts(ops, dtype, t, hidden, ff, experts, top, groups, keep):
    """Softmax scores over all experts, the choice limited to the best groups, the scores themselves as weights, and
    experts with a SiLU gate, against the plain ones; the logits are spread so that no choice is a rounding apart, and
    the best expert of a token often lies in a group that loses."""
    from from_scratch_inference_engine_amd.parts import RoutedExperts

    x = rnd((t, hidden), 1).to(dtype)
    w = {"mlp.router": rnd((experts, hidden), 2, 3.0 / math.sqrt(hidden)).to(dtype)}
    for j in range(experts):
        w[f"mlp.e{j}.gate"], w[f"mlp.e{j}.up"] = rnd((ff, hidden), 10 + j, hidden ** -0.5).to(dtype), rnd((ff, hidden), 40 + j, hidden ** -0.5).to(dtype)
        w[f"mlp.e{j}.down"] = rnd((hidden, ff), 70 + j, ff ** -0.5).to(dtype)
    part = RoutedExperts(hidden, ff, experts, top, scores="softmax", groups=groups, keep=keep, renorm=False, correction=False, gated="silu")
    part.router_weight = w["mlp.router"].cuda()
    part.up_weight = torch.cat([torch.stack([w[f"mlp.e{j}.gate"], w[f"mlp.e{j}.up"]], 1).reshape(2 * ff, hidden) for j in range(experts)]).cuda()
    part.down_weight = torch.cat([w[f"mlp.e{j}.down"] for j in range(experts)]).cuda()
    got = part.forward(x.cuda(), None).cpu()
    w64 = {k: v.double().numpy() for k, v in w.items()}
    mlp = {"router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}
    ref = plain.expert_ff(x.double().numpy(), w64, "mlp.", mlp)
    ids, weights = ops.moe_route(x.cuda(), part.router_weight, None, top, 1.0, scores="softmax", groups=groups, keep=keep, renorm=False)
    ref_ids, ref_w = plain.route(x.double().numpy() @ w64["mlp.router"].T, top, groups, keep)
    z = np.sort(x.double().numpy() @ w64["mlp.router"].T, axis=-1)
    sure = np.ones(t, bool) if experts == 1 else (np.abs(np.diff(z, axis=-1)).min(-1) > (1e-4 if dtype == torch.float32 else 0.05))
    assert sure.sum() >= t // 3
    assert (np.sort(ids.cpu().numpy()[sure], -1) == np.sort(ref_ids[sure], -1)).all()
    assert rel(np.sort(weights.cpu().numpy()[sure], -1), np.sort(ref_w[sure], -1)) <= tol(dtype, 1e-5, 2.0 ** -6)
    assert rel(got.numpy()[sure], ref[sure]) <= tol(dtype, 2e-5, 2.0 ** -5)


@pytest.mark.parametrize("dtype", DTYPES)
def test_dense_feed_forward_with_a_relu_gate(ops, dtype):
    from from_scratch_inference_engine_amd.parts import SwiGLU, prepare_parts

    for t, hidden, ff in ((1, 64, 40), (5, 128, 320), (200, 72, 50)):
        x = rnd((t, hidden), 1).to(dtype)
        w = {"mlp.gate": rnd((ff, hidden), 2, hidden ** -0.5).to(dtype), "mlp.up": rnd((ff, hidden), 3, hidden ** -0.5).to(dtype),
             "mlp.down": rnd((hidden, ff), 4, ff ** -0.5).to(dtype)}
        part = SwiGLU(hidden, ff, activation="relu")
        part.gate_up_weight = torch.stack([w["mlp.gate"], w["mlp.up"]], 1).reshape(2 * ff, hidden).contiguous().cuda()
        part.down_weight = w["mlp.down"].cuda()
        prepare_parts(part, "cuda", dtype, {"weight_copies": True})
        got = part.forward(x.cuda(), SimpleNamespace(partial_sums_ok=False)).float().cpu()
        ref = plain.dense_ff(x.double().numpy(), {k: v.double().numpy() for k, v in w.items()}, "mlp.")
        assert rel(got, ref) <= tol(dtype, 1e-5, 2.0 ** -6), (t, hidden, ff)


# ------------------------------------------------------------------------------------------------
# whole models
# ------------------------------------------------------------------------------------------------
def rotation(base, dims, scaling=None):
    r = {"base": base, "dims": dims}
    if scaling:
        r["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return r


def attention(heads, kv, dim, vdim, scale, size, pool=None, cap=None, rot=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": size}}
    if pool:
        m["mask"]["pool"] = pool
    if cap:
        m["softcap"] = cap
    if rot:
        m["rot"] = rot
    return m


def retention_of(heads, dim, vdim, decay, rot=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}
    if rot:
        m["rot"] = rot
    return m


def side_by_side(left, right, ls, rs):
    return {"left": left, "right": right, "left_scale": ls, "right_scale": rs}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, n, top, groups, keep):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": n, "top": top, "groups": {"count": groups, "keep": keep}}}


def layer(kind, mixer, mlp):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


# A: both kinds of layer, windows and chunks far shorter than the prompts, blocks larger than the window in one layer,
#    values wider and narrower than keys, partly rotated heads with rescaled frequencies
CONFIG_A = {"architecture": "Mafosun", "width": 72, "vocab": 150, "norm": {"eps": 1e-6}, "layers": [
    layer("parallel", side_by_side(attention(6, 3, 24, 40, 0.3, 16), retention_of(3, 24, 16, (0.9, 0.99, 1.0), rotation(500.0, 16)), 1.3, 0.4),
          moe(40, 6, 2, 3, 1)),
    layer("attention", attention(4, 2, 32, 20, 0.25, 10, 4, 6.0, rotation(1000.0, 20, (4.0, 1.0, 4.0, 64))), dense(100)),
    layer("attention", attention(2, 1, 16, 16, 0.3, 5, 7, None, rotation(77.0, 16)), None),
    layer("parallel", side_by_side(attention(2, 2, 16, 16, 0.4, 33), retention_of(2, 40, 36, (0.5, 0.999)), 1.0, 1.0), dense(50)),
]}
# B: attention only; no rotation in one layer, one kv head a query head, blocks and a window of one position, a window
#    without blocks, top 1, one group
CONFIG_B = {"architecture": "Mafosun", "width": 64, "vocab": 97, "norm": {"eps": 1e-5}, "layers": [
    layer("attention", attention(4, 4, 16, 24, 0.3, 1, 1, 3.0), moe(24, 1, 1, 1, 1)),
    layer("attention", attention(4, 1, 32, 32, 0.2, 12, 12, 30.0, rotation(10000.0, 32, (6.0, 1.0, 3.0, 32))), moe(32, 5, 1, 1, 1)),
    layer("attention", attention(2, 2, 48, 48, 0.15, 21, None, None, rotation(200.0, 24)), dense(72)),  # a window alone
]}
# C: two mixers side by side only, heads of sizes the matrix-core kernels take, a chunk of one page, every head with
#    its own decay, all experts chosen
CONFIG_C = {"architecture": "Mafosun", "width": 128, "vocab": 300, "norm": {"eps": 1e-5}, "layers": [
    layer("parallel", side_by_side(attention(4, 2, 64, 128, 0.15, 8), retention_of(4, 32, 32, (0.7, 0.9, 0.97, 0.995), rotation(2e5, 32)), 0.7, 1.9),
          moe(48, 4, 4, 2, 2)),
    layer("parallel", side_by_side(attention(8, 2, 32, 64, 0.2, 40), retention_of(1, 64, 128, (0.99,), rotation(100.0, 8)), 2.0, 0.25), dense(96)),
]}
# D: sizes that are multiples of nothing
CONFIG_D = {"architecture": "Mafosun", "width": 90, "vocab": 101, "norm": {"eps": 1e-4}, "layers": [
    layer("attention", attention(6, 2, 20, 12, 0.4, 9, 5, 9.0, rotation(50.0, 10)), moe(34, 9, 3, 3, 1)),
    layer("parallel", side_by_side(attention(3, 1, 10, 14, 0.5, 11), retention_of(5, 10, 14, (0.6, 0.8, 0.9, 0.95, 1.0), rotation(300.0, 6)), 0.9, 1.1),
          moe(26, 3, 2, 1, 1)),
]}
CONFIGS = {"A": CONFIG_A, "B": CONFIG_B, "C": CONFIG_C, "D": CONFIG_D}


def mafosun_tensors(cfg, seed, sharp=True):
    """``sharp``: head norms that make the softmax rows peaked (the float32 tests: a key that is missed shows at once).
    Not sharp: the same tensors with mild head norms, for bfloat16, where a peaked row turns a rounding of the input
    into another key, which says nothing about the kernels (those models also use all their experts: ``without_choices``)."""
    g = torch.Generator().manual_seed(seed)
    w = cfg["width"]

    def mat(rows, cols, gain=1.0):
        return torch.randn((rows, cols), generator=g) * (gain / math.sqrt(cols))

    def vec(n, centre, spread):
        return centre + torch.randn((n,), generator=g) * spread
    out = {"embed": torch.randn((cfg["vocab"], w), generator=g), "embed.norm": vec(w, 1.0, 0.2), "final.norm": vec(w, 1.0, 0.2)}

    def attention_tensors(p, m):
        h, kv, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        out.update({p + "q": mat(h * d, w), p + "k": mat(kv * d, w), p + "v": mat(kv * e, w), p + "o": mat(w, h * e),
                    p + "q.norm": vec(d, 2.0 if sharp else 1.0, 0.3), p + "k.norm": vec(d, 2.0 if sharp else 1.0, 0.3)})
    for i, lay in enumerate(cfg["layers"]):
        m, p = lay["mixer"], f"l{i}.mix."
        out[f"l{i}.norm1"] = vec(w, 1.0, 0.2)
        if lay["type"] == "attention":
            attention_tensors(p, m)
        else:
            attention_tensors(p + "left.", m["left"])
            r, q = m["right"], p + "right."
            out.update({q + "q": mat(r["heads"] * r["dim"], w, 2.0), q + "k": mat(r["heads"] * r["dim"], w, 2.0),
                        q + "v": mat(r["heads"] * r["vdim"], w), q + "g": mat(r["heads"] * r["vdim"], w, 2.0),
                        q + "o": mat(w, r["heads"] * r["vdim"])})
        mlp = lay["mlp"]
        if mlp is not None:
            q = f"l{i}.mlp."
            out[f"l{i}.norm2"] = vec(w, 1.0, 0.2)
            if mlp["kind"] == "dense":
                out.update({q + "gate": mat(mlp["ff"], w, 1.5), q + "up": mat(mlp["ff"], w, 1.5), q + "down": mat(w, mlp["ff"], 1.5)})
            else:
                ff = mlp["expert"]["ff"]
                out[q + "router"] = mat(mlp["router"]["experts"], w, 10.0)  # (logits far apart: few choices are a rounding apart)
                for j in range(mlp["router"]["experts"]):
                    out.update({f"{q}e{j}.gate": mat(ff, w, 1.5), f"{q}e{j}.up": mat(ff, w, 1.5), f"{q}e{j}.down": mat(w, ff, 1.5)})
    return {k: v.to(torch.bfloat16).contiguous() for k, v in out.items()}


def without_choices(cfg):
    """The same configuration with every expert chosen (all groups kept, top = experts): the weights are the softmax
    scores, a continuous function of the input.  For whole models in bfloat16, where a choice between two groups of
    experts that is made by a hair falls either way and the other group is another function; the choice itself is
    tested alone in both types and in whole models in float32."""
    cfg = copy.deepcopy(cfg)
    for lay in cfg["layers"]:
        if lay["mlp"] is not None and lay["mlp"]["kind"] == "moe":
            r = lay["mlp"]["router"]
            r["top"], r["groups"]["keep"] = r["experts"], r["groups"]["count"]
    return cfg


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = tmp_path_factory.mktemp("mafosun")
    out = {}
    for name, cfg in CONFIGS.items():
        for tag, sharp in (("", True), ("~", False)):
            d = helpers.make_model_dir(root / (name + tag), cfg if sharp else without_choices(cfg), 0,
                                       tensors=mafosun_tensors(cfg, seed=ord(name), sharp=sharp))
            out[name + tag] = (d, plain.read_config(d), plain.read_weights(d))
    return out


def clear_rows(cfg, w, ids, least=0.03):
    """The first positions of a sequence up to the first token whose choice of experts, in any layer, is made by less
    than ``least`` of its logits' spread.  In bfloat16 such a choice can fall the other way; the other group of experts
    is another function, and what it writes reaches every later position through keys, values and states."""
    margins = []
    plain.forward(cfg, w, ids, margins=margins)
    if not margins:
        return len(ids)
    close = np.nonzero(np.min(np.stack(margins), axis=0) < least)[0]
    return int(close[0]) if len(close) else len(ids)


def close_enough(got, ref, dtype, what):
    """float32: 1e-4 of the largest logit at every position.  bfloat16: the difference's root mean square against the
    logits'; with random weights the router's choice between two groups of experts is now and then a rounding apart,
    and the other group is another function whose output the layer's norm brings to full size, so a few positions may
    be far off while the typical one must be close."""
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape and np.isfinite(got).all(), what
    if dtype == "float32":
        bad = np.abs(got - ref).max(-1) > 1e-4 * np.abs(ref).max()
        assert not bad.any(), f"{what}: first wrong position {int(np.argmax(bad))}, {np.abs(got - ref).max():.3e}"
    else:
        err = np.sqrt(((got - ref) ** 2).mean(-1)) / np.sqrt((ref ** 2).mean())
        far = int((err > 0.12).sum())
        assert far <= max(1, len(err) // 10) and np.median(err) <= 0.06, \
            f"{what}: {far} of {len(err)} rows far off, the median row by {np.median(err):.3f} of the logits' size"


def step_through(runner, plan, seqs):
    """``plan``: steps of [(request, tokens)]; returns {request: logits of all its positions}.  A request is
    opened at its first entry and closed after its last token."""
    from from_scratch_inference_engine_amd.engine.context import StepEntry

    fed, caches, got = {r: 0 for r in seqs}, {}, {r: [] for r in seqs}
    for step in plan:
        entries = []
        for r, n in step:
            if r not in caches:
                caches[r] = runner.manager.open(r)
            entries.append(StepEntry(caches[r], seqs[r][fed[r]:fed[r] + n], list(range(n))))
            fed[r] += n
        out = runner.step(entries).cpu().numpy()
        row = 0
        for (r, n) in step:
            got[r].append(out[row:row + n])
            row += n
            if fed[r] == len(seqs[r]):
                runner.manager.close(caches.pop(r))
        runner.manager.check_invariants()
    return {r: np.concatenate(v) for r, v in got.items() if v}


def test_the_plain_model_feels_every_mechanism(models):
    """The oracle itself: taking a mechanism away (the sink, the pooled blocks, a window's or a chunk's edge, the cap, the
    rescaled frequencies, the decay, the value norm, the groups of the router, a scale of the two mixers, the norm of the
    embedding) moves its logits by far more than the tolerances of the tests below."""
    d, cfg, w = models["A"]
    ids = helpers.token_ids(cfg["vocab"], 90, 1)
    ref = plain.forward(cfg, w, ids)
    size = np.abs(ref).max()

    def moved(cfg2, w2, forward=plain.forward):
        return np.abs(forward(cfg2, w2, ids) - ref).max() / size
    edits = {
        "pool": lambda c, x: c["layers"][1]["mixer"]["mask"].pop("pool"),
        "pool size": lambda c, x: c["layers"][1]["mixer"]["mask"].update(pool=5),
        "window": lambda c, x: c["layers"][1]["mixer"]["mask"].update(size=11),
        "large blocks": lambda c, x: c["layers"][2]["mixer"]["mask"].update(pool=8),
        "chunk": lambda c, x: c["layers"][0]["mixer"]["left"]["mask"].update(size=17),
        "cap": lambda c, x: c["layers"][1]["mixer"].pop("softcap"),
        "frequencies": lambda c, x: c["layers"][1]["mixer"]["rot"].pop("scaling"),
        "rotated part": lambda c, x: c["layers"][1]["mixer"]["rot"].update(dims=16),
        "decay": lambda c, x: c["layers"][0]["mixer"]["right"].update(decay=[0.9, 0.99, 0.99]),
        "retention's rotation": lambda c, x: c["layers"][0]["mixer"]["right"].pop("rot"),
        "left scale": lambda c, x: c["layers"][0]["mixer"].update(left_scale=1.0),
        "right scale": lambda c, x: c["layers"][0]["mixer"].update(right_scale=1.0),
        "groups": lambda c, x: c["layers"][0]["mlp"]["router"]["groups"].update(keep=3),
        "head norm": lambda c, x: x.update({"l1.mix.k.norm": x["l1.mix.k.norm"] * 0 + 1}),
        "embedding norm": lambda c, x: x.update({"embed.norm": x["embed.norm"] * 0 + 1}),
        "output norm": lambda c, x: x.update({"l3.norm2": x["l3.norm2"] * 0 + 1}),
    }
    for name, edit in edits.items():
        c2, w2 = copy.deepcopy(cfg), dict(w)
        edit(c2, w2)
        assert moved(c2, w2) > 1e-3, name
    # mechanisms that are functions of the oracle: the sink, the value norm, the layout of the rotation
    import unittest.mock as mock

    real = plain.window_pool_attention
    with mock.patch.object(plain, "window_pool_attention", lambda *a: real(*a[:-1], False)):
        assert moved(cfg, w) > 1e-3
    with mock.patch.object(plain, "value_norm", lambda x, eps: x):
        assert moved(cfg, w) > 1e-3
    real_rotate = plain.rotate
    with mock.patch.object(plain, "rotate", lambda x, p, f, d, layout: real_rotate(x, p, f, d, "half")):
        assert moved(cfg, w) > 1e-3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_model_whole_in_portions_decoded_and_batched(models, name, dtype):
    """The same requests whole, token by token (through the captured decode graphs), in portions down to two tokens
    and one, and in batches of unequal requests that start and end at different steps in a pool so small that pages
    and state slots are taken again."""
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine.model import Runner

    d, cfg, w = models[name if dtype == "float32" else name + "~"]
    vocab = cfg["vocab"]
    seqs = {"a": helpers.token_ids(vocab, 75, 1), "b": helpers.token_ids(vocab, 1, 2), "c": helpers.token_ids(vocab, 33, 3),
            "d": helpers.token_ids(vocab, 130, 4), "e": helpers.token_ids(vocab, 18, 5)}
    ref = {r: plain.forward(cfg, w, ids) for r, ids in seqs.items()}
    # bfloat16: a request is compared up to its first token whose choice of experts is a close call
    upto = {r: len(ids) if dtype == "float32" else clear_rows(cfg, w, ids) for r, ids in seqs.items()}
    assert dtype == "float32" or sum(upto.values()) >= sum(len(ids) for ids in seqs.values()) // 3
    model = load_model(d, dtype=dtype)
    runner = Runner(model, page_size=8, num_pages=40, max_requests=3)
    assert runner.graphs.enabled

    def check(got, r, what):
        if upto[r]:
            close_enough(got[r][:upto[r]], ref[r][:upto[r]], dtype, what)
    got = step_through(runner, [[(r, len(ids))] for r, ids in seqs.items()], seqs)
    for r in seqs:
        check(got, r, f"{name} whole {r}")
    for r, head in (("a", 10), ("c", 1)):
        got = step_through(runner, [[(r, head)]] + [[(r, 1)]] * (len(seqs[r]) - head), {r: seqs[r]})
        check(got, r, f"{name} decode {r}")
    assert runner.graphs.replays > 50
    sizes, plan, left = [2, 7, 1, 16, 3, 2, 33, 8, 64], [], len(seqs["d"])
    while left:
        n = min(sizes[len(plan) % len(sizes)], left)
        plan.append([("d", n)])
        left -= n
    check(step_through(runner, plan, {"d": seqs["d"]}), "d", f"{name} portions")
    plan = [[("a", 30), ("c", 2), ("b", 1)], [("a", 1), ("c", 20), ("e", 3)], [("c", 11), ("a", 44), ("e", 1)],
            [("e", 14), ("d", 9)], [("d", 120)], [("d", 1)]]
    got = step_through(runner, plan, seqs)
    for r in seqs:
        check(got, r, f"{name} batched {r}")
    assert all(a.pages_issued_again() for a in runner.manager.allocators)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_output_product_or_two_for_mixers_side_by_side(models, dtype):
    """The mixers of a side-by-side layer share one output product over their heads laid side by side, the scales on the
    activations; with ``joint_output`` off they keep their own products and a kernel adds the results.  Both are the
    plain model's logits."""
    from pathlib import Path

    from from_scratch_inference_engine_amd.config.base import read_config_json
    from from_scratch_inference_engine_amd.engine.model import Model, Runner
    from from_scratch_inference_engine_amd.models.registry import build_model_spec, parse_config
    from from_scratch_inference_engine_amd.parts import SideBySide
    from from_scratch_inference_engine_amd.weights.loader import load_weights

    d, cfg, w = models["C" if dtype == "float32" else "C~"]
    ids = helpers.token_ids(cfg["vocab"], 45, 9)
    ref = plain.forward(cfg, w, ids)
    for joint in (True, False):
        spec = build_model_spec(parse_config(read_config_json(d)))
        pairs = [b.mixer for b in spec.layers if isinstance(b.mixer, SideBySide)]
        assert pairs and all(m.joint for m in pairs)
        if not joint:
            for m in pairs:
                m.joint, m.o = False, None
        model = Model(spec, dtype, "cuda:0")
        load_weights(Path(d), spec.bindings, model.dtype, model.device, spec.ignore_unexpected)
        model._prepare(True)
        runner = Runner(model, page_size=8, num_pages=40, max_requests=2)
        got = step_through(runner, [[("a", 30)], [("a", 2)]] + [[("a", 1)]] * 13, {"a": ids})["a"]
        close_enough(got, ref, dtype, f"joint {joint}")


def test_long_decoding_with_a_far_first_token(models):
    """Five hundred decoded tokens in float32, page after page: every logit is the plain one, with a retention head
    that never forgets the request's first tokens, windows that hand their pages back and pooled blocks that stay."""
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine.model import Runner

    d, cfg, w = models["A"]
    ids = helpers.token_ids(cfg["vocab"], 500, 11)
    ref = plain.forward(cfg, w, ids)
    runner = Runner(load_model(d, dtype="float32"), page_size=8, num_pages=70, max_requests=1)
    got = step_through(runner, [[("a", 5)]] + [[("a", 1)]] * 495, {"a": ids})
    close_enough(got["a"], ref, "float32", "long decode")
    other = plain.forward(cfg, w, [(ids[0] + 1) % cfg["vocab"]] + ids[1:])
    assert np.abs(other[-1] - ref[-1]).max() > 1e-3 * np.abs(ref).max()  # the first token still matters at the end


@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_engine(models, name):
    """Prompts of unequal length generated together through the LLM entry point and its scheduler (three at a
    time, portions of at most 16 tokens), in float32: the tokens are the plain implementation's greedy ones."""
    from from_scratch_inference_engine_amd import GenerationConfig, LLM

    d, cfg, w = models[name]
    prompts = [helpers.token_ids(cfg["vocab"], n, 20 + n) for n in (1, 9, 40, 23)]
    n_new = 48
    llm = LLM(d, dtype="float32", block_size=8, num_blocks=64, max_batch=3, eos_id=-1, prefill_chunk=16)
    got = llm.generate_ids_batch(prompts, GenerationConfig(max_tokens=n_new))
    for prompt, mine in zip(prompts, got):
        assert len(mine) == n_new
        logits = plain.forward(cfg, w, prompt + mine)[len(prompt) - 1:-1]
        for i, tok in enumerate(mine):  # the plain choice, unless the two best are a rounding apart
            assert tok == int(logits[i].argmax()) or (logits[i].max() - logits[i, tok]) <= 1e-4 * np.abs(logits).max(), (len(prompt), i)
    assert llm.engine.runner.graphs.replays > 0


@pytest.mark.parametrize("name", ["A", "D"])
def test_replay_program_runs_the_model(models, tmp_path, name):
    """bin/trace_run on the architecture: a prompt in portions beside another request's single tokens, then a third
    request in the slot and pages that the second gave back."""
    d, cfg, w = models[name]
    a, b, c = (helpers.token_ids(cfg["vocab"], n, 7 + n) for n in (50, 20, 9))
    tb = helpers.TraceBuilder()
    tb.step([("a", a[:17], [16]), ("b", b[:1], [0])])
    for i in range(1, 20):
        lo, hi = 17 + (i - 1) * 2, min(50, 17 + i * 2)
        entries = [("b", b[i:i + 1], [0])] + ([("a", a[lo:hi], list(range(hi - lo)))] if lo < 50 else [])
        tb.step(entries, end=["b"] if i == 19 else [])
    tb.step([("c", c, list(range(9)))], end=["a", "c"])
    for dtype in ("float32", "bfloat16"):
        d, cfg, w = models[name if dtype == "float32" else name + "~"]
        per = helpers.collect(tb, helpers.run_trace(d, dtype, tb.steps, 128, tmp_path / dtype))
        for rid, ids in (("a", a), ("b", b), ("c", c)):
            ref = plain.forward(cfg, w, ids)
            upto = len(ids) if dtype == "float32" else clear_rows(cfg, w, ids)
            pos = [p for p in sorted(per[rid]) if p < upto]
            if pos:
                close_enough(np.stack([per[rid][p] for p in pos]), ref[pos], dtype, f"replay {rid}")


def test_command_line_writes_a_random_model_and_generates(tmp_path):
    """random-model from a config.json, then generate from that folder and, without a folder, from the configuration
    and the seed: the architecture is served by the same command line as the others."""
    (tmp_path / "cfg.json").write_text(json.dumps(CONFIG_A))
    env = dict(os.environ, PYTHONPATH=str(helpers.ROOT))
    base = [sys.executable, "-m", "from_scratch_inference_engine_amd"]
    made = subprocess.run(base + ["random-model", "--config", str(tmp_path / "cfg.json"), "--out", str(tmp_path / "m"), "--seed", "5"],
                          capture_output=True, text=True, env=env, timeout=300)
    assert made.returncode == 0, made.stderr[-2000:]
    common = ["--prompt-ids", "3 1 4 1 5 9 2 6", "--max-tokens", "12", "--num-blocks", "64", "--max-batch", "4", "--dtype", "float32"]
    a = subprocess.run(base + ["generate", "--model-dir", str(tmp_path / "m")] + common, capture_output=True, text=True, env=env, timeout=300)
    b = subprocess.run(base + ["generate", "--config", str(tmp_path / "cfg.json"), "--random-weights", "5"] + common,
                       capture_output=True, text=True, env=env, timeout=300)
    assert a.returncode == 0 and b.returncode == 0, a.stderr[-2000:] + b.stderr[-2000:]
    tokens = a.stdout.strip().splitlines()[-1].split()
    assert len(tokens) == 12 and all(0 <= int(t) < CONFIG_A["vocab"] for t in tokens)
    cfg, w = plain.read_config(tmp_path / "m"), plain.read_weights(tmp_path / "m")
    ids = [3, 1, 4, 1, 5, 9, 2, 6] + [int(t) for t in tokens]
    logits = plain.forward(cfg, w, ids)[7:-1]
    for i, t in enumerate(tokens):
        assert int(t) == int(logits[i].argmax()) or (logits[i].max() - logits[i, int(t)]) <= 1e-4 * np.abs(logits).max(), i
    assert len(b.stdout.strip().splitlines()[-1].split()) == 12
