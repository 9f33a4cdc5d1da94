"""Fiterax on the GPU against the plain implementation (plain_fiterax.py): every mechanism alone, then whole models
of small configurations through the step function, the scheduler and the replay program.

The weights are drawn here with a spread that keeps activations of order one (standard deviation fan_in^-1/2, wide
norm weights and biases), temperatures and scales that make softmax rows peaked and reach the scores' cap, gate
biases that let some heads of the matrix memory forget at once and others keep a loud first token to the end, and
router corrections that move the choice of experts: a key that is missed, a state that is lost, an input of the
convolution that is dropped at a portion's start then moves the logits far beyond rounding."""

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
import plain_fiterax as plain

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
@pytest.mark.parametrize("hidden, groups, kinds, scale", [(96, 2, (None, None), 1.0), (257, 1, ("same", "f32"), 0.35),
                                                          (4104, 8, ("f32", "same"), 2.25), (90, 3, ("same", None), 0.7),
                                                          (72, 72, (None, "f32"), 1.0), (15000, 2, ("same", "same"), 0.35)])
def test_group_rms_norm_adds_two_scaled_deltas_and_gives_two_outputs(ops, dtype, hidden, groups, kinds, scale):
    """residual + scale * (delta + delta2), each delta absent, in the output's type or float32; every group by its
    own root mean square; one pass for two weights; the sum written back; and chosen rows without writing back."""
    t, eps = 7, 1e-3
    res = rnd((t, hidden), 1, 3.0)
    res[:, :hidden // groups] *= 9.0  # a loud first group: a norm over the whole row would flatten the others

    def delta(kind, seed):
        return None if kind is None else rnd((t, hidden), seed).to(torch.float32 if kind == "f32" else dtype)
    d1, d2 = delta(kinds[0], 2), delta(kinds[1], 3)
    w1, w2 = rnd((hidden,), 4) + 1.0, rnd((hidden,), 6) + 1.0
    total = res.double()
    both = sum(d.double() for d in (d1, d2) if d is not None)
    if d1 is not None or d2 is not None:
        total = total + scale * both
    ref1 = plain.group_rms_norm(total.numpy(), w1.double().numpy(), eps, groups)
    ref2 = plain.group_rms_norm(total.numpy(), w2.double().numpy(), eps, groups)
    dev = lambda x: None if x is None else x.cuda()
    r = res.clone().cuda()
    o1, o2 = ops.group_rmsnorm(r, w1.cuda(), eps, groups, dtype, delta=dev(d1), delta2=dev(d2), delta_scale=scale,
                               weight2=w2.cuda(), write_back=True)
    assert rel(o1.float().cpu(), ref1) <= tol(dtype) and rel(o2.float().cpu(), ref2) <= tol(dtype)
    assert rel(r.cpu(), total) <= 1e-6
    rows = torch.tensor([5, 0, 5, 2], dtype=torch.int32)
    r = res.clone().cuda()
    o = ops.group_rmsnorm(r, w1.cuda(), eps, groups, dtype, delta=dev(d1), delta2=dev(d2), delta_scale=scale, rows=rows.cuda())
    assert rel(o.float().cpu(), ref1[rows.long().numpy()]) <= tol(dtype)
    assert torch.equal(r.cpu(), res)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("pair", [False, True])
@pytest.mark.parametrize("taps, hidden", [(4, 40), (2, 7), (7, 300), (1, 12), (3, 520)])
def test_convolution_over_portions_steps_and_slots(ops, dtype, taps, hidden, pair):
    """Three requests fed in unequal portions (single tokens, portions shorter than the convolution is long) over
    several steps, one of them in a slot that another has used, two convolutions sharing the slots: every output is
    the input plus the convolution over the request's own earlier inputs, zeros before its start.  ``pair``: both
    convolutions in the same launches, each with its own inputs, weights and state."""
    seqs = {"a": rnd((19, hidden), 1), "b": rnd((5, hidden), 2), "c": rnd((8, hidden), 3)}
    w = rnd((hidden, taps), 4)
    seqs0, w0 = {r: rnd(tuple(x.shape), 10 + i) for i, (r, x) in enumerate(seqs.items())}, rnd((hidden, taps), 14)
    got0 = {r: [] for r in seqs}
    state = torch.full((4, 2, max(taps - 1, 0), hidden), 77.0).cuda() if taps > 1 else None
    slot = {"a": 0, "b": 2, "c": 1}
    plan = [[("a", 1), ("b", 1)], [("b", 2), ("a", 2)], [("a", 1), ("b", 1)], [("a", 9), ("b", 1)], [("c", 3), ("a", 1)],
            [("c", 1), ("a", 5)], [("c", 4)]]
    fed, got = {r: 0 for r in seqs}, {r: [] for r in seqs}
    for step in plan:
        rows, starts, slots = [], [0], []
        for r, n in step:
            if r == "c":
                slot["c"] = slot["b"]  # b has ended: c takes its slot
            if fed[r] == 0 and state is not None:
                state[slot[r], 1] = 0.0  # (the engine zeroes the slots of the requests that start)
                if pair:
                    state[slot[r], 0] = 0.0
            rows.append(seqs[r][fed[r]:fed[r] + n])
            starts.append(starts[-1] + n)
            slots.append(slot[r])
        view = None if state is None else state[:, 1]
        if pair:
            rows0 = torch.cat([seqs0[r][fed[r]:fed[r] + n] for r, n in step]).cuda()
            out0, out = ops.causal_conv(rows0, w0.cuda(), None if state is None else state[:, 0], i32(starts), i32(slots), dtype,
                                        torch.cat(rows).cuda(), w.cuda(), view)
            out0, out = out0.float().cpu(), out.float().cpu()
        else:
            out = ops.causal_conv(torch.cat(rows).cuda(), w.cuda(), view, i32(starts), i32(slots), dtype).float().cpu()
        at = 0
        for r, n in step:
            got[r].append(out[at:at + n])
            if pair:
                got0[r].append(out0[at:at + n])
            at += n
            fed[r] += n
    for r, x in seqs.items():
        ref = plain.input_convolution(x.double().numpy(), w.double().numpy())
        assert rel(torch.cat(got[r]), ref) <= tol(dtype, 1e-6), r
        if pair:
            ref0 = plain.input_convolution(seqs0[r].double().numpy(), w0.double().numpy())
            assert rel(torch.cat(got0[r]), ref0) <= tol(dtype, 1e-6), r
    if state is not None and not pair:
        assert bool((state[:, 0] == 77.0).all())  # the other convolution's inputs were left alone


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m, n, k", [(1, 2, 8), (70, 16, 256), (5, 9, 37), (300, 3, 1030)])
def test_a_few_float32_outputs_a_row(ops, dtype, m, n, k):
    """The gates' projection: float32 results of a handful of outputs a row, with a bias, at sizes that are multiples
    of nothing; a row's numbers do not depend on the other rows."""
    x, w, b = rnd((m, k), 1).to(dtype), rnd((n, k), 2, k ** -0.5).to(dtype), rnd((n,), 3)
    y = ops.gemm(x.cuda(), w.cuda(), b.cuda(), out_dtype=torch.float32, kind=ops.GEMM_NARROW)
    assert y.dtype == torch.float32
    ref = x.double().numpy() @ w.double().numpy().T + b.double().numpy()
    assert rel(y.cpu(), ref) <= 2e-6
    alone = ops.gemm(x[m // 2:m // 2 + 1].cuda(), w.cuda(), b.cuda(), out_dtype=torch.float32, kind=ops.GEMM_NARROW)
    assert torch.equal(alone[0], y[m // 2])


@pytest.mark.parametrize("planes, m, n, with_bias", [(1, 3, 8, False), (4, 37, 100, True), (9, 64, 6144, True)])
def test_partial_sums_added_in_order_and_rounded_once(ops, planes, m, n, with_bias):
    parts, bias = rnd((planes, m, n), 1, 3.0), rnd((n,), 2)
    y = ops.sum_round(parts.cuda(), bias.cuda() if with_bias else None)
    ref = parts[0].clone()
    for p in range(1, planes):
        ref += parts[p]
    if with_bias:
        ref += bias
    assert y.dtype == torch.bfloat16 and torch.equal(y.cpu(), ref.to(torch.bfloat16))


@pytest.mark.parametrize("m", [17, 40, 64])
def test_products_of_a_few_dozen_rows_from_the_engine(ops, m):
    """17 to 64 rows with a bfloat16 result: partial sums of the engine's product, added and rounded once, against
    float64; a row's numbers do not depend on the other rows."""
    from from_scratch_inference_engine_amd.parts.linear import Linear

    lin = Linear(512, 1544, bias=True)
    lin.weight, lin.bias = rnd((1544, 512), 1, 512 ** -0.5).to(torch.bfloat16).cuda(), rnd((1544,), 2).cuda()
    lin.prepare(True)
    x = rnd((m, 512), 3).to(torch.bfloat16)
    y = lin(x.cuda())
    ref = x.double().numpy() @ lin.weight.cpu().double().numpy().T + lin.bias.cpu().double().numpy()
    assert y.dtype == torch.bfloat16 and rel(y.float().cpu(), ref) <= 2.0 ** -7
    fewer = lin(x[:m - 7].cuda())
    assert rel(fewer.float().cpu(), y[:m - 7].float().cpu()) <= 2.0 ** -7


def attention_case(seqs, heads, kv, hd, page, dtype, seed, scalar, edit=None):
    """Pools, tables and the planner's items for requests (past, new) of a causal attention without a window."""
    from from_scratch_inference_engine_amd.parts.attention import AttentionPlanner

    g = torch.Generator().manual_seed(seed)
    n_pages = sum(-(-(p + n) // page) for p, n in seqs) + 2
    order = torch.randperm(n_pages, generator=g).tolist()
    k_pool, v_pool = torch.full((n_pages, kv, page, hd), 7.0), torch.full((n_pages, kv, hd, page), -9.0)
    tables = torch.full((len(seqs), max(-(-(p + n) // page) for p, n in seqs)), -1, dtype=torch.int32)
    qs, ks, vs = [], [], []
    for p, n in seqs:
        qs.append(torch.randn(n, heads * hd, generator=g).to(dtype).float())
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
                           page_size=page, compute_dtype=torch.float32 if scalar else dtype, pad=None)
    for _, n in seqs:
        host.q_starts.append(host.q_starts[-1] + n)
    host.n_tokens = host.q_starts[-1]
    plan = AttentionPlanner(heads, kv, hd, None).plan(host)
    return dict(q=torch.cat(qs).to(dtype), k_pool=k_pool.to(dtype), v_pool=v_pool.to(dtype), tables=tables, plan=plan,
                qs=qs, ks=ks, vs=vs)


def run_attention(case, heads, kv, hd, scale, cap, share_keys=True):
    from from_scratch_inference_engine_amd.parts.attention import paged_attention

    plan = {k: (torch.from_numpy(v).cuda() if isinstance(v, np.ndarray) else v) for k, v in case["plan"].items()}
    cache = SimpleNamespace(k_pool=case["k_pool"].cuda(), v_pool=case["v_pool"].cuda(), block_tables=case["tables"].cuda(),
                            page_size=case["k_pool"].shape[2])
    q = case["q"].cuda()
    return paged_attention(q, heads * hd, cache, SimpleNamespace(**plan), heads, kv, hd, None, scale, q.shape[0],
                           share_keys=share_keys, softcap=cap).float().cpu().numpy()


def oracle_attention(q, k, v, heads, kv, hd, past, scale, cap):
    n, total = q.shape[0], k.shape[0]
    out = plain.capped_attention(q.double().numpy().reshape(n, heads, hd), k.double().numpy().reshape(total, kv, hd),
                                 v.double().numpy().reshape(total, kv, hd), scale, None, cap, past)
    return out.reshape(n, heads * hd)


FAMILIES = [(torch.float32, True), (torch.bfloat16, True), (torch.bfloat16, False)]  # (type, float32-arithmetic kernel)


@pytest.mark.parametrize("family", range(3))
@pytest.mark.parametrize("heads, kv, hd, page, cap", [(4, 2, 64, 16, 5.0), (6, 1, 32, 8, 2.0), (2, 2, 48, 16, 30.0),
                                                      (8, 2, 128, 16, 3.0), (4, 4, 64, 16, None)])
def test_capped_scores_on_every_attention_kernel(ops, family, heads, kv, hd, page, cap):
    """Random queries and keys whose scores reach well beyond the cap: decoded tokens against long contexts (cut into
    items and merged, on an idle and on a full device), short and long portions, first tokens."""
    from from_scratch_inference_engine_amd.parts.attention import AttentionPlanner

    dtype, scalar = FAMILIES[family]
    scale = 0.9  # (scores of standard deviation 0.9 sqrt(hd): most of them beyond a cap of 5)
    seqs = [(0, 1), (0, 2), (700, 1), (0, 150), (300, 2), (123, 70), (2100, 1), (500, 200)]
    outs = []
    for units in (4096, 1):
        AttentionPlanner.compute_units = units
        try:
            case = attention_case(seqs, heads, kv, hd, page, dtype, seed=hd + heads, scalar=scalar)
        finally:
            AttentionPlanner.compute_units = None
        assert case["plan"]["mfma"] == (not scalar)
        outs.append(run_attention(case, heads, kv, hd, scale, cap))
        if not scalar and ops.attention_mfma_lds_ok(hd, page):
            outs.append(run_attention(case, heads, kv, hd, scale, cap, share_keys=False))
    uncapped = run_attention(case, heads, kv, hd, scale, None)
    row = 0
    for (p, n), q, k, v in zip(seqs, case["qs"], case["ks"], case["vs"]):
        ref = oracle_attention(q, k, v, heads, kv, hd, p, scale, cap)
        for out in outs:
            err = np.abs(out[row:row + n] - ref).max()
            assert err <= (3e-6 if dtype == torch.float32 else 2.0 ** -7) * v.abs().max().item(), f"past {p} new {n}: {err}"
        if cap is not None and p + n > 100:  # the cap is felt: without it the rows are far away
            assert np.abs(uncapped[row:row + n] - ref).max() > 0.05
        row += n


@pytest.mark.parametrize("family", range(3))
def test_attention_finds_far_keys_page_borders_and_itself(ops, family):
    """For every query one key carries the softmax although the cap flattens everything beyond it: the very first key
    of a long context, a key on either side of a page's border, the query's own position; a louder key just after the
    query must stay unseen."""
    dtype, scalar = FAMILIES[family]
    heads, kv, hd, page, scale, cap = 4, 2, 64, 16, 1.0, 12.0
    seqs = [(1500, 1), (640, 4), (0, 40), (63, 3)]
    targets = {0: [0], 1: [15, 16, 642, 0], 2: [min(i, 3) if i < 20 else (i if i % 2 else 15) for i in range(40)], 3: [63, 31, 32]}

    def edit(qs, ks, vs):
        for s, (p, n) in enumerate(seqs):
            ks[s].mul_(0.05)
            for i in range(n):
                pos, key = p + i, targets[s][i]
                assert key <= pos
                direction = torch.zeros(hd)
                direction[(7 * s + 3 * i) % hd] = 1.0
                ks[s][key] += (5.0 * direction).repeat(kv)
                qs[s][i] = (2.0 * direction).repeat(heads) + 0.05 * qs[s][i]
                if pos + 1 < p + n:
                    ks[s][pos + 1] += (9.0 * direction).repeat(kv)  # louder, and not to be seen
            for t in (qs[s], ks[s]):
                t.copy_(t.to(dtype).float())
    case = attention_case(seqs, heads, kv, hd, page, dtype, seed=5, scalar=scalar, edit=edit)
    out = run_attention(case, heads, kv, hd, scale, cap)
    row = 0
    for s, ((p, n), q, k, v) in enumerate(zip(seqs, case["qs"], case["ks"], case["vs"])):
        ref = oracle_attention(q, k, v, heads, kv, hd, p, scale, cap)
        got = out[row:row + n]
        assert np.abs(got - ref).max() <= (1e-5 if dtype == torch.float32 else 2.0 ** -6) * v.abs().max().item(), s
        if p + n < 200:  # (among a thousand flattened keys the one key holds part of the weight only: the oracle decides there)
            for i in range(n):
                chosen = v[targets[s][i]].double().numpy().reshape(kv, hd)
                for h in range(heads):
                    mine = got[i, h * hd:(h + 1) * hd]
                    assert np.abs(mine - chosen[h // (heads // kv)]).max() <= 0.1 * np.abs(chosen).max() + 0.05, (s, i, h)
        row += n


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv, dim, vdim, rot", [(6, 3, 24, 40, 16), (4, 4, 64, 64, 64), (2, 1, 32, 16, 0), (3, 1, 20, 7, 10)])
def test_attention_prep_unit_norm_with_a_temperature_a_head(ops, dtype, heads, kv, dim, vdim, rot):
    """Queries: rotated, divided by their root mean square, times their head's temperature; keys likewise without a
    temperature, in the pool beside the values; the gates' sigmoid."""
    t, page, eps, base = 37, 8, 1e-4, 300.0
    padded = dim if dim == vdim else -(-max(dim, vdim) // 16) * 16
    width = heads * dim + kv * dim + kv * vdim + heads
    proj = rnd((t, width), 1, 2.0).to(dtype)
    temps = rnd((heads,), 2).abs() + 0.5
    pos = torch.arange(5, 5 + t)
    pairs = rot // 2
    table = None
    if pairs:
        f = torch.tensor([base ** (-2.0 * i / rot) for i in range(pairs)], dtype=torch.float64)
        a = pos.double()[:, None] * f[None, :]
        table = torch.stack([a.cos(), a.sin()], dim=-1).float().cuda()
    units = -(-t // page) + 2
    k_pool, v_pool = torch.zeros((units, kv, page, padded), dtype=dtype).cuda(), torch.zeros((units, kv, padded, page), dtype=dtype).cuda()
    slots = torch.randperm((units - 1) * page, generator=torch.Generator().manual_seed(3))[:t].to(torch.int32) + page
    q_w = (torch.ones((heads, dim)) * temps[:, None]).contiguous().cuda()
    q, gate = ops.attention_prep(proj.cuda(), 0, heads * dim, heads * dim + kv * dim, width - heads, heads, kv, dim, vdim, padded,
                                 q_w, torch.ones(dim).cuda(), eps, pairs, table, True, slots=slots.cuda(), k_pool=k_pool, v_pool=v_pool)
    x = proj.double().numpy()
    qr = plain.unit_rms(plain.rotate_half(x[:, :heads * dim].reshape(t, heads, dim), pos.numpy(), base, rot), eps) * temps.double().numpy()[None, :, None]
    kr = plain.unit_rms(plain.rotate_half(x[:, heads * dim:heads * dim + kv * dim].reshape(t, kv, dim), pos.numpy(), base, rot), eps)
    got_q = q.float().cpu().numpy().reshape(t, heads, padded)
    assert rel(got_q[..., :dim], qr) <= tol(dtype) and not got_q[..., dim:].any()
    assert rel(gate.cpu(), plain.sigmoid(x[:, width - heads:])) <= 1e-5
    kp, vp = k_pool.float().cpu().numpy(), v_pool.float().cpu().numpy()
    for i in range(t):
        unit, off = divmod(int(slots[i]), page)
        assert rel(kp[unit, :, off, :dim], kr[i]) <= tol(dtype)
        vv = x[i, heads * dim + kv * dim:width - heads].reshape(kv, vdim)
        assert rel(vp[unit, :, :vdim, off], vv) <= tol(dtype, 1e-6, 1e-6)


def memory_inputs(t, heads, dim, vdim, seed, dtype):
    """A fused projection (q, k, v side by side) and gate logits; head 0 forgets nearly everything at every token,
    head 1 nearly nothing and takes its first token loudly, the others are in between."""
    proj = rnd((t, heads * (2 * dim + vdim)), seed).to(dtype)
    gates = rnd((t, 2 * heads), seed + 1, 2.0)
    gates[:, heads] -= 9.0          # head 0's forget gate: closed
    if heads > 1:
        gates[:, heads + 1] += 9.0  # head 1's: open
        gates[0, 1] += 14.0         # and a loud first token
        gates[1:, 1] -= 3.0
    return proj, gates


def oracle_memory(proj, gates, heads, dim, vdim, cap, pieces=False):
    t = proj.shape[0]
    x = proj.double().numpy()
    q = x[:, :heads * dim].reshape(t, heads, dim) * dim ** -0.5
    k = x[:, heads * dim:2 * heads * dim].reshape(t, heads, dim)
    v = x[:, 2 * heads * dim:].reshape(t, heads, vdim)
    gi, gf = plain.capped_gates(gates.double().numpy()[:, :heads], gates.double().numpy()[:, heads:], cap)
    return plain.matrix_memory(q, k, v, gi, gf, pieces)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, dim, vdim, cap", [(4, 40, 56, 11.0), (1, 20, 7, 3.0), (3, 130, 33, 15.0), (2, 256, 64, 8.0),
                                                   (1, 300, 70, 5.0)])
def test_matrix_memory_over_portions_steps_and_slots(ops, dtype, heads, dim, vdim, cap):
    """Requests fed whole, token by token and in unequal portions, in slots that are used again: numerator, the
    normaliser's product and the running maximum of every token are those of the walk over the whole request, with
    heads that forget at once beside heads that keep a loud first token.  (The three are compared one by one: their
    quotient is as ill-conditioned as n . q is close to zero, which is nobody's fault.)"""
    lens = {"a": 70, "b": 9, "c": 31, "d": 333}
    data = {r: memory_inputs(n, heads, dim, vdim, 10 * i, dtype) for i, (r, n) in enumerate(lens.items())}
    ref = {r: oracle_memory(p, g, heads, dim, vdim, cap, pieces=True) for r, (p, g) in data.items()}
    record = ops.mlstm_state_floats(dim, vdim)
    state = torch.full((4, heads, record), 5.0).cuda()
    slot = {"a": 0, "b": 1, "c": 1, "d": 3}
    # portions of sixteen tokens and more go chunk by chunk on the matrix cores, the others token by token
    plan = [[("a", 1), ("b", 2)], [("b", 7), ("a", 17), ("d", 16)], [("a", 1)], [("a", 2), ("c", 30), ("d", 15)],
            [("d", 290), ("c", 1), ("a", 49)], [("d", 12)]]
    fed, got = {r: 0 for r in lens}, {r: [] for r in lens}
    for step in plan:
        rows, gts, starts, slots = [], [], [0], []
        for r, n in step:
            if fed[r] == 0:
                state[slot[r]] = 0.0
            rows.append(data[r][0][fed[r]:fed[r] + n])
            gts.append(data[r][1][fed[r]:fed[r] + n])
            starts.append(starts[-1] + n)
            slots.append(slot[r])
        proj = torch.cat(rows).cuda()
        num, den, coef = ops.mlstm_scan(proj, 0, heads * dim, 2 * heads * dim, torch.cat(gts).cuda(), cap, dim ** -0.5, state,
                                        i32(starts), i32(slots), heads, dim, vdim)
        num, den, coef = num.cpu(), den.cpu(), coef.cpu()
        at = 0
        for r, n in step:
            got[r].append((num[at:at + n], den[at:at + n], coef[at:at + n]))
            at += n
            fed[r] += n
    for r in lens:
        num, den, coef = (torch.cat([g[i] for g in got[r]]).numpy() for i in range(3))
        _, ref_num, ref_den, ref_m = ref[r]
        for h in range(heads):  # head by head: their sizes differ by orders of magnitude
            assert rel(num[:, h], ref_num[:, h]) <= 2e-5 and rel(den[:, h], ref_den[:, h]) <= 2e-5, (r, h)
            assert np.abs(coef[:, h, 3] - ref_m[:, h]).max() <= 1e-5, (r, h)
            assert np.abs(coef[1:, h, 2] - ref_m[:-1, h]).max() <= 1e-5 and coef[0, h, 2] == 0.0, (r, h)  # m before the token
    assert bool((state[2] == 5.0).all())  # a slot of no request was not touched
    # the first token is still felt by head 1 at the request's end, and not at all by head 0
    if heads > 1:
        p, g = data["a"]
        p2 = p.clone()
        p2[0, 2 * heads * dim:] *= -1.0  # the first token's values
        other = oracle_memory(p2, g, heads, dim, vdim, cap)
        mine = ref["a"][0]
        assert np.abs(other[-1, 1] - mine[-1, 1]).max() > 0.05 * np.abs(mine[-1, 1]).max()
        assert np.abs(other[-1, 0] - mine[-1, 0]).max() < 1e-6 * np.abs(mine[-1, 0]).max()


@pytest.mark.parametrize("dim, vdim", [(24, 40), (140, 20), (64, 100)])
def test_matrix_memory_of_many_requests_a_step(ops, dim, vdim):
    """Steps of 128 requests (two tokens each, then single tokens): with that many the walk holds whole rows of the
    memory a wave; the same numbers as with a few requests, against the plain walk."""
    n, heads, cap, dtype = 128, 8, 9.0, torch.float32
    data = [memory_inputs(5, heads, dim, vdim, 7 * r, dtype) for r in range(n)]
    state = torch.zeros((n, heads, ops.mlstm_state_floats(dim, vdim))).cuda()
    got = [[] for _ in range(n)]
    fed = 0
    for size in (2, 1, 1, 1):
        proj = torch.cat([p[fed:fed + size] for p, _ in data]).cuda()
        gates = torch.cat([g[fed:fed + size] for _, g in data]).cuda()
        num, den, coef = ops.mlstm_scan(proj, 0, heads * dim, 2 * heads * dim, gates, cap, dim ** -0.5, state,
                                        i32(list(range(0, n * size + 1, size))), i32(list(range(n))), heads, dim, vdim)
        num, den = num.cpu(), den.cpu()
        for r in range(n):
            got[r].append((num[r * size:(r + 1) * size], den[r * size:(r + 1) * size]))
        fed += size
    for r in range(0, n, 9):
        _, ref_num, ref_den, _ = oracle_memory(*data[r], heads, dim, vdim, cap, pieces=True)
        num, den = (torch.cat([g[i] for g in got[r]]).numpy() for i in range(2))
        for h in range(heads):
            assert rel(num[:, h], ref_num[:, h]) <= 2e-5 and rel(den[:, h], ref_den[:, h]) <= 2e-5, (r, h)


@pytest.mark.parametrize("dtype", DTYPES)
def test_matrix_memory_output_norm_and_gate(ops, dtype):
    t, heads, vdim, eps = 11, 3, 20, 1e-3
    num, den = rnd((t, heads, vdim), 1, 4.0), rnd((t, heads), 2)
    coef = rnd((t, heads, 4), 3)  # (f, i, m before, m): the last one alone is read
    den[0] = 1e-4  # the floor exp(-m) takes over
    gate, w = rnd((t, 2 * heads * vdim), 4).to(dtype), rnd((heads * vdim,), 5) + 1.0
    y = ops.mlstm_out(num.cuda(), den.cuda(), coef.cuda(), gate.cuda()[:, heads * vdim:], w.cuda(), eps, dtype).float().cpu()
    o = num.double().numpy() / (np.maximum(np.abs(den.double().numpy()), np.exp(-coef[..., 3].double().numpy())) + 1e-6)[..., None]
    ref = plain.unit_rms(o, eps).reshape(t, -1) * w.double().numpy() * plain.sigmoid(gate.double().numpy()[:, heads * vdim:])
    assert rel(y, ref) <= tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("t, hidden, ff, experts, top", [(50, 64, 96, 8, 3), (7, 90, 34, 5, 5), (300, 40, 17, 3, 1), (1, 32, 32, 1, 1),
                                                         (130, 128, 272, 16, 2), (600, 48, 40, 2, 1)])
def test_routed_experts_against_the_plain_ones(ops, dtype, t, hidden, ff, experts, top):
    """Router (corrections that move the choice and leave the weights alone), grouping, both products and the sum,
    as the part does them, at sizes that are multiples of nothing."""
    from from_scratch_inference_engine_amd.parts.moe import RoutedExperts

    x = rnd((t, hidden), 1).to(dtype)
    router, corr = rnd((experts, hidden), 2, 0.5).to(dtype), rnd((experts,), 3, 0.6)
    up, down = rnd((experts, ff, hidden), 4, hidden ** -0.5).to(dtype), rnd((experts, hidden, ff), 5, ff ** -0.5).to(dtype)
    part = RoutedExperts(hidden, ff, experts, top, route_scale=1.75)
    part.router_weight, part.correction = router.cuda(), corr.cuda()
    part.up_weight, part.down_weight = up.reshape(-1, hidden).cuda(), down.reshape(-1, ff).cuda()
    got = part.forward(x.cuda(), None).cpu()
    w = {"m.router": router.double().numpy(), "m.correction": corr.double().numpy()}
    for e in range(experts):
        w[f"m.e{e}.up"], w[f"m.e{e}.down"] = up[e].double().numpy(), down[e].double().numpy()
    mlp = {"router": {"experts": experts, "top": top, "scale": 1.75}}
    ref = plain.moe_feed_forward(x.double().numpy(), w, "m.", mlp)
    ids, weights = ops.moe_route(x.cuda(), router.cuda(), corr.cuda(), top, 1.75)
    ref_ids, ref_w = plain.route(x.double().numpy(), w["m.router"], w["m.correction"], top, 1.75)
    same = (ids.cpu().numpy() == ref_ids).all(-1)
    assert same.mean() > 0.97  # (a choice may differ where two scores are a rounding apart)
    assert rel(weights.cpu().numpy()[same], ref_w[same]) <= 1e-5
    no_corr = plain.route(x.double().numpy(), w["m.router"], 0 * w["m.correction"], top, 1.75)[0]
    assert experts == top or t < 8 or (no_corr != ref_ids).any()
    rows = np.nonzero(same)[0]
    assert rel(got.numpy()[rows], ref[rows]) <= tol(dtype, 2e-5, 2.0 ** -5)
    order, slot_of, tiles = ops.moe_group(ids, experts)
    order, slot_of, tiles = order.cpu().numpy(), slot_of.cpu().numpy(), tiles.cpu().numpy()
    flat = ids.cpu().numpy().reshape(-1)
    assert sorted(order.tolist()) == list(range(t * top)) and (order[slot_of] == np.arange(t * top)).all()
    assert (np.diff(flat[order]) >= 0).all()  # slots of an expert are consecutive
    covered = np.zeros(t * top, dtype=int)
    for e, first, n in tiles:
        assert 0 <= n <= ops.moe_tile_rows(t * top, experts) and (n == 0 or (flat[order[first:first + n]] == e).all())
        covered[first:first + n] += 1
    assert (covered == 1).all()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden, ff", [(72, 50), (64, 192), (128, 64)])
def test_experts_products_do_not_depend_on_the_tiles(ops, dtype, hidden, ff):
    """Tiles of 16, 32, 64 and 128 rows (a few rows an expert, many, very many) over the same pairs: the same products
    up to the order of their sums, whichever expert is crowded or empty, at sizes that are multiples of nothing and
    at sizes that the vector loads take."""
    t, top, n_experts = 333, 2, 5
    assert [ops.moe_tile_rows(n, 8) for n in (16, 8 * 8, 8 * 9, 8 * 47, 8 * 48, 8 * 255, 8 * 256)] == [16, 16, 32, 32, 64, 64, 128]
    x = rnd((t, hidden), 1).to(dtype).cuda()
    up = rnd((n_experts, ff, hidden), 2, hidden ** -0.5).to(dtype).cuda()
    down = rnd((n_experts, hidden, ff), 3, ff ** -0.5).to(dtype).cuda()
    ids = torch.randint(0, n_experts - 1, (t, top), generator=torch.Generator().manual_seed(4), dtype=torch.int32)  # the last: empty
    ids[:200, 0] = 1  # a crowded one
    weights = rnd((t * top,), 5).abs().cuda()
    got = {}
    for rows in (16, 32, 64, 128):
        order, slot_of, tiles = ops.moe_group(ids.cuda(), n_experts, tile_rows=rows)
        act = ops.moe_gemm(x, up, tiles, order, gather_div=top, tile_rows=rows)
        out = ops.moe_gemm(act, down, tiles, order, pair_weight=weights, tile_rows=rows)
        got[rows] = ops.moe_combine(out, slot_of, t, top).cpu().double().numpy()
    xs, e = x.cpu().double().numpy(), ids.numpy()
    ref = np.zeros((t, hidden))
    for i in range(t):
        for c in range(top):
            hid = plain.gelu_erf(up[e[i, c]].cpu().double().numpy() @ xs[i])
            if dtype == torch.bfloat16:
                hid = torch.tensor(hid).to(dtype).double().numpy()
            ref[i] += float(weights[i * top + c]) * (down[e[i, c]].cpu().double().numpy() @ hid)
    for rows in (16, 32, 64, 128):
        assert rel(got[rows], ref) <= tol(dtype, 2e-5, 2.0 ** -6), rows
        assert rel(got[rows], got[16]) <= tol(dtype, 2e-6, 2.0 ** -7), rows


# ------------------------------------------------------------------------------------------------
# whole models
# ------------------------------------------------------------------------------------------------
def attention(heads, kv, dim, vdim, scale, cap, rot_dims, base=10000.0):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "rot": {"base": base, "dims": rot_dims}}
    if cap is not None:
        m["softcap"] = cap
    return m


def memory(heads, dim, vdim, cap):
    return {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}


def experts(ff, n, top, scale):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": n, "top": top, "scale": scale}}


def layer(kind, mixer, mlp):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


# A: both mixers, values wider and narrower than keys, partly rotated heads, caps that are reached, three groups
CONFIG_A = {"architecture": "Fiterax", "width": 72, "vocab": 150, "norm": {"eps": 1e-6, "groups": 3}, "embedding": {"scale": 3.5},
            "residual_mult": 0.5, "canon": {"taps": 3}, "layers": [
    layer("attention", attention(6, 3, 24, 40, 0.4, 6.0, 16, 500.0), experts(40, 5, 2, 1.7)),
    layer("mlstm", memory(3, 24, 16, 6.0), experts(56, 4, 4, 1.0)),
    layer("attention", attention(2, 1, 32, 32, 0.3, 20.0, 32), None),
    layer("mlstm", memory(2, 40, 36, 15.0), experts(24, 6, 1, 3.0)),
]}
# B: matrix memories only (no pages at all), one group, no convolution, no factor, one expert
CONFIG_B = {"architecture": "Fiterax", "width": 64, "vocab": 97, "norm": {"eps": 1e-5, "groups": 1}, "embedding": {"scale": 1.0},
            "residual_mult": 1.0, "canon": {"taps": 1}, "layers": [
    layer("mlstm", memory(1, 64, 64, 10.0), experts(64, 1, 1, 1.0)),
    layer("mlstm", memory(4, 16, 8, 4.0), None),
]}
# C: attention only, heads of 128 that the matrix-core kernels take unpadded, no cap in one layer, no rotation in
#    another, one kv head a query head, a long convolution
CONFIG_C = {"architecture": "Fiterax", "width": 128, "vocab": 300, "norm": {"eps": 1e-5, "groups": 8}, "embedding": {"scale": 8.0},
            "residual_mult": 0.25, "canon": {"taps": 6}, "layers": [
    layer("attention", attention(4, 2, 128, 128, 0.12, None, 64), experts(80, 8, 3, 2.25)),
    layer("attention", attention(4, 4, 64, 16, 0.2, 4.0, 0), experts(32, 3, 2, 0.5)),
]}
# D: sizes that are multiples of nothing
CONFIG_D = {"architecture": "Fiterax", "width": 90, "vocab": 101, "norm": {"eps": 1e-4, "groups": 5}, "embedding": {"scale": 0.5},
            "residual_mult": 1.5, "canon": {"taps": 2}, "layers": [
    layer("mlstm", memory(5, 10, 14, 2.0), experts(34, 3, 2, 1.0)),
    layer("attention", attention(6, 2, 20, 12, 0.5, 9.0, 10, 77.0), experts(50, 7, 3, 2.0)),
]}


def fiterax_tensors(cfg, seed):
    g = torch.Generator().manual_seed(seed)
    w = cfg["width"]

    def mat(rows, cols, gain=1.0):
        return torch.randn((rows, cols), generator=g) * (gain / math.sqrt(cols))

    def vec(n, centre, spread):
        return centre + torch.randn((n,), generator=g) * spread
    taps = cfg["canon"]["taps"]
    out = {"embed": torch.randn((cfg["vocab"], w), generator=g) / cfg["embedding"]["scale"], "final.norm": vec(w, 1.0, 0.2),
           "head": mat(cfg["vocab"], w, 2.0)}
    for i, lay in enumerate(cfg["layers"]):
        m, p = lay["mixer"], f"l{i}.mix."
        out[f"l{i}.norm1"] = vec(w, 1.0, 0.2)
        out[f"l{i}.canon1"] = torch.randn((w, taps), generator=g) * 0.4
        h, d, e = m["heads"], m["dim"], m["vdim"]
        if lay["type"] == "attention":
            kv = m["kv_heads"]
            out.update({p + "q": mat(h * d, w), p + "k": mat(kv * d, w), p + "v": mat(kv * e, w), p + "g": mat(h, w, 2.0),
                        p + "q.b": vec(h * d, 0.0, 0.3), p + "k.b": vec(kv * d, 0.0, 0.3), p + "v.b": vec(kv * e, 0.0, 0.3),
                        p + "temp": vec(h, 6.0, 1.5), p + "o": mat(w, h * e), p + "o.b": vec(w, 0.0, 0.2)})
        else:
            out.update({p + "q": mat(h * d, w, 2.0), p + "k": mat(h * d, w, 2.0), p + "v": mat(h * e, w), p + "g": mat(h * e, w, 2.0),
                        p + "i": mat(h, w, 3.0), p + "f": mat(h, w, 3.0), p + "norm": vec(h * e, 1.0, 0.2), p + "o": mat(w, h * e)})
            # forget gates from nearly closed (the first head) to nearly open (the last), input gates spread out
            out[p + "i.b"] = vec(h, 0.0, 2.0)
            out[p + "f.b"] = torch.linspace(-3.0, 5.0, h) if h > 1 else torch.tensor([2.0])
        if lay["mlp"] is not None:
            r, ff = lay["mlp"]["router"], lay["mlp"]["expert"]["ff"]
            q = f"l{i}.mlp."
            out[f"l{i}.norm2"] = vec(w, 1.0, 0.2)
            out[f"l{i}.canon2"] = torch.randn((w, taps), generator=g) * 0.4
            out[q + "router"], out[q + "correction"] = mat(r["experts"], w, 1.5), vec(r["experts"], 0.0, 0.5)
            for j in range(r["experts"]):
                out[f"{q}e{j}.up"], out[f"{q}e{j}.down"] = mat(ff, w, 1.5), mat(w, ff, 1.5)
    return {k: v.to(torch.bfloat16).contiguous() for k, v in out.items()}


CONFIGS = {"A": CONFIG_A, "B": CONFIG_B, "C": CONFIG_C, "D": CONFIG_D}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = tmp_path_factory.mktemp("fiterax")
    out = {}
    for name, cfg in CONFIGS.items():
        d = helpers.make_model_dir(root / name, cfg, 0, tensors=fiterax_tensors(cfg, seed=ord(name)))
        out[name] = (d, plain.read_config(d), plain.read_weights(d))
    return out


def close_enough(got, ref, dtype, what):
    """float32: 1e-4 of the largest logit at every position.  bfloat16: the difference's root mean square against the
    logits'; with random weights the router's choice between two experts is now and then a rounding apart, and the
    other expert is another function, so a few positions may be far off while the typical one must be close."""
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
    """The oracle itself: taking a mechanism away (the convolution, the groups of the norm, the cap, a temperature,
    the corrections of the router, the factor on the sublayers, the forget gates' biases) moves its logits by far more
    than the tolerances of the tests below."""
    import copy

    d, cfg, w = models["A"]
    ids = helpers.token_ids(cfg["vocab"], 90, 1)
    ref = plain.forward(cfg, w, ids)
    size = np.abs(ref).max()

    def moved(cfg2, w2):
        return np.abs(plain.forward(cfg2, w2, ids) - ref).max() / size
    edits = {
        "groups": lambda c, x: c["norm"].update(groups=1),
        "cap": lambda c, x: c["layers"][0]["mixer"].pop("softcap"),
        "factor": lambda c, x: c.update(residual_mult=1.0),
        "gate cap": lambda c, x: c["layers"][1]["mixer"].update(gate_cap=60.0),
        "convolution": lambda c, x: x.update({"l0.canon1": x["l0.canon1"] * 0}),
        "second convolution": lambda c, x: x.update({"l1.canon2": x["l1.canon2"] * 0}),
        "temperature": lambda c, x: x.update({"l0.mix.temp": x["l0.mix.temp"] * 0 + 1}),
        "correction": lambda c, x: x.update({"l0.mlp.correction": x["l0.mlp.correction"] * 0}),
        "forget bias": lambda c, x: x.update({"l1.mix.f.b": x["l1.mix.f.b"] * 0}),
        "output bias": lambda c, x: x.update({"l2.mix.o.b": x["l2.mix.o.b"] * 0}),
    }
    for name, edit in edits.items():
        c2, w2 = copy.deepcopy(cfg), dict(w)
        edit(c2, w2)
        assert moved(c2, w2) > 1e-3, name


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_model_whole_in_portions_decoded_and_batched(models, name, dtype):
    """The same requests whole, token by token (through the captured decode graphs), in portions down to two tokens
    and one, and in batches of unequal requests that start and end at different steps in a pool so small that pages
    and state slots are taken again."""
    from from_scratch_inference_engine_amd import load_model
    from from_scratch_inference_engine_amd.engine.model import Runner

    d, cfg, w = models[name]
    vocab = cfg["vocab"]
    seqs = {"a": helpers.token_ids(vocab, 75, 1), "b": helpers.token_ids(vocab, 1, 2), "c": helpers.token_ids(vocab, 33, 3),
            "d": helpers.token_ids(vocab, 130, 4), "e": helpers.token_ids(vocab, 18, 5)}
    ref = {r: plain.forward(cfg, w, ids) for r, ids in seqs.items()}
    model = load_model(d, dtype=dtype)
    runner = Runner(model, page_size=8, num_pages=40, max_requests=3)
    assert runner.graphs.enabled
    got = step_through(runner, [[(r, len(ids))] for r, ids in seqs.items()], seqs)
    for r in seqs:
        close_enough(got[r], ref[r], dtype, f"{name} whole {r}")
    for r, head in (("a", 10), ("c", 1)):
        got = step_through(runner, [[(r, head)]] + [[(r, 1)]] * (len(seqs[r]) - head), {r: seqs[r]})
        close_enough(got[r], ref[r], dtype, f"{name} decode {r}")
    assert runner.graphs.replays > 50
    sizes, plan, left = [2, 7, 1, 16, 3, 2, 33, 8, 64], [], len(seqs["d"])
    while left:
        n = min(sizes[len(plan) % len(sizes)], left)
        plan.append([("d", n)])
        left -= n
    close_enough(step_through(runner, plan, {"d": seqs["d"]})["d"], ref["d"], dtype, f"{name} portions")
    plan = [[("a", 30), ("c", 2), ("b", 1)], [("a", 1), ("c", 20), ("e", 3)], [("c", 11), ("a", 44), ("e", 1)],
            [("e", 14), ("d", 9)], [("d", 120)], [("d", 1)]]
    got = step_through(runner, plan, seqs)
    for r in seqs:
        close_enough(got[r], ref[r], dtype, f"{name} batched {r}")
    assert all(a.pages_issued_again() for a in runner.manager.allocators)


def test_long_decoding_with_a_far_first_token(models):
    """Five hundred decoded tokens in float32, page after page: every logit is the plain one, with matrix memories
    that still hold the request's first tokens and attention that reads all the pages."""
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


@pytest.mark.parametrize("name", ["A", "B"])
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
        per = helpers.collect(tb, helpers.run_trace(d, dtype, tb.steps, 128, tmp_path / dtype))
        for rid, ids in (("a", a), ("b", b), ("c", c)):
            ref = plain.forward(cfg, w, ids)
            pos = sorted(per[rid])
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
