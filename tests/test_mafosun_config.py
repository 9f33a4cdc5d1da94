"""Mafosun without a GPU: the configuration, the expected tensors, the parts the builder makes, the attention plan for
chunks and pooled blocks, and the rescaled frequencies."""

import copy
import math
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import plain_mafosun as plain
from test_mafosun_gpu import CONFIG_A, CONFIG_B, CONFIG_C, CONFIG_D, mafosun_tensors

from from_scratch_inference_engine_amd.cache.manager import CacheManager, PagedNeed, PooledNeed, StateNeed
from from_scratch_inference_engine_amd.config.base import ConfigError
from from_scratch_inference_engine_amd.models.registry import build_model_spec, known_architectures, parse_config
from from_scratch_inference_engine_amd.ops.functions import ATTN_KEEP_WALK, ATTN_POOL_WALK
from from_scratch_inference_engine_amd.parts.attention import AttentionPlanner
from from_scratch_inference_engine_amd.parts.rope import RotaryEncoding
from from_scratch_inference_engine_amd.weights.loader import expected_tensors


@pytest.mark.parametrize("raw", [CONFIG_A, CONFIG_B, CONFIG_C, CONFIG_D])
def test_configuration_round_trip_and_expected_tensors(raw):
    assert "Mafosun" in known_architectures()
    cfg = parse_config(raw)
    assert parse_config(cfg.to_dict()) == cfg and cfg.width == raw["width"] and len(cfg.layers) == len(raw["layers"])
    spec = build_model_spec(cfg)
    want = {k: tuple(v.shape) for k, v in mafosun_tensors(raw, 0).items()}
    got = {k: tuple(s.shape) for k, s in expected_tensors(spec.bindings).items()}
    assert got == want


def test_what_the_builder_makes():
    spec = build_model_spec(parse_config(CONFIG_A))
    blocks = spec.layers
    assert [type(b).__name__ for b in blocks] == ["BranchNormBlock"] * 4 and blocks[2].ffn is None
    pair = blocks[0].mixer
    assert pair.left_scale == 1.3 and pair.right_scale == 0.4 and pair.joint and pair.o.in_features == 6 * 40 + 3 * 16
    assert pair.cache_need() == {"left": PagedNeed(3, 48, 16, 0), "right": StateNeed((3, 24, 16), "float32")}
    assert pair.left.chunk == 16 and pair.left.value_unit_norm_eps == 1e-6 and not pair.left.position.rotates
    assert pair.right.decay == [0.9, 0.99, 1.0] and pair.right.position.rotary_dim == 16
    att = blocks[1].mixer
    assert att.window == 10 and att.pool == 4 and att.softcap == 6.0 and att.unit_sink and att.interleaved_pairs
    assert att.cache_need() == {"tokens": PagedNeed(2, 32, 10, 0), "blocks": PooledNeed(2, 32, None, 0, 4)}
    assert att.position.bands == (4.0, 1.0, 4.0, 64.0)
    # blocks larger than the window: the keys stay until a block's means are made
    assert blocks[2].mixer.cache_need()["tokens"] == PagedNeed(1, 16, 7, 0)
    ffn = blocks[0].ffn
    assert (ffn.scores, ffn.groups, ffn.keep, ffn.renorm, ffn.gated, ffn.has_correction) == ("softmax", 3, 1, False, "silu", False)
    assert blocks[1].ffn.activation == "relu"
    assert spec.lm_head.param_decls()["weight"].shape == (150, 72)


@pytest.mark.parametrize("edit, word", [
    (lambda c: c["layers"][0].update(type="mamba"), "not a mixer"),
    (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][1]["mixer"]["mask"].pop("size"), "size"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=21), "even"),
    (lambda c: c["layers"][1]["mixer"].update(heads=3), "multiple"),
    (lambda c: c["layers"][0]["mixer"]["right"].update(decay=[0.5]), "decay"),
    (lambda c: c["layers"][0]["mixer"]["right"].update(decay=[0.5, 0.5, 1.5]), "at most 1"),
    (lambda c: c["layers"][0]["mixer"]["left"]["mask"].update(pool=3), "chunked"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=4), "groups"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=5), "choices"),
    (lambda c: c["layers"][1]["mlp"].update(kind="conv"), "feed-forward"),
    (lambda c: c.pop("vocab"), "vocab"),
])
def test_refusals(edit, word):
    raw = copy.deepcopy(CONFIG_A)
    edit(raw)
    with pytest.raises(ConfigError, match=word):
        parse_config(raw)


def test_rescaled_frequencies():
    for dims, base, bands in ((64, 300000.0, (6.0, 1.0, 3.0, 2048)), (20, 1000.0, (4.0, 1.0, 4.0, 64)), (6, 50.0, (2.0, 0.5, 3.0, 16))):
        enc = RotaryEncoding(dims + 4, base, rotary_dim=dims, bands=bands)
        ref = plain.rotary_frequencies(dims, base, dict(zip(("factor", "low", "high", "original"), bands)))
        assert np.allclose(enc.frequencies(), ref, rtol=1e-14, atol=0)
        plain_ones = plain.rotary_frequencies(dims, base)
        assert (ref <= plain_ones).all() and (ref < plain_ones).any()


def visible_by_definition(pos, window, chunk, pool):
    if chunk:
        return set(range(pos // chunk * chunk, pos + 1)), set()
    keys = set(range(max(0, pos - window + 1), pos + 1)) if window else set(range(pos + 1))
    blocks = {b for b in range(pos // pool + 1) if (b + 1) * pool - 1 <= pos - window} if pool else set()
    return keys, blocks


@pytest.mark.parametrize("window, chunk, pool", [(None, 16, None), (None, 1, None), (None, 7, None), (10, None, 4), (5, None, 7), (1, None, 1),
                                                 (80, None, 10), (None, None, None)])
@pytest.mark.parametrize("units", [1, 256])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_plan_covers_what_a_query_reads(window, chunk, pool, units, dtype):
    """From the items alone, with the kernels' mask (causal, the window, the pooled blocks of flagged items): every query
    of a step reads exactly the keys and blocks of its definition, each once, and every block that the step completes is
    made."""
    planner = AttentionPlanner(4, 2, 64, window, chunk=chunk, pool=pool)
    planner.compute_units = units
    rng = np.random.default_rng(3)
    for trial in range(30):
        n_seqs = int(rng.integers(1, 5))
        past = [int(rng.choice([0, 1, 15, 16, 17, 95, 96, 97, 300, 1500])) for _ in range(n_seqs)]
        new = [int(rng.choice([1, 1, 2, 3, 16, 33, 150])) for _ in range(n_seqs)]
        host = SimpleNamespace(n_seqs=n_seqs, q_lens=new, past_lens=past, q_starts=list(np.cumsum([0] + new)), page_size=16,
                               compute_dtype=dtype, pad=None, memo={})
        host.n_tokens = host.q_starts[-1]
        plan = planner.plan(host)
        seen = {}  # row -> [keys list, blocks list]
        assert plan["mfma"] == (dtype == torch.bfloat16)
        every = list(plan["items"]) + list(plan.get("pool_items", []))
        assert not any(int(it[7]) & ATTN_POOL_WALK for it in plan["items"]) or not plan["mfma"]
        slots = {}  # row -> slots of the partial records that items leave for it
        for it in every:
            if int(it[6]) >= 0:
                for t in range(int(it[2])):
                    slots.setdefault(int(it[1]) + t, []).append(int(it[6]) + t)
        for row, first, n, stride in (tuple(int(v) for v in m) for m in plan["merges"]):
            assert sorted(slots.pop(row)) == [first + i * stride for i in range(n)]
        assert not slots and plan["n_merges"] == len(plan["merges"])
        taken = [s for it in every if int(it[6]) >= 0 for s in range(int(it[6]), int(it[6]) + int(it[2]))]
        assert len(taken) == len(set(taken)) and all(s < plan["n_partial"] for s in taken)
        for it in every:
            s, row0, n, p, kb, ke, partial, flags = (int(v) for v in it)
            keep = flags & ~(ATTN_KEEP_WALK | ATTN_POOL_WALK)
            assert keep == 0
            for t in range(n):
                pos = p + t
                assert pos == past[s] + (row0 + t - host.q_starts[s])
                keys, blocks = seen.setdefault(row0 + t, ([], []))
                keys += [k for k in range(kb, ke) if k <= pos and (not window or k > pos - window)]
                if flags & ATTN_POOL_WALK:
                    blocks += [b for b in range(max(0, p + n - window) // pool) if (b + 1) * pool <= pos - window + 1]
        merged = {int(m[0]) for m in plan["merges"]}
        for s in range(n_seqs):
            for t in range(new[s]):
                row, pos = host.q_starts[s] + t, past[s] + t
                keys, blocks = seen[row]
                want_keys, want_blocks = visible_by_definition(pos, window, chunk, pool)
                assert sorted(keys) == sorted(want_keys) and sorted(blocks) == sorted(want_blocks), (trial, s, t)
        for it in every:
            rows = range(int(it[1]), int(it[1]) + int(it[2]))
            assert all((r in merged) == (int(it[6]) >= 0) for r in rows)
        if pool:
            jobs = {(int(a), int(b)) for a, b in plan["pool_jobs"]}
            want = {(s, b) for s in range(n_seqs) for b in range((past[s] + new[s]) // pool) if (b + 1) * pool - 1 >= past[s]}
            assert jobs == want and plan["n_pool_jobs"] == len(want)


def test_cache_manager_counts_pooled_blocks_by_their_own_pages():
    """Keys of a window that hands pages back beside pooled blocks that stay: a page of the blocks' group holds
    page_size blocks of ``pool`` positions each."""
    needs = [PagedNeed(2, 32, 12, 0), PooledNeed(2, 32, None, 0, 4)]
    manager = CacheManager(needs, page_size=8, num_pages=[10, 3], max_requests=2)
    assert manager.tokens_per_page(0) == 8 and manager.tokens_per_page(1) == 32
    rc = manager.open("a")
    total = 0
    for n in (5, 30, 1, 40, 3):
        assert manager.can_reserve([(rc, n)])
        manager.reserve(rc, n)
        manager.commit(rc, n)
        total += n
        assert len(rc.tables[1]) == -(-total // 32) and all(p >= 0 for p in rc.tables[1])
        assert rc.pages_held(0) <= -(-(12 + 8) // 8) + 1
        manager.check_invariants()
    manager.close(rc)
    assert manager.free_pages(0) == 10 and manager.free_pages(1) == 3
