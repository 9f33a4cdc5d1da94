"""Grouped-query attention over the paged cache."""

from __future__ import annotations

import math
from typing import Dict, Optional

import numpy as np
import torch

from .. import ops
from ..cache.manager import PagedNeed, PooledNeed
from ..ops.functions import ATTN_ITEM_INTS, ATTN_KEEP_WALK, ATTN_MERGE_INTS, ATTN_POOL_WALK
from ..ops.functions import GEMM_MFMA_SKINNY_BEST_M
from .base import Mixer, Norm, ParamDecl, Part, PositionEncoding, register_part
from .linear import Linear


class AttentionPlanner:
    """Cuts a step into the work items of the attention kernels (host side, once per step for all
    layers with the same geometry).

    A request's portion of n tokens at past length p becomes tiles of query tokens; a tile reads
    the keys from the start of its window to its last token.  A portion of at most
    ``small_tokens`` tokens is one *small* item.  A small item that reads more than ``split_keys``
    keys (decoding against a long context) is split over the keys into several items and merged
    afterwards in the order of the splits: 256 keys an item for the float32-arithmetic kernel (128
    or 64 by the same rule as below); for
    the matrix-core kernel, which gives every 128 keys to a wave of the item's workgroup and
    combines those inside, 1,024 keys, or 512, 256 or 128 while that leaves the step with at most
    as many workgroups as the device has compute units (every wave still sums the same 128 keys;
    only where their sums meet changes).  Longer portions are cut into *large* tiles of ``large_tokens``; how they are
    cut depends on the portion alone, never on what else is in the batch.  The item table lists
    the small items first.

    Two geometries exist: the matrix-core kernel (bfloat16, head size a multiple of 16, page size
    a multiple of 4) and the float32-arithmetic kernel for everything else; which one a step
    uses follows from the step's dtype and page size."""

    # Keys above which a large tile is given four waves that split its keys.  Off: idle waves in
    # the four-wave workgroups cost more than the balance gains.
    long_keys: Optional[int] = None
    # Compute units to fill with the workgroups of small items; None: those of the device.
    compute_units: Optional[int] = None

    def __init__(self, n_heads: int, n_kv: int, head_dim: int, window: Optional[int], keep_first: int = 0,
                 chunk: Optional[int] = None, pool: Optional[int] = None):
        """``keep_first`` (with a window): the first positions of a request stay visible to every later query.
        Items say so in their last field (``ATTN_ITEM_KEEP``); an item whose window has left those keys behind
        reads them first and then its own range (flag ``ATTN_KEEP_WALK``), and where a request's keys are split
        over several items the kept keys are an item of their own that is merged with the rest.

        ``chunk`` (instead of a window): a query reads the keys of its own chunk of that many positions, counted
        from the request's start, up to itself.  The kernels know nothing of it: a portion is cut where a chunk
        ends, so all queries of an item share a chunk, and the item's range of keys starts where the chunk does.

        ``pool`` (with a window): beside the window a query reads one pooled key and value for every block of
        ``pool`` positions that lies wholly before its window.  Items carry the flag ``ATTN_POOL_WALK``; where a
        request's keys are split over several items the pooled blocks are an item of their own.  The plan also
        lists the blocks that the step completes (``pool_jobs``: request of the step, block), whose means the
        mixer has computed before attention runs."""
        if chunk and (window or keep_first):
            raise ValueError("attention plan: chunks go without a window")
        if pool and not window:
            raise ValueError("attention plan: pooled blocks go with a window")
        self.n_heads, self.n_kv, self.head_dim, self.window = n_heads, n_kv, head_dim, window
        self.keep_first = int(keep_first) if window else 0
        self.chunk, self.pool = (int(chunk) if chunk else None), (int(pool) if pool else None)
        self.key = ("attention", n_heads, n_kv, head_dim, window, self.keep_first, self.chunk, self.pool)
        self._geometry = {}

    def _portions(self, p: int, n: int):
        """A request's n tokens from position p as (offset, tokens, position) runs whose queries share their first
        key's rule: the portion itself, or with chunks its pieces between the chunks' ends."""
        if not self.chunk or (p % self.chunk) + n <= self.chunk:
            return [(0, n, p)]
        runs, off = [], 0
        while off < n:
            here = min(n - off, self.chunk - (p + off) % self.chunk)
            runs.append((off, here, p + off))
            off += here
        return runs

    def _pooled_seen(self, last_pos: int) -> int:
        """Pooled blocks that the query at ``last_pos`` reads."""
        return max(0, last_pos - self.window + 1) // self.pool if self.pool else 0

    def _first_key(self, p: int):
        """(first key of the window of the query at position p, kept keys that lie before it)."""
        if self.chunk:
            return p // self.chunk * self.chunk, 0
        first = max(0, p - self.window + 1) if self.window else 0
        if self.keep_first and first <= self.keep_first:
            return 0, 0  # the kept keys and the window touch: one range, the mask does the rest
        return first, (self.keep_first if first else 0)

    def geometry(self, mfma: bool):
        """(small_tokens, large_tokens, split_keys) of a kernel family."""
        if mfma not in self._geometry:
            group = self.n_heads // self.n_kv
            if mfma:
                small = max(1, ops.attention_mfma_rows(self.head_dim, False) // min(group, 16))
                rows = ops.attention_mfma_rows(self.head_dim, True)
                large = max(1, rows // min(group, rows))
                # at most 1,024 keys (eight waves of 128) an item
                self._geometry[mfma] = (small, large, 128 * min(8, ops.attention_mfma_max_waves(self.head_dim)))
            else:
                t = ops.attention_tile_tokens(self.n_heads, self.n_kv)
                self._geometry[mfma] = (t, t, 256)
        return self._geometry[mfma]

    def uses_mfma(self, compute_dtype, page_size: int) -> bool:
        return (compute_dtype == torch.bfloat16 and self.head_dim % 16 == 0 and self.head_dim <= 256
                and page_size % 4 == 0 and (not self.keep_first or self.mfma_keeps_first))

    mfma_keeps_first = True  # whether the matrix-core kernels read an item's kept first keys

    def _waves_for(self, keys: int, max_waves: int) -> int:
        """Waves of a workgroup for an item of ``keys`` keys: one per 128 keys, a power of two."""
        need = max(1, -(-keys // 128))
        w = 1
        while w < need and w < max_waves:
            w *= 2
        return min(w, max_waves)

    def _small_keys(self, host, small_tokens):
        """Keys that each small portion of the step reads."""
        keys = []
        for s in range(host.n_seqs):
            for _, n, p in self._portions(host.past_lens[s], host.q_lens[s]):
                if n <= small_tokens:
                    first, kept = self._first_key(p)
                    keys.append(p + n - first + kept)
        return keys

    def split_keys(self, host, mfma: bool) -> int:
        """Keys per small item in this step.  A workgroup draws only so much from memory, so a step
        with few requests is faster with more, shorter items although they cost a merge, and a full
        device keeps the long ones."""
        memo = getattr(host, "memo", None)
        if memo is not None and (self.key, mfma, self.compute_units) in memo:
            return memo[(self.key, mfma, self.compute_units)]
        split = self._split_keys(host, mfma)
        if memo is not None:
            memo[(self.key, mfma, self.compute_units)] = split
        return split

    def _split_keys(self, host, mfma: bool) -> int:
        small_tokens, _, longest = self.geometry(mfma)
        units = self.compute_units if self.compute_units is not None else ops.compute_units()
        keys = self._small_keys(host, small_tokens)
        group = self.n_heads // self.n_kv
        # the float32-arithmetic kernel takes 32 keys a pass and up to 16 heads of a group a workgroup:
        # its items shorten to 64 keys (two passes) while compute units are idle
        rows, shortest, room = (ops.attention_mfma_rows(self.head_dim, False), 128, 1) if mfma else (16, 64, 2)
        per_item = self.n_kv * -(-group // min(group, rows))  # workgroups of one item
        split = longest
        if mfma and keys and len(keys) <= self.whole_requests and max(keys) <= longest:
            # one or two requests whose keys fit one item: the item stays whole and the step has no
            # merge at all; the waves of its workgroup deal the keys and combine through LDS
            return longest
        # halved while the halves' workgroups still number at most the compute units: beyond that a
        # split only adds a merge.  The float32-arithmetic kernel's workgroups are slower and several
        # share a unit: twice the units.
        # (the matrix-core kernel: up to exactly one workgroup a unit)
        most_groups = units * room + (1 if mfma else 0)
        while split > shortest and sum(-(-k // (split // 2)) for k in keys) * per_item < most_groups:
            split //= 2
        if self.fine_items and mfma and keys and split > shortest:
            # between that length and its half: the shortest multiple of 32 whose workgroups still number at most the units
            lo, hi = 0, (split - split // 2) // 32 - 1
            while lo < hi:
                mid = (lo + hi + 1) // 2
                if sum(-(-k // (split - 32 * mid)) for k in keys) * per_item < most_groups:
                    lo = mid
                else:
                    hi = mid - 1
            split -= 32 * lo
        # requests that fit one item each need no merge at all while they stay whole: cutting them in
        # two is not worth one, in three or more it is
        if keys and split < longest and max(keys) <= longest and -(-max(keys) // split) <= 2:
            return longest
        # Items of the matrix-core kernel may be longer: the waves of a workgroup deal an item's keys
        # among themselves, and an item more for a request costs the work before the walk again and
        # a merge.  Where the requests alone give every compute unit a workgroup they stay whole,
        # however long.  Fewer requests take the longest items of which the full ones still number the
        # units; fewer workgroups than units lose.
        if self.long_items and mfma and keys and split == longest and units > 0 and max(keys) > longest:
            long = longest
            while long < max(keys):
                long *= 2
            # (no item longer than the keys a unit gets when they are dealt evenly, as a power of two:
            # one request of 100,000 keys among 63 short ones is cut, or its workgroups would run long
            # after the others)
            even = sum(keys) * per_item / units
            most = longest
            while most < even:
                most *= 2
            long = min(long, most)
            if len(keys) * per_item < units:
                while long > longest and sum(max(1, k // long) for k in keys) * per_item < units:
                    long //= 2
            split = long
        # Two cases in which shorter items are faster (measured at 28/4 and 40/8 heads of 128):
        # * more workgroups than units, in rounds of which the last is mostly empty: the items shorten
        #   as far as the same number of rounds still holds all their workgroups.  Items of less than a
        #   quarter of the length (the one key by which a request has passed a multiple) do not count
        #   as workgroups here: they are over at once.
        # * long items (twice the usual longest and more) whose workgroups leave the units half empty: a
        #   unit holds two such workgroups, so the items shorten as far as two a unit allow.  Not where
        #   no request is cut at all: whole requests that fill the units read at the memory's rate as
        #   they are, and cut in two they only gain a merge.
        # Both in steps of a 64th of the length (at least 32 keys) and to no less than half of it.
        if self.fill_rounds and mfma and keys and units > 0:
            def groups_of(length, least=0):
                return sum(k // length + (1 if k % length > least else 0) for k in keys) * per_item
            everyone, large_ones = groups_of(split), groups_of(split, split // 4)
            rounds = -(-large_ones // units)
            room_for = 0
            if large_ones > units and large_ones * 10 < rounds * units * 9:
                room_for = rounds * units
            elif split >= 2 * longest and everyone * 2 <= units * 3 and max(keys) > split:
                room_for = 2 * units
            if room_for:
                step = max(32, split // 64 // 32 * 32)
                # the shortest length on the grid whose workgroups still fit (their number only grows as
                # the items shorten): by halving the range
                lo, hi = 0, (split - split // 2) // step  # steps below `split`: lo fits, hi is the most
                while lo < hi:
                    mid = (lo + hi + 1) // 2
                    if groups_of(split - mid * step) <= room_for:
                        lo = mid
                    else:
                        hi = mid - 1
                shorter = split - lo * step
                if groups_of(shorter, shorter // 4) > large_ones:  # (shorter items that are no more items gain nothing)
                    split = shorter
        return split

    long_items = True  # items beyond the longest of `geometry` where they still fill the device
    # Steps of up to so many requests keep items that fit the longest whole (no merge launch).  0:
    # never, which is faster: the one-wave item asks for all its blocks of keys at once, a wave of the
    # many-wave workgroup for two at a time.
    whole_requests = 0
    # items shorten so that the last round of their workgroups is a full one (see split_keys)
    fill_rounds = True
    # between a power of two and its half, the shortest items whose workgroups still number at most the units
    fine_items = True

    @staticmethod
    def _items_of(keys: int, split_keys: int, longest: int) -> int:
        """Items that the ``keys`` keys of a small portion are cut into: runs of ``split_keys``."""
        return max(1, -(-keys // split_keys))

    def graph_bucket(self, host):
        """What a captured graph of this step's shape must fix: the number of (small) work items,
        the waves per item and the keys per item; None if the step has portions that do not fit
        small items."""
        mfma = self.uses_mfma(host.compute_dtype, host.page_size)
        small_tokens = self.geometry(mfma)[0]
        split_keys = self.split_keys(host, mfma)
        most = self.geometry(mfma)[2]
        n, longest = 0, 1
        for s in range(host.n_seqs):
            if host.q_lens[s] > small_tokens:
                return None
            first_key, kept = self._first_key(host.past_lens[s])
            keys = host.past_lens[s] + host.q_lens[s] - first_key
            mine = self._items_of(keys, split_keys, most)
            longest = max(longest, keys - (mine - 1) * split_keys)  # (the last item; the others have split_keys, if any)
            if mine > 1:
                longest = max(longest, split_keys)
                mine += 1 if kept else 0  # (the kept first keys are an item of their own)
                if not mfma:  # (and the pooled blocks; the matrix-core geometry keeps them in a table of their own)
                    mine += 1 if self._pooled_seen(host.past_lens[s] + host.q_lens[s] - 1) else 0
            elif kept:
                longest = max(longest, keys + 32 * -(-kept // 32))
            n += mine
        if mfma:
            # items: a multiple of the number of requests and of a quarter of what gives every unit a
            # workgroup, so that one graph serves a batch while its requests grow: their items grow
            # longer, not more (the captured graph pads with empty items, whose workgroups leave at
            # once).  The length of the items is data of the step, not of the graph.
            units = self.compute_units if self.compute_units is not None else ops.compute_units()
            group = self.n_heads // self.n_kv
            per_item = self.n_kv * -(-group // min(group, ops.attention_mfma_rows(self.head_dim, False)))
            step = max(host.n_seqs, units // per_item // 4, 1)
            return (-(-n // step) * step,
                    self._waves_for(longest, ops.attention_mfma_max_waves(self.head_dim)), 0)
        step = host.n_seqs * max(1, 1024 // split_keys)
        return (-(-n // step) * step, 1, split_keys)

    def plan(self, host) -> Dict[str, object]:
        mfma = self.uses_mfma(host.compute_dtype, host.page_size)
        small_tokens, large_tokens, most = self.geometry(mfma)
        padded = getattr(host, "pad", None) is not None
        split_keys = self.split_keys(host, mfma)
        small, merges = [], []
        large_runs = []  # per long portion: its tiles as rows of an array (a prompt of thousands of tokens has hundreds)
        n_partial = 0
        pool_flag = ATTN_POOL_WALK if self.pool else 0
        pool_jobs = []
        # The matrix-core kernels read keys and values of one pool.  With pooled blocks they leave partial records for
        # the queries that see blocks, the float32-arithmetic kernel leaves the blocks' records (items of their own,
        # ``pool_items``, cut to its tiles of queries), and the merge joins the two in one softmax.
        two_pass = bool(mfma and self.pool)
        pool_tile = ops.attention_tile_tokens(self.n_heads, self.n_kv) if two_pass else 0
        pool_items, pool_item_runs, pooled_runs, merge_runs = [], [], [], []

        def blocks_items(s, row0, n, p, base):
            """The pooled blocks of n queries as items of the float32-arithmetic kernel, slots base .. base + n."""
            for off in range(0, n, pool_tile):
                pool_items.append((s, row0 + off, min(pool_tile, n - off), p + off, 0, 0, base + off, pool_flag))
        for s in range(host.n_seqs):
            if self.pool:
                # the blocks whose last position this step brings: their means are made before attention runs
                p_all, n_all = host.past_lens[s], host.q_lens[s]
                pool_jobs += [(s, b) for b in range(p_all // self.pool, (p_all + n_all) // self.pool)]
            for off, n, p in self._portions(host.past_lens[s], host.q_lens[s]):
                row0 = host.q_starts[s] + off
                first_key, kept = self._first_key(p)
                keep = self.keep_first
                total = p + n
                n_splits = self._items_of(total - first_key, split_keys, most) if split_keys is not None else 1
                pooled = self._pooled_seen(total - 1) > 0
                if n <= small_tokens and (n_splits > 1 or (two_pass and pooled)):
                    base = n_partial
                    if kept:
                        small.append((s, row0, n, p, 0, kept, base, keep))
                        base += n
                    if pooled and two_pass:
                        blocks_items(s, row0, n, p, base)
                        base += n
                    elif pooled:  # the pooled blocks: an item with no keys of its own
                        small.append((s, row0, n, p, 0, 0, base, keep | pool_flag))
                        base += n
                    for i in range(n_splits):
                        kb = first_key + i * split_keys
                        small.append((s, row0, n, p, kb, total if i == n_splits - 1 else kb + split_keys, base + i * n, keep))
                    n_splits += (1 if kept else 0) + (1 if pooled else 0)
                    for t in range(n):
                        merges.append((row0 + t, n_partial + t, n_splits, n))
                    n_partial += n_splits * n
                elif n <= small_tokens:
                    small.append((s, row0, n, p, first_key, total, -1,
                                  (keep | ATTN_KEEP_WALK if keep else 0) | (0 if two_pass else pool_flag)))
                else:
                    # (the short tile that a long portion may end with stays with the portion's other tiles:
                    # as a small item it would walk all the portion's keys in one workgroup a kv head, alone
                    # on the device, while as the last of a group of four it shares their blocks of keys)
                    t0 = np.arange(0, n, large_tokens, dtype=np.int64)
                    run = np.empty((t0.shape[0], ATTN_ITEM_INTS), dtype=np.int64)
                    pos0 = p + t0
                    run[:, 0] = s
                    run[:, 1] = row0 + t0
                    run[:, 2] = np.minimum(large_tokens, n - t0)
                    run[:, 3] = pos0
                    run[:, 4] = np.maximum(0, pos0 - self.window + 1) if self.window else (first_key if self.chunk else 0)
                    if self.keep_first:
                        run[:, 4] = np.where(run[:, 4] <= self.keep_first, 0, run[:, 4])
                    run[:, 5] = pos0 + run[:, 2]
                    run[:, 6] = -1
                    run[:, 7] = (self.keep_first | ATTN_KEEP_WALK if self.keep_first else 0) | (0 if two_pass else pool_flag)
                    if two_pass:
                        # the tiles whose last query sees a block (the later ones of the run) leave partial records:
                        # a tile of n_t queries has the slots base .. base + n_t for its keys, the next n_t for the blocks
                        sees = np.maximum(0, run[:, 5] - self.window) // self.pool > 0
                        mine, run = run[sees], run[~sees]
                        if len(mine):
                            n_t = mine[:, 2]
                            ends = np.cumsum(2 * n_t)
                            bases = n_partial + ends - 2 * n_t
                            mine[:, 6] = bases
                            tile = np.repeat(np.arange(len(mine)), n_t)
                            t_in = np.arange(int(n_t.sum())) - np.repeat(np.cumsum(n_t) - n_t, n_t)
                            merge_runs.append(np.stack([mine[tile, 1] + t_in, bases[tile] + t_in, np.full_like(t_in, 2), n_t[tile]], axis=1))
                            pieces = -(-n_t // pool_tile)
                            tile = np.repeat(np.arange(len(mine)), pieces)
                            at = (np.arange(int(pieces.sum())) - np.repeat(np.cumsum(pieces) - pieces, pieces)) * pool_tile
                            zeros = np.zeros_like(at)
                            pool_item_runs.append(np.stack([mine[tile, 0], mine[tile, 1] + at, np.minimum(pool_tile, n_t[tile] - at),
                                                            mine[tile, 3] + at, zeros, zeros, bases[tile] + n_t[tile] + at,
                                                            zeros + pool_flag], axis=1))
                            n_partial += int(ends[-1])
                            pooled_runs.append(mine)
                    if len(run):
                        large_runs.append(run)
        large = np.concatenate(large_runs) if large_runs else np.zeros((0, ATTN_ITEM_INTS), dtype=np.int64)
        waves = 1
        if mfma and small:
            waves = self._waves_for(max(it[5] - it[4] + (32 * -(-min(it[7] & ~(ATTN_KEEP_WALK | ATTN_POOL_WALK), it[4]) // 32)
                                                            if it[7] & ATTN_KEEP_WALK else 0) for it in small),
                                    ops.attention_mfma_max_waves(self.head_dim))
        if padded:
            # a captured graph launches fixed grids: pad with items and merges that do nothing
            n_items, waves, _ = host.pad[self.key]
            if len(large) or len(small) > n_items:
                raise RuntimeError("attention plan does not fit the captured graph")
            small += [(0, 0, 0, 0, 0, 0, -1, 0)] * (n_items - len(small))
            if two_pass:
                # one item of pooled blocks a request at most (a step of single tokens), and every row merged
                if len(pool_items) > host.n_seqs:
                    raise RuntimeError("attention plan: more items of pooled blocks than the captured graph has room for")
                pool_items += [(0, 0, 0, 0, 0, 0, -1, 0)] * (host.n_seqs - len(pool_items))
            if n_items > host.n_seqs or two_pass:
                # the graph has room for items that share a request's keys: it merges every row
                # (rows that need none get an empty merge)
                merged = {m[0] for m in merges}
                merges += [(row, 0, 0, 0) for row in range(host.n_tokens) if row not in merged]
                n_partial = (n_items + (host.n_seqs if two_pass else 0)) * small_tokens
        # consecutive large tiles of one request, four at a time, for the kernel that shares the
        # keys of a block among four waves
        groups = np.zeros((0, 2), dtype=np.int64)
        if mfma and large_runs:
            firsts, counts, at = [], [], 0
            for run in large_runs:
                f = np.arange(0, run.shape[0], 4, dtype=np.int64)
                firsts.append(at + f)
                counts.append(np.minimum(4, run.shape[0] - f))
                at += run.shape[0]
            firsts, counts = np.concatenate(firsts), np.concatenate(counts)
            # by the number of keys a group goes through, ascending: the kernel starts its workgroups
            # from the back of this list, the longest first (with several requests in a step the
            # order of the requests would otherwise decide)
            order = np.argsort(large[firsts + counts - 1, 5] - large[firsts, 4], kind="stable")
            groups = np.stack([firsts[order], counts[order]], axis=1)
        n_long, long_waves = 0, 4
        if pooled_runs:
            # the tiles that leave partial records: a class of their own behind the others, a wave a workgroup
            n_long, long_waves = sum(len(r) for r in pooled_runs), 1
            large = np.concatenate([large] + pooled_runs)
        elif mfma and self.long_keys is not None:
            # large tiles that read more than ``long_keys`` keys go to workgroups of four waves
            is_long = large[:, 5] - large[:, 4] > self.long_keys
            large = np.concatenate([large[~is_long], large[is_long]])
            n_long = int(is_long.sum())
        small_items = np.asarray(small, dtype=np.int64).reshape(-1, ATTN_ITEM_INTS)
        extra = {}
        if self.pool:
            if padded:  # (a step of single tokens completes at most a block a request)
                if len(pool_jobs) > host.n_seqs:
                    raise RuntimeError("attention plan: more completed blocks than the captured graph has room for")
                pool_jobs += [(-1, 0)] * (host.n_seqs - len(pool_jobs))
            extra = {"pool_jobs": np.asarray(pool_jobs, dtype=np.int32).reshape(-1, 2), "n_pool_jobs": len(pool_jobs),
                     "pool_items": np.concatenate([np.asarray(pool_items, dtype=np.int64).reshape(-1, ATTN_ITEM_INTS)]
                                                  + pool_item_runs).astype(np.int32),
                     "n_pool_items": len(pool_items) + sum(len(r) for r in pool_item_runs)}
        return {
            **extra,
            "items": np.concatenate([small_items, large]).astype(np.int32),
            "merges": np.concatenate([np.asarray(merges, dtype=np.int64).reshape(-1, ATTN_MERGE_INTS)] + merge_runs).astype(np.int32),
            "groups": groups.astype(np.int32), "n_groups": len(groups),
            "n_small": len(small), "n_large": len(large) - n_long, "n_long": n_long, "long_waves": long_waves,
            "n_merges": len(merges) + sum(len(m) for m in merge_runs),
            "n_partial": n_partial, "mfma": mfma, "waves": waves,
            "single": all(host.q_lens[s] == 1 for s in range(host.n_seqs)),  # one token a request
        }


def paged_attention(q: torch.Tensor, q_stride: int, cache, plan, n_heads: int, n_kv: int, head_dim: int,
                    window: Optional[int], scale: float, n_tokens: int, sinks: Optional[torch.Tensor] = None,
                    share_keys: bool = True, softcap: Optional[float] = None, pooled=None) -> torch.Tensor:
    """Causal attention of a step's queries over the paged cache, by the work items of ``plan`` (an
    ``AttentionPlanner``'s): [n_tokens, n_heads * head_dim] in the queries' type.  ``q``: rows of ``q_stride``
    values whose first n_heads * head_dim are the heads' queries; the keys and values of the step's own
    tokens are in the cache already.  ``sinks`` (float32 [n_heads] or None): a term exp(sinks[h]) more in the
    denominator of head h's softmax.  ``softcap`` (a positive number or None): the scaled scores become
    softcap * tanh(score / softcap) before the mask and the softmax.  ``pooled`` = (k_pool, v_pool, block_tables,
    block_tokens): the pools of pooled blocks that items flagged ``ATTN_POOL_WALK`` read beside their keys (a planner
    with ``pool``).  Every mixer whose cache is pages of keys and values calls this."""
    cap = float(softcap or 0.0)
    if pooled is not None and plan.mfma and plan.n_pool_items and not plan.n_partial:
        raise RuntimeError("attention: items of pooled blocks without partial records to leave them in")
    out = torch.empty((n_tokens, n_heads * head_dim), dtype=q.dtype, device=q.device)
    partials = None
    if plan.n_partial:
        partials = torch.empty((plan.n_partial * n_heads * (head_dim + 2),), dtype=torch.float32, device=q.device)
    args = (partials, n_heads, n_kv, head_dim, window, scale, n_tokens)
    if plan.mfma:
        if plan.n_small:
            ops.attention_mfma(q, q_stride, cache.k_pool, cache.v_pool, cache.block_tables, plan.items,
                               plan.n_small, out, *args, large=False, waves=plan.waves, sinks=sinks, softcap=cap)
        if (plan.n_large and (not plan.n_long or getattr(plan, "long_waves", 4) == 1) and share_keys
                and ops.attention_mfma_lds_ok(head_dim, cache.page_size)):
            ops.attention_mfma_lds(q, q_stride, cache.k_pool, cache.v_pool, cache.block_tables,
                                   plan.items[plan.n_small:], plan.groups, plan.n_groups, out, n_heads,
                                   n_kv, head_dim, window, scale, n_tokens, sinks=sinks, softcap=cap)
        elif plan.n_large:
            ops.attention_mfma(q, q_stride, cache.k_pool, cache.v_pool, cache.block_tables,
                               plan.items[plan.n_small:], plan.n_large, out, *args, large=True, sinks=sinks, softcap=cap)
        if plan.n_long:
            ops.attention_mfma(q, q_stride, cache.k_pool, cache.v_pool, cache.block_tables,
                               plan.items[plan.n_small + plan.n_large:], plan.n_long, out, *args, large=True,
                               waves=getattr(plan, "long_waves", 4), sinks=sinks, softcap=cap)
        if pooled is not None and plan.n_pool_items:
            # the pooled blocks of the queries that see any: partial records beside those of their keys
            ops.attention_scalar(q, q_stride, cache.k_pool, cache.v_pool, cache.block_tables, plan.pool_items,
                                 plan.n_pool_items, out, *args, softcap=cap, pooled=pooled)
    else:
        ops.attention_scalar(q, q_stride, cache.k_pool, cache.v_pool, cache.block_tables, plan.items,
                             plan.n_small + plan.n_large, out, *args, sinks=sinks, softcap=cap, pooled=pooled)
    if plan.n_merges:
        ops.attention_merge(partials, plan.merges, plan.n_merges, out, n_heads, head_dim, sinks=sinks)
    return out


@register_part("mixer", "gqa_attention")
class GQAttention(Mixer):
    """q/k/v projections (one matrix, optional bias), optional norms of every q and k head,
    position encoding, causal attention with kv head = q head // (heads / kv heads) and scale
    1/sqrt(head_dim), output projection without bias (src/model/model.cpp:110-129,
    src/model/nn.cpp:151-226).  ``window`` = number of latest positions a query reads (None: all).
    ``sink=True``: a learned number per head (parameter ``sink``) whose exponential joins the softmax's
    denominator; it has no key and no value.  ``keep_first``: with a window, the first positions of a request
    that every later query still reads.  ``scale``: the factor on the scores (None: 1/sqrt(head_dim)).
    ``value_dim``: the size of a head's values where it is not the keys' (the cache and the attention kernels then
    work on heads of ``padded`` values, the larger of the two rounded up to 16, zeros at their end).
    ``gate=True``: the projection has one more row a head, and head h's result is multiplied by the sigmoid of
    its row's product with x before the output projection.  ``value_mix``: "source" publishes this layer's
    values of the step's tokens, "mixed" replaces its own by (1 - w) v + w v_source (parameter
    ``value_mix_weight``, one number) before they are cached; both ends must agree in kv heads and value size.
    ``o_bias=True``: the output projection has a bias.  ``unit_norm_eps``: every q and k head is divided by its root
    mean square (eps inside the root; no weight; a rotation does not change a head's root mean square, so the kernel's
    order, norm then rotation, gives the same head as rotation then norm).  ``head_temperature=True`` (with
    ``unit_norm_eps``): a number per query head (parameter ``temperature``) multiplies its scores.  ``softcap``: the
    scaled scores become softcap * tanh(score / softcap).
    ``interleaved_pairs=True``: the encoding rotates neighbours (2i, 2i + 1) of the checkpoint's heads; the rows of the
    q and k projections and the head norms' weights are reordered once, when the weights are loaded (even values of the
    rotated part first, then the odd ones), so that the rotation is that of the pairs (i, i + rotary_dim / 2): the scores
    do not change when q and k are reordered alike, and nothing else reads them.  ``value_unit_norm_eps``: every kv
    head's values are divided by their root mean square (eps inside the root, no weight) before they are cached.
    ``unit_sink=True``: one is added to the softmax's denominator (a sink whose score is 0, without a value).
    ``chunk`` (instead of a window): a query reads the keys of its own chunk of that many positions, counted from the
    request's start.  ``pool`` (with a window): beside the window a query reads the mean key and mean value of every
    block of ``pool`` positions that lies wholly before its window; the means are kept in pages of their own (an entry a
    block, a second cache need) and made by a kernel from the cached keys and values when a block's last position
    arrives.  ``fused_prep=True`` takes the one-kernel path below also where none of its reasons holds.
    With any of gate, mixed values, another value size or the unit norm, what stands between projection and attention is one kernel
    (``ops.attention_prep``: head norms, rotation of the first ``rotary_dim`` values from the step's table, value
    mixing, gates, cache write) and one after it (``ops.gate_heads``).

    What happens between the projection and attention, in this order: bias, ``q_norm`` / ``k_norm``
    (a norm as wide as a head, applied to every head through ``Norm.plain``; None: none), the
    position encoding's ``rotate``, the write of k and v into the cache.  The mixer owns all of it;
    the encoding only rotates.  Where nothing stands between the projection and a rotation that
    the encoding can describe by a table of cosines and sines (``rotation_table``), the mixer's own
    kernels do several of these steps at once: for steps of one token a request the attention
    kernel itself finishes the projection's partial sums (bias, rotation, cache write); for up to 16
    rows the projection's epilogue does; for 17 to 128 rows the kernel that writes the cache adds
    the partial sums up.  With head norms, or an encoding without a table, the steps run one after
    the other (projection, bias, norms, ``rotate``, cache write), which every combination can take."""

    share_keys = True  # long portions: four tiles of a request share each block of keys through LDS
    # steps of one token a request: the attention kernel adds up the q/k/v product's partial sums,
    # rotates and writes the cache itself (one launch fewer a layer)
    finish_qkv_in_attention = True

    @property
    def graph_safe(self) -> bool:
        """forward reads the step only through device tables; its sub-parts must too."""
        return all(p.graph_safe for p in self.sub_parts().values())

    def __init__(self, hidden_size: int, n_heads: int, n_kv_heads: int, head_dim: int, qkv_bias: bool,
                 position: PositionEncoding, window: Optional[int] = None, q_norm: Optional[Norm] = None,
                 k_norm: Optional[Norm] = None, sink: bool = False, keep_first: int = 0, scale: Optional[float] = None,
                 value_dim: Optional[int] = None, gate: bool = False, value_mix: Optional[str] = None,
                 o_bias: bool = False, unit_norm_eps: Optional[float] = None, head_temperature: bool = False,
                 softcap: Optional[float] = None, interleaved_pairs: bool = False,
                 value_unit_norm_eps: Optional[float] = None, unit_sink: bool = False, chunk: Optional[int] = None,
                 pool: Optional[int] = None, fused_prep: bool = False):
        if n_heads % n_kv_heads:
            raise ValueError(f"attention: heads {n_heads} must be a multiple of kv heads {n_kv_heads}")
        self.value_dim = head_dim if value_dim is None else int(value_dim)
        self.padded = head_dim if self.value_dim == head_dim else -(-max(head_dim, self.value_dim) // 16) * 16
        if self.padded > 256 or self.value_dim < 1:
            raise ValueError(f"attention: head_dim {head_dim} is larger than the kernels take (256)" if self.value_dim == head_dim
                             else f"attention: heads of {head_dim} and values of {self.value_dim} are larger than the kernels take (256)")
        if value_mix not in (None, "source", "mixed"):
            raise ValueError(f"attention: value_mix '{value_mix}' is neither 'source' nor 'mixed'")
        if keep_first < 0 or (keep_first and not window):
            raise ValueError("attention: keep_first goes with a window")
        self.hidden_size, self.n_heads, self.n_kv, self.head_dim = hidden_size, n_heads, n_kv_heads, head_dim
        self.window, self.keep_first = window, int(keep_first)
        self.position = position
        self.q_norm, self.k_norm = q_norm, k_norm
        self.has_gate, self.value_mix = bool(gate), value_mix
        self.unit_norm_eps = None if unit_norm_eps is None else float(unit_norm_eps)
        self.has_temperature = bool(head_temperature)
        if self.unit_norm_eps is not None and (q_norm is not None or k_norm is not None):
            raise ValueError("attention: the heads take norm parts or the unit norm, not both")
        if self.has_temperature and self.unit_norm_eps is None:
            raise ValueError("attention: a temperature a head goes with the unit norm of the heads")
        if softcap is not None and not softcap > 0:
            raise ValueError(f"attention: softcap {softcap} must be positive")
        self.softcap = None if softcap is None else float(softcap)
        self.temperature: Optional[torch.Tensor] = None
        self._unit_q = self._unit_k = None  # the unit norm's weights: the temperature (or 1) for q, 1 for k
        self.interleaved_pairs = bool(interleaved_pairs)
        self._reordered = False
        self.value_unit_norm_eps = None if value_unit_norm_eps is None else float(value_unit_norm_eps)
        self.unit_sink = bool(unit_sink)
        if unit_sink and sink:
            raise ValueError("attention: a learned sink or the sink of score 0, not both")
        if chunk is not None and (chunk < 1 or window or keep_first):
            raise ValueError("attention: a chunk is a positive number of positions and goes without a window")
        if pool is not None and (pool < 1 or not window or keep_first):
            raise ValueError("attention: pooled blocks are a positive number of positions and go with a plain window")
        self.chunk, self.pool = chunk, pool
        self.prepared = (self.has_gate or value_mix is not None or self.value_dim != head_dim or self.unit_norm_eps is not None
                         or self.value_unit_norm_eps is not None or pool is not None or bool(fused_prep) or self.interleaved_pairs)
        if self.prepared:
            if position.rotates and getattr(position, "layout", None) != "half":
                raise ValueError("attention: with a gate, mixed values or values of another size the position encoding "
                                 "must be the rotation of the pairs (i, i + rotary_dim / 2), or none")
            if q_norm is not None and k_norm is not None and q_norm.eps != k_norm.eps:
                raise ValueError("attention: the norms of the q and k heads must share their eps")
        self.rot_pairs = (getattr(position, "rotary_dim", 0) // 2) if position.rotates else 0
        self.q_dim, self.kv_dim, self.v_dim = n_heads * head_dim, n_kv_heads * head_dim, n_kv_heads * self.value_dim
        self.qkv = Linear(hidden_size, self.q_dim + self.kv_dim + self.v_dim + (n_heads if gate else 0), bias=qkv_bias)
        self.o = Linear(n_heads * self.value_dim, hidden_size, bias=o_bias)
        self.scale = 1.0 / math.sqrt(head_dim) if scale is None else float(scale)
        self._planner: Optional[AttentionPlanner] = None
        self.has_sink = bool(sink)
        self.sink: Optional[torch.Tensor] = None
        self.value_mix_weight: Optional[torch.Tensor] = None

    def sub_parts(self) -> Dict[str, Part]:
        parts: Dict[str, Part] = {"position": self.position}
        if self.q_norm is not None:
            parts["q_norm"] = self.q_norm
        if self.k_norm is not None:
            parts["k_norm"] = self.k_norm
        return parts

    # parameters -------------------------------------------------------------------------
    def param_decls(self) -> Dict[str, ParamDecl]:
        rows = self.qkv.out_features
        decls = {"qkv_weight": ParamDecl((rows, self.hidden_size)),
                 "o_weight": ParamDecl((self.hidden_size, self.n_heads * self.value_dim))}
        if self.qkv.has_bias:
            # (the gates' rows have no bias in a checkpoint: theirs is zero, added in ``prepare``)
            decls["qkv_bias"] = ParamDecl((rows - (self.n_heads if self.has_gate else 0),), "vector", "bias")
        if self.o.has_bias:
            decls["o_bias"] = ParamDecl((self.hidden_size,), "vector", "bias")
        if self.has_temperature:
            decls["temperature"] = ParamDecl((self.n_heads,), "vector", "norm")
        if self.has_sink:
            decls["sink"] = ParamDecl((self.n_heads,), "vector", "bias")
        if self.value_mix is not None:
            # (the source layer's number exists in checkpoints and is not used)
            decls["value_mix_weight"] = ParamDecl((), "vector", "bias")
        return decls

    qkv_weight = property(lambda s: s.qkv.weight, lambda s, t: setattr(s.qkv, "weight", t))
    qkv_bias = property(lambda s: s.qkv.bias, lambda s, t: setattr(s.qkv, "bias", t))
    o_weight = property(lambda s: s.o.weight, lambda s, t: setattr(s.o, "weight", t))
    o_bias = property(lambda s: s.o.bias, lambda s, t: setattr(s.o, "bias", t))

    def prepare(self, device, compute_dtype) -> None:
        bias = self.qkv.bias
        if self.has_gate and bias is not None and bias.shape[0] == self.qkv.out_features - self.n_heads:
            self.qkv.bias = torch.cat([bias, torch.zeros((self.n_heads,), dtype=bias.dtype, device=bias.device)])
        if self.interleaved_pairs and not self._reordered and self.rot_pairs:
            # neighbours (2i, 2i + 1) of the rotated part become the pairs (i, i + pairs): q and k rows and the head
            # norms' weights alike
            hd, rot = self.head_dim, 2 * self.rot_pairs
            order = torch.cat([torch.arange(0, rot, 2), torch.arange(1, rot, 2), torch.arange(rot, hd)]).to(device)
            heads = torch.arange(self.n_heads + self.n_kv, device=device)
            rows = torch.arange(self.qkv.out_features, device=device)
            rows[:self.q_dim + self.kv_dim] = (heads[:, None] * hd + order[None, :]).reshape(-1)
            self.qkv.weight = self.qkv.weight[rows].contiguous()
            if self.qkv.bias is not None:
                self.qkv.bias = self.qkv.bias[rows[:self.qkv.bias.shape[0]]].contiguous()
            for norm in {id(n): n for n in (self.q_norm, self.k_norm) if n is not None}.values():
                norm.weight = norm.weight[order].contiguous()
            self._reordered = True
        if self.unit_sink:
            self.sink = torch.zeros((self.n_heads,), dtype=torch.float32, device=device)
        if self.unit_norm_eps is not None:
            ones = torch.ones((self.n_heads, self.head_dim), dtype=torch.float32, device=device)
            self._unit_k = ones[0].contiguous()
            self._unit_q = ones if self.temperature is None else (ones * self.temperature.to(device)[:, None]).contiguous()
        copies = bool(self.options.get("weight_copies", True))
        self.o.prepare(copies)
        self.qkv.prepare(copies)  # (read by the product of 17 to 64 rows; the few-rows product with the rotation reads rows)

    def release_optional_memory(self) -> int:
        return self.qkv.drop_copy() + self.o.drop_copy()

    # cache and plan ---------------------------------------------------------------------
    def cache_need(self):
        if self.chunk:
            # (a query reads no key before its chunk's start: the pages a chunk's length back go to the pool again)
            return PagedNeed(self.n_kv, self.padded, self.chunk, 0)
        if self.pool:
            # keys and values of the window (a block's positions stay until its means are made), and the pooled blocks
            return {"tokens": PagedNeed(self.n_kv, self.padded, max(self.window, self.pool), 0),
                    "blocks": PooledNeed(self.n_kv, self.padded, None, 0, self.pool)}
        return PagedNeed(self.n_kv, self.padded, self.window, self.keep_first if self.window else 0)

    def planner(self) -> AttentionPlanner:
        if self._planner is None:
            self._planner = AttentionPlanner(self.n_heads, self.n_kv, self.padded, self.window, self.keep_first,
                                             chunk=self.chunk, pool=self.pool)
        return self._planner

    # compute ----------------------------------------------------------------------------
    def _fused_table(self, ctx) -> Optional[torch.Tensor]:
        """The rotation as a table, if the mixer's fused kernels may stand for bias + rotate + write:
        nothing between the projection and the rotation, and an encoding that is such a rotation
        (or none at all: then the kernels only add the bias and write)."""
        if self.q_norm is not None or self.k_norm is not None or self.head_dim % 8:
            return None
        return self.position.rotation_table(self.head_dim, ctx)

    def _from_sums(self, x: torch.Tensor, ctx, cache, plan, table) -> Optional[torch.Tensor]:
        """Attention of a step of one token a request straight from the q/k/v product's partial sums
        (None: not such a step, or the kernels do not take the sizes)."""
        if not (self.finish_qkv_in_attention and self.sink is None and not self.keep_first and self.softcap is None and table is not None and cache.writes and plan.mfma and plan.single
                and plan.n_small and not plan.n_large and not plan.n_long and x.dtype == torch.bfloat16
                and ops.attention_mfma_qkv_ok(self.head_dim, cache.page_size)):
            return None
        sums = self.qkv.partial_sums(x, few_rows=True)
        if sums is None:
            return None
        out = torch.empty((x.shape[0], self.q_dim), dtype=x.dtype, device=x.device)
        partials = None
        if plan.n_partial:
            partials = torch.empty((plan.n_partial * self.n_heads * (self.head_dim + 2),), dtype=torch.float32,
                                   device=x.device)
        ops.attention_mfma_qkv(sums, self.qkv.bias, table, cache.slots, cache.k_pool, cache.v_pool,
                               cache.block_tables, plan.items, plan.n_small, out, partials, self.n_heads, self.n_kv,
                               self.head_dim, self.window, self.scale, waves=plan.waves)
        if plan.n_merges:
            ops.attention_merge(partials, plan.merges, plan.n_merges, out, self.n_heads, self.head_dim)
        return out

    def _project_rotate_store(self, x: torch.Tensor, ctx, cache, table) -> torch.Tensor:
        """q/k/v [T, (heads + 2 kv heads) head_dim] of which attention reads the q columns: projected,
        with the bias, the head norms and the rotation applied, and k and v written into the cache
        (unless this call only reads another call's cache)."""
        nh, nkv, hd = self.n_heads, self.n_kv, self.head_dim
        store = dict(slots=cache.slots, k_pool=cache.k_pool, v_pool=cache.v_pool,
                     page_size=cache.page_size) if cache.writes else {}
        bias = self.qkv.bias
        if table is not None:
            if x.dtype == torch.bfloat16 and 0 < x.shape[0] <= GEMM_MFMA_SKINNY_BEST_M and x.shape[1] % 8 == 0 and hd % 16 == 0:
                # a few rows of a step that is not one token a request: the projection's own epilogue
                # adds the bias, rotates and stores
                return ops.gemm_mfma_skinny_rope(x, self.qkv.weight, bias, ctx.positions, nh, nkv, hd, None,
                                                 cos_sin=table, **store)
            sums = self.qkv.partial_sums(x)
            if sums is not None:
                # 17 to 128 rows: the engine's product in slices of K, added up by the kernel that rotates
                qkv = torch.empty(sums.shape[1:], dtype=ctx.compute_dtype, device=x.device)
                return ops.rope_kv_write(qkv, ctx.positions, nh, nkv, hd, None, bias=bias, cos_sin=table,
                                         parts=sums, **store)
        qkv = self.qkv(x, skip_bias=True)
        if table is not None:
            return ops.rope_kv_write(qkv, ctx.positions, nh, nkv, hd, None, bias=bias, cos_sin=table, **store)
        # one step after the other
        plain_write = not self.position.rotates and self.q_norm is None and self.k_norm is None
        if bias is not None and not plain_write:
            ops.bias_add(qkv, bias)
            bias = None
        if self.q_norm is not None:
            q = qkv[:, :self.q_dim]
            self.q_norm.plain(q, out=q)
        if self.k_norm is not None:
            k = qkv[:, self.q_dim:self.q_dim + self.kv_dim]
            self.k_norm.plain(k, out=k)
        if self.position.rotates:
            self.position.rotate(qkv, nh, nkv, hd, ctx)
        if store or bias is not None:
            ops.rope_kv_write(qkv, ctx.positions, nh, nkv, hd, None, bias=bias, **store)  # (no rotation: bias, write)
        return qkv

    @property
    def heads_width(self) -> int:
        """Values a token has behind attention, in front of the output projection."""
        return self.n_heads * self.value_dim

    def forward_heads(self, x: torch.Tensor, ctx, cache, out: torch.Tensor, scale: float = 1.0) -> None:
        """``forward`` without the output projection: the heads' results times ``scale`` into ``out`` [T, heads_width]
        (columns of wider rows may do).  For a mixer that runs this one beside another and projects both at once."""
        if not self.prepared:
            raise NotImplementedError("attention: the heads' results alone come from the one-kernel path (fused_prep=True)")
        self._forward_prepared(x, ctx, cache, ctx.plan(self.planner()), heads_out=out, heads_scale=scale)

    def _forward_prepared(self, x: torch.Tensor, ctx, cache, plan, heads_out=None, heads_scale: float = 1.0):
        """Gate, mixed values or values of another size than the keys: the fused projection, one kernel for all
        that stands between it and attention, attention over heads of ``padded`` values, the gate."""
        nh, nkv, hd, vd, pd = self.n_heads, self.n_kv, self.head_dim, self.value_dim, self.padded
        blocks = None
        if self.pool:
            cache, blocks = cache["tokens"], cache["blocks"]
        proj = self.qkv(x)
        k_off, v_off = self.q_dim, self.q_dim + self.kv_dim
        g_off = v_off + self.v_dim
        table = self.position.table(ctx) if self.rot_pairs else None
        other, other_stride = None, 0
        memo = ("attention values", nkv, vd)
        if self.value_mix == "source":
            ctx.memo[memo] = proj[:, v_off:v_off + self.v_dim]  # (a view: the projection lives as long as the step's memo)
        elif self.value_mix == "mixed":
            other = ctx.memo.get(memo)
            if other is None:
                raise RuntimeError("attention: no earlier layer of this step has published values to mix with")
            other_stride = other.stride(0)
        norm = self.q_norm if self.q_norm is not None else self.k_norm
        q_weight = None if self.q_norm is None else self.q_norm.weight
        k_weight = None if self.k_norm is None else self.k_norm.weight
        eps = norm.eps if norm is not None else 0.0
        if self.unit_norm_eps is not None:
            q_weight, k_weight, eps = self._unit_q, self._unit_k, self.unit_norm_eps
        store = dict(slots=cache.slots, k_pool=cache.k_pool, v_pool=cache.v_pool) if cache.writes else {}
        q, gate = ops.attention_prep(proj, 0, k_off, v_off, g_off, nh, nkv, hd, vd, pd, q_weight, k_weight, eps,
                                     self.rot_pairs, table, self.has_gate,
                                     v_other=other, v_other_stride=other_stride,
                                     mix=self.value_mix_weight if other is not None else None,
                                     v_unit_norm_eps=self.value_unit_norm_eps, **store)
        pooled = None
        if blocks is not None:
            if cache.writes and plan.n_pool_jobs:
                ops.pool_blocks(cache.k_pool, cache.v_pool, cache.block_tables, blocks.k_pool, blocks.v_pool,
                                blocks.block_tables, plan.pool_jobs, plan.n_pool_jobs, self.pool)
            pooled = (blocks.k_pool, blocks.v_pool, blocks.block_tables, self.pool)
        out = paged_attention(q, nh * pd, cache, plan, nh, nkv, pd, self.window, self.scale, x.shape[0], sinks=self.sink,
                              share_keys=self.share_keys, softcap=self.softcap, pooled=pooled)
        if heads_out is not None:
            ops.gate_heads(out, pd, vd, nh, gate, out=heads_out, scale=heads_scale)
            return None
        if gate is not None or pd != vd:
            out = ops.gate_heads(out, pd, vd, nh, gate)
        return self.o.for_residual(out, ctx)

    def forward(self, x: torch.Tensor, ctx, cache) -> torch.Tensor:
        plan = ctx.plan(self.planner())
        if self.prepared:
            return self._forward_prepared(x, ctx, cache, plan)
        table = self._fused_table(ctx)
        out = self._from_sums(x, ctx, cache, plan, table)
        if out is not None:
            return self.o.for_residual(out, ctx)
        qkv = self._project_rotate_store(x, ctx, cache, table)
        out = paged_attention(qkv, qkv.shape[1], cache, plan, self.n_heads, self.n_kv, self.head_dim, self.window,
                              self.scale, x.shape[0], sinks=self.sink, share_keys=self.share_keys, softcap=self.softcap)
        return self.o.for_residual(out, ctx)
