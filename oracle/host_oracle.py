"""Pure-Python restatement of the reference's host-side bookkeeping for the paged attention path.

TEST INFRASTRUCTURE ONLY: imported by tests/ (and nothing in the shipped package).  Small-case
integer logic, written to follow the reference's control flow so that each step can be compared
with the cited Rust:

  default_buckets / ReplayBucketPolicy     crates/inference-executor-core/src/replay.rs:1-87
  SplitKVSelector                          crates/inference-backend-metal/src/components/gqa_split_kv.rs:86-156
  build_single_q_kv_splits                 crates/inference-executor-metal/src/attn/gqa/batch_metadata.rs:352-424
  build_tiled_q_kv_splits                  crates/inference-executor-metal/src/attn/gqa/batch_metadata.rs:433-523
  metadata_update                          crates/inference-executor-metal/src/attn/gqa/batch_metadata.rs:192-317
  select_split_kv_variant (+ work model)   crates/inference-executor-metal/src/attn/gqa/mod.rs:64-316
  page_table_start_index                   crates/inference-executor-metal/src/attn/gqa/request_page_table.rs:112-117
  U32IDAllocator                           crates/inference-runtime-core/src/memory/u32_id_allocator.rs:40-173
  DecoderBlocks (L cache lanes, no trie)   crates/inference-runtime-core/src/runtime/decoder/trie_cache/blocks/trie/{api,mod}.rs,
                                           blocks/util.rs, block/mutable_block.rs

Pinned by the reference's own test vectors (see tests/test_host_plan.py, tests/test_runtime_blocks.py).
The allocator's FIFO reuse order comes from crossbeam-queue 0.3.13 `SegQueue` (not in the reference
tree); the reference asserts only counts and bitmaps, so the order is stated here and pinned by this
repo's own known answer.
"""
from collections import deque

U32_MAX = 0xFFFFFFFF
BASE_BUCKETS = [1, 2, 4, 6, 8, 12, 16, 20, 24, 32, 40, 48, 56, 64]


def div_ceil(a, b):
    return -(-a // b)


# ---------------------------------------------------------------- replay buckets


def default_buckets(max_capacity):
    buckets = [b for b in BASE_BUCKETS if b <= max_capacity]
    lower = 64
    while lower < max_capacity:
        step = lower // 4
        for part in range(1, 5):
            candidate = min(lower + step * part, U32_MAX)
            if candidate >= max_capacity:
                return buckets
            buckets.append(candidate)
        lower = min(lower * 2, U32_MAX)
    return buckets


class ReplayBucketPolicy:
    def __init__(self, max_capacity, topology_boundaries=()):
        assert max_capacity > 0, "replay bucket capacity must be positive"
        buckets = default_buckets(max_capacity)
        for boundary in topology_boundaries:
            assert boundary > 0, "replay topology boundary must be positive"
            if 1 < boundary <= max_capacity:
                buckets.append(boundary - 1)
        buckets.append(max_capacity)
        self.max_capacity = max_capacity
        self.buckets = sorted(set(buckets))

    def capacity(self, active):
        assert active > 0, "replay bucket requires active work"
        assert active <= self.max_capacity, "replay active work exceeds capacity"
        return next(b for b in self.buckets if b >= active)


# ---------------------------------------------------------------- variant selection


def next_pow2(v):
    p = 1
    while p < v:
        p <<= 1
    return p


class SplitKVSelector:
    """variant tuples: ("SingleQ", kv_tile, threads, q_head_tile) / ("TiledQ", q_tile, kv_tile, q_head_tile)."""

    def __init__(self, two_byte, head_dim, tokens_per_page, group, dspark_history=False):
        profile = (head_dim, tokens_per_page)
        self.group = group
        self.supports_tiled_q = (not dspark_history and two_byte and profile in ((128, 8), (256, 8), (256, 16))
                                 and group <= 8)
        self.full_group = not dspark_history and profile == (128, 8)
        self.single_tile = next_pow2(max(min(head_dim, 256), 32))
        self.tiled_q_tile, self.tiled_kv_tile = 8, 16
        self.max_q_head_tile = 256 // (self.tiled_q_tile // 8 * 32)

    def single_q(self):
        return ("SingleQ", self.single_tile, self.single_tile, min(self.group, self.max_q_head_tile))

    def max_q_tokens_per_partial_output(self):
        return self.tiled_q_tile if self.supports_tiled_q else 1

    def select(self, num_tokens, num_q_token_tiles):
        assert num_tokens > 0 and 0 < num_q_token_tiles <= num_tokens
        if not self.supports_tiled_q or num_tokens < 2 * num_q_token_tiles:
            return self.single_q()
        desired = div_ceil(self.group, 2) if (not self.full_group and num_tokens < 4 * num_q_token_tiles) \
            else self.group
        return ("TiledQ", self.tiled_q_tile, self.tiled_kv_tile, min(desired, self.max_q_head_tile))


# ---------------------------------------------------------------- split plans


def _greedy(tiles, kv_tile, budget, cost_is_tokens):
    """tiles: list of dicts {len, ctx, n}.  The reference's rescan loop, literally."""
    used = sum(t["len"] if cost_is_tokens else 1 for t in tiles)
    while used < budget:
        best = None
        for i, t in enumerate(tiles):
            cost = t["len"] if cost_is_tokens else 1
            if used + cost > budget:
                continue
            kv_tiles = div_ceil(t["ctx"], kv_tile)
            if t["n"] >= kv_tiles:
                continue
            per_split = div_ceil(kv_tiles, t["n"])
            if best is None or per_split > best[1]:
                best = (i, per_split)
        if best is None:
            break
        t = tiles[best[0]]
        used += t["len"] if cost_is_tokens else 1
        t["n"] += 1
    return tiles


def _emit(tiles, kv_tile):
    kv_splits, cu = [], [0]
    for i, t in enumerate(tiles):
        kv_tiles = div_ceil(t["ctx"], kv_tile)
        for s in range(t["n"]):
            tb, te = kv_tiles * s // t["n"], kv_tiles * (s + 1) // t["n"]
            kv_splits += [i, tb * kv_tile, min(t["ctx"], te * kv_tile)]
        cu.append(len(kv_splits) // 3)
    return kv_splits, cu


def build_single_q_kv_splits(flat_token_indices, kv_tile, max_kv_splits):
    assert flat_token_indices and max_kv_splits >= len(flat_token_indices)
    tiles = [{"len": 1, "ctx": t + 1, "n": 1} for t in flat_token_indices]
    return _emit(_greedy(tiles, kv_tile, max_kv_splits, False), kv_tile)


def q_token_tiles_of(token_indices, cu_tokens, q_tile):
    tiles = []
    for r, start_pos in enumerate(token_indices):
        begin, req_end = cu_tokens[r], cu_tokens[r + 1]
        while begin < req_end:
            end = begin + min(req_end - begin, q_tile)
            tiles.append({"begin": begin, "end": end, "len": end - begin, "ctx": start_pos + (end - cu_tokens[r]),
                          "n": 1})
            begin = end
    return tiles


def build_tiled_q_kv_splits(token_indices, cu_tokens, q_tile, kv_tile, max_partial_tokens):
    tiles = q_token_tiles_of(token_indices, cu_tokens, q_tile)
    assert tiles and sum(t["len"] for t in tiles) <= max_partial_tokens
    _greedy(tiles, kv_tile, max_partial_tokens, True)
    q_token_tiles = [v for t in tiles for v in (t["begin"], t["end"])]
    kv_splits, cu = _emit(tiles, kv_tile)
    return q_token_tiles, kv_splits, cu


def metadata_update(max_tokens, req_slots, token_indices, cu_tokens, variant, mode="exact", caller_tokens=0,
                    boundaries=()):
    """Returns dict(req_slots, flat_token_indices, q_token_tiles, kv_splits (padded), cu_kv_splits, shape)."""
    assert len(req_slots) == len(token_indices) and len(cu_tokens) == len(req_slots) + 1 and cu_tokens[0] == 0
    for r in range(len(req_slots)):
        assert cu_tokens[r] <= cu_tokens[r + 1], "GQA batch cu_tokens must be nondecreasing"
        assert token_indices[r] + (cu_tokens[r + 1] - cu_tokens[r]) <= U32_MAX
    num_tokens = cu_tokens[-1]
    assert 0 < num_tokens <= max_tokens
    if mode == "caller":
        assert num_tokens <= caller_tokens, "GQA active token count must not exceed the caller-owned token capacity"
        assert caller_tokens <= max_tokens, "GQA caller-owned token capacity must not exceed the metadata capacity"
    slots_by_token, flat = [], []
    for r in range(len(req_slots)):
        for i in range(cu_tokens[r + 1] - cu_tokens[r]):
            slots_by_token.append(req_slots[r])
            flat.append(token_indices[r] + i)
    tiled = variant[0] == "TiledQ"
    if tiled:
        q_tiles, kv_splits, cu = build_tiled_q_kv_splits(token_indices, cu_tokens, variant[1], variant[2], max_tokens)
        num_tiles = len(q_tiles) // 2
    else:
        q_tiles = []
        kv_splits, cu = build_single_q_kv_splits(flat, variant[1], max_tokens)
        num_tiles = num_tokens
    num_splits = len(kv_splits) // 3
    if mode == "exact":
        totals = (num_tokens, num_tiles, min(next_pow2(num_splits), max_tokens))
    else:
        plain = ReplayBucketPolicy(max_tokens)
        tokens_policy = ReplayBucketPolicy(max_tokens, boundaries)
        total_tokens = tokens_policy.capacity(num_tokens) if mode == "bucketed" else caller_tokens
        totals = (total_tokens, plain.capacity(num_tiles), plain.capacity(num_splits))
    kv_splits = kv_splits + [U32_MAX] * (3 * (totals[2] - num_splits))
    shape = (num_tokens, totals[0], num_tiles, totals[1], num_splits, totals[2], tiled or num_splits > num_tokens)
    return dict(req_slots=slots_by_token, flat_token_indices=flat, q_token_tiles=q_tiles, kv_splits=kv_splits,
                cu_kv_splits=cu, shape=shape)


def fixed_partition_splits(flat_token_indices, partition):
    kv_splits, cu = [], [0]
    for i, t in enumerate(flat_token_indices):
        ctx = t + 1
        for s in range(div_ceil(ctx, partition)):
            kv_splits += [i, s * partition, min(ctx, (s + 1) * partition)]
        cu.append(len(kv_splits) // 3)
    return kv_splits, cu


# ---------------------------------------------------------------- batch selector (attn/gqa/mod.rs)


def _padded_kv_splits(num_kv_splits, max_tokens, policy):
    if policy is not None:
        return policy.capacity(num_kv_splits)
    return min(next_pow2(num_kv_splits), max_tokens)


def _selection_work(tiles, kv_tile, scheduled_q_tokens, blocks_per_split, waves_per_block, max_tokens, policy):
    assert tiles
    active = sum(t["len"] for t in tiles)
    assert active <= max_tokens
    while active < max_tokens:
        candidates = [(div_ceil(div_ceil(t["ctx"], kv_tile), t["n"]), -i, i) for i, t in enumerate(tiles)
                      if active + t["len"] <= max_tokens and t["n"] < div_ceil(t["ctx"], kv_tile)]
        if not candidates:
            break
        i = max(candidates)[2]
        active += tiles[i]["len"]
        tiles[i]["n"] += 1
    num_splits = sum(t["n"] for t in tiles)
    scheduled = sum(div_ceil(t["ctx"], kv_tile) * kv_tile * scheduled_q_tokens for t in tiles)
    active_work = sum(div_ceil(t["ctx"], kv_tile) * kv_tile * t["len"] for t in tiles)
    blocks = num_splits * blocks_per_split
    return dict(num_kv_splits=num_splits, scheduled_map_work=scheduled, active_map_work=active_work,
                bookkeeping=blocks + blocks * waves_per_block + active +
                _padded_kv_splits(num_splits, max_tokens, policy) * scheduled_q_tokens,
                active_partial_states=active,
                padded_replay_work=_padded_kv_splits(num_splits, max_tokens, policy) * scheduled_q_tokens)


def tiled_q_selection_work(variant, q_heads_per_kv_head, max_tokens, policy, token_indices, cu_tokens):
    _, q_tile, kv_tile, q_head_tile = variant
    tiles = q_token_tiles_of(token_indices, cu_tokens, q_tile)
    return _selection_work(tiles, kv_tile, q_tile, div_ceil(q_heads_per_kv_head, q_head_tile),
                           q_tile // 8 * q_head_tile, max_tokens, policy)


def select_split_kv_variant(selector, use_d256_page8_selector, max_tokens, bucket_max_tokens, token_indices,
                            cu_tokens):
    assert len(cu_tokens) == len(token_indices) + 1 and cu_tokens[0] == 0
    num_tokens = cu_tokens[-1]
    assert num_tokens > 0
    num_tiles = sum(div_ceil(cu_tokens[r + 1] - cu_tokens[r], selector.tiled_q_tile)
                    for r in range(len(token_indices)))
    candidate = selector.select(num_tokens, num_tiles)
    if not use_d256_page8_selector or candidate[0] != "TiledQ":
        return candidate
    single = selector.select(num_tokens, num_tokens)
    policy = ReplayBucketPolicy(bucket_max_tokens) if bucket_max_tokens else None
    flat_ctx = [token_indices[r] + i + 1 for r in range(len(token_indices))
                for i in range(cu_tokens[r + 1] - cu_tokens[r])]
    single_tiles = [{"len": 1, "ctx": c, "n": 1} for c in flat_ctx]
    single_work = _selection_work(single_tiles, single[1], 1, 1, single[2] // 32, max_tokens, policy)
    tiled_work = tiled_q_selection_work(candidate, single[3], max_tokens, policy, token_indices, cu_tokens)
    complete = sum(flat_ctx) + min(single_work["bookkeeping"], tiled_work["bookkeeping"])
    enough = tiled_work["active_map_work"] * 2 >= tiled_work["scheduled_map_work"]
    return candidate if (enough and complete >= 2048) else single


# ---------------------------------------------------------------- page table


def page_table_start_index(layout, req_slot, layer, block):
    slots, layers, blocks, ids = layout
    assert req_slot < slots and layer < layers and block < blocks
    return ((req_slot * layers + layer) * blocks + block) * ids


def page_ids_by_layer(block_ids, num_layers, ids_per_block):
    assert len(block_ids) == num_layers * ids_per_block
    return [list(block_ids[l * ids_per_block:(l + 1) * ids_per_block]) for l in range(num_layers)]


# ---------------------------------------------------------------- page-ID allocator


class ResourceExhausted(Exception):
    pass


class U32IDAllocator:
    def __init__(self, capacity):
        assert capacity <= U32_MAX
        self._capacity, self.counter = capacity, 0
        self.free_ids = deque()
        self.bitmap = [0] * div_ceil(capacity, 64)

    def _mark(self, i, allocated):
        assert i < self._capacity, "U32 ID allocator ID is out of range"
        word, mask = i >> 6, 1 << (i & 63)
        assert bool(self.bitmap[word] & mask) != allocated
        self.bitmap[word] ^= mask

    def alloc_one(self):
        if self.free_ids:
            i = self.free_ids.popleft()
        elif self.counter < self._capacity:
            i, self.counter = self.counter, self.counter + 1
        else:
            raise ResourceExhausted("not enough ID")
        self._mark(i, True)
        return i

    def alloc_many(self, count):
        ids = []
        while len(ids) < count and self.free_ids:
            ids.append(self.free_ids.popleft())
        rest = count - len(ids)
        if rest:
            if self.counter + rest > self._capacity:
                for i in ids:
                    self.free_ids.append(i)  # popped IDs go back to the tail, as the reference does
                raise ResourceExhausted("not enough ID")
            ids += list(range(self.counter, self.counter + rest))
            self.counter += rest
        for i in ids:
            self._mark(i, True)
        return ids

    def free_many(self, ids):
        for i in ids:
            self._mark(i, False)
            self.free_ids.append(i)

    def free_one(self, i):
        self.free_many([i])

    def free(self):
        return len(self.free_ids) + max(self._capacity - self.counter, 0)

    def used(self):
        return self._capacity - self.free()

    def capacity(self):
        return self._capacity


# ---------------------------------------------------------------- decoder blocks (token window state machine)


class Block:
    """`MutableBlock<N>` (block/mutable_block.rs:13-167); a full block keeps the same bookkeeping
    after it is committed (kind "immutable") -- without a trie nothing else distinguishes it."""

    def __init__(self, n, page_ids, kind="mutable"):
        self.n, self.page_ids, self.kind = n, page_ids, kind
        self.tokens, self.scheduled_index, self.ready_index = [], 0, 0

    cached = property(lambda s: s.tokens[:s.scheduled_index])
    scheduled = property(lambda s: s.tokens[s.scheduled_index:s.ready_index])
    ready = property(lambda s: s.tokens[s.ready_index:])

    def ready_token_slots(self):
        return self.n - self.ready_index

    def push_tokens(self, tokens):
        size = min(self.n - len(self.tokens), len(tokens))
        self.tokens += tokens[:size]
        return tokens[size:]

    def schedule_tokens(self, num):
        num = min(num, len(self.tokens) - self.ready_index)
        out = self.tokens[self.ready_index:self.ready_index + num]
        self.ready_index += num
        return out

    def unschedule_tokens(self, tokens):
        assert self.tokens[self.ready_index - len(tokens):self.ready_index] == tokens
        self.ready_index -= len(tokens)

    def cache_tokens(self, tokens):
        assert self.tokens[self.scheduled_index:self.scheduled_index + len(tokens)] == tokens
        self.scheduled_index += len(tokens)


class DecoderBlocks:
    """`TrieDecoderBlocks<N, P, L, BC>` without prefix sharing: every logical block owns its pages;
    a committed full block becomes immutable with the pages it already had (the reference's
    `CommitMultiLaneMutableBlockResult::Immutable` outcome); lookups never hit.  A full block of
    queued tokens reserved at init time goes to the semi-immutable list, as the reference does on
    a cache miss (trie/api.rs:67-129)."""

    def __init__(self, n, lanes, allocator, pages_per_kv_block, tokens):
        assert tokens and lanes - 1 <= len(tokens)
        self.n, self.lanes, self.alloc, self.ppb = n, lanes, allocator, pages_per_kv_block
        self.immutable, self.semi_immutable, self.mutable = [], deque(), deque()
        self.queued = deque(tokens)
        self.spec_tokens = []
        self.num_in_sync_blocks = 0
        self.epoch = 0

    # -- views over lane 0
    def _all(self):
        return list(self.immutable) + list(self.semi_immutable) + list(self.mutable)

    def cached_tokens(self):
        return [t for b in self._all() for t in b[0].cached]

    def scheduled_tokens(self):
        return [t for b in list(self.semi_immutable) + list(self.mutable) for t in b[0].scheduled]

    def ready_tokens(self):
        return [t for b in list(self.semi_immutable) + list(self.mutable) for t in b[0].ready]

    def queued_tokens(self):
        return list(self.queued)

    def state(self):
        return (self.num_in_sync_blocks, self.cached_tokens(), self.scheduled_tokens(), self.ready_tokens(),
                self.queued_tokens(), list(self.spec_tokens))

    def block_counts(self):
        return len(self.immutable), len(self.semi_immutable), len(self.mutable)

    def ready_token_slots(self):
        return sum(b[0].ready_token_slots() for b in list(self.semi_immutable) + list(self.mutable))

    # -- helpers (blocks/util.rs)
    def _pop_front_queued(self, num):
        num = min(len(self.queued) - (self.lanes - 1), num)
        tokens = [self.queued[i] for i in range(num + self.lanes - 1)]  # the head of the deque: O(num)
        for _ in range(num):
            self.queued.popleft()
        return tokens

    def _push_front_queued(self, tokens, lanes):
        for t in reversed(tokens[:len(tokens) - (lanes - 1)] if lanes > 1 else tokens):
            self.queued.appendleft(t)

    def _push_tokens(self, block_vec, tokens):
        if not tokens:
            return
        window = len(tokens) - (self.lanes - 1)
        for lane, block in enumerate(block_vec):
            assert block.push_tokens(tokens[lane:lane + window]) == []

    def _alloc_block_vec(self, kind):
        """Lanes in index order, each lane's KV pages from the shared allocator; on failure the
        lanes already allocated are released in index order (cache/multi_lane_impl.rs:57-79).
        The reference also draws state pages per lane after the KV pages; the attention path has
        none, so that draw is a zero-length allocation here."""
        got = []
        try:
            for _ in range(self.lanes):
                got.append(self.alloc.alloc_many(self.ppb))
        except ResourceExhausted:
            for ids in got:
                self.alloc.free_many(ids)
            return None
        return [Block(self.n, ids, kind) for ids in got]

    def _free_block_vec(self, block_vec):
        for block in block_vec:
            self.alloc.free_many(block.page_ids)

    # -- trie/api.rs:48-136
    def init_block_once(self):
        cachable = max(len(self.queued) - (self.lanes - 1), 0)
        num = min(cachable, self.n)
        tokens = self._pop_front_queued(num) if num else []
        use_cache = num == self.n and len(self.queued) > 0 and not self.mutable and not self.semi_immutable
        block_vec = self._alloc_block_vec("semi_immutable" if use_cache else "mutable")
        if block_vec is None:
            self._push_front_queued(tokens, self.lanes)
            return "ResourceLimitExceeded"
        self._push_tokens(block_vec, tokens)
        (self.semi_immutable if use_cache else self.mutable).append(block_vec)
        return self.ready_token_slots()

    # -- trie/api.rs:138-153
    def uninit_block_once(self):
        for blocks in (self.mutable, self.semi_immutable):
            if blocks:
                block_vec = blocks.pop()
                self._push_front_queued(list(block_vec[0].tokens), 1)
                self._free_block_vec(block_vec)
                return len(self.cached_tokens())
        if self.immutable:
            # The reference leaves an immutable block's pages with the prefix trie (unpinned, to be
            # evicted later); with no trie the pages go straight back to the allocator.
            block_vec = self.immutable.pop()
            self._push_front_queued(list(block_vec[0].tokens), 1)
            self._free_block_vec(block_vec)
        return len(self.cached_tokens())

    # -- trie/api.rs:184-273
    def prepare(self, budget):
        assert 0 < budget <= self.ready_token_slots()
        validated = len(self.ready_tokens()) + len(self.queued)
        assert validated != 0
        if budget < validated:
            # implied by the reference's debug assertions (tokens.len() == budget; lanes' windows line up)
            num_ready = len(self.ready_tokens())
            assert budget <= num_ready, "prefill chunk must fit in the ready tokens"
            assert self.lanes == 1 or budget == num_ready, \
                "prefill chunk must take every ready token when L > 1 (the lookahead comes from the queue)"
        token_index, block_index, tokens = None, len(self.immutable), []
        for block_vec in list(self.semi_immutable) + list(self.mutable):
            main = block_vec[0]
            if len(main.ready) == 0:
                block_index += 1
                continue
            if token_index is None:
                token_index = block_index * self.n + len(main.cached) + len(main.scheduled)
            take = min(len(main.ready), budget - len(tokens))
            for lane_block in block_vec[1:]:
                lane_block.schedule_tokens(take)
            tokens += main.schedule_tokens(take)
            if len(tokens) >= budget:
                break
            block_index += 1
        if budget < validated:
            tokens += list(self.queued)[:self.lanes - 1]
            return ("Prefill", self.epoch, token_index, tokens, budget)
        assert len(self.queued) < self.lanes
        tokens += list(self.queued)
        selected = budget - len(tokens)
        assert selected <= len(self.spec_tokens)
        del self.spec_tokens[selected:]
        if token_index is None:
            token_index = len(self.cached_tokens()) + len(self.scheduled_tokens())
        return ("Decode", self.epoch, token_index, tokens, list(self.spec_tokens))

    # -- trie/api.rs:276-331
    def cancel(self, query):
        tokens = query[3]
        index_end = max(len(tokens) - (self.lanes - 1), 0)
        for block_vec in list(reversed(self.mutable)) + list(reversed(self.semi_immutable)):
            if index_end == 0:
                break
            index_start = index_end - min(index_end, len(block_vec[0].scheduled))
            if index_start != index_end:
                for lane, block in enumerate(block_vec):
                    count = index_end - index_start
                    scheduled = block.scheduled[len(block.scheduled) - count:]
                    assert tokens[index_start + lane:index_end + lane] == scheduled
                    block.unschedule_tokens(scheduled)
            index_end = index_start
        assert index_end == 0

    def _cache(self, block_vec, tokens, start, end):
        if start == end:
            return
        for lane, block in enumerate(block_vec):
            scheduled = block.scheduled[:end - start]
            assert tokens[start + lane:end + lane] == scheduled
            block.cache_tokens(scheduled)

    def _commit_full(self, block_vec):
        for block in block_vec:
            block.kind = "immutable"
        self.immutable.append(block_vec)

    # -- trie/api.rs:334-549
    def commit(self, query, sampled):
        kind, _, _, input_tokens = query[0], query[1], query[2], query[3]
        lm1 = self.lanes - 1
        if kind == "Prefill":
            ready_to_cached, ready_window = input_tokens, max(len(input_tokens) - lm1, 0)
            queued_to_cached, queued_window = input_tokens[max(len(input_tokens) - lm1, 0):], 0
        else:
            validated, sampled_token, new_spec = sampled
            assert query[4][:len(validated)] == validated, \
                "validated tokens must equal a prefix of the speculative input suffix"
            ready_window = max(len(input_tokens) - lm1, 0)
            queued_window = min(len(input_tokens) + len(validated),
                                max(len(input_tokens) + len(validated) + 1 - lm1, 0)) - ready_window
            self.queued.extend(validated)
            self.queued.append(sampled_token)
            for _ in range(queued_window):
                self.queued.popleft()
            self.spec_tokens = list(new_spec)
            ready_to_cached = input_tokens
            queued_to_cached = input_tokens[max(len(input_tokens) - lm1, 0):] + list(validated) + [sampled_token]
        index_start = 0
        done = False
        for blocks in (self.semi_immutable, self.mutable):
            while blocks and not done:
                block_vec = blocks.popleft()
                index_end = index_start + min(ready_window - index_start, len(block_vec[0].scheduled))
                self._cache(block_vec, ready_to_cached, index_start, index_end)
                index_start = index_end
                if len(block_vec[0].cached) != self.n:
                    blocks.appendleft(block_vec)
                    done = True
                else:
                    self._commit_full(block_vec)
            if done:
                break
        extra_start = 0
        while self.mutable:
            block_vec = self.mutable.popleft()
            num = min(queued_window - extra_start, self.n - len(block_vec[0].tokens))
            extra_end = extra_start + num
            if extra_start != extra_end:
                self._push_tokens(block_vec, queued_to_cached[extra_start:extra_end + lm1])
                for block in block_vec:
                    block.schedule_tokens(num)
                self._cache(block_vec, queued_to_cached, extra_start, extra_end)
            extra_start = extra_end
            if len(block_vec[0].cached) != self.n:
                self.mutable.appendleft(block_vec)
                break
            self._commit_full(block_vec)
        self._try_mark_ready()
        assert index_start == ready_window and extra_start == queued_window

    def _try_mark_ready(self):
        cachable = max(len(self.queued) - (self.lanes - 1), 0)
        for block_vec in self.mutable:
            if cachable == 0:
                break
            if len(block_vec[0].tokens) == self.n:
                continue
            num = min(cachable, self.n - len(block_vec[0].tokens))
            cachable -= num
            self._push_tokens(block_vec, self._pop_front_queued(num))

    # -- trie/mod.rs:176-229
    def prepare_blocks(self):
        start = self.num_in_sync_blocks
        blocks = self._all()
        kv_page_ids = [[list(b[lane].page_ids) for b in blocks[start:]] for lane in range(self.lanes)]
        self.num_in_sync_blocks = len(blocks)
        return (start, kv_page_ids)

    def cancel_blocks(self, sync_blocks):
        self.num_in_sync_blocks = sync_blocks[0]

    def drop(self):
        for block_vec in list(reversed(self.mutable)) + list(reversed(self.semi_immutable)):
            self._free_block_vec(block_vec)
        for block_vec in reversed(self.immutable):
            self._free_block_vec(block_vec)  # no trie to keep them
        self.mutable.clear()
        self.semi_immutable.clear()
        self.immutable.clear()
