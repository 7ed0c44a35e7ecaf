// Host-side planning of a GQA batch: replay capacity buckets, SplitKV variant selection and the
// per-batch metadata (per-token slots/positions, Q-token tiles, KV splits).  Pure integer logic,
// no device work.  Follows
//   crates/inference-executor-core/src/replay.rs:4-87                      (buckets)
//   crates/inference-backend-metal/src/components/gqa_split_kv.rs:86-156   (variant geometry)
//   crates/inference-executor-metal/src/attn/gqa/mod.rs:64-316             (batch selector)
//   crates/inference-executor-metal/src/attn/gqa/batch_metadata.rs:192-523 (metadata + split plans)
#include <algorithm>
#include <functional>
#include <queue>

#include "split_kv.h"

namespace psi {

// ---------------------------------------------------------------- replay buckets (replay.rs)

static const uint32_t kBaseBuckets[] = {1, 2, 4, 6, 8, 12, 16, 20, 24, 32, 40, 48, 56, 64};

struct BucketPolicy {
    uint32_t max_capacity = 0;
    std::vector<uint32_t> buckets;

    // First bucket that holds `active` (replay.rs:56-61).
    int capacity(uint32_t active, uint32_t* out) const {
        PSI_REQUIRE(active > 0, "replay bucket requires active work");
        PSI_REQUIRE(active <= max_capacity, "replay active work exceeds capacity");
        *out = *std::lower_bound(buckets.begin(), buckets.end(), active);
        return PSI_HIP_OK;
    }
};

static int make_bucket_policy(uint32_t max_capacity, const uint32_t* boundaries, uint32_t num_boundaries,
                              BucketPolicy* policy) {
    PSI_REQUIRE(max_capacity > 0, "replay bucket capacity must be positive");
    std::vector<uint32_t>& b = policy->buckets;
    b.clear();
    for (uint32_t base : kBaseBuckets)
        if (base <= max_capacity) b.push_back(base);
    // Above 64: quarters of each power-of-two interval, stopping before max_capacity (replay.rs:69-87).
    bool done = false;
    for (uint64_t lower = 64; !done && lower < max_capacity; lower *= 2) {
        const uint64_t step = lower / 4;
        for (uint64_t part = 1; part <= 4; ++part) {
            const uint64_t candidate = std::min<uint64_t>(lower + step * part, UINT32_MAX);
            if (candidate >= max_capacity) {
                done = true;
                break;
            }
            b.push_back((uint32_t)candidate);
        }
    }
    for (uint32_t i = 0; i < num_boundaries; ++i) {
        PSI_REQUIRE(boundaries[i] > 0, "replay topology boundary must be positive");
        if (boundaries[i] > 1 && boundaries[i] <= max_capacity) b.push_back(boundaries[i] - 1);
    }
    b.push_back(max_capacity);
    std::sort(b.begin(), b.end());
    b.erase(std::unique(b.begin(), b.end()), b.end());
    policy->max_capacity = max_capacity;
    return PSI_HIP_OK;
}

// ---------------------------------------------------------------- variant geometry (gqa_split_kv.rs)

struct SplitKVSelector {
    uint32_t group;
    bool supports_tiled_q;
    bool full_group_for_tiled_q;
    uint32_t single_q_tile;  // = threads per threadblock
    uint32_t tiled_q_token_tile = 8;
    uint32_t tiled_kv_token_tile = 16;
    uint32_t max_q_head_tile;

    psi_hip_split_kv_variant single_q() const {
        psi_hip_split_kv_variant v{};
        v.kind = PSI_HIP_VARIANT_SINGLE_Q;
        v.q_token_tile_size = 1;
        v.kv_token_tile_size = single_q_tile;
        v.num_threads_per_threadblock = single_q_tile;
        v.q_head_tile_size = std::min(group, max_q_head_tile);
        return v;
    }

    int select(uint32_t num_tokens, uint32_t num_q_token_tiles, psi_hip_split_kv_variant* out) const {
        PSI_REQUIRE(num_tokens > 0, "GQA SplitKV selection requires tokens");
        PSI_REQUIRE(num_q_token_tiles > 0 && num_q_token_tiles <= num_tokens,
                    "GQA SplitKV selection requires 0 < q_token_tiles <= tokens");
        if (!supports_tiled_q || (uint64_t)num_tokens < 2ull * num_q_token_tiles) {
            *out = single_q();
            return PSI_HIP_OK;
        }
        const uint32_t desired = (!full_group_for_tiled_q && (uint64_t)num_tokens < 4ull * num_q_token_tiles)
                                     ? (group + 1) / 2
                                     : group;
        psi_hip_split_kv_variant v{};
        v.kind = PSI_HIP_VARIANT_TILED_Q;
        v.q_token_tile_size = tiled_q_token_tile;
        v.kv_token_tile_size = tiled_kv_token_tile;
        v.num_threads_per_threadblock = 0;
        v.q_head_tile_size = std::min(desired, max_q_head_tile);
        *out = v;
        return PSI_HIP_OK;
    }
};

static uint32_t next_pow2_u32(uint32_t v) {
    uint32_t p = 1;
    while (p < v) p <<= 1;
    return p;
}

static int make_selector(const psi_hip_gqa_config* cfg, bool dspark_history, SplitKVSelector* sel,
                         Geometry* geometry_out = nullptr) {
    Geometry g;
    int rc = make_geometry(cfg, &g);
    if (rc != PSI_HIP_OK) return rc;
    // The reference's attention kernels accept f32 and bf16 only; f16 shares the bf16 geometry here.
    const bool two_byte = g.dtype != PSI_HIP_F32;
    const bool profile = (g.d == 128 && g.tokens_per_page == 8) ||
                         (g.d == 256 && (g.tokens_per_page == 8 || g.tokens_per_page == 16));
    sel->group = g.group;
    sel->supports_tiled_q = !dspark_history && two_byte && profile && g.group <= 8;
    sel->full_group_for_tiled_q = !dspark_history && g.d == 128 && g.tokens_per_page == 8;
    sel->single_q_tile = next_pow2_u32(std::max(std::min(g.d, 256u), 32u));
    sel->max_q_head_tile = 256 / (sel->tiled_q_token_tile / 8 * 32);
    if (geometry_out) *geometry_out = g;
    return PSI_HIP_OK;
}

// ---------------------------------------------------------------- split plans (batch_metadata.rs)

struct QTile {
    uint32_t flat_begin, flat_end, context_len;
    uint64_t num_splits;
};

static inline uint64_t div_ceil_u64(uint64_t a, uint64_t b) { return (a + b - 1) / b; }

// Greedy budgeted split count assignment shared by both variants (batch_metadata.rs:364-386 and
// :466-488): repeatedly give one more split to the tile whose splits currently span the most KV
// tiles; ties go to the lowest tile index; a tile is skipped when its partial-state cost no longer
// fits.  `cost(tile)` is 1 for SingleQ and the tile's token count for TiledQ.
static void assign_greedy_splits(std::vector<QTile>& tiles, uint32_t kv_tile, uint64_t budget, bool cost_is_tokens) {
    uint64_t used = 0;
    for (auto& t : tiles) used += cost_is_tokens ? (t.flat_end - t.flat_begin) : 1;
    // Max-heap on (kv tiles per split, lowest index first).  Popping the best candidate, bumping it
    // and pushing it back reproduces the reference's full rescan: priorities of other tiles do not
    // change between steps, and a tile rejected for cost can never fit later (the budget only shrinks).
    struct Entry {
        uint64_t per_split;
        uint32_t index;
        bool operator<(const Entry& o) const {
            return per_split != o.per_split ? per_split < o.per_split : index > o.index;
        }
    };
    std::priority_queue<Entry> heap;
    auto kv_tiles = [&](const QTile& t) { return div_ceil_u64(t.context_len, kv_tile); };
    for (uint32_t i = 0; i < tiles.size(); ++i)
        if (tiles[i].num_splits < kv_tiles(tiles[i])) heap.push({div_ceil_u64(kv_tiles(tiles[i]), tiles[i].num_splits), i});
    while (used < budget && !heap.empty()) {
        const Entry e = heap.top();
        heap.pop();
        QTile& t = tiles[e.index];
        const uint64_t cost = cost_is_tokens ? (t.flat_end - t.flat_begin) : 1;
        if (used + cost > budget) continue;  // cannot fit now or later
        t.num_splits += 1;
        used += cost;
        if (t.num_splits < kv_tiles(t)) heap.push({div_ceil_u64(kv_tiles(t), t.num_splits), e.index});
    }
}

static int emit_splits(const std::vector<QTile>& tiles, uint32_t kv_tile, std::vector<uint32_t>* kv_splits,
                       std::vector<uint32_t>* cu) {
    kv_splits->clear();
    cu->assign(1, 0u);
    for (uint32_t i = 0; i < tiles.size(); ++i) {
        const QTile& t = tiles[i];
        const uint64_t n_tiles = div_ceil_u64(t.context_len, kv_tile);
        for (uint64_t s = 0; s < t.num_splits; ++s) {
            const uint64_t tb = n_tiles * s / t.num_splits, te = n_tiles * (s + 1) / t.num_splits;
            const uint64_t begin = tb * kv_tile, end = te * kv_tile;
            PSI_REQUIRE(begin <= UINT32_MAX, "GQA map KV split KV-token begin must fit u32");
            PSI_REQUIRE(end <= UINT32_MAX, "GQA map KV split KV-token end must fit u32");
            kv_splits->push_back(i);
            kv_splits->push_back((uint32_t)begin);
            kv_splits->push_back(std::min(t.context_len, (uint32_t)end));
        }
        PSI_REQUIRE(kv_splits->size() / 3 <= UINT32_MAX, "GQA map KV split count must fit u32");
        cu->push_back((uint32_t)(kv_splits->size() / 3));
    }
    return PSI_HIP_OK;
}

static std::vector<QTile> single_q_tiles(const std::vector<uint32_t>& flat_token_indices) {
    std::vector<QTile> tiles;
    tiles.reserve(flat_token_indices.size());
    for (uint32_t i = 0; i < flat_token_indices.size(); ++i)
        tiles.push_back({i, i + 1, flat_token_indices[i] + 1, 1});
    return tiles;
}

// Request-local chunks of at most q_tile tokens (batch_metadata.rs:443-461).
static std::vector<QTile> tiled_q_tiles(const uint32_t* token_indices, const uint32_t* cu_tokens, uint32_t num_reqs,
                                        uint32_t q_tile) {
    std::vector<QTile> tiles;
    for (uint32_t r = 0; r < num_reqs; ++r) {
        uint32_t begin = cu_tokens[r];
        const uint32_t req_end = cu_tokens[r + 1];
        while (begin < req_end) {
            const uint32_t end = begin + std::min(req_end - begin, q_tile);
            tiles.push_back({begin, end, token_indices[r] + (end - cu_tokens[r]), 1});
            begin = end;
        }
    }
    return tiles;
}

// ---------------------------------------------------------------- batch selector (attn/gqa/mod.rs)

struct SelectionWork {
    uint64_t num_kv_splits, scheduled_map_work, active_map_work, map_blocks_per_kv_head, map_waves_per_kv_head,
        active_partial_states, padded_replay_work;
    uint64_t bookkeeping() const {
        return map_blocks_per_kv_head + map_waves_per_kv_head + active_partial_states + padded_replay_work;
    }
};

static int padded_kv_splits(uint64_t num_kv_splits, uint32_t max_tokens, const BucketPolicy* policy, uint64_t* out) {
    if (policy) {
        uint32_t cap;
        PSI_REQUIRE(num_kv_splits <= UINT32_MAX, "GQA active KV-split count must fit u32");
        int rc = policy->capacity((uint32_t)num_kv_splits, &cap);
        if (rc != PSI_HIP_OK) return rc;
        *out = cap;
        return PSI_HIP_OK;
    }
    uint64_t p = 1;
    while (p < num_kv_splits) p <<= 1;
    *out = std::min<uint64_t>(p, max_tokens);
    return PSI_HIP_OK;
}

// mod.rs:221-274: the same greedy loop as the metadata builder, priced in partial-state tokens.
static int selection_work(std::vector<QTile> tiles, uint32_t kv_tile, uint32_t scheduled_q_tokens,
                          uint32_t map_blocks_per_split, uint32_t waves_per_map_block, uint32_t max_tokens,
                          const BucketPolicy* policy, SelectionWork* out) {
    PSI_REQUIRE(!tiles.empty(), "GQA SplitKV selection requires tiles");
    uint64_t active = 0;
    for (auto& t : tiles) active += t.flat_end - t.flat_begin;
    PSI_REQUIRE(active <= max_tokens, "GQA SplitKV selection tokens exceed max_tokens");
    assign_greedy_splits(tiles, kv_tile, max_tokens, true);
    SelectionWork w{};
    for (auto& t : tiles) {
        const uint64_t n_tiles = div_ceil_u64(t.context_len, kv_tile);
        w.num_kv_splits += t.num_splits;
        w.scheduled_map_work += n_tiles * ((uint64_t)kv_tile * scheduled_q_tokens);
        w.active_map_work += n_tiles * ((uint64_t)kv_tile * (t.flat_end - t.flat_begin));
        w.active_partial_states += (uint64_t)(t.flat_end - t.flat_begin) * t.num_splits;
    }
    w.map_blocks_per_kv_head = w.num_kv_splits * map_blocks_per_split;
    w.map_waves_per_kv_head = w.map_blocks_per_kv_head * waves_per_map_block;
    uint64_t padded;
    int rc = padded_kv_splits(w.num_kv_splits, max_tokens, policy, &padded);
    if (rc != PSI_HIP_OK) return rc;
    w.padded_replay_work = padded * scheduled_q_tokens;
    *out = w;
    return PSI_HIP_OK;
}

static int check_batch(const uint32_t* token_indices, const uint32_t* cu_tokens, uint32_t num_reqs) {
    PSI_REQUIRE(token_indices && cu_tokens, "GQA batch arrays must not be null");
    PSI_REQUIRE(cu_tokens[0] == 0, "GQA batch cu_tokens must start at zero");
    for (uint32_t r = 0; r < num_reqs; ++r) {
        PSI_REQUIRE(cu_tokens[r] <= cu_tokens[r + 1], "GQA batch cu_tokens must be nondecreasing");
        PSI_REQUIRE((uint64_t)token_indices[r] + (cu_tokens[r + 1] - cu_tokens[r]) <= UINT32_MAX,
                    "GQA request context length must fit u32");
    }
    return PSI_HIP_OK;
}

}  // namespace psi

using namespace psi;

extern "C" int psi_hip_replay_buckets(uint32_t max_capacity, const uint32_t* topology_boundaries,
                                      uint32_t num_boundaries, uint32_t* out_buckets, uint32_t buckets_capacity,
                                      uint32_t* out_num_buckets) {
    BucketPolicy policy;
    int rc = make_bucket_policy(max_capacity, topology_boundaries, num_boundaries, &policy);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(out_num_buckets != nullptr, "out_num_buckets must not be null");
    *out_num_buckets = (uint32_t)policy.buckets.size();
    if (out_buckets) {
        PSI_REQUIRE(buckets_capacity >= policy.buckets.size(), "bucket output array too small");
        std::copy(policy.buckets.begin(), policy.buckets.end(), out_buckets);
    }
    return PSI_HIP_OK;
}

extern "C" int psi_hip_replay_bucket_capacity(uint32_t max_capacity, const uint32_t* topology_boundaries,
                                              uint32_t num_boundaries, uint32_t active, uint32_t* out_capacity) {
    BucketPolicy policy;
    int rc = make_bucket_policy(max_capacity, topology_boundaries, num_boundaries, &policy);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(out_capacity != nullptr, "out_capacity must not be null");
    return policy.capacity(active, out_capacity);
}

extern "C" int psi_hip_split_kv_select(const psi_hip_gqa_config* cfg, int dspark_history, uint32_t num_tokens,
                                       uint32_t num_q_token_tiles, psi_hip_split_kv_variant* out_variant) {
    SplitKVSelector sel;
    int rc = make_selector(cfg, dspark_history != 0, &sel);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(out_variant != nullptr, "out_variant must not be null");
    return sel.select(num_tokens, num_q_token_tiles, out_variant);
}

extern "C" int psi_hip_split_kv_max_q_tokens_per_partial_output(const psi_hip_gqa_config* cfg, int dspark_history,
                                                                uint32_t* out) {
    SplitKVSelector sel;
    int rc = make_selector(cfg, dspark_history != 0, &sel);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(out != nullptr, "out pointer must not be null");
    *out = sel.supports_tiled_q ? sel.tiled_q_token_tile : 1;
    return PSI_HIP_OK;
}

extern "C" int psi_hip_split_kv_select_batch(const psi_hip_gqa_config* cfg, uint32_t max_tokens,
                                             uint32_t bucket_max_tokens, const uint32_t* token_indices,
                                             const uint32_t* cu_tokens, uint32_t num_reqs,
                                             psi_hip_split_kv_variant* out_variant) {
    SplitKVSelector sel;
    Geometry g;
    int rc = make_selector(cfg, false, &sel, &g);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(out_variant != nullptr, "out_variant must not be null");
    rc = check_batch(token_indices, cu_tokens, num_reqs);
    if (rc != PSI_HIP_OK) return rc;
    const uint32_t num_tokens = cu_tokens[num_reqs];
    PSI_REQUIRE(num_tokens > 0, "GQA batch metadata requires tokens");
    uint64_t num_q_token_tiles = 0;
    for (uint32_t r = 0; r < num_reqs; ++r)
        num_q_token_tiles += div_ceil_u64(cu_tokens[r + 1] - cu_tokens[r], sel.tiled_q_token_tile);
    psi_hip_split_kv_variant candidate;
    rc = sel.select(num_tokens, (uint32_t)num_q_token_tiles, &candidate);
    if (rc != PSI_HIP_OK) return rc;
    const bool d256_page8 = g.d == 256 && g.tokens_per_page == 8;
    if (!d256_page8 || candidate.kind != PSI_HIP_VARIANT_TILED_Q) {
        *out_variant = candidate;
        return PSI_HIP_OK;
    }
    // mod.rs:96-127: compare both plans' bookkeeping and require enough useful map work.
    BucketPolicy policy;
    const BucketPolicy* policy_ptr = nullptr;
    if (bucket_max_tokens > 0) {
        rc = make_bucket_policy(bucket_max_tokens, nullptr, 0, &policy);
        if (rc != PSI_HIP_OK) return rc;
        policy_ptr = &policy;
    }
    const psi_hip_split_kv_variant single = sel.single_q();
    std::vector<uint32_t> flat;
    uint64_t logical_pairs = 0;
    for (uint32_t r = 0; r < num_reqs; ++r)
        for (uint32_t i = 0; i < cu_tokens[r + 1] - cu_tokens[r]; ++i) {
            flat.push_back(token_indices[r] + i);
            logical_pairs += (uint64_t)token_indices[r] + i + 1;
        }
    SelectionWork single_work, tiled_work;
    rc = selection_work(single_q_tiles(flat), single.kv_token_tile_size, 1, 1, single.num_threads_per_threadblock / 32,
                        max_tokens, policy_ptr, &single_work);
    if (rc != PSI_HIP_OK) return rc;
    rc = selection_work(tiled_q_tiles(token_indices, cu_tokens, num_reqs, candidate.q_token_tile_size),
                        candidate.kv_token_tile_size, candidate.q_token_tile_size,
                        (uint32_t)div_ceil_u64(single.q_head_tile_size, candidate.q_head_tile_size),
                        candidate.q_token_tile_size / 8 * candidate.q_head_tile_size, max_tokens, policy_ptr,
                        &tiled_work);
    if (rc != PSI_HIP_OK) return rc;
    const uint64_t complete_plan_work = logical_pairs + std::min(single_work.bookkeeping(), tiled_work.bookkeeping());
    const bool enough_utilization = tiled_work.active_map_work * 2 >= tiled_work.scheduled_map_work;
    *out_variant = (enough_utilization && complete_plan_work >= 2048) ? candidate : single;
    return PSI_HIP_OK;
}

extern "C" int psi_hip_gqa_metadata_update(uint32_t max_tokens, const uint32_t* req_slots,
                                           const uint32_t* token_indices, const uint32_t* cu_tokens,
                                           uint32_t num_reqs, const psi_hip_split_kv_variant* variant,
                                           uint32_t capacity_mode, uint32_t caller_num_total_tokens,
                                           const uint32_t* topology_boundaries, uint32_t num_boundaries,
                                           uint32_t partition_tokens, uint32_t kv_splits_capacity,
                                           uint32_t* req_slots_by_token, uint32_t* flat_token_indices,
                                           uint32_t* q_token_tiles, uint32_t* kv_splits, uint32_t* cu_kv_splits,
                                           psi_hip_gqa_replay_shape* out_shape) {
    PSI_REQUIRE(max_tokens > 0, "GQA batch metadata requires tokens");
    PSI_REQUIRE(req_slots && variant && req_slots_by_token && flat_token_indices && kv_splits && cu_kv_splits &&
                    out_shape,
                "GQA batch metadata arrays must not be null");
    int rc = check_batch(token_indices, cu_tokens, num_reqs);
    if (rc != PSI_HIP_OK) return rc;
    const bool tiled = variant->kind == PSI_HIP_VARIANT_TILED_Q;
    PSI_REQUIRE(variant->kind == PSI_HIP_VARIANT_SINGLE_Q || tiled, "unknown SplitKV variant kind %u", variant->kind);
    PSI_REQUIRE(variant->kv_token_tile_size > 0, "GQA KV-token tile size must be positive");
    PSI_REQUIRE(!tiled || variant->q_token_tile_size > 0, "GQA Q-token tile size must be positive");
    PSI_REQUIRE(!tiled || q_token_tiles != nullptr, "GQA Q-token tile array must not be null");
    const uint32_t num_tokens = cu_tokens[num_reqs];
    PSI_REQUIRE(num_tokens > 0, "GQA batch metadata requires tokens");
    PSI_REQUIRE(num_tokens <= max_tokens, "GQA batch tokens exceed the metadata capacity");
    const bool fixed = capacity_mode == PSI_HIP_CAPACITY_FIXED_PARTITION;
    const uint32_t max_kv_splits = fixed ? kv_splits_capacity : max_tokens;
    if (capacity_mode == PSI_HIP_CAPACITY_CALLER_TOKENS) {
        PSI_REQUIRE(num_tokens <= caller_num_total_tokens,
                    "GQA active token count must not exceed the caller-owned token capacity");
        PSI_REQUIRE(caller_num_total_tokens <= max_tokens,
                    "GQA caller-owned token capacity must not exceed the metadata capacity");
    }
    PSI_REQUIRE(capacity_mode <= PSI_HIP_CAPACITY_FIXED_PARTITION, "unknown capacity mode %u", capacity_mode);

    // Per-token expansion (batch_metadata.rs:234-246).
    std::vector<uint32_t> flat;
    flat.reserve(num_tokens);
    for (uint32_t r = 0; r < num_reqs; ++r)
        for (uint32_t i = 0; i < cu_tokens[r + 1] - cu_tokens[r]; ++i) {
            req_slots_by_token[flat.size()] = req_slots[r];
            flat_token_indices[flat.size()] = token_indices[r] + i;
            flat.push_back(token_indices[r] + i);
        }

    std::vector<QTile> tiles = tiled ? tiled_q_tiles(token_indices, cu_tokens, num_reqs, variant->q_token_tile_size)
                                     : single_q_tiles(flat);
    if (fixed) {
        PSI_REQUIRE(partition_tokens > 0 && partition_tokens % variant->kv_token_tile_size == 0,
                    "partition_tokens must be a positive multiple of the KV-token tile size");
        for (auto& t : tiles) t.num_splits = div_ceil_u64(t.context_len, partition_tokens);
    } else if (tiled) {
        uint64_t partial_tokens = 0;
        for (auto& t : tiles) partial_tokens += t.flat_end - t.flat_begin;
        PSI_REQUIRE(partial_tokens <= max_tokens, "GQA tiled partial-output tokens exceed the metadata capacity");
        assign_greedy_splits(tiles, variant->kv_token_tile_size, max_tokens, true);
    } else {
        PSI_REQUIRE(max_kv_splits >= flat.size(), "GQA KV-split capacity is smaller than the token count");
        assign_greedy_splits(tiles, variant->kv_token_tile_size, max_kv_splits, false);
    }
    std::vector<uint32_t> splits, cu;
    if (fixed) {
        // Fixed partitions cut on partition boundaries rather than on even tile shares.
        uint64_t rows = 0;
        for (const auto& t : tiles) rows += t.num_splits;
        splits.reserve((size_t)rows * 3);
        cu.reserve(tiles.size() + 1);
        cu.assign(1, 0u);
        for (uint32_t i = 0; i < tiles.size(); ++i) {
            for (uint64_t s = 0; s < tiles[i].num_splits; ++s) {
                splits.push_back(i);
                splits.push_back((uint32_t)(s * partition_tokens));
                splits.push_back((uint32_t)std::min<uint64_t>(tiles[i].context_len, (s + 1) * partition_tokens));
            }
            cu.push_back((uint32_t)(splits.size() / 3));
        }
    } else {
        rc = emit_splits(tiles, variant->kv_token_tile_size, &splits, &cu);
        if (rc != PSI_HIP_OK) return rc;
    }
    const uint32_t num_kv_splits = (uint32_t)(splits.size() / 3);
    const uint32_t num_q_token_tiles = tiled ? (uint32_t)tiles.size() : num_tokens;
    PSI_REQUIRE(num_kv_splits <= max_kv_splits, "GQA KV-split plan exceeds the KV-split capacity: %u > %u",
                num_kv_splits, max_kv_splits);

    // Recorded capacities (batch_metadata.rs:277-294).
    uint32_t total_tokens = num_tokens, total_tiles = num_q_token_tiles, total_splits = num_kv_splits;
    if (capacity_mode == PSI_HIP_CAPACITY_EXACT || fixed) {
        total_splits = (uint32_t)std::min<uint64_t>(next_pow2_u32(num_kv_splits), max_kv_splits);
        if (fixed) total_splits = num_kv_splits;  // fixed partitions launch exactly the planned splits
    } else {
        BucketPolicy tokens_policy, plain_policy;
        rc = make_bucket_policy(max_tokens, topology_boundaries, num_boundaries, &tokens_policy);
        if (rc != PSI_HIP_OK) return rc;
        rc = make_bucket_policy(max_tokens, nullptr, 0, &plain_policy);
        if (rc != PSI_HIP_OK) return rc;
        if (capacity_mode == PSI_HIP_CAPACITY_BUCKETED) {
            rc = tokens_policy.capacity(num_tokens, &total_tokens);
            if (rc != PSI_HIP_OK) return rc;
        } else {
            total_tokens = caller_num_total_tokens;
        }
        rc = plain_policy.capacity(num_q_token_tiles, &total_tiles);
        if (rc != PSI_HIP_OK) return rc;
        rc = plain_policy.capacity(num_kv_splits, &total_splits);
        if (rc != PSI_HIP_OK) return rc;
    }
    PSI_REQUIRE(total_splits >= num_kv_splits, "GQA recorded KV-split capacity is below the plan");

    if (tiled)
        for (uint32_t i = 0; i < tiles.size(); ++i) {
            q_token_tiles[2 * i] = tiles[i].flat_begin;
            q_token_tiles[2 * i + 1] = tiles[i].flat_end;
        }
    std::copy(splits.begin(), splits.end(), kv_splits);
    std::fill(kv_splits + splits.size(), kv_splits + (size_t)total_splits * 3, PSI_HIP_SENTINEL);
    std::copy(cu.begin(), cu.end(), cu_kv_splits);

    out_shape->num_tokens = num_tokens;
    out_shape->num_total_tokens = total_tokens;
    out_shape->num_q_token_tiles = num_q_token_tiles;
    out_shape->num_total_q_token_tiles = total_tiles;
    out_shape->num_kv_splits = num_kv_splits;
    out_shape->num_total_kv_splits = total_splits;
    out_shape->reduce_sdpa_partial_outputs = (tiled || num_kv_splits > num_tokens) ? 1u : 0u;
    return PSI_HIP_OK;
}

extern "C" int psi_hip_split_kv_balanced_workers(const psi_hip_gqa_config* cfg, uint32_t* out_num_workers) {
    Geometry g;
    int rc = make_geometry(cfg, &g);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(out_num_workers != nullptr, "out pointer must not be null");
    // One 4-wave workgroup per compute unit (256 of them): equal shares of the tiles with as few rows, i.e.
    // partial states and row starts, as the batch allows.  Measured on B=32, ctx 1k-8k, 24/4 heads: 256
    // workgroups 93.7 us, 512 97.7 us, 768 101.6 us, against 104.0 us for a workgroup per 512-token row.
    *out_num_workers = std::max(1u, 256u / g.hkv);
    return PSI_HIP_OK;
}

extern "C" int psi_hip_split_kv_balance_plan(const uint32_t* kv_splits_in, uint32_t num_rows_in,
                                             const uint32_t* cu_in, uint32_t num_tokens, uint32_t num_workers,
                                             uint32_t* kv_splits_out, uint32_t rows_capacity, uint32_t* cu_out,
                                             uint32_t* worker_cu_out, uint32_t* out_num_rows) {
    PSI_REQUIRE(kv_splits_in && cu_in && kv_splits_out && cu_out && worker_cu_out && out_num_rows,
                "balanced plan arrays must not be null");
    PSI_REQUIRE(num_workers > 0 && num_tokens > 0, "balanced plan needs workers and tokens");
    PSI_REQUIRE(cu_in[0] == 0 && cu_in[num_tokens] == num_rows_in, "cu_kv_splits must cover every input row");
    constexpr uint32_t kTile = 16;
    // The cut depends on the tiles alone, and adjacent rows of one token that meet on a tile boundary are cut as if
    // they were one row (a piece runs on across such a boundary at no cost): they are merged first, so that the
    // passes below walk a batch's tokens rather than its partitions.
    struct Run {
        uint32_t token, begin, end;
    };
    std::vector<Run> runs;
    runs.reserve(num_rows_in);
    for (uint32_t r = 0; r < num_rows_in; ++r) {
        const uint32_t token = kv_splits_in[3 * r], b = kv_splits_in[3 * r + 1], e = kv_splits_in[3 * r + 2];
        PSI_REQUIRE(token < num_tokens, "balanced plan input must not hold padding rows");
        if (!runs.empty() && e > b && runs.back().token == token && runs.back().end == b && b % kTile == 0 &&
            runs.back().end > runs.back().begin)
            runs.back().end = e;
        else
            runs.push_back(Run{token, b, e});
    }
    auto tiles_of = [&](const Run& run) -> uint64_t {
        return run.end > run.begin ? (uint64_t)(run.end + kTile - 1) / kTile - run.begin / kTile : 0;
    };
    uint64_t total = 0;
    for (const Run& run : runs) total += tiles_of(run);
    // A worker's cost is its tiles plus kRowStartTiles per row it starts (split record -> slot -> page ID ->
    // first keys, the pipeline running empty and filling again, and the partial state written at the end: about
    // 6 us against 0.62 us per tile on MI355X; with a weight of five tiles the workgroups of C2's decode map that
    // serve two rows ended 3 us after those that serve one).
    // Workers are filled in order up to a common budget; the budget is the smallest one that leaves the last
    // worker no more than the others.
    constexpr uint64_t kRowStartTiles = 10;
    struct Piece {
        uint32_t token, begin, end, worker;
    };
    std::vector<Piece> pieces;
    // One pass over the rows for a budget.  The search for the budget only needs the cost that lands on the last
    // worker, so it runs with `emit` off and keeps the last piece alone; the pass that follows it writes the pieces.
    auto fill = [&](uint64_t budget, bool emit) -> uint64_t {
        if (emit) {
            pieces.clear();
            pieces.reserve((size_t)num_tokens + num_workers);
        }
        Piece last{0u, 0u, 0u, 0u};
        bool have_last = false;
        uint32_t w = 0;
        uint64_t used = 0;
        bool open_row = false;  // the worker's last piece can still be extended (same token, adjacent keys)
        for (const Run& run : runs) {
            const uint32_t row_token = run.token, b = run.begin, e = run.end;
            uint64_t remaining = tiles_of(run);
            uint32_t tile_cursor = b / kTile;
            if (remaining == 0) {  // degenerate row: keep it so that row counts per token stay positive
                last = Piece{row_token, b, e, w};
                have_last = true;
                if (emit) pieces.push_back(last);
                open_row = false;
                continue;
            }
            while (remaining > 0) {
                const uint32_t piece_begin = std::max<uint32_t>(b, tile_cursor * kTile);
                const bool extends =
                    open_row && have_last && last.worker == w && last.token == row_token && last.end == piece_begin;
                const uint64_t start_cost = extends ? 0 : kRowStartTiles;
                if (w + 1 < num_workers && used + start_cost >= budget) {  // no room for even one tile: next worker
                    ++w;
                    used = 0;
                    open_row = false;
                    continue;
                }
                const uint64_t room = w + 1 < num_workers ? budget - used - start_cost : remaining;
                const uint64_t take = std::min<uint64_t>(remaining, std::max<uint64_t>(room, 1));
                const uint32_t piece_end = (uint32_t)std::min<uint64_t>(e, (uint64_t)(tile_cursor + take) * kTile);
                if (extends) {
                    last.end = piece_end;  // same worker, same token, adjacent keys: one row, one partial state
                    if (emit) pieces.back().end = piece_end;
                } else {
                    last = Piece{row_token, piece_begin, piece_end, w};
                    have_last = true;
                    if (emit) pieces.push_back(last);
                }
                open_row = true;
                tile_cursor += (uint32_t)take;
                remaining -= take;
                used += start_cost + take;
            }
        }
        return w + 1 == num_workers ? used : 0;
    };
    // The smallest budget that leaves the last worker no more than the others: a larger one only moves work from
    // the last worker to the rest (with a budget 1.5 % above it the last of C2's 64 workers got 24 tiles of 148).
    uint64_t high = std::max<uint64_t>((total + kRowStartTiles * ((uint64_t)num_tokens + num_workers)) / num_workers,
                                      kRowStartTiles + 1);  // room for at least one tile
    while (fill(high, false) > high) high += std::max<uint64_t>(high / 64, 1);
    uint64_t low = std::max<uint64_t>(total / num_workers, kRowStartTiles + 1);  // below the mean nothing fits
    if (low > high) low = high;
    while (low < high) {
        const uint64_t mid = low + (high - low) / 2;
        if (fill(mid, false) > mid) low = mid + 1;
        else high = mid;
    }
    const uint64_t budget = high;
    fill(budget, true);

    uint32_t out_rows = 0, worker = 0;
    worker_cu_out[0] = 0;
    uint32_t token = 0;
    cu_out[0] = 0;
    PSI_REQUIRE(pieces.size() <= rows_capacity, "balanced plan exceeds the row capacity");
    for (const Piece& piece : pieces) {
        while (token < piece.token) cu_out[++token] = out_rows;
        while (worker < piece.worker) worker_cu_out[++worker] = out_rows;
        kv_splits_out[3 * out_rows] = piece.token;
        kv_splits_out[3 * out_rows + 1] = piece.begin;
        kv_splits_out[3 * out_rows + 2] = piece.end;
        ++out_rows;
    }
    while (token < num_tokens) cu_out[++token] = out_rows;
    while (worker < num_workers) worker_cu_out[++worker] = out_rows;
    *out_num_rows = out_rows;
    return PSI_HIP_OK;
}

extern "C" int psi_hip_split_kv_order_longest_first(uint32_t* kv_splits, uint32_t num_kv_splits,
                                                    uint32_t* partial_row_index) {
    PSI_REQUIRE(kv_splits != nullptr && partial_row_index != nullptr, "split arrays must not be null");
    std::vector<uint32_t> order(num_kv_splits);
    for (uint32_t i = 0; i < num_kv_splits; ++i) order[i] = i;
    auto length = [&](uint32_t row) -> uint64_t {
        const uint32_t* r = kv_splits + (size_t)row * 3;
        if (r[0] == PSI_HIP_SENTINEL) return 0;  // padding rows stay last
        return (uint64_t)r[2] - r[1] + 1;
    };
    std::stable_sort(order.begin(), order.end(), [&](uint32_t x, uint32_t y) { return length(x) > length(y); });
    std::vector<uint32_t> sorted((size_t)num_kv_splits * 3);
    for (uint32_t pos = 0; pos < num_kv_splits; ++pos) {
        std::copy(kv_splits + (size_t)order[pos] * 3, kv_splits + (size_t)order[pos] * 3 + 3, sorted.begin() + (size_t)pos * 3);
        partial_row_index[order[pos]] = pos;
    }
    std::copy(sorted.begin(), sorted.end(), kv_splits);
    return PSI_HIP_OK;
}

// Partition length for prefill chunks: a model of the row-group map's launch.  An item = (token group of a request,
// partition, KV head, head subset) costs its KV tiles plus a fixed share (its start, its partial rows); the units
// take items heaviest first as they become free; every item's partial rows are written once and read once by the
// combine.  The figures are this library's own measurements on MI355X: an item's fixed cost is that of nine tiles,
// and the partial rows of an item of 256 columns at head_dim 256 cost the launch 0.06 tiles.
extern "C" int psi_hip_split_kv_chunk_partition_tokens(const psi_hip_gqa_config* cfg, uint32_t q_token_tile_size,
                                                       const uint32_t* token_indices, const uint32_t* cu_tokens,
                                                       uint32_t num_reqs, uint32_t num_compute_units,
                                                       uint32_t* out_partition_tokens) {
    Geometry g;
    int rc = make_geometry(cfg, &g);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(out_partition_tokens != nullptr, "out_partition_tokens must not be null");
    PSI_REQUIRE(num_reqs == 0 || (token_indices && cu_tokens), "request arrays must not be null");
    *out_partition_tokens = 0;
    if (num_reqs == 0 || !chunk_map_supported(g, q_token_tile_size)) return PSI_HIP_OK;
    const uint32_t units = num_compute_units ? num_compute_units : 256u;
    const uint32_t tile_keys = chunk_tile_keys(g.d);
    uint32_t longest_chunk = 0;
    for (uint32_t r = 0; r < num_reqs; ++r)
        if (cu_tokens[r + 1] >= cu_tokens[r]) longest_chunk = std::max(longest_chunk, cu_tokens[r + 1] - cu_tokens[r]);
    // (as psi_hip_split_kv_tiled_q_group_rows and the launch have it: no head subsets when every chunk fits one
    // workgroup with all the heads)
    const uint32_t chunk_tiles = (longest_chunk + q_token_tile_size - 1) / q_token_tile_size;
    const uint32_t width = std::max(std::min(chunk_tiles, chunk_group_tiles(g.group, q_token_tile_size)), 1u);
    const uint32_t subsets = chunk_launch_subsets(g.group, width, q_token_tile_size);
    const uint32_t group_tokens =
        (subsets == 1 ? std::max(std::min(chunk_all_heads_tiles(g.group, q_token_tile_size),
                                          chunk_group_tiles(g.group, q_token_tile_size)), 1u)
                      : chunk_group_tiles(g.group, q_token_tile_size)) * q_token_tile_size;
    const uint32_t copies = g.hkv * subsets;  // items of equal cost per (group, partition)
    constexpr double kItemTiles = 9.0;
    const double partial_tiles = 0.06 * g.d / 256.0;
    uint64_t longest = 0;
    for (uint32_t r = 0; r < num_reqs; ++r) {
        PSI_REQUIRE(cu_tokens[r + 1] >= cu_tokens[r], "cu_tokens must not decrease (request %u)", r);
        longest = std::max<uint64_t>(longest, (uint64_t)token_indices[r] + (cu_tokens[r + 1] - cu_tokens[r]));
    }
    if (longest == 0) return PSI_HIP_OK;
    const uint32_t unsplit = (uint32_t)std::min<uint64_t>((longest + 255) / 256 * 256, 1u << 20);
    std::vector<uint32_t> candidates;
    for (uint32_t p = 256; p < unsplit && p <= 32768; p += p < 2048 ? 256 : (p < 8192 ? 1024 : 2048)) candidates.push_back(p);
    candidates.push_back(unsplit);
    double best = 0.0;
    std::vector<double> costs;
    std::vector<double> free_at;
    for (uint32_t partition : candidates) {
        // (more than 64 partitions of a request are never the answer)
        if ((uint64_t)partition * 64 < longest && partition != unsplit) continue;
        costs.clear();
        for (uint32_t r = 0; r < num_reqs; ++r) {
            const uint32_t prefix = token_indices[r], chunk = cu_tokens[r + 1] - cu_tokens[r];
            for (uint32_t a = 0; a < chunk; a += group_tokens) {
                const uint64_t kv_end = (uint64_t)prefix + std::min(a + group_tokens, chunk);  // causal limit of the group's last token
                for (uint64_t lo = 0; lo < kv_end; lo += partition) {
                    const uint64_t keys = std::min<uint64_t>(lo + partition, kv_end) - lo;
                    costs.push_back((double)((keys + tile_keys - 1) / tile_keys) + kItemTiles);
                }
            }
        }
        std::sort(costs.begin(), costs.end(), std::greater<double>());
        const double items = (double)costs.size() * copies;
        double total = 0.0;
        for (double c : costs) total += c * copies;
        double end;
        if (items > 8.0 * units) {
            // so many items that the units end within the lightest item of each other
            end = std::max(total / units + 0.5 * costs.back(), costs.front());
        } else {
            free_at.assign(units, 0.0);  // a min-heap of the times at which the units become free
            std::make_heap(free_at.begin(), free_at.end(), std::greater<double>());
            end = 0.0;
            for (double c : costs)
                for (uint32_t k = 0; k < copies; ++k) {
                    std::pop_heap(free_at.begin(), free_at.end(), std::greater<double>());
                    free_at.back() += c;
                    end = std::max(end, free_at.back());
                    std::push_heap(free_at.begin(), free_at.end(), std::greater<double>());
                }
        }
        const double cost = end + partial_tiles * items;
        if (*out_partition_tokens == 0 || cost <= best) {  // (ties go to the longer partition: fewer partial rows)
            best = cost;
            *out_partition_tokens = partition;
        }
    }
    return PSI_HIP_OK;
}

// Row groups for the prefill-chunk map.  Rows are sorted by (request slot, first key, Q-token tile); a
// group is a run of rows of consecutive, contiguous tiles of one request that start at the same key,
// every tile but the last one full, at most `max_tiles` of them.
extern "C" int psi_hip_split_kv_tiled_q_group_rows(const psi_hip_gqa_config* cfg, uint32_t q_token_tile_size,
                                                   const uint32_t* kv_splits, uint32_t num_kv_splits,
                                                   const uint32_t* q_token_tiles, uint32_t num_q_token_tiles,
                                                   const uint32_t* req_slots, uint32_t* row_groups,
                                                   uint64_t row_groups_capacity, uint32_t* out_group_tiles,
                                                   uint32_t* out_num_groups) {
    Geometry g;
    int rc = make_geometry(cfg, &g);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(kv_splits && q_token_tiles && req_slots && row_groups && out_group_tiles && out_num_groups,
                "row-group arrays must not be null");
    PSI_REQUIRE(q_token_tile_size > 0 && q_token_tile_size <= 64, "GQA Q-token tile size must be in 1..64");
    *out_group_tiles = 0;
    *out_num_groups = 0;
    if (!chunk_map_supported(g, q_token_tile_size)) return PSI_HIP_OK;  // no grouped kernel for this shape
    const uint32_t max_tiles = chunk_group_tiles(g.group, q_token_tile_size);

    struct Row {
        uint32_t slot, kv_begin, tile, row, kv_end;
    };
    std::vector<Row> rows;
    rows.reserve(num_kv_splits);
    for (uint32_t r = 0; r < num_kv_splits; ++r) {
        const uint32_t* s = kv_splits + (size_t)r * 3;
        if (s[0] == PSI_HIP_SENTINEL) continue;
        PSI_REQUIRE(s[0] < num_q_token_tiles, "kv_split row %u names Q-token tile %u of %u", r, s[0], num_q_token_tiles);
        PSI_REQUIRE(s[2] > s[1], "kv_split row %u is empty", r);
        const uint32_t flat_begin = q_token_tiles[(size_t)s[0] * 2];
        rows.push_back(Row{req_slots[flat_begin], s[1], s[0], r, s[2]});
    }
    std::sort(rows.begin(), rows.end(), [](const Row& x, const Row& y) {
        if (x.slot != y.slot) return x.slot < y.slot;
        if (x.kv_begin != y.kv_begin) return x.kv_begin < y.kv_begin;
        if (x.tile != y.tile) return x.tile < y.tile;
        return x.row < y.row;
    });
    struct Group {
        uint32_t first, count;  // range of `rows`
        uint32_t keys;          // its longest KV range: what an item of the group costs, and the dispatch-order key
        uint64_t work;          // query tokens x keys: the order among groups of equal range
    };
    std::vector<Group> groups;
    auto tile_tokens = [&](uint32_t tile) { return q_token_tiles[(size_t)tile * 2 + 1] - q_token_tiles[(size_t)tile * 2]; };
    for (uint32_t i = 0; i < rows.size(); ++i) {
        bool join = false;
        if (!groups.empty()) {
            const Group& cur = groups.back();
            const Row& prev = rows[i - 1];
            join = cur.count < max_tiles && prev.slot == rows[i].slot && prev.kv_begin == rows[i].kv_begin &&
                   prev.tile + 1 == rows[i].tile && tile_tokens(prev.tile) == q_token_tile_size &&
                   q_token_tiles[(size_t)prev.tile * 2 + 1] == q_token_tiles[(size_t)rows[i].tile * 2];
        }
        if (!join) groups.push_back(Group{i, 0, 0, 0});
        groups.back().count += 1;
        groups.back().keys = std::max(groups.back().keys, rows[i].kv_end - rows[i].kv_begin);
        groups.back().work += (uint64_t)tile_tokens(rows[i].tile) * (rows[i].kv_end - rows[i].kv_begin);
    }
    // Longest groups first, so that the short ones fill the end of the launch.  A work item walks the group's KV
    // range whatever the number of its query tokens (a request's last group may hold a few), so the range is the
    // key, not the tokens x keys product, by which such a group was claimed last and ended the launch.
    std::stable_sort(groups.begin(), groups.end(), [](const Group& x, const Group& y) {
        return x.keys != y.keys ? x.keys > y.keys : x.work > y.work;
    });
    // No group wider than what fits one workgroup with all the heads of a KV head (short chunks, verify steps): the
    // table is written that narrow, which tells the launch to deal no heads to separate work items.
    uint32_t stride = max_tiles;
    const uint32_t all_heads_tiles = chunk_all_heads_tiles(g.group, q_token_tile_size);
    if (all_heads_tiles >= 1 && all_heads_tiles < max_tiles) {
        uint32_t widest = 0;
        for (const Group& grp : groups) widest = std::max(widest, grp.count);
        if (widest <= all_heads_tiles) stride = all_heads_tiles;
    }
    PSI_REQUIRE((uint64_t)groups.size() * stride <= row_groups_capacity,
                "row-group table too small: %llu groups of %u rows, capacity %llu words",
                (unsigned long long)groups.size(), stride, (unsigned long long)row_groups_capacity);
    for (size_t gi = 0; gi < groups.size(); ++gi) {
        uint32_t* out = row_groups + gi * stride;
        for (uint32_t m = 0; m < stride; ++m)
            out[m] = m < groups[gi].count ? rows[groups[gi].first + m].row : PSI_HIP_SENTINEL;
    }
    *out_group_tiles = stride;
    *out_num_groups = (uint32_t)groups.size();
    return PSI_HIP_OK;
}
