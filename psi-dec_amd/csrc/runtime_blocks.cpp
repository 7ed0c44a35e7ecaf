// Host-side cache ownership for the paged attention path: the page-ID allocator and the per-request
// token-window state machine that decides which tokens a step runs and which pages a request owns.
// No device work happens here; the page IDs it hands out are what psi_hip_page_table_write_page_ids
// uploads and what the append / attention kernels dereference.
//
// Reference behaviour followed:
//   U32IDAllocator        crates/inference-runtime-core/src/memory/u32_id_allocator.rs:40-173
//   TPKVBlockAllocator    crates/inference-runtime-core/src/runtime/decoder/allocator/tp_kv_block_allocator.rs:24-36
//   DeviceBlock (Drop)    crates/inference-runtime-core/src/memory/device_kv_block.rs:44-51
//   MutableBlock          crates/inference-runtime-core/src/runtime/decoder/trie_cache/block/mutable_block.rs:13-167
//   TrieDecoderBlocks     crates/inference-runtime-core/src/runtime/decoder/trie_cache/blocks/trie/api.rs:34-571,
//                         .../blocks/trie/mod.rs:176-229, .../blocks/util.rs:8-89
// Prefix sharing between requests (the trie, its eviction queue and reservations) is not part of this
// library: every logical block owns its pages from allocation until the request releases it.
#include <algorithm>
#include <atomic>
#include <deque>
#include <memory>
#include <mutex>
#include <vector>

#include "common.h"

struct psi_hip_id_allocator {
    std::atomic<int> refs{1};  // the creator's handle plus one per decoder-blocks object drawing from it
    std::mutex mu;
    uint64_t capacity = 0;
    uint64_t counter = 0;             // next never-issued ID
    std::deque<uint32_t> free_ids;    // FIFO: first freed, first reused; preferred over fresh IDs
    std::vector<uint64_t> bitmap;     // bit i set <=> ID i is allocated

    bool bit(uint32_t id) const { return (bitmap[id >> 6] >> (id & 63)) & 1u; }
    void flip(uint32_t id) { bitmap[id >> 6] ^= (1ull << (id & 63)); }
};

namespace {

using psi::fail;

int alloc_many_locked(psi_hip_id_allocator* a, size_t count, uint32_t* ids) {
    size_t got = 0;
    while (got < count && !a->free_ids.empty()) {
        ids[got++] = a->free_ids.front();
        a->free_ids.pop_front();
    }
    const size_t fresh = count - got;
    if (fresh != 0) {
        if (a->counter + fresh > a->capacity) {
            // Popped IDs return to the tail of the queue, as the reference does.
            for (size_t i = 0; i < got; ++i) a->free_ids.push_back(ids[i]);
            return fail(PSI_HIP_ERR_RESOURCE_EXHAUSTED, "not enough ID");
        }
        for (size_t i = 0; i < fresh; ++i) ids[got + i] = static_cast<uint32_t>(a->counter + i);
        a->counter += fresh;
    }
    for (size_t i = 0; i < count; ++i) a->flip(ids[i]);
    return PSI_HIP_OK;
}

int free_many_locked(psi_hip_id_allocator* a, const uint32_t* ids, size_t count) {
    for (size_t i = 0; i < count; ++i) {
        PSI_REQUIRE(ids[i] < a->capacity, "U32 ID allocator ID is out of range");
        PSI_REQUIRE(a->bit(ids[i]), "U32 ID allocator cannot free an unallocated ID");
        a->flip(ids[i]);
        a->free_ids.push_back(ids[i]);
    }
    return PSI_HIP_OK;
}

// One lane's view of a logical block: tokens split into cached | scheduled | ready by two indices.
struct LaneBlock {
    std::vector<uint32_t> tokens;
    size_t scheduled_index = 0;  // tokens[..scheduled_index] are cached
    size_t ready_index = 0;      // tokens[scheduled_index..ready_index] are scheduled
    std::vector<uint32_t> page_ids;
};

using BlockVec = std::vector<LaneBlock>;  // one entry per cache lane

}  // namespace

struct psi_hip_decoder_blocks {
    psi_hip_id_allocator* alloc = nullptr;
    size_t n = 0, lanes = 0, pages_per_block = 0;
    std::vector<BlockVec> immutable_blocks;
    std::deque<BlockVec> semi_immutable_blocks, mutable_blocks;
    std::deque<uint32_t> queued;
    std::vector<uint32_t> spec;
    size_t num_in_sync_blocks = 0;
    uint64_t epoch = 0;

    size_t cached(const BlockVec& b) const { return b[0].scheduled_index; }
    size_t scheduled(const BlockVec& b) const { return b[0].ready_index - b[0].scheduled_index; }
    size_t ready(const BlockVec& b) const { return b[0].tokens.size() - b[0].ready_index; }

    size_t ready_token_slots() const {
        size_t s = 0;
        for (const auto& b : semi_immutable_blocks) s += n - b[0].ready_index;
        for (const auto& b : mutable_blocks) s += n - b[0].ready_index;
        return s;
    }
    size_t num_cached() const {
        size_t s = 0;
        for (const auto& b : immutable_blocks) s += cached(b);
        for (const auto& b : semi_immutable_blocks) s += cached(b);
        for (const auto& b : mutable_blocks) s += cached(b);
        return s;
    }
    size_t num_scheduled() const {
        size_t s = 0;
        for (const auto& b : semi_immutable_blocks) s += scheduled(b);
        for (const auto& b : mutable_blocks) s += scheduled(b);
        return s;
    }
    size_t num_ready() const {
        size_t s = 0;
        for (const auto& b : semi_immutable_blocks) s += ready(b);
        for (const auto& b : mutable_blocks) s += ready(b);
        return s;
    }
    size_t num_total() const {
        size_t s = queued.size();
        for (const auto& b : immutable_blocks) s += b[0].tokens.size();
        for (const auto& b : semi_immutable_blocks) s += b[0].tokens.size();
        for (const auto& b : mutable_blocks) s += b[0].tokens.size();
        return s;
    }

    // Takes up to `num` tokens off the queue front; returns them plus the L-1 tokens of lookahead the
    // other lanes need (those stay queued).
    std::vector<uint32_t> pop_front_queued(size_t num) {
        num = std::min(queued.size() - (lanes - 1), num);
        std::vector<uint32_t> out(queued.begin(), queued.begin() + num + lanes - 1);
        queued.erase(queued.begin(), queued.begin() + num);
        return out;
    }
    // Inverse of pop_front_queued: `lookahead` trailing tokens never left the queue.
    void push_front_queued(const std::vector<uint32_t>& tokens, size_t lookahead) {
        if (tokens.size() <= lookahead) return;
        for (size_t i = tokens.size() - lookahead; i-- > 0;) queued.push_front(tokens[i]);
    }
    // Lane l receives the window tokens[l .. l + len - (L-1)).
    void push_tokens(BlockVec& b, const uint32_t* tokens, size_t len) {
        if (len == 0) return;
        const size_t window = len - (lanes - 1);
        for (size_t lane = 0; lane < lanes; ++lane)
            b[lane].tokens.insert(b[lane].tokens.end(), tokens + lane, tokens + lane + window);
    }
    void schedule(BlockVec& b, size_t num) {
        for (auto& lane : b) lane.ready_index += std::min(num, lane.tokens.size() - lane.ready_index);
    }
    bool alloc_block_vec(BlockVec* out) {
        std::lock_guard<std::mutex> lock(alloc->mu);
        BlockVec b(lanes);
        for (size_t lane = 0; lane < lanes; ++lane) {
            b[lane].page_ids.resize(pages_per_block);
            if (alloc_many_locked(alloc, pages_per_block, b[lane].page_ids.data()) != PSI_HIP_OK) {
                for (size_t done = 0; done < lane; ++done)
                    free_many_locked(alloc, b[done].page_ids.data(), pages_per_block);
                return false;
            }
        }
        *out = std::move(b);
        return true;
    }
    void free_block_vec(const BlockVec& b) {
        std::lock_guard<std::mutex> lock(alloc->mu);
        for (const auto& lane : b) free_many_locked(alloc, lane.page_ids.data(), lane.page_ids.size());
    }
    // Moves `end - start` scheduled tokens of every lane to cached after checking them against the
    // step's token list (lane l sees the list shifted by l).
    bool cache_tokens(BlockVec& b, const std::vector<uint32_t>& tokens, size_t start, size_t end) {
        if (start == end) return true;
        for (size_t lane = 0; lane < lanes; ++lane) {
            LaneBlock& lb = b[lane];
            if (lb.scheduled_index + (end - start) > lb.ready_index || end + lane > tokens.size()) return false;
            if (!std::equal(tokens.begin() + start + lane, tokens.begin() + end + lane,
                            lb.tokens.begin() + lb.scheduled_index))
                return false;
            lb.scheduled_index += end - start;
        }
        return true;
    }
    void try_mark_ready() {
        size_t cachable = queued.size() > lanes - 1 ? queued.size() - (lanes - 1) : 0;
        for (auto& b : mutable_blocks) {
            if (cachable == 0) break;
            if (b[0].tokens.size() == n) continue;
            const size_t num = std::min(cachable, n - b[0].tokens.size());
            cachable -= num;
            const std::vector<uint32_t> tokens = pop_front_queued(num);
            push_tokens(b, tokens.data(), tokens.size());
        }
    }
};

namespace {

void copy_tokens(const std::vector<uint32_t>& src, uint32_t* dst) { std::copy(src.begin(), src.end(), dst); }

int check_query(const psi_hip_decoder_blocks* b, const psi_hip_query_tokens* q) {
    PSI_REQUIRE(q != nullptr, "query tokens must not be null");
    PSI_REQUIRE(q->kind == PSI_HIP_QUERY_PREFILL || q->kind == PSI_HIP_QUERY_DECODE, "unknown query kind %u", q->kind);
    PSI_REQUIRE(q->epoch == b->epoch, "query epoch %llu does not match the blocks' epoch %llu",
                (unsigned long long)q->epoch, (unsigned long long)b->epoch);
    PSI_REQUIRE(q->num_tokens != 0 && q->tokens != nullptr, "query tokens must not be empty");
    PSI_REQUIRE(q->token_index < b->num_total(), "query token_index is past the request's tokens");
    PSI_REQUIRE(q->num_spec_tokens == 0 || q->spec_tokens != nullptr, "spec_tokens pointer is null");
    if (q->kind == PSI_HIP_QUERY_PREFILL)
        PSI_REQUIRE(q->window >= 1 && q->window == q->num_tokens - (b->lanes - 1),
                    "prefill window must equal tokens.len() - (L - 1)");
    return PSI_HIP_OK;
}

}  // namespace

extern "C" {

int psi_hip_id_allocator_create(uint64_t capacity, psi_hip_id_allocator** out) {
    PSI_REQUIRE(out != nullptr, "out must not be null");
    PSI_REQUIRE(capacity <= 0xFFFFFFFFull, "U32 ID allocator capacity must fit u32");
    auto a = std::make_unique<psi_hip_id_allocator>();
    a->capacity = capacity;
    a->bitmap.assign((capacity + 63) / 64, 0);
    *out = a.release();
    return PSI_HIP_OK;
}

int psi_hip_id_allocator_destroy(psi_hip_id_allocator* a) {
    // Shared ownership, like the reference's Arc<U32IDAllocator>: the memory goes when the last
    // decoder-blocks object that draws from it has gone too.
    if (a != nullptr && a->refs.fetch_sub(1) == 1) delete a;
    return PSI_HIP_OK;
}

int psi_hip_id_allocator_alloc_one(psi_hip_id_allocator* a, uint32_t* id) {
    PSI_REQUIRE(a != nullptr && id != nullptr, "allocator and id must not be null");
    std::lock_guard<std::mutex> lock(a->mu);
    return alloc_many_locked(a, 1, id);
}

int psi_hip_id_allocator_alloc_many(psi_hip_id_allocator* a, size_t count, uint32_t* ids) {
    PSI_REQUIRE(a != nullptr && (count == 0 || ids != nullptr), "allocator and ids must not be null");
    PSI_REQUIRE(count <= 0xFFFFFFFFull, "count must fit u32");
    std::lock_guard<std::mutex> lock(a->mu);
    return alloc_many_locked(a, count, ids);
}

int psi_hip_id_allocator_free_one(psi_hip_id_allocator* a, uint32_t id) {
    PSI_REQUIRE(a != nullptr, "allocator must not be null");
    std::lock_guard<std::mutex> lock(a->mu);
    return free_many_locked(a, &id, 1);
}

int psi_hip_id_allocator_free_many(psi_hip_id_allocator* a, const uint32_t* ids, size_t count) {
    PSI_REQUIRE(a != nullptr && (count == 0 || ids != nullptr), "allocator and ids must not be null");
    std::lock_guard<std::mutex> lock(a->mu);
    // All-or-nothing: validate before the first bit is cleared (a repeated ID within the call is
    // caught by the second pass because the first occurrence already cleared its bit).
    for (size_t i = 0; i < count; ++i) {
        PSI_REQUIRE(ids[i] < a->capacity, "U32 ID allocator ID is out of range");
        PSI_REQUIRE(a->bit(ids[i]), "U32 ID allocator cannot free an unallocated ID");
    }
    for (size_t i = 0; i < count; ++i) {
        if (!a->bit(ids[i])) {
            for (size_t j = 0; j < i; ++j) {  // undo
                a->flip(ids[j]);
                a->free_ids.pop_back();
            }
            return fail(PSI_HIP_ERR_INVALID_ARGUMENT, "U32 ID allocator cannot free an unallocated ID");
        }
        a->flip(ids[i]);
        a->free_ids.push_back(ids[i]);
    }
    return PSI_HIP_OK;
}

int psi_hip_id_allocator_counts(psi_hip_id_allocator* a, uint64_t* used, uint64_t* free_count, uint64_t* capacity) {
    PSI_REQUIRE(a != nullptr, "allocator must not be null");
    std::lock_guard<std::mutex> lock(a->mu);
    const uint64_t f = a->free_ids.size() + (a->capacity - a->counter);
    if (used) *used = a->capacity - f;
    if (free_count) *free_count = f;
    if (capacity) *capacity = a->capacity;
    return PSI_HIP_OK;
}

int psi_hip_id_allocator_bitmap(psi_hip_id_allocator* a, uint64_t* words, size_t num_words) {
    PSI_REQUIRE(a != nullptr && (num_words == 0 || words != nullptr), "allocator and words must not be null");
    std::lock_guard<std::mutex> lock(a->mu);
    PSI_REQUIRE(num_words == a->bitmap.size(), "bitmap has %zu words, caller asked for %zu", a->bitmap.size(),
                num_words);
    std::copy(a->bitmap.begin(), a->bitmap.end(), words);
    return PSI_HIP_OK;
}

int psi_hip_bitmap_allocated_ranges(const uint64_t* words, size_t num_words, uint32_t* ranges, size_t capacity_pairs,
                                    size_t* num_pairs) {
    PSI_REQUIRE((num_words == 0 || words != nullptr) && num_pairs != nullptr, "words and num_pairs must not be null");
    size_t pairs = 0;
    bool open = false;
    uint64_t begin = 0;
    const uint64_t bits = static_cast<uint64_t>(num_words) * 64;
    for (uint64_t i = 0; i <= bits; ++i) {
        const bool set = i < bits && ((words[i >> 6] >> (i & 63)) & 1u);
        if (set && !open) {
            open = true;
            begin = i;
        } else if (!set && open) {
            open = false;
            if (ranges != nullptr) {
                PSI_REQUIRE(pairs < capacity_pairs, "range buffer holds %zu pairs, more are needed", capacity_pairs);
                ranges[2 * pairs] = static_cast<uint32_t>(begin);
                ranges[2 * pairs + 1] = static_cast<uint32_t>(i);
            }
            ++pairs;
        }
    }
    *num_pairs = pairs;
    return PSI_HIP_OK;
}

int psi_hip_decoder_blocks_create(psi_hip_id_allocator* allocator, const psi_hip_decoder_blocks_config* cfg,
                                  const uint32_t* tokens, size_t num_tokens, psi_hip_decoder_blocks** out) {
    PSI_REQUIRE(allocator != nullptr && cfg != nullptr && out != nullptr, "allocator, cfg and out must not be null");
    PSI_REQUIRE(cfg->tokens_per_block > 0, "tokens_per_block must be positive");
    PSI_REQUIRE(cfg->num_cache_lanes >= 1, "num_cache_lanes must be at least 1");
    PSI_REQUIRE(num_tokens != 0 && tokens != nullptr, "a request starts with at least one token");
    PSI_REQUIRE(cfg->num_cache_lanes - 1 <= num_tokens, "a request needs at least L - 1 tokens");
    auto b = std::make_unique<psi_hip_decoder_blocks>();
    b->alloc = allocator;
    allocator->refs.fetch_add(1);
    b->n = cfg->tokens_per_block;
    b->lanes = cfg->num_cache_lanes;
    b->pages_per_block = cfg->pages_per_kv_block;
    b->queued.assign(tokens, tokens + num_tokens);
    *out = b.release();
    return PSI_HIP_OK;
}

int psi_hip_decoder_blocks_destroy(psi_hip_decoder_blocks* b) {
    if (b == nullptr) return PSI_HIP_OK;
    // Release order of the reference's Drop: mutable blocks last to first, then semi-immutable ones.
    for (auto it = b->mutable_blocks.rbegin(); it != b->mutable_blocks.rend(); ++it) b->free_block_vec(*it);
    for (auto it = b->semi_immutable_blocks.rbegin(); it != b->semi_immutable_blocks.rend(); ++it)
        b->free_block_vec(*it);
    // With no trie to keep them, committed blocks are released too.
    for (auto it = b->immutable_blocks.rbegin(); it != b->immutable_blocks.rend(); ++it) b->free_block_vec(*it);
    psi_hip_id_allocator_destroy(b->alloc);
    delete b;
    return PSI_HIP_OK;
}

int psi_hip_decoder_blocks_ready_token_slots(const psi_hip_decoder_blocks* b, size_t* out) {
    PSI_REQUIRE(b != nullptr && out != nullptr, "blocks and out must not be null");
    *out = b->ready_token_slots();
    return PSI_HIP_OK;
}

int psi_hip_decoder_blocks_init_block_once(psi_hip_decoder_blocks* b, size_t* ready_token_slots) {
    PSI_REQUIRE(b != nullptr, "blocks must not be null");
    const size_t lookahead = b->lanes - 1;
    const size_t cachable = b->queued.size() > lookahead ? b->queued.size() - lookahead : 0;
    const size_t num = std::min(cachable, b->n);
    std::vector<uint32_t> tokens;
    if (num != 0) tokens = b->pop_front_queued(num);
    // A whole block of known tokens with more behind it, and nothing partially filled before it, is
    // the case the reference offers to its prefix cache; on a miss it becomes a semi-immutable block.
    const bool full_known_block =
        num == b->n && !b->queued.empty() && b->mutable_blocks.empty() && b->semi_immutable_blocks.empty();
    BlockVec block;
    if (!b->alloc_block_vec(&block)) {
        b->push_front_queued(tokens, lookahead);
        return fail(PSI_HIP_ERR_RESOURCE_EXHAUSTED, "no free pages for another block");
    }
    b->push_tokens(block, tokens.data(), tokens.size());
    (full_known_block ? b->semi_immutable_blocks : b->mutable_blocks).push_back(std::move(block));
    if (ready_token_slots) *ready_token_slots = b->ready_token_slots();
    return PSI_HIP_OK;
}

int psi_hip_decoder_blocks_uninit_block_once(psi_hip_decoder_blocks* b, size_t* cached_token_slots) {
    PSI_REQUIRE(b != nullptr, "blocks must not be null");
    BlockVec block;
    bool have = true;
    if (!b->mutable_blocks.empty()) {
        block = std::move(b->mutable_blocks.back());
        b->mutable_blocks.pop_back();
    } else if (!b->semi_immutable_blocks.empty()) {
        block = std::move(b->semi_immutable_blocks.back());
        b->semi_immutable_blocks.pop_back();
    } else if (!b->immutable_blocks.empty()) {
        block = std::move(b->immutable_blocks.back());
        b->immutable_blocks.pop_back();
    } else {
        have = false;
    }
    if (have) {
        b->push_front_queued(block[0].tokens, 0);
        b->free_block_vec(block);
        const size_t total = b->immutable_blocks.size() + b->semi_immutable_blocks.size() + b->mutable_blocks.size();
        b->num_in_sync_blocks = std::min(b->num_in_sync_blocks, total);
    }
    if (cached_token_slots) *cached_token_slots = b->num_cached();
    return PSI_HIP_OK;
}

int psi_hip_decoder_blocks_set_spec_tokens(psi_hip_decoder_blocks* b, const uint32_t* spec_tokens, size_t count) {
    PSI_REQUIRE(b != nullptr && (count == 0 || spec_tokens != nullptr), "blocks and spec_tokens must not be null");
    b->spec.assign(spec_tokens, spec_tokens + count);
    return PSI_HIP_OK;
}

int psi_hip_decoder_blocks_prepare(psi_hip_decoder_blocks* b, size_t token_budget, psi_hip_query_tokens* out) {
    PSI_REQUIRE(b != nullptr && out != nullptr, "blocks and out must not be null");
    PSI_REQUIRE(token_budget > 0, "token budget must be positive");
    PSI_REQUIRE(token_budget <= b->ready_token_slots(),
                "token budget %zu exceeds the %zu ready token slots; init more blocks first", token_budget,
                b->ready_token_slots());
    const size_t validated = b->num_ready() + b->queued.size();
    PSI_REQUIRE(validated != 0, "nothing to run: no ready or queued tokens");
    const size_t lookahead = b->lanes - 1;
    const bool prefill = token_budget < validated;
    // Size check before any state changes.
    const size_t need_tokens = prefill ? token_budget + lookahead : validated;
    PSI_REQUIRE(out->tokens != nullptr && out->tokens_capacity >= need_tokens,
                "query token buffer holds %zu tokens, %zu are needed", out->tokens_capacity, need_tokens);
    if (prefill) {
        PSI_REQUIRE(lookahead <= b->queued.size(), "prefill needs L - 1 queued lookahead tokens");
        PSI_REQUIRE(token_budget <= b->num_ready(), "prefill chunk of %zu tokens exceeds the %zu ready tokens",
                    token_budget, b->num_ready());
        // The lookahead is read from the queue, so with L > 1 the chunk must end at the last ready token.
        PSI_REQUIRE(lookahead == 0 || token_budget == b->num_ready(),
                    "prefill chunk must take every ready token when L > 1");
    } else {
        PSI_REQUIRE(b->queued.size() < b->lanes, "a decode step carries fewer than L queued tokens");
        const size_t selected = token_budget - validated;
        PSI_REQUIRE(selected <= b->spec.size(), "token budget asks for %zu speculative tokens, %zu are stored",
                    selected, b->spec.size());
        PSI_REQUIRE(selected == 0 || (out->spec_tokens != nullptr && out->spec_tokens_capacity >= selected),
                    "spec token buffer holds %zu tokens, %zu are needed", out->spec_tokens_capacity, selected);
    }

    bool have_index = false;
    size_t token_index = 0, block_index = b->immutable_blocks.size();
    std::vector<uint32_t> tokens;
    auto visit = [&](BlockVec& block) -> bool {  // true = budget reached
        const size_t ready = b->ready(block);
        if (ready == 0) {
            ++block_index;
            return false;
        }
        if (!have_index) {
            have_index = true;
            token_index = block_index * b->n + b->cached(block) + b->scheduled(block);
        }
        const size_t take = std::min(ready, token_budget - tokens.size());
        const size_t from = block[0].ready_index;
        b->schedule(block, take);
        tokens.insert(tokens.end(), block[0].tokens.begin() + from, block[0].tokens.begin() + from + take);
        if (tokens.size() >= token_budget) return true;
        ++block_index;
        return false;
    };
    bool done = false;
    for (auto& block : b->semi_immutable_blocks)
        if ((done = visit(block))) break;
    if (!done)
        for (auto& block : b->mutable_blocks)
            if (visit(block)) break;

    out->epoch = b->epoch;
    out->num_spec_tokens = 0;
    out->window = 0;
    if (prefill) {
        tokens.insert(tokens.end(), b->queued.begin(), b->queued.begin() + lookahead);
        out->kind = PSI_HIP_QUERY_PREFILL;
        out->token_index = token_index;
        out->window = static_cast<uint32_t>(token_budget);
    } else {
        tokens.insert(tokens.end(), b->queued.begin(), b->queued.end());
        const size_t selected = token_budget - tokens.size();
        b->spec.resize(selected);
        out->kind = PSI_HIP_QUERY_DECODE;
        out->token_index = have_index ? token_index : b->num_cached() + b->num_scheduled();
        out->num_spec_tokens = selected;
        if (selected) copy_tokens(b->spec, out->spec_tokens);
    }
    out->num_tokens = tokens.size();
    copy_tokens(tokens, out->tokens);
    return PSI_HIP_OK;
}

int psi_hip_decoder_blocks_cancel(psi_hip_decoder_blocks* b, const psi_hip_query_tokens* q) {
    PSI_REQUIRE(b != nullptr, "blocks must not be null");
    if (int rc = check_query(b, q)) return rc;
    const size_t lookahead = b->lanes - 1;
    const size_t total = q->num_tokens > lookahead ? q->num_tokens - lookahead : 0;
    // Dry run first so that a mismatching query changes nothing.
    for (int pass = 0; pass < 2; ++pass) {
        size_t index_end = total;
        auto visit = [&](BlockVec& block) -> int {
            const size_t count = std::min(index_end, b->scheduled(block));
            const size_t index_start = index_end - count;
            for (size_t lane = 0; lane < b->lanes && count != 0; ++lane) {
                LaneBlock& lb = block[lane];
                if (pass == 0) {
                    PSI_REQUIRE(lb.ready_index - lb.scheduled_index >= count &&
                                    std::equal(q->tokens + index_start + lane, q->tokens + index_end + lane,
                                               lb.tokens.begin() + (lb.ready_index - count)),
                                "cancelled query does not match the scheduled tokens");
                } else {
                    lb.ready_index -= count;
                }
            }
            index_end = index_start;
            return PSI_HIP_OK;
        };
        for (auto it = b->mutable_blocks.rbegin(); it != b->mutable_blocks.rend() && index_end != 0; ++it)
            if (int rc = visit(*it)) return rc;
        for (auto it = b->semi_immutable_blocks.rbegin(); it != b->semi_immutable_blocks.rend() && index_end != 0; ++it)
            if (int rc = visit(*it)) return rc;
        PSI_REQUIRE(index_end == 0, "cancelled query covers more tokens than are scheduled");
    }
    return PSI_HIP_OK;
}

int psi_hip_decoder_blocks_commit(psi_hip_decoder_blocks* b, const psi_hip_query_tokens* q,
                                  const psi_hip_sampled_tokens* s) {
    PSI_REQUIRE(b != nullptr && s != nullptr, "blocks and sampled tokens must not be null");
    if (int rc = check_query(b, q)) return rc;
    PSI_REQUIRE(s->kind == q->kind, "sampled tokens kind does not match the query kind");
    PSI_REQUIRE(s->epoch == b->epoch, "sampled tokens epoch does not match the blocks' epoch");
    const size_t lookahead = b->lanes - 1;
    const std::vector<uint32_t> input(q->tokens, q->tokens + q->num_tokens);
    const size_t ready_window = input.size() > lookahead ? input.size() - lookahead : 0;
    {   // Dry run: the query's window must be the oldest scheduled tokens, lane by lane.
        size_t idx = 0;
        bool stop = false;
        auto check = [&](const BlockVec& block) -> bool {
            const size_t count = std::min(ready_window - idx, b->scheduled(block));
            for (size_t lane = 0; lane < b->lanes && count != 0; ++lane) {
                const LaneBlock& lb = block[lane];
                if (lb.ready_index - lb.scheduled_index < count || idx + count + lane > input.size() ||
                    !std::equal(input.begin() + idx + lane, input.begin() + idx + count + lane,
                                lb.tokens.begin() + lb.scheduled_index))
                    return false;
            }
            idx += count;
            stop = b->cached(block) + count != b->n;
            return true;
        };
        bool ok = true;
        for (auto it = b->semi_immutable_blocks.begin(); ok && !stop && it != b->semi_immutable_blocks.end(); ++it)
            ok = check(*it);
        for (auto it = b->mutable_blocks.begin(); ok && !stop && it != b->mutable_blocks.end(); ++it) ok = check(*it);
        PSI_REQUIRE(ok && idx == ready_window, "committed query does not match the scheduled tokens");
    }
    std::vector<uint32_t> queued_to_cached(input.begin() + ready_window, input.end());
    size_t queued_window = 0;
    if (q->kind == PSI_HIP_QUERY_DECODE) {
        PSI_REQUIRE(s->num_validated_tokens == 0 || s->validated_tokens != nullptr, "validated_tokens is null");
        PSI_REQUIRE(s->num_spec_tokens == 0 || s->spec_tokens != nullptr, "sampled spec_tokens is null");
        PSI_REQUIRE(s->num_validated_tokens <= q->num_spec_tokens &&
                        std::equal(s->validated_tokens, s->validated_tokens + s->num_validated_tokens, q->spec_tokens),
                    "validated tokens must equal a prefix of the speculative input suffix");
        PSI_REQUIRE(input.size() >= b->queued.size() &&
                        std::equal(b->queued.begin(), b->queued.end(), input.end() - b->queued.size()),
                    "decode query must end with the queued tokens");
        const size_t v = s->num_validated_tokens;
        const size_t with_sample = input.size() + v + 1;
        queued_window =
            std::min(input.size() + v, with_sample > lookahead ? with_sample - lookahead : 0) - ready_window;
        b->queued.insert(b->queued.end(), s->validated_tokens, s->validated_tokens + v);
        b->queued.push_back(s->sampled_token);
        b->queued.erase(b->queued.begin(), b->queued.begin() + queued_window);
        b->spec.assign(s->spec_tokens, s->spec_tokens + s->num_spec_tokens);
        queued_to_cached.insert(queued_to_cached.end(), s->validated_tokens, s->validated_tokens + v);
        queued_to_cached.push_back(s->sampled_token);
    }

    // Scheduled -> cached, front to back; a block whose every token is cached becomes immutable.
    size_t index_start = 0;
    bool stop = false;
    for (auto* blocks : {&b->semi_immutable_blocks, &b->mutable_blocks}) {
        while (!stop && !blocks->empty()) {
            BlockVec& block = blocks->front();
            const size_t index_end = index_start + std::min(ready_window - index_start, b->scheduled(block));
            if (!b->cache_tokens(block, input, index_start, index_end))
                return fail(PSI_HIP_ERR_INVALID_ARGUMENT, "committed query does not match the scheduled tokens");
            index_start = index_end;
            if (b->cached(block) != b->n) {
                stop = true;
            } else {
                b->immutable_blocks.push_back(std::move(block));
                blocks->pop_front();
            }
        }
        if (stop) break;
    }
    // Accepted drafts and the lanes' lookahead go straight from the queue into the cache.
    size_t extra_start = 0;
    while (!b->mutable_blocks.empty()) {
        BlockVec& block = b->mutable_blocks.front();
        const size_t num = std::min(queued_window - extra_start, b->n - block[0].tokens.size());
        const size_t extra_end = extra_start + num;
        if (num != 0) {
            b->push_tokens(block, queued_to_cached.data() + extra_start, num + lookahead);
            b->schedule(block, num);
            if (!b->cache_tokens(block, queued_to_cached, extra_start, extra_end))
                return fail(PSI_HIP_ERR_RUNTIME, "internal: accepted tokens do not line up with the block");
        }
        extra_start = extra_end;
        if (b->cached(block) != b->n) break;
        b->immutable_blocks.push_back(std::move(block));
        b->mutable_blocks.pop_front();
    }
    b->try_mark_ready();
    if (index_start != ready_window || extra_start != queued_window)
        return fail(PSI_HIP_ERR_RUNTIME, "internal: commit windows not consumed (%zu/%zu, %zu/%zu)", index_start,
                    ready_window, extra_start, queued_window);
    return PSI_HIP_OK;
}

int psi_hip_decoder_blocks_prepare_blocks(psi_hip_decoder_blocks* b, size_t* block_index, size_t* num_blocks,
                                          uint32_t* kv_page_ids, size_t capacity_ids) {
    PSI_REQUIRE(b != nullptr && block_index != nullptr && num_blocks != nullptr, "arguments must not be null");
    const size_t total = b->immutable_blocks.size() + b->semi_immutable_blocks.size() + b->mutable_blocks.size();
    PSI_REQUIRE(b->num_in_sync_blocks <= total, "num_in_sync_blocks exceeds the number of blocks");
    const size_t start = b->num_in_sync_blocks, count = total - start;
    *block_index = start;
    *num_blocks = count;
    if (kv_page_ids == nullptr) return PSI_HIP_OK;  // size query only, nothing marked as synced
    PSI_REQUIRE(capacity_ids >= b->lanes * count * b->pages_per_block,
                "page-id buffer holds %zu IDs, %zu are needed", capacity_ids, b->lanes * count * b->pages_per_block);
    size_t i = 0;
    auto emit = [&](const BlockVec& block) {
        if (i >= start) {
            for (size_t lane = 0; lane < b->lanes; ++lane)
                std::copy(block[lane].page_ids.begin(), block[lane].page_ids.end(),
                          kv_page_ids + (lane * count + (i - start)) * b->pages_per_block);
        }
        ++i;
    };
    for (const auto& block : b->immutable_blocks) emit(block);
    for (const auto& block : b->semi_immutable_blocks) emit(block);
    for (const auto& block : b->mutable_blocks) emit(block);
    b->num_in_sync_blocks = total;
    return PSI_HIP_OK;
}

int psi_hip_decoder_blocks_cancel_blocks(psi_hip_decoder_blocks* b, size_t block_index) {
    PSI_REQUIRE(b != nullptr, "blocks must not be null");
    PSI_REQUIRE(block_index <= b->num_in_sync_blocks, "cancelled sync starts past the synced blocks");
    b->num_in_sync_blocks = block_index;
    return PSI_HIP_OK;
}

int psi_hip_decoder_blocks_counts(const psi_hip_decoder_blocks* b, size_t* immutable_blocks,
                                  size_t* semi_immutable_blocks, size_t* mutable_blocks, size_t* in_sync_blocks) {
    PSI_REQUIRE(b != nullptr, "blocks must not be null");
    if (immutable_blocks) *immutable_blocks = b->immutable_blocks.size();
    if (semi_immutable_blocks) *semi_immutable_blocks = b->semi_immutable_blocks.size();
    if (mutable_blocks) *mutable_blocks = b->mutable_blocks.size();
    if (in_sync_blocks) *in_sync_blocks = b->num_in_sync_blocks;
    return PSI_HIP_OK;
}

int psi_hip_decoder_blocks_tokens(const psi_hip_decoder_blocks* b, uint32_t which, uint32_t* out, size_t capacity,
                                  size_t* count) {
    PSI_REQUIRE(b != nullptr && count != nullptr, "blocks and count must not be null");
    std::vector<uint32_t> v;
    auto add = [&](const BlockVec& block) {
        const LaneBlock& lb = block[0];
        if (which == PSI_HIP_TOKENS_CACHED) v.insert(v.end(), lb.tokens.begin(), lb.tokens.begin() + lb.scheduled_index);
        if (which == PSI_HIP_TOKENS_SCHEDULED)
            v.insert(v.end(), lb.tokens.begin() + lb.scheduled_index, lb.tokens.begin() + lb.ready_index);
        if (which == PSI_HIP_TOKENS_READY) v.insert(v.end(), lb.tokens.begin() + lb.ready_index, lb.tokens.end());
    };
    switch (which) {
        case PSI_HIP_TOKENS_CACHED:
        case PSI_HIP_TOKENS_SCHEDULED:
        case PSI_HIP_TOKENS_READY:
            for (const auto& block : b->immutable_blocks) add(block);
            for (const auto& block : b->semi_immutable_blocks) add(block);
            for (const auto& block : b->mutable_blocks) add(block);
            break;
        case PSI_HIP_TOKENS_QUEUED:
            v.assign(b->queued.begin(), b->queued.end());
            break;
        case PSI_HIP_TOKENS_SPEC:
            v = b->spec;
            break;
        default:
            return fail(PSI_HIP_ERR_INVALID_ARGUMENT, "unknown token class %u", which);
    }
    *count = v.size();
    if (out == nullptr) return PSI_HIP_OK;
    PSI_REQUIRE(capacity >= v.size(), "token buffer holds %zu tokens, %zu are needed", capacity, v.size());
    copy_tokens(v, out);
    return PSI_HIP_OK;
}

}  // extern "C"
