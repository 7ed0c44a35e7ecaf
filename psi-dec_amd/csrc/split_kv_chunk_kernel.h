// gfx950 split-KV map for prefill chunks: many query tokens of one request against one KV range,
// 2-byte K/V (bf16 / f16), head_dim 128 or 256, pages of 8 * 2^k tokens.  Same results as the
// multi-query map (semantics of
// crates/inference-backend-metal/src/components/metal/gqa_split_kv_tiled_q.metal:49-319), other
// decomposition: here the matrix cores and the LDS are the bound, not HBM.
//
// Work decomposition
//   one workgroup = one (row group, kv_head [, part of the query heads]).  A row group is a run of consecutive
//   Q-token tiles of one request whose kv_split rows start at the same key (the rows of one KV partition).  With
//   more than 5 query heads per KV head the heads are dealt to two or three workgroups.  The workgroup's query
//   columns, column c = token_in_group * heads + head, are dealt out 16 per multiplying wave: a wave keeps the
//   online-softmax state and the accumulators of its columns for the whole KV range, so wave states never merge.
//
//   Twelve waves: eight that multiply (two per SIMD) and four that load (one per SIMD), around four LDS stages of
//   32 keys.  A loading wave fetches its quarter of a tile into registers four tiles
//   ahead (the tiles come from other compute units' L2 slices or from HBM, two microseconds away under load),
//   stores it into the stage once every multiplying wave has said that it is through with the stage's previous
//   tile, and announces it; a multiplying wave waits for the four announcements of its next tile, multiplies, and
//   says so.  No barrier inside the range: the multiplying waves drift apart, and one wave's matrix work runs
//   beside another's softmax and operand reads.  Every wait on another wave's word gives up after
//   65536 polls: the wave then tells the host through MapArgs::status and waits no more, and the
//   multiplying waves store empty states for the workgroup's columns; no wave stays behind.
//
// Per 32-key tile and wave (16 columns)
//   QK^T  S[key][column] on v_mfma_f32_16x16x32 of the storage type: A = K rows from LDS (key 16 * b + i in row i of
//         key block b), B = the query columns, held in registers for the whole kernel.  A lane ends up with keys
//         16 * b + 4 * (lane / 16) + r, r = 0..3, b = 0, 1, of its column.
//   softmax  per column, in-lane over those 8 keys; masks only on tiles that touch the start of the range
//         or a column's causal limit.  The reference maximum of a column moves only when a tile
//         exceeds it by more than 2^8; a wave-wide vote guards the cross-lane maximum and the
//         rescaling of the accumulators, which therefore run a handful of times per range.
//         Probabilities stay below 2^8.  The row sum adds the probabilities as rounded for the product
//         (v_dot2_f32_f16 with ones), so that numerator and denominator carry the same weights.
//   PV    O^T[dim][column] += V^T[dim][key] * P^T[key][column] on v_mfma_f32_16x16x32_f16: B = the probabilities,
//         rounded once to f16 (11 significant bits; one bf16 term alone, 8 bits, costs the whole output tolerance,
//         and two bf16 terms cost half as many matrix instructions again), A = V^T read straight out of the
//         row-major V tile with the transposing LDS read of gfx950 (ds_read_b64_tr_b16: the 16 lanes of a quarter
//         wave hand in 16 addresses of 4 elements each, a 16 x 4 block, and get it back transposed - lane 4a + c
//         receives element c of the addresses a, a + 4, a + 8, a + 12), so no instruction of the kernel
//         transposes V.  The V tile is kept as f16 in LDS: bf16 pages are converted once per tile, to nearest, on
//         their way from the load registers into LDS (exact for 6.1e-5 <= |v| <= 65504; smaller magnitudes keep
//         an absolute spacing of 6e-8; larger ones become Inf, reach the accumulators as Inf or NaN, and are
//         reported to the host through MapArgs::status).  The accumulators keep a column per lane, so rescaling
//         needs no cross-lane traffic.
//
// LDS layout per stage
//   K    [32 keys][D] elements, 16-byte chunk index XOR (key % 16): the 16 lanes of an operand read (16 rows, one
//        chunk) then hit 16 different bank groups, and a row-wise store stays a permutation of its row.
//   V    [32 keys][D] f16, rows padded to D * 2 + 32 bytes: the four keys of a quarter wave's transposing read
//        (32 bytes each, 16 dims) then fall into different bank groups, and so do the eight keys of two quarters.
//   and thirteen words: tiles stored, per loading wave; tiles read, per multiplying wave; and one that says that
//   some wave's wait ran out (and four that nobody reads).
#pragma once
#include <atomic>

#include "split_kv_tiled_kernel.h"

namespace psi {

constexpr int kChunkKeys = 32;         // keys per KV tile
constexpr int kChunkWaves = 8;          // multiplying waves
constexpr int kChunkLoaders = 4;        // loading waves
constexpr int kChunkStages = 4;         // KV tiles in LDS
constexpr int kChunkWaveCols = 16;      // query columns of a multiplying wave
static_assert(kChunkWaves * kChunkWaveCols == kChunkCols, "128 query columns per workgroup");
constexpr uint32_t kNoRow = 0xffffffffu;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;  // 128-bit word that stays in registers

// Probabilities of 8 keys -> B operand of the 16x16x32 f16 contraction: one term, rounded to nearest.
__device__ __forceinline__ uint4 prob_operand_f16(const float (&p)[8]) {
    const f16x8_t h = {(_Float16)p[0], (_Float16)p[1], (_Float16)p[2], (_Float16)p[3],
                       (_Float16)p[4], (_Float16)p[5], (_Float16)p[6], (_Float16)p[7]};
    return __builtin_bit_cast(uint4, h);
}

// sum + the eight f16 values of `packed`, in f32.
__device__ __forceinline__ float add_f16x8(uint4 packed, float sum) {
    const f16x2_t ones = {(_Float16)1.0f, (_Float16)1.0f};
    sum = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, packed.x), ones, sum, false);
    sum = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, packed.y), ones, sum, false);
    sum = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, packed.z), ones, sum, false);
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, packed.w), ones, sum, false);
}

// max(a, b, c) in one instruction.  The logits are matrix-core results: a NaN among them (NaN in K or Q) ends up in
// the probabilities either way, so the operands need not be canonicalised first, as fmaxf would have them.
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// 8 elements of the storage type -> 8 f16.  bf16: widening is exact, the narrowing is exact inside the range of
// f16's normal numbers (see the header).
template <typename Tag>
__device__ __forceinline__ u32x4_t to_f16x8(u32x4_t w);
template <>
__device__ __forceinline__ u32x4_t to_f16x8<F16Tag>(u32x4_t w) { return w; }
template <>
__device__ __forceinline__ u32x4_t to_f16x8<BF16Tag>(u32x4_t w) {
    u32x4_t out;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float lo = __uint_as_float(w[i] << 16), hi = __uint_as_float(w[i] & 0xffff0000u);
        const f16x2_t h = {(_Float16)lo, (_Float16)hi};  // to nearest: what f16 cannot hold becomes Inf
        out[i] = __builtin_bit_cast(uint32_t, h);
    }
    return out;
}

__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) {
#pragma unroll
    for (int s = 1; s < 64; s <<= 1) v = min(v, (uint32_t)__shfl_xor((int)v, s, 64));
    return v;
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
#pragma unroll
    for (int s = 1; s < 64; s <<= 1) v = max(v, (uint32_t)__shfl_xor((int)v, s, 64));
    return v;
}

template <int D>
struct ChunkLds {
    static constexpr int kKBytes = kChunkKeys * D * 2;
    static constexpr int kVStride = D * 2 + 32;  // bytes per key row of the V tile
    static constexpr int kVtBytes = kChunkKeys * kVStride;
    static constexpr int kStageBytes = kKBytes + kVtBytes;
    static constexpr int kFlagsOffset = kChunkStages * kStageBytes;
    // tiles stored per loading wave [4], tiles read per multiplying wave [8], a wait ran out [1]
    static constexpr int bytes = kFlagsOffset + 64;
};

// kPage8: pages of eight tokens (a tile then spans four pages instead of one or two).
template <typename Tag, int D, bool kPage8>
__global__ __launch_bounds__(64 * (kChunkWaves + kChunkLoaders), 1) void split_kv_chunk_map(
    MapArgs a, const uint32_t* __restrict__ page_ids, const uint32_t* __restrict__ kv_splits,
    const uint32_t* __restrict__ req_slots, const uint16_t* __restrict__ q, const uint16_t* __restrict__ pages,
    const uint32_t* __restrict__ q_token_tiles, const uint32_t* __restrict__ flat_token_indices,
    const uint32_t* __restrict__ row_groups, uint32_t group_tiles, uint32_t num_groups, uint32_t head_subsets) {
    resolve_active(a);
    static_assert(D == 256 || D == 128, "head_dim 128 or 256");
    constexpr int kKSteps = D / 32;
    constexpr int kDimBlocks = D / 16;
    constexpr int kRowChunks = D / 8;                      // 16-byte chunks per key row
    constexpr int kSubs = 64 * kChunkLoaders / kRowChunks;  // keys that the loading threads cover at a time (8 or 16)
    constexpr int kLoads = kChunkKeys / kSubs;               // 128-bit loads per loading thread and operand (4 or 2)
    constexpr int kKBytes = ChunkLds<D>::kKBytes;
    constexpr int kVStride = ChunkLds<D>::kVStride;
    constexpr int kStageBytes = ChunkLds<D>::kStageBytes;
    constexpr float kSlack = 8.0f;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    // Progress words, addressed as LDS: through a generic pointer a volatile access becomes a flat one, which
    // counts as a global load too, and waiting for its value would wait for every tile load in flight.
    typedef volatile __attribute__((address_space(3))) uint32_t* LdsWords;
    const LdsWords landed = (LdsWords)(lds + ChunkLds<D>::kFlagsOffset);  // tiles stored, per loading wave
    const LdsWords done = landed + kChunkLoaders;                          // tiles read, per multiplying wave
    const LdsWords failed = done + kChunkWaves;                            // some wave's wait ran out

    const uint32_t TS = a.rows_per_split_head;
    const uint32_t subset = blockIdx.x % head_subsets;
    const uint32_t kv_head = (blockIdx.x / head_subsets) % a.walk.hkv;
    const uint32_t group = blockIdx.x / (head_subsets * a.walk.hkv);
    const uint32_t heads_per_subset = (a.group + head_subsets - 1) / head_subsets;
    const uint32_t head_first = kv_head * a.group + subset * heads_per_subset;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t mt = lane & 15, mc = lane >> 4;
    if (group >= num_groups || subset * heads_per_subset >= a.group) return;
    const uint32_t G = min(heads_per_subset, a.group - subset * heads_per_subset);

    const uint32_t* rows = row_groups + (uint64_t)group * group_tiles;
    const uint32_t my_row = lane < group_tiles ? rows[lane] : kNoRow;
    const bool my_row_ok = my_row != kNoRow && my_row < a.num_active_kv_splits;
    const uint32_t num_tiles = __builtin_amdgcn_readfirstlane(__popcll(__ballot(my_row_ok)));
    if (num_tiles == 0) return;
    const uint32_t row0 = __builtin_amdgcn_readfirstlane(rows[0]);
    if (row0 >= a.num_active_kv_splits) return;
    const uint32_t q_tile0 = kv_splits[row0 * 3];
    if (q_tile0 >= a.num_active_q_token_tiles || q_tile0 + num_tiles > a.num_active_q_token_tiles) return;
    const uint32_t kv_begin = kv_splits[row0 * 3 + 1];
    const uint32_t kv_end_max = __builtin_amdgcn_readfirstlane(
        wave_max_u32(my_row_ok && lane < num_tiles ? kv_splits[my_row * 3 + 2] : 0u));
    const uint32_t flat_begin = q_token_tiles[q_tile0 * 2];
    const uint32_t flat_end = q_token_tiles[(q_tile0 + num_tiles - 1) * 2 + 1];
    if (flat_end <= flat_begin || flat_end > a.num_active_tokens || kv_end_max <= kv_begin) return;
    const uint32_t ncols = (flat_end - flat_begin) * G;
    if (ncols > (uint32_t)kChunkCols || flat_end - flat_begin > num_tiles * TS) return;
    const uint32_t req_slot = req_slots[flat_begin];
    const uint32_t key_base0 = kv_begin & ~(uint32_t)(kChunkKeys - 1);
    const uint32_t num_kv_tiles = (kv_end_max - key_base0 + kChunkKeys - 1) / kChunkKeys;

    if (tid < kChunkLoaders + kChunkWaves + 1) landed[tid] = 0u;
    __syncthreads();
    // Both roles poll with the word of wave (lane % count) in each lane and a wave-wide vote.  A wait that runs out
    // marks the workgroup's results as void (every multiplying wave looks at `failed` when it is through, tells the
    // host and stores empty states); the wave itself goes on without waiting any more, so that nothing of this
    // costs the tile loops a branch.
    // The bound is a constant and the loop the only one, so that it stays the plain unrolled poll: a run-time bound
    // in it, a second loop or a second path next to it each cost 1 to 5 % of the launch.
    bool impatient = false;
    auto wait_all_above = [&](LdsWords words, uint32_t count_mask, uint32_t value) __attribute__((always_inline)) {
        bool there = impatient;
        if (!impatient) {
            for (uint32_t polls = 0; polls < kDefaultWaitPolls; ++polls) {
                there = __all(words[lane & count_mask] > value);
                if (there) break;
                __builtin_amdgcn_s_sleep(1);
            }
        }
        if (!there) {
            // Only an LDS word here: a global store on this path would make every count of outstanding loads that
            // the compiler keeps for the loading waves a guess, and its partial waits full ones.
            impatient = true;  // `there` stays true from here on: the wave waits no more
            if (lane == 0) *failed = 1u;
        }
        asm volatile("" ::: "memory");
    };

    if (wave >= (uint32_t)kChunkWaves) {
        // =========================== a loading wave ===========================
        // A loading thread takes one 16-byte chunk of the keys sub, sub + kSubs, ... of every tile, so that a wave's
        // load covers whole rows (two of 512 bytes, or four of 256).
        const uint32_t lw = wave - kChunkWaves;
        const uint32_t log2p = 31 - __builtin_clz(a.walk.tokens_per_page);
        const uint32_t page_mask = a.walk.tokens_per_page - 1;
        const uint32_t* table_row = page_ids + ((uint64_t)req_slot * a.walk.num_layers + a.layer) *
                                                          a.walk.num_blocks * a.walk.ids_per_block;
        const uint32_t last_page = (kv_end_max - 1) >> log2p;
        const uint64_t page_bytes = a.walk.page_elems * 2;
        const unsigned char* base = reinterpret_cast<const unsigned char*>(pages);
        // Page ids come through the scalar cache: a vector load would queue behind the tile loads in flight, and
        // waiting for it would wait for all of them.  A tile's ids are fetched one step before its loads are
        // issued.  Tiles past the end of the range are clamped to the last one, so that loads stay unconditional.
        typedef const __attribute__((address_space(4))) uint32_t* ConstantIds;
        const ConstantIds ids_row = (ConstantIds)(uintptr_t)table_row;
        constexpr int kIds = kPage8 ? 4 : 2;  // pages under a tile's 32 keys
        struct TileIds {
            uint32_t id[kIds];
        };
        auto tile_key = [&](uint32_t t) { return key_base0 + min(t, num_kv_tiles - 1) * kChunkKeys; };
        auto fetch_ids = [&](uint32_t t) -> TileIds {
            const uint32_t kb = tile_key(t);
            TileIds ids;
#pragma unroll
            for (int j = 0; j < kIds; ++j) ids.id[j] = ids_row[min((kb + (kChunkKeys / kIds) * j) >> log2p, last_page)];
            return ids;
        };
        const uint32_t ltid = tid - 64 * kChunkWaves;
        const uint32_t ld_chunk = ltid % kRowChunks;
        const uint32_t ld_sub = ltid / kRowChunks;  // 0 .. kSubs - 1; load i takes key ld_sub + kSubs * i of the tile
        // The keys of one load of a wave lie in one run of eight (ld_sub / 8 is the same for the whole wave): the
        // run's rows are found with scalar arithmetic, and a lane adds a constant.
        const uint32_t run_first = kSubs == 8 ? 0u : __builtin_amdgcn_readfirstlane(ld_sub & ~7u);
        const uint32_t lane_off = (ld_sub & 7) * (D * 2) + ld_chunk * 16;
        const uint32_t k_off = kv_head * a.walk.tokens_per_page * (D * 2) + lane_off;
        const uint32_t v_off = (a.walk.hkv + kv_head) * a.walk.tokens_per_page * (D * 2) + lane_off;
        struct Staging {
            u32x4_t k[kLoads], v[kLoads];
        };
        auto issue_loads = [&](uint32_t t, const TileIds& ids) __attribute__((always_inline)) -> Staging {
            const uint32_t kb = tile_key(t);
            Staging st;
            const unsigned char* rows_of_run[kLoads];
#pragma unroll
            for (int i = 0; i < kLoads; ++i) {
                const uint32_t first = kSubs * i + run_first;  // of the tile's keys
                uint32_t id;
                if constexpr (kSubs == 8 || !kPage8) id = ids.id[(kSubs * i) / (kChunkKeys / kIds)];
                else id = run_first == 0 ? ids.id[2 * i] : ids.id[2 * i + 1];
                rows_of_run[i] = base + id * page_bytes + (uint64_t)((kb + first) & page_mask) * (D * 2);
            }
#pragma unroll
            for (int i = 0; i < kLoads; ++i) st.k[i] = *reinterpret_cast<const u32x4_t*>(rows_of_run[i] + k_off);
#pragma unroll
            for (int i = 0; i < kLoads; ++i) st.v[i] = *reinterpret_cast<const u32x4_t*>(rows_of_run[i] + v_off);
            return st;
        };
        // Where this wave says that a tile is stored.  A harness that wants to see waits run out (MapArgs::
        // mute_loaders) has the word written where no wave looks.
        const LdsWords announce = a.mute_loaders ? failed + 1 + lw : landed + lw;
        uint32_t k_store[kLoads], v_store[kLoads];
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            const uint32_t key = ld_sub + kSubs * i;
            k_store[i] = key * (D * 2) + ((ld_chunk ^ (key & 15)) * 16);
            v_store[i] = kKBytes + key * kVStride + ld_chunk * 16;
        }
        auto store_tile = [&](uint32_t it, Staging& st) __attribute__((always_inline)) {
            if (it >= (uint32_t)kChunkStages) wait_all_above(done, kChunkWaves - 1, it - kChunkStages);
            unsigned char* stage = lds + (it % kChunkStages) * kStageBytes;
            const uint32_t kb = key_base0 + it * kChunkKeys;
            const bool edge = kb < kv_begin || kb + kChunkKeys > kv_end_max;  // first or last tile of the range
#pragma unroll
            for (int i = 0; i < kLoads; ++i) *reinterpret_cast<u32x4_t*>(stage + k_store[i]) = st.k[i];
#pragma unroll
            for (int i = 0; i < kLoads; ++i) {
                u32x4_t w = to_f16x8<Tag>(st.v[i]);
                const uint32_t token = kb + ld_sub + kSubs * i;
                // V rows outside the range are zeroed: their probability is 0 but their bytes may be NaN / Inf
                if (edge && (token < kv_begin || token >= kv_end_max)) w = u32x4_t{0u, 0u, 0u, 0u};
                *reinterpret_cast<u32x4_t*>(stage + v_store[i]) = w;
            }
            if (lane == 0) *announce = it + 1;  // behind the stores in the LDS queue
        };
        // Four tiles of loads in flight per wave (one register set per stage): the tiles come from the other
        // compute units' L2 slices or from HBM, two microseconds away under load, and a tile is used up in less
        // than one.
        Staging st_a = issue_loads(0, fetch_ids(0));
        Staging st_b = issue_loads(1, fetch_ids(1));
        Staging st_c = issue_loads(2, fetch_ids(2));
        Staging st_d = issue_loads(3, fetch_ids(3));
        TileIds ids = fetch_ids(4);
        auto step = [&](uint32_t it, Staging& st) __attribute__((always_inline)) {
            if (it < num_kv_tiles) store_tile(it, st);
            st = issue_loads(it + kChunkStages, ids);
            ids = fetch_ids(it + kChunkStages + 1);
        };
        for (uint32_t it = 0; it < num_kv_tiles; it += 4) {
            step(it, st_a);
            step(it + 1, st_b);
            step(it + 2, st_c);
            step(it + 3, st_d);
        }
        return;
    }

    // =========================== a multiplying wave ===========================
    const uint32_t c = wave * kChunkWaveCols + mt;
    const bool used = c < ncols;
    uint32_t lim = 0;
    uint64_t part_row = 0;
    uint4 qreg[kKSteps];
    {
        const uint32_t t = used ? c / G : 0u, h = used ? c % G : 0u;
        const uint32_t m = t / TS, r = t % TS;
        const uint32_t row = rows[m];
        if (used) {
            lim = min(kv_splits[row * 3 + 2], flat_token_indices[flat_begin + t] + 1);
            part_row = ((uint64_t)row * a.hq + head_first + h) * TS + r;
        }
        const uint16_t* q_row = q + ((uint64_t)(flat_begin + t) * a.hq + head_first + h) * D + mc * 8;
#pragma unroll
        for (int ks = 0; ks < kKSteps; ++ks)
            qreg[ks] = used ? *reinterpret_cast<const uint4*>(q_row + ks * 32) : make_uint4(0, 0, 0, 0);
    }
    const uint32_t wave_lo = __builtin_amdgcn_readfirstlane(wave_min_u32(used ? lim : 0xffffffffu));
    const uint32_t wave_hi = __builtin_amdgcn_readfirstlane(wave_max_u32(lim));
    // tiles that hold a visible key of this wave
    const uint32_t my_tiles = wave_hi > key_base0 ? min(num_kv_tiles, (wave_hi - key_base0 + kChunkKeys - 1) / kChunkKeys) : 0u;

    const uint32_t k_row0 = mt * (D * 2);
    const uint32_t vt_base = (4 * mc + (mt >> 2)) * kVStride + (mt & 3) * 8;
    float run_max = -INFINITY, lane_sum = 0.0f;
    f32x4_t o[kDimBlocks];
#pragma unroll
    for (int db = 0; db < kDimBlocks; ++db) o[db] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

    constexpr int kAhead = kKSteps < 4 ? kKSteps : 4;  // k-steps between an operand's read and its product
    for (uint32_t it = 0; it < my_tiles; ++it) {
        wait_all_above(landed, kChunkLoaders - 1, it);
        const unsigned char* kbuf = lds + (it % kChunkStages) * kStageBytes;
        const unsigned char* vbuf = kbuf + kKBytes;
        const uint32_t kb = key_base0 + it * kChunkKeys;
        const bool masked = !(kb >= kv_begin && kb + kChunkKeys <= wave_lo);
        f32x4_t s0 = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f}, s1 = s0;
        uint4 k0[kKSteps], k1[kKSteps];
        auto read_k = [&](int ks) __attribute__((always_inline)) {
            const uint32_t off = k_row0 + (((4 * ks + mc) ^ mt) * 16);
            k0[ks] = *reinterpret_cast<const uint4*>(kbuf + off);
            k1[ks] = *reinterpret_cast<const uint4*>(kbuf + off + 16 * (D * 2));
        };
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < kAhead; ++ks) read_k(ks);
#pragma unroll
        for (int ks = 0; ks < kKSteps; ++ks) {
            s0 = mfma_16x16x32<Tag>(k0[ks], qreg[ks], s0);
            s1 = mfma_16x16x32<Tag>(k1[ks], qreg[ks], s1);
            if (ks + kAhead < kKSteps) read_k(ks + kAhead);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, 2 * kAhead, 0);  // the first reads
#pragma unroll
        for (int ks = 0; ks < kKSteps - kAhead; ++ks) {
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);  // two products
            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // the reads kAhead steps on
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 2 * kAhead, 0);
        __builtin_amdgcn_sched_barrier(0);
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = j < 4 ? s0[j] : s1[j - 4];
        if (masked) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t token = kb + 16 * (j >> 2) + 4 * mc + (j & 3);
                if (token < kv_begin || token >= lim) v[j] = -INFINITY;
            }
        }
        float m = max3(max3(v[0], v[1], v[2]), max3(v[3], v[4], v[5]), fmaxf(v[6], v[7])) * a.scale_log2;
        if (__any(m > run_max + kSlack)) {
            m = fmaxf(m, __shfl_xor(m, 16, 64));
            m = fmaxf(m, __shfl_xor(m, 32, 64));
            if (m > run_max + kSlack) {
                const float alpha = run_max > -INFINITY ? __builtin_amdgcn_exp2f(run_max - m) : 0.0f;
                run_max = m;
                lane_sum *= alpha;
#pragma unroll
                for (int db = 0; db < kDimBlocks; ++db)
#pragma unroll
                    for (int r = 0; r < 4; ++r) o[db][r] *= alpha;
            }
        }
        const float neg_ref = run_max > -INFINITY ? -run_max : 0.0f;
        float p[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) p[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(v[j], a.scale_log2, neg_ref));
        const uint4 pb = prob_operand_f16(p);
        lane_sum = add_f16x8(pb, lane_sum);
#pragma unroll
        for (int g = 0; g < kDimBlocks; g += 4) {
            uint4 vt[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const unsigned char* src = vbuf + vt_base + (g + i) * 32;
                const uint2 lo = lds_read_tr16_b64(src), hi = lds_read_tr16_b64(src + 16 * kVStride);
                vt[i] = make_uint4(lo.x, lo.y, hi.x, hi.y);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) o[g + i] = mfma_16x16x32<F16Tag>(vt[i], pb, o[g + i]);
        }
        if (lane == 0) done[wave] = it + 1;  // behind this tile's reads in the LDS queue
    }
    if (lane == 0) done[wave] = 0xffffffffu;

    lane_sum += __shfl_xor(lane_sum, 16, 64);
    lane_sum += __shfl_xor(lane_sum, 32, 64);
    // A V element that f16 cannot hold has reached the accumulators as Inf or NaN (the conversion rounds to nearest,
    // so that it overflows instead of saturating): the host is told, and the rows stay as they are, visibly wrong.
    {
        float probe = 0.0f;
#pragma unroll
        for (int db = 0; db < kDimBlocks; ++db)
#pragma unroll
            for (int r = 0; r < 4; ++r) probe = __builtin_fmaf(o[db][r], 0.0f, probe);
        if (__any(lim != 0 && probe != probe) && lane == 0)
            __hip_atomic_store(a.status + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    if (*failed != 0u) {  // some wave's wait ran out: the host is told, and the columns get empty states
        if (lane == 0) __hip_atomic_store(a.status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        run_max = -INFINITY;
        lane_sum = 0.0f;
#pragma unroll
        for (int db = 0; db < kDimBlocks; ++db) o[db] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    }
    if (lim != 0) {
        if (mc == 0) {
            a.part_max[part_row] = run_max;
            a.part_sum[part_row] = lane_sum;
        }
        float* dst = a.part_acc + part_row * D + mc * 4;
#pragma unroll
        for (int db = 0; db < kDimBlocks; ++db)
            *reinterpret_cast<float4*>(dst + db * 16) = make_float4(o[db][0], o[db][1], o[db][2], o[db][3]);
    }
}

template <typename Tag, int D>
inline int launch_chunk_map_typed(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a, const uint32_t* row_groups,
                                  uint32_t group_tiles, uint32_t num_groups) {
    const uint32_t subsets = chunk_head_subsets(g.group);
    const dim3 grid(num_groups * g.hkv * subsets);
    const bool page8 = g.tokens_per_page == 8;
    auto* kernel = page8 ? &split_kv_chunk_map<Tag, D, true> : &split_kv_chunk_map<Tag, D, false>;
    // The kernel's LDS is above the default limit of a launch; the limit is raised once per GPU and kernel (a
    // function's attributes belong to the device it is loaded on).
    static std::atomic<uint64_t> raised_on[2] = {{0}, {0}};
    const uint64_t device_bit = 1ull << (ctx->device & 63);
    if ((raised_on[page8].load(std::memory_order_relaxed) & device_bit) == 0) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                ChunkLds<D>::bytes) != hipSuccess)
            return PSI_HIP_ERR_UNSUPPORTED;
        raised_on[page8].fetch_or(device_bit, std::memory_order_relaxed);
    }
    hipLaunchKernelGGL(kernel, grid, dim3(64 * (kChunkWaves + kChunkLoaders)), ChunkLds<D>::bytes, ctx->stream, a,
                       a.walk.page_ids, a.kv_splits, a.req_slots, reinterpret_cast<const uint16_t*>(a.q),
                       reinterpret_cast<const uint16_t*>(a.kv_pages), a.q_token_tiles, a.flat_token_indices, row_groups,
                       group_tiles, num_groups, subsets);
    return PSI_HIP_OK;
}

}  // namespace psi
