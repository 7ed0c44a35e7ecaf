// gfx950 split-KV map for prefill chunks: many query tokens of one request against one KV range,
// 2-byte K/V (bf16 / f16), head_dim 128 or 256, pages of 8 * 2^k tokens.  Same results as the
// multi-query map (semantics of
// crates/inference-backend-metal/src/components/metal/gqa_split_kv_tiled_q.metal:49-319), other
// decomposition: here the matrix cores and the LDS are the bound, not HBM.
//
// Work decomposition
//   one work item = one (row group, kv_head [, part of the query heads]); the launch is one workgroup per compute
//   unit, and a workgroup takes items until none is left (see the kernel at the end of this file).  A row group is
//   a run of consecutive Q-token tiles of one request whose kv_split rows start at the same key (the rows of one KV
//   partition).  With more than 5 query heads per KV head the heads are dealt to two or three items.  An item's query
//   columns, column c = token_in_group * heads + head, are dealt out 32 per wave, as two blocks of 16: a wave keeps
//   the online-softmax state and the accumulators of its columns for the whole KV range, so wave states never merge.
//
//   Eight waves, two per SIMD, each with half of the SIMD's registers.  Every operand of every product is read
//   from LDS, and an operand read serves both column blocks of a wave, so a tile's K and V cross the LDS port once
//   per 32 columns.  With 16 columns per wave (and then room for waves that only load) the same kernel's time
//   followed its LDS traffic: taking the loading waves' stores away, or their loads, each bought back a tenth of
//   the launch, and the products alone ran as long as the tile reads take at the LDS port's rate.  With one wave
//   per SIMD nothing hides the latencies of a wave's own chain (operand reads, matrix results, exponentials);
//   with two, each fills the other's gaps.
//
//   A KV tile is 16 KiB of K and 16 KiB of V: 32 keys at head_dim 256, 64 at head_dim 128.  No wave only loads:
//   every wave fetches an eighth of the rows of K and of V of every tile.  K goes straight to LDS
//   with `global_load_lds_dwordx4`, which moves 16 bytes per lane from a per-lane global address to LDS address
//   M0 + 16 * lane with no register in between, three tiles ahead, into a ring of four K tiles.  V goes through
//   registers, two tiles ahead (two register sets, taken in turn), where bf16 becomes f16, into a ring of two V
//   tiles.  One barrier per tile, B(t): before it a wave has stored its V rows of tile t and seen its K rows of
//   tile t + 1 land (a wave's loads complete in the order of their issue); behind it everybody has, and every
//   wave is through with tile t - 1.  No wait between waves other than the barrier, so none that could run out.
//
// Per tile and wave (2 x 16 columns), for each 32 keys of the tile
//   QK^T  S[key][column] on v_mfma_f32_16x16x32 of the storage type: A = K rows from LDS (key 16 * b + i in row i of
//         key block b), B = the query columns: the first block's held in registers for the whole kernel, the second
//         block's too at head_dim 128, and read from LDS with the K operands at head_dim 256 (64 registers of
//         queries next to 128 accumulators and the V rows under way are more than a wave has).  A lane ends up with keys 16 * b + 4 * (lane / 16) + r,
//         r = 0..3, b = 0, 1, of its column.
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
//         transposes V.  The V tile is kept as f16 in LDS: bf16 rows are converted once per tile, to nearest, by
//         the wave that fetched them (exact for 6.1e-5 <= |v| <= 65504; smaller magnitudes keep
//         an absolute spacing of 6e-8; larger ones become Inf, reach the accumulators as Inf or NaN, and are
//         reported to the host through MapArgs::status).  The accumulators keep a column per lane, so rescaling
//         needs no cross-lane traffic.
//
// LDS layout
//   K    four tiles of [32 or 64 keys][D] elements, 16-byte chunk index XOR (key % 16): the 16 lanes of an operand read
//        (16 rows, one chunk) then hit 16 different bank groups.  (The loads write 1 KiB in lane order, so the
//        layout can permute 16-byte chunks within a row, through the choice of each lane's global address, but
//        cannot pad rows.)
//   V    two tiles of [32 or 64 keys][D] f16, 32-byte chunk index XOR (key % 8): the four keys of a quarter wave's
//        transposing read (32 bytes each, 16 dims) then fall into different bank groups, and so do the eight keys
//        of two quarters.
//   Q    at head_dim 256, the second column block's query operands, 8 KiB per wave.
#pragma once
#include <algorithm>
#include <atomic>
#include <type_traits>

#include "split_kv_tiled_kernel.h"

namespace psi {

// Keys per KV tile: 32 at head_dim 256, 64 at head_dim 128 (the same 16 KiB of K and of V, and as many matrix
// instructions between two barriers; with 32 keys at head_dim 128 a tile's fixed costs - barrier, first operand reads,
// the way from the last product of K * Q^T to the first of V^T * P^T - weighed twice as much).
template <int D>
constexpr int kChunkKeysOf = (int)chunk_tile_keys(D);
constexpr int kChunkColBlocks = 2;  // 16-column blocks of a wave
constexpr int kChunkWaves = 8;
constexpr int kChunkStages = 4;   // K tiles in LDS
constexpr int kChunkVStages = 2;  // V tiles in LDS
constexpr int kChunkWaveCols = 16 * kChunkColBlocks;
static_assert(kChunkWaves * kChunkWaveCols == kChunkCols, "the workgroup's query columns");
constexpr uint32_t kNoRow = 0xffffffffu;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;  // 128-bit word that stays in registers

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

// 16 bytes per lane from rows + lane_offset to LDS address lds_dst + 16 * lane.  `rows` and `lds_dst` are the same
// in every lane (scalar registers).  Assembly, and so are the waits for these loads: the compiler does not know that
// they write LDS, and where it does (the builtin) it waits for every outstanding one before any LDS read, which
// would undo the prefetch.
__device__ __forceinline__ void dma_16_bytes_per_lane(uint32_t lds_dst, const void* rows, uint32_t lane_offset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_dst), "v"(lane_offset), "s"(rows)
                 : "memory", "m0");
}

template <int D>
struct ChunkLds {
    static constexpr int kKBytes = kChunkKeysOf<D> * D * 2;  // a tile of K, and of V
    static constexpr int kVOffset = kChunkStages * kKBytes;
    static constexpr int kQOffset = kVOffset + kChunkVStages * kKBytes;
    // k-steps of a wave's second column block whose query operands live here: all of them at head_dim 256 (128
    // accumulators + 64 registers of queries + the V rows under way are more than a wave has), none at 128
    static constexpr int kQSteps = D == 256 ? D / 32 : 0;
    static constexpr int bytes = kQOffset + kChunkWaves * kQSteps * 1024;
};

// One work item: (row group, kv_head, part of the query heads) = item / (head_subsets * hkv), item / head_subsets %
// hkv, item % head_subsets.  `next_item` (thread 0's) and `claimed`: see the kernel below.
template <typename Tag, int D, bool kTable>
__device__ __forceinline__ void chunk_map_item(
    const MapArgs& a, const uint32_t* __restrict__ page_ids, const uint32_t* __restrict__ kv_splits,
    const uint32_t* __restrict__ req_slots, const uint16_t* __restrict__ q, const uint16_t* __restrict__ pages,
    const uint32_t* __restrict__ q_token_tiles, const uint32_t* __restrict__ flat_token_indices,
    const uint32_t* __restrict__ row_groups, uint32_t group_tiles, uint32_t num_groups, uint32_t head_subsets,
    uint32_t item, uint32_t& next_item, bool& claimed) {
    static_assert(D == 256 || D == 128, "head_dim 128 or 256");
    constexpr int NB = kChunkColBlocks;
    constexpr int kKSteps = D / 32;
    constexpr int kDimBlocks = D / 16;
    constexpr int kRowBytes = D * 2;
    constexpr int kRowChunks = D / 8;                    // 16-byte chunks per key row: 32 or 16
    constexpr int kRowsPerLoad = 64 / kRowChunks;        // key rows that one load of a wave covers: 2 or 4
    constexpr int kKeys = kChunkKeysOf<D>;
    constexpr int kSub = kKeys / 32;                     // 32-key halves of a tile (what one V^T * P^T product spans)
    constexpr int kKeyBlocks = kKeys / 16;               // 16-key blocks of a tile (what one K * Q^T product spans)
    constexpr int kWaveRows = kKeys / kChunkWaves;       // rows of K, and of V, that a wave fetches per tile: 4 or 8
    constexpr int kLoads = kWaveRows / kRowsPerLoad;     // loads per wave, tile and operand: 2 or 1
    constexpr int kKBytes = ChunkLds<D>::kKBytes;
    constexpr int kVOffset = ChunkLds<D>::kVOffset;
    constexpr int kQSteps = ChunkLds<D>::kQSteps;
    constexpr bool kQInLds = kQSteps != 0;
    static_assert(kQSteps == kKSteps || kQSteps == 0, "the second block's queries live in LDS, or in registers");
    // k-steps of the second block whose queries are in registers.  (At head_dim 256 two of the eight fit instead of
    // the second set of operand registers below, and bought less than that set does; three spill inside the loop.)
    constexpr int kQ1Regs = kQInLds ? 0 : kKSteps;
    constexpr float kSlack = 8.0f;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const uint32_t TS = a.rows_per_split_head;
    const uint32_t subset = item % head_subsets;
    const uint32_t kv_head = (item / head_subsets) % a.walk.hkv;
    const uint32_t group = item / (head_subsets * a.walk.hkv);
    const uint32_t heads_per_subset = (a.group + head_subsets - 1) / head_subsets;
    const uint32_t head_first = kv_head * a.group + subset * heads_per_subset;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t mt = lane & 15, mc = lane >> 4;
    // (every exit before the tile loop is taken by the whole workgroup or by none of it)
    if (group >= num_groups || subset * heads_per_subset >= a.group) return;
    const uint32_t G = min(heads_per_subset, a.group - subset * heads_per_subset);

    // (kTable false: no table, every kv_split row is a group of its own, group_tiles is 1)
    const uint32_t* rows = row_groups + (uint64_t)group * group_tiles;
    auto row_of = [&](uint32_t i) -> uint32_t { return kTable ? rows[i] : group; };
    const uint32_t my_row = lane < group_tiles ? row_of(lane) : kNoRow;
    const bool my_row_ok = my_row != kNoRow && my_row < a.num_active_kv_splits;
    const uint32_t num_tiles = __builtin_amdgcn_readfirstlane(__popcll(__ballot(my_row_ok)));
    if (num_tiles == 0) return;
    const uint32_t row0 = __builtin_amdgcn_readfirstlane(row_of(0));
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
    const uint32_t key_base0 = kv_begin & ~(uint32_t)(kKeys - 1);
    const uint32_t num_kv_tiles = (kv_end_max - key_base0 + kKeys - 1) / kKeys;

    // ---------------- the wave's columns ----------------
    // The partial row of column block j of this lane's column: (row of the tile's split, head, token in the tile).
    // Worked out where it is needed, at either end of the kernel, rather than kept in registers through the loop.
    auto column_of = [&](int j, uint32_t* t, uint32_t* h) -> bool {
        const uint32_t c = wave * kChunkWaveCols + 16 * j + mt;
        *t = c < ncols ? c / G : 0u;
        *h = c < ncols ? c % G : 0u;
        return c < ncols;
    };
    bool used[NB];
    uint32_t lim[NB];
    unsigned char* q_lds = lds + ChunkLds<D>::kQOffset + wave * (kQSteps * 1024) + lane * 16;
    uint4 qreg[kKSteps];                     // the first block's
    uint4 qreg1[kQ1Regs > 0 ? kQ1Regs : 1];  // the second block's, as far as they live in registers
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        uint32_t t, h;
        used[j] = column_of(j, &t, &h);
        lim[j] = 0;
        if (used[j]) lim[j] = min(kv_splits[row_of(t / TS) * 3 + 2], flat_token_indices[flat_begin + t] + 1);
        const uint16_t* q_row = q + ((uint64_t)(flat_begin + t) * a.hq + head_first + h) * D + mc * 8;
#pragma unroll
        for (int ks = 0; ks < kKSteps; ++ks) {
            const uint4 operand = used[j] ? *reinterpret_cast<const uint4*>(q_row + ks * 32) : make_uint4(0, 0, 0, 0);
            if (j == 0) qreg[ks] = operand;
            else if (ks < kQ1Regs) qreg1[ks] = operand;
            else *reinterpret_cast<uint4*>(q_lds + ks * 1024) = operand;
        }
    }
    uint32_t lo = 0xffffffffu, hi = 0;
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        lo = min(lo, used[j] ? lim[j] : 0xffffffffu);
        hi = max(hi, lim[j]);
    }
    const uint32_t wave_lo = __builtin_amdgcn_readfirstlane(wave_min_u32(lo));
    const uint32_t wave_hi = __builtin_amdgcn_readfirstlane(wave_max_u32(hi));
    // tiles that hold a visible key of this wave, and of any wave of the workgroup
    const uint32_t my_tiles =
        wave_hi > key_base0 ? min(num_kv_tiles, (wave_hi - key_base0 + kKeys - 1) / kKeys) : 0u;
    uint32_t* tile_counts = reinterpret_cast<uint32_t*>(lds);  // (where the first tile will land)
    if (lane == 0) tile_counts[wave] = my_tiles;
    __syncthreads();
    const uint32_t group_kv_tiles =
        __builtin_amdgcn_readfirstlane(wave_max_u32(lane < (uint32_t)kChunkWaves ? tile_counts[lane] : 0u));
    __syncthreads();
    // None of the loads above may be outstanding when the tile loads begin: the compiler's waits count the loads it
    // knows of, and the tile loads are not among them.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    // ---------------- the wave's share of the tile loads ----------------
    const uint32_t log2p = 31 - __builtin_clz(a.walk.tokens_per_page);
    const uint32_t page_mask = a.walk.tokens_per_page - 1;
    const uint32_t* table_row = page_ids + ((uint64_t)req_slot * a.walk.num_layers + a.layer) * a.walk.num_blocks *
                                               a.walk.ids_per_block;
    const uint64_t page_bytes = a.walk.page_elems * 2;
    const unsigned char* base = reinterpret_cast<const unsigned char*>(pages);
    // Page ids come through the scalar cache.  The wave's four or eight rows of a tile lie in one page (pages hold
    // at least 8 tokens).  Rows past the end of the range (the last tile's) are taken from the range's last page: the table
    // need not hold a page for them, and nobody looks at what they hold.  Tiles past the last one are clamped to it,
    // so that every iteration issues the same number of loads and the counts of outstanding ones stay constants.
    const uint32_t last_page = (kv_end_max - 1) >> log2p;
    typedef const __attribute__((address_space(4))) uint32_t* ConstantIds;
    const ConstantIds ids_row = (ConstantIds)(uintptr_t)table_row;
    auto first_key = [&](uint32_t t) { return key_base0 + min(t, group_kv_tiles - 1) * kKeys + kWaveRows * wave; };
    auto page_of = [&](uint32_t t) -> uint32_t { return ids_row[min(first_key(t) >> log2p, last_page)]; };
    auto rows_of = [&](uint32_t t, uint32_t id) -> const unsigned char* {
        return base + id * page_bytes + (uint64_t)(first_key(t) & page_mask) * kRowBytes;
    };
    const uint32_t k_plane = kv_head * a.walk.tokens_per_page * kRowBytes;
    const uint32_t v_plane = (a.walk.hkv + kv_head) * a.walk.tokens_per_page * kRowBytes;
    const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char*)(lds);
    const uint32_t row_in_load = lane / kRowChunks, slot = lane % kRowChunks;
    // K goes from global memory straight to LDS; where in the wave's rows a lane's 16 bytes come from:
    uint32_t k_lane[kLoads];
    // V goes through registers, where bf16 becomes f16; where in the wave's rows of a stage a lane's 16 bytes go:
    uint32_t v_lane[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
        const uint32_t key = kWaveRows * wave + kRowsPerLoad * i + row_in_load;  // in the tile
        k_lane[i] = (kRowsPerLoad * i + row_in_load) * kRowBytes + ((slot ^ (key & 15)) * 16);
        v_lane[i] = kVOffset + (kWaveRows * wave + kRowsPerLoad * i + row_in_load) * kRowBytes +
                    (((((slot >> 1) ^ (key & 7)) << 1) | (slot & 1)) * 16);
    }
    const uint32_t v_from = row_in_load * kRowBytes + slot * 16;  // (the rows of load i begin kRowsPerLoad * i rows on)
    auto issue_k_loads = [&](uint32_t t, uint32_t id) __attribute__((always_inline)) {
        const unsigned char* rows_at = rows_of(t, id) + k_plane;
        const uint32_t dst = lds0 + (t % kChunkStages) * kKBytes + kWaveRows * wave * kRowBytes;
#pragma unroll
        for (int i = 0; i < kLoads; ++i) dma_16_bytes_per_lane(dst + i * 1024, rows_at, k_lane[i]);
    };
    struct VRows {
        u32x4_t w[kLoads];
    };
    auto load_v_rows = [&](uint32_t t, uint32_t id, VRows& r) __attribute__((always_inline)) {
        const unsigned char* rows_at = rows_of(t, id) + v_plane + v_from;
#pragma unroll
        for (int i = 0; i < kLoads; ++i)
            r.w[i] = *reinterpret_cast<const u32x4_t*>(rows_at + i * (kRowsPerLoad * kRowBytes));
    };
    // The wave's V rows of tile t into their stage: as f16, and zero where a row lies outside the range - its
    // probability is 0, but its bytes may be NaN or Inf.
    // (the stage, t % kChunkVStages, is a constant where this is called: it goes into the store's immediate offset)
    auto store_v_rows = [&](uint32_t t, auto stage, const VRows& r) __attribute__((always_inline)) {
        const uint32_t kb = key_base0 + t * kKeys;
        const bool edge = kb < kv_begin || kb + kKeys > kv_end_max;  // first or last tile of the range
        unsigned char* mine = lds + decltype(stage)::value * kKBytes;
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            u32x4_t w = to_f16x8<Tag>(r.w[i]);
            const uint32_t token = kb + kWaveRows * wave + kRowsPerLoad * i + row_in_load;
            if (edge && (token < kv_begin || token >= kv_end_max)) w = u32x4_t{0u, 0u, 0u, 0u};
            *reinterpret_cast<u32x4_t*>(mine + v_lane[i]) = w;
        }
    };
    // everything this wave has written to LDS is there, and every wave has come this far
    auto barrier = []() __attribute__((always_inline)) { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    // Where a lane reads its K operand of k-step ks: chunk (4 * ks + mc) ^ mt of row mt.  4 * ks and mc share no bit,
    // so that is the lane's chunk of k-step 0 with ks * 64 bytes XORed in: one register, not one per k-step.
    const uint32_t k_lane0 = mt * kRowBytes + ((mc ^ mt) * 16);
    // transposing reads: key 4 * mc + mt / 4 (and 16 on), dims 16 * db + 4 * (mt % 4) ..; the 32-byte chunk db of a
    // row sits at chunk db ^ (key % 8)
    const uint32_t v_key = 4 * mc + (mt >> 2);
    // (likewise one register: the lane's place in chunk 0 ^ (key % 8), with (db % 8) * 32 XORed in and db / 8 * 256 added)
    const uint32_t v_lane0 = kVOffset + v_key * kRowBytes + (mt & 3) * 8 + (v_key & 7) * 32;
    float run_max[NB], lane_sum[NB];
    f32x4_t o[NB][kDimBlocks];
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        run_max[j] = -INFINITY;
        lane_sum[j] = 0.0f;
#pragma unroll
        for (int db = 0; db < kDimBlocks; ++db) o[j][db] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    }

    // ---------------- the tile loop ----------------
    // One barrier per tile, B(t).  Before it a wave has stored its V rows of tile t (in the middle of the tile
    // before) and seen its K rows of tile t + 1 land; behind it everybody has, and every wave is through with tile
    // t - 1: its K stage takes the loads of tile t + 3, and its V stage the rows of tile t + 1.  So behind B(t) a
    // wave asks for its K rows of tile t + 3 and multiplies K * Q^T of tile t; then it stores its V rows of tile
    // t + 1, which it asked for two tiles ago (two register sets, taken in turn), and asks for those of tile t + 3;
    // then the softmax and the products with V.  The loads complete in the order of their issue: at the barrier
    // the K rows of tile t + 1 are followed by the V rows of tile t + 1, the K rows of tile t + 2 and the V rows
    // of tile t + 2.
    // k-steps between an operand's read and its product
    constexpr int kAhead = 1;
    // whether those reads are issued ahead of the products of the step before them (a second set of operand
    // registers) or behind them (the same registers again, and the products' 64 cycles to cover the read)
    constexpr bool kReadsFirst = true;
    uint32_t next_id = 0;
    auto tile = [&](uint32_t it, auto v_stage, VRows& v_rows) __attribute__((always_inline)) {
        constexpr int kVStage = decltype(v_stage)::value;  // it % kChunkVStages
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * kLoads) : "memory");
        barrier();
        const uint32_t id = next_id;   // of tile it + 3, asked for a tile ago: a page id takes as long as an LDS round trip,
        next_id = page_of(it + 4);     // and waiting for it waits for every LDS read in flight as well
        issue_k_loads(it + 3, id);
        const bool mine = it < my_tiles;  // (a wave that sees none of the tile's keys still does its share of the loads)

        const uint32_t k_at = (it % kChunkStages) * kKBytes + k_lane0;
        const uint32_t kb = key_base0 + it * kKeys;
        const bool masked = !(kb >= kv_begin && kb + kKeys <= wave_lo);
        float logits[NB][4 * kKeyBlocks];
        if (mine) {
        // (zeroed here, where the first products can take the zeros as a constant operand, not from registers)
        f32x4_t sc[kKeyBlocks][NB];
#pragma unroll
        for (int b = 0; b < kKeyBlocks; ++b)
#pragma unroll
            for (int j = 0; j < NB; ++j) sc[b][j] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        uint4 kk[kKeyBlocks][kKSteps], q1[kKSteps];
        // the operands of k-step ks: the key blocks of K, and the second column block's queries
        auto read_k = [&](int ks) __attribute__((always_inline)) {
            const unsigned char* src = lds + (k_at ^ (ks * 64));
#pragma unroll
            for (int b = 0; b < kKeyBlocks; ++b) kk[b][ks] = *reinterpret_cast<const uint4*>(src + 16 * b * kRowBytes);
            if (ks < kQ1Regs) q1[ks] = qreg1[ks];
            else q1[ks] = *reinterpret_cast<const uint4*>(q_lds + ks * 1024);
        };
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < kAhead; ++ks) read_k(ks);
#pragma unroll
        for (int ks = 0; ks < kKSteps; ++ks) {
            if (ks + kAhead < kKSteps) read_k(ks + kAhead);
#pragma unroll
            for (int j = 0; j < NB; ++j)
#pragma unroll
                for (int b = 0; b < kKeyBlocks; ++b)
                    sc[b][j] = mfma_16x16x32<Tag>(kk[b][ks], j == 0 ? qreg[ks] : q1[ks], sc[b][j]);
        }
        // LDS reads of k-step ks: the K operands, and the second block's queries unless they are in registers
        static_assert(kKeyBlocks == 2 || (kKeyBlocks == 4 && kQ1Regs == kKSteps), "the literal counts below");
        auto reads_of = [](int ks) __attribute__((always_inline)) {
            if (kKeyBlocks == 4) __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
            else if (ks < kQ1Regs) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            else __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
        };
        auto products_of_a_step = []() __attribute__((always_inline)) {
            if (kKeyBlocks == 4) __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
            else __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
        };
#pragma unroll
        for (int ks = 0; ks < kAhead; ++ks) reads_of(ks);  // the first reads
#pragma unroll
        for (int ks = 0; ks < kKSteps - kAhead; ++ks) {
            if constexpr (kReadsFirst) reads_of(ks + kAhead);  // the reads kAhead steps on
            products_of_a_step();
            if constexpr (!kReadsFirst) reads_of(ks + kAhead);
        }
#pragma unroll
        for (int ks = 0; ks < kAhead; ++ks) products_of_a_step();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int i = 0; i < 4 * kKeyBlocks; ++i) logits[j][i] = sc[i >> 2][j][i & 3];
        }
        if (it + 1 < group_kv_tiles) store_v_rows(it + 1, std::integral_constant<int, 1 - kVStage>{}, v_rows);
        load_v_rows(it + 3, id, v_rows);
        if (!mine) return;
        uint4 pb[NB][kSub];
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            constexpr int kMine = 4 * kKeyBlocks;  // the lane's keys of its column: 4 * mc + r of every key block
            float (&v)[kMine] = logits[j];
            if (masked) {
#pragma unroll
                for (int i = 0; i < kMine; ++i) {
                    const uint32_t token = kb + 16 * (i >> 2) + 4 * mc + (i & 3);
                    if (token < kv_begin || token >= lim[j]) v[i] = -INFINITY;
                }
            }
            float m = max3(max3(v[0], v[1], v[2]), max3(v[3], v[4], v[5]), max3(v[6], v[7], v[7]));
            if constexpr (kMine == 16)
                m = max3(m, max3(max3(v[8], v[9], v[10]), max3(v[11], v[12], v[13]), v[14]), v[15]);
            m *= a.scale_log2;
            if (__any(m > run_max[j] + kSlack)) {
                m = fmaxf(m, __shfl_xor(m, 16, 64));
                m = fmaxf(m, __shfl_xor(m, 32, 64));
                if (m > run_max[j] + kSlack) {
                    const float alpha = run_max[j] > -INFINITY ? __builtin_amdgcn_exp2f(run_max[j] - m) : 0.0f;
                    run_max[j] = m;
                    lane_sum[j] *= alpha;
#pragma unroll
                    for (int db = 0; db < kDimBlocks; ++db)
#pragma unroll
                        for (int r = 0; r < 4; ++r) o[j][db][r] *= alpha;
                }
            }
            const float neg_ref = run_max[j] > -INFINITY ? -run_max[j] : 0.0f;
            uint32_t words[kMine / 2];
#pragma unroll
            for (int i = 0; i < kMine; i += 2) {
                // rounded to nearest, once, for the product and for the sum alike
                const f16x2_t h = {(_Float16)__builtin_amdgcn_exp2f(__builtin_fmaf(v[i], a.scale_log2, neg_ref)),
                                   (_Float16)__builtin_amdgcn_exp2f(__builtin_fmaf(v[i + 1], a.scale_log2, neg_ref))};
                const f16x2_t ones = {(_Float16)1.0f, (_Float16)1.0f};
                lane_sum[j] = __builtin_amdgcn_fdot2(h, ones, lane_sum[j], false);
                words[i / 2] = __builtin_bit_cast(uint32_t, h);
            }
#pragma unroll
            for (int sub = 0; sub < kSub; ++sub)
                pb[j][sub] = make_uint4(words[4 * sub], words[4 * sub + 1], words[4 * sub + 2], words[4 * sub + 3]);
        }
        constexpr int kVGroup = 2;  // V operands read ahead of their products
#pragma unroll
        for (int sub = 0; sub < kSub; ++sub) {
#pragma unroll
            for (int g = 0; g < kDimBlocks; g += kVGroup) {
                uint4 vt[kVGroup];
#pragma unroll
                for (int i = 0; i < kVGroup; ++i) {
                    const unsigned char* src = lds + (v_lane0 ^ (((g + i) & 7) * 32)) +
                                               (kVStage * kKBytes + 32 * sub * kRowBytes + ((g + i) & 8) * 32);
                    const uint2 lo2 = lds_read_tr16_b64(src), hi2 = lds_read_tr16_b64(src + 16 * kRowBytes);
                    vt[i] = make_uint4(lo2.x, lo2.y, hi2.x, hi2.y);
                }
#pragma unroll
                for (int i = 0; i < kVGroup; ++i)
#pragma unroll
                    for (int j = 0; j < NB; ++j) o[j][g + i] = mfma_16x16x32<F16Tag>(vt[i], pb[j][sub], o[j][g + i]);
            }
        }
    };
    if (group_kv_tiles != 0) {
        VRows first, even, odd;  // `odd` holds the rows of the odd tiles, and is taken in the even tiles
        const uint32_t id0 = page_of(0), id1 = page_of(1), id2 = page_of(2);
        next_id = page_of(3);
        issue_k_loads(0, id0);
        load_v_rows(0, id0, first);
        issue_k_loads(1, id1);
        load_v_rows(1, id1, odd);
        issue_k_loads(2, id2);
        load_v_rows(2, id2, even);
        store_v_rows(0, std::integral_constant<int, 0>{}, first);
        uint32_t it = 0;
        for (; it + 1 < group_kv_tiles; it += 2) {
            tile(it, std::integral_constant<int, 0>{}, odd);
            tile(it + 1, std::integral_constant<int, 1>{}, even);
        }
        if (it < group_kv_tiles) tile(it, std::integral_constant<int, 0>{}, odd);
        // The loads of tiles past the end go to LDS: they must be through before the workgroup gives it back.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }

    // The workgroup's next item is asked for here, so that the answer travels while the results are stored.
    if (tid == 0) next_item = gridDim.x + atomicAdd(a.work_claim, 1u);
    claimed = true;

    // Where the columns' partial rows go.  Both blocks' rows are known before either block's stores are issued: the
    // row numbers come from memory, and a wait for a load waits for every store issued before it as well.  (A row
    // number fits 32 bits: the partial accumulators, D floats a row, fit the GPU's memory.)
    uint32_t part_row[NB];
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        uint32_t t, h;
        column_of(j, &t, &h);
        part_row[j] = (row_of(t / TS) * a.hq + head_first + h) * TS + t % TS;
    }
#pragma unroll
    for (int j = 0; j < NB; ++j) asm volatile("" : "+v"(part_row[j]));
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        lane_sum[j] += __shfl_xor(lane_sum[j], 16, 64);
        lane_sum[j] += __shfl_xor(lane_sum[j], 32, 64);
        if (lim[j] != 0) {
            if (mc == 0) {
                a.part_max[part_row[j]] = run_max[j];
                a.part_sum[part_row[j]] = lane_sum[j];
            }
            float* dst = a.part_acc + (uint64_t)part_row[j] * D + mc * 4;
#pragma unroll
            for (int db = 0; db < kDimBlocks; ++db)
                *reinterpret_cast<float4*>(dst + db * 16) = make_float4(o[j][db][0], o[j][db][1], o[j][db][2], o[j][db][3]);
        }
    }
    // A V element that f16 cannot hold has reached the accumulators as Inf or NaN (the conversion rounds to nearest,
    // so that it overflows instead of saturating): the host is told, and the rows stay as they are, visibly wrong.
    // (Looked for behind the stores, which do not wait for it, and along eight chains rather than one.)
    float probe[NB][4];
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            probe[j][r] = 0.0f;
#pragma unroll
            for (int db = 0; db < kDimBlocks; ++db) probe[j][r] = __builtin_fmaf(o[j][db][r], 0.0f, probe[j][r]);
        }
    bool out_of_range = false;
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const float all = (probe[j][0] + probe[j][1]) + (probe[j][2] + probe[j][3]);
        out_of_range |= lim[j] != 0 && all != all;
    }
    if (__any(out_of_range) && lane == 0)
        __hip_atomic_store(a.status + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// The grid is as many workgroups as the GPU holds at once, and a workgroup takes items until there are none left:
// the first is its own number, the others come from a counter, in the order of the list (longest first).  The
// hardware hands the workgroups of a larger grid to the compute units in a fixed rotation, and a workgroup waits for
// the unit whose turn it is while others stand idle: with items of 4 to 128 tiles a launch then ended a tenth later
// than with items taken as units become free.
//   work_claim[0] counts the items handed out beyond the first of each workgroup, work_claim[1] the workgroups that
// are through; the last one out sets both back to zero for the next launch (launches of a context run one after
// the other, on its stream).
template <typename Tag, int D, bool kTable>
__global__ __launch_bounds__(64 * kChunkWaves, 1) void split_kv_chunk_map(
    MapArgs a, const uint32_t* __restrict__ page_ids, const uint32_t* __restrict__ kv_splits,
    const uint32_t* __restrict__ req_slots, const uint16_t* __restrict__ q, const uint16_t* __restrict__ pages,
    const uint32_t* __restrict__ q_token_tiles, const uint32_t* __restrict__ flat_token_indices,
    const uint32_t* __restrict__ row_groups, uint32_t group_tiles, uint32_t num_groups, uint32_t head_subsets,
    uint32_t num_items) {
    resolve_active(a);
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    volatile uint32_t* mailbox = reinterpret_cast<volatile uint32_t*>(lds + 1024);  // (clear of the item's first LDS words)
    uint32_t item = blockIdx.x;
    while (item < num_items) {
        uint32_t next_item = 0;
        bool claimed = false;
        chunk_map_item<Tag, D, kTable>(a, page_ids, kv_splits, req_slots, q, pages, q_token_tiles, flat_token_indices, row_groups,
                               group_tiles, num_groups, head_subsets, item, next_item, claimed);
        if (!claimed && threadIdx.x == 0) next_item = gridDim.x + atomicAdd(a.work_claim, 1u);
        __syncthreads();  // every wave is through with the item's LDS
        if (threadIdx.x == 0) *mailbox = next_item;
        __syncthreads();
        item = __builtin_amdgcn_readfirstlane(*mailbox);
    }
    if (threadIdx.x == 0 && atomicAdd(a.work_claim + 1, 1u) == gridDim.x - 1) {
        __hip_atomic_store(a.work_claim, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(a.work_claim + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

template <typename Tag, int D, bool kTable>
inline int launch_chunk_map_form(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a, const uint32_t* row_groups,
                                 uint32_t group_tiles, uint32_t num_groups) {
    const uint32_t subsets = chunk_launch_subsets(g.group, group_tiles, a.rows_per_split_head);
    const uint32_t num_items = num_groups * g.hkv * subsets;
    if (num_items == 0) return PSI_HIP_OK;
    auto* kernel = &split_kv_chunk_map<Tag, D, kTable>;
    // The kernel's LDS is above the default limit of a launch; the limit is raised once per GPU and kernel (a
    // function's attributes belong to the device it is loaded on).  How many workgroups the GPU holds at once is
    // asked then, too.
    static std::atomic<uint64_t> raised_on{0};
    static std::atomic<int> resident_per_cu{0};
    const uint64_t device_bit = 1ull << (ctx->device & 63);
    if ((raised_on.load(std::memory_order_relaxed) & device_bit) == 0) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                ChunkLds<D>::bytes) != hipSuccess)
            return PSI_HIP_ERR_UNSUPPORTED;
        int per_cu = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 64 * kChunkWaves, ChunkLds<D>::bytes) !=
                hipSuccess ||
            per_cu < 1)
            return PSI_HIP_ERR_UNSUPPORTED;
        resident_per_cu.store(per_cu, std::memory_order_relaxed);
        raised_on.fetch_or(device_bit, std::memory_order_relaxed);
    }
    const uint32_t resident = (uint32_t)resident_per_cu.load(std::memory_order_relaxed) * (uint32_t)ctx->num_cus;
    const dim3 grid(std::min(num_items, resident));
    hipLaunchKernelGGL(kernel, grid, dim3(64 * kChunkWaves), ChunkLds<D>::bytes, ctx->stream, a, a.walk.page_ids,
                       a.kv_splits, a.req_slots, reinterpret_cast<const uint16_t*>(a.q),
                       reinterpret_cast<const uint16_t*>(a.kv_pages), a.q_token_tiles, a.flat_token_indices, row_groups,
                       group_tiles, num_groups, subsets, num_items);
    return PSI_HIP_OK;
}

// With a table, or without one: every kv_split row a group of its own (group_tiles 1), which is how the plain and the
// balanced multi-query entry points launch this kernel for tiles of more than 48 query columns.
template <typename Tag, int D>
inline int launch_chunk_map_typed(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a, const uint32_t* row_groups,
                                  uint32_t group_tiles, uint32_t num_groups) {
    if (row_groups == nullptr) {
        if (group_tiles != 1) return PSI_HIP_ERR_UNSUPPORTED;
        return launch_chunk_map_form<Tag, D, false>(ctx, g, a, nullptr, 1, num_groups);
    }
    return launch_chunk_map_form<Tag, D, true>(ctx, g, a, row_groups, group_tiles, num_groups);
}

}  // namespace psi
