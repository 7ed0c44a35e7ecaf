// gfx950 split-KV multi-query map (speculative verify, prefill chunks) for 2-byte K/V (bf16 / f16),
// head_dim 128 or 256, pages of 8 or 16*2^k tokens.  Semantics of
// crates/inference-backend-metal/src/components/metal/gqa_split_kv_tiled_q.metal:49-319.
//
// Work decomposition
//   one workgroup = one (kv_split row, kv_head), or a worker's range of rows in the balanced launch.  The row
//   names a request-local tile of up to 8 query tokens; with the G query heads that share the KV head this gives
//   up to 8*G query columns, column c = token_in_tile * G + head, handled as blocks of 16 columns.  Every K and V
//   byte of the split is therefore fetched from HBM once for all of them.  Four streams of KV tiles per workgroup
//   (stream p takes the 16-token tiles p, p + 4, ...), each with its own online-softmax state per column; the
//   states merge through LDS at the end of the row.
//   Up to 48 columns (three blocks): split_kv_tiled_paired_map, two waves per stream, KV tiles through LDS by
//   global_load_lds.  49 to 64 columns (8 tokens x 7 or 8 heads per KV head) are more than its stages and registers
//   hold: those launches go to the row-group kernel (split_kv_chunk_kernel.h) with every row a group of its own.
//
// Per 16-token KV tile
//   QK^T  S[token][column] on v_mfma_f32_16x16x32: A = the K tile (lane = token lane%16, 8 contiguous dims), B =
//         the query columns staged once per row in LDS in operand order (or kept in registers).
//   softmax  the MFMA leaves each lane with 4 tokens of one column; causal / range masks per column;
//         probabilities stay in registers: that register layout is exactly the A operand of
//         v_mfma_f32_16x16x16 (row = column, k = 4 tokens).
//   PV    O[column][dim] += P^T * V on v_mfma_f32_16x16x16.  The contraction runs over tokens, the strided axis
//         of V, so the V tile is read out of LDS with the transposing read (4 tokens x 1 dim per lane).  bf16
//         probabilities are split into two bf16 terms (two MFMAs) so that P carries 16 mantissa bits; f16
//         carries 11 in one.
//
// Algorithmic bytes per (kv token, kv head): 2 * head_dim * 2, read once per (Q tile, split).
#pragma once
#include <type_traits>

#include "split_kv_decode_kernel.h"

namespace psi {

typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4_t;

// D(16x16, f32) += A(16x16) * B(16x16).  Lane l holds A[row l%16][k 4*(l/16)..+4],
// B[k 4*(l/16)..+4][col l%16] and D[row 4*(l/16)+r][col l%16], r = 0..3.
template <typename Tag>
__device__ __forceinline__ f32x4_t mfma_16x16x16(uint2 a, uint2 b, f32x4_t c);
template <>
__device__ __forceinline__ f32x4_t mfma_16x16x16<BF16Tag>(uint2 a, uint2 b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4_t, a), __builtin_bit_cast(s16x4_t, b), c,
                                                     0, 0, 0);
}
template <>
__device__ __forceinline__ f32x4_t mfma_16x16x16<F16Tag>(uint2 a, uint2 b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4_t, a), __builtin_bit_cast(f16x4_t, b), c, 0,
                                                 0, 0);
}

// Probabilities of 4 tokens -> A operand(s).  bf16: p = hi + lo with both terms truncated to bf16,
// 16 mantissa bits in total; f16: one rounded term.
template <typename Tag>
struct ProbOperand;
template <>
struct ProbOperand<BF16Tag> {
    static constexpr int kTerms = 2;
    uint2 term[2];
    __device__ __forceinline__ void set(const float (&p)[4]) {
        uint32_t hi[4], lo[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            hi[r] = __float_as_uint(p[r]) & 0xffff0000u;
            lo[r] = __float_as_uint(p[r] - __uint_as_float(hi[r])) & 0xffff0000u;
        }
        term[0] = make_uint2((hi[0] >> 16) | hi[1], (hi[2] >> 16) | hi[3]);
        term[1] = make_uint2((lo[0] >> 16) | lo[1], (lo[2] >> 16) | lo[3]);
    }
};
template <>
struct ProbOperand<F16Tag> {
    static constexpr int kTerms = 1;
    uint2 term[1];
    __device__ __forceinline__ void set(const float (&p)[4]) {
        const f16x4_t h = {(_Float16)p[0], (_Float16)p[1], (_Float16)p[2], (_Float16)p[3]};
        term[0] = __builtin_bit_cast(uint2, h);
    }
};

typedef __attribute__((ext_vector_type(4))) short tr_s16x4_t;
// Transposing LDS read of gfx950 (ds_read_b64_tr_b16): the 16 lanes of a quarter wave hand in 16 addresses of 4
// consecutive 2-byte elements each, a 16 x 4 block, and get it back transposed: lane 4 * a + c receives element c of
// the addresses a, a + 4, a + 8, a + 12.
__device__ __forceinline__ uint2 lds_read_tr16_b64(const void* p) {
    const tr_s16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) tr_s16x4_t*)(const_cast<void*>(p)));
    return __builtin_bit_cast(uint2, v);
}

// The reference maximum of a column moves only when a tile exceeds it by more than kMaxSlack (log2 domain), a few
// times per range: probabilities stay below 2^kMaxSlack, and the rescaling of the accumulators is rare.
constexpr float kMaxSlack = 8.0f;
constexpr int kTiledTileWaves = 4;  // waves that share the KV tiles of a split among them


// ---------------------------------------------------------------------------------------------------------------
// KV tiles through LDS without registers (tiles of up to 48 query columns; see split_kv_tiled_paired_map below).
//
// A 16-token tile of K (and of V) is 16 rows of D elements.  `global_load_lds_dwordx4` moves 16 bytes per lane from
// a per-lane global address to LDS address M0 + instruction offset + 16 * lane, with no register in between.  One
// instruction covers 8 rows x 128 bytes (whole lines): lane p = 8 * c + t fetches chunk c (8 elements) of row t, and
// lands at slot p of a 1 KiB block; a tile is 2 * D / 64 such blocks, [row half][line of the row].  Read back, the A
// operand of K * Q^T (16 rows x 8 elements per quarter wave) and the transposed V block of a quarter wave both
// gather whole 16-byte slots, conflict-free.
//
// The loads are inline assembly, and so are the waits for them: the compiler does not know that they write LDS, and
// where it does (the builtin) it waits for every outstanding one before any LDS read, which would undo the prefetch.
// ---------------------------------------------------------------------------------------------------------------

// Line `kLine` (64 elements) of the 8 + 8 rows of a tile: two loads of 1 KiB, one per half tile.  The instruction
// offset is added to the global and to the LDS address alike, hence 1024 - 128 between the M0 values of consecutive
// lines.
template <int kLine, int kHalfBytes>
__device__ __forceinline__ void dma_tile_line(uint32_t lds_tile, const void* rows0, const void* rows1) {
    asm volatile(
        "s_add_u32 m0, %0, %3\n\ts_nop 0\n\t"
        "global_load_lds_dwordx4 %1, off offset:%5 nt\n\t"
        "s_add_u32 m0, %0, %4\n\ts_nop 0\n\t"
        "global_load_lds_dwordx4 %2, off offset:%5 nt"
        :
        : "s"(lds_tile), "v"(rows0), "v"(rows1), "n"(kLine * 896), "n"(kHalfBytes + kLine * 896), "n"(kLine * 128)
        : "memory", "m0", "scc");
}
template <int kDQ, int kHalfBytes>
__device__ __forceinline__ void dma_tile(uint32_t lds_tile, const void* rows0, const void* rows1) {
    dma_tile_line<0, kHalfBytes>(lds_tile, rows0, rows1);
    dma_tile_line<1, kHalfBytes>(lds_tile, rows0, rows1);
    if constexpr (kDQ == 4) {
        dma_tile_line<2, kHalfBytes>(lds_tile, rows0, rows1);
        dma_tile_line<3, kHalfBytes>(lds_tile, rows0, rows1);
    }
}

// Waits until at most `kLoads * groups` of the wave's loads are outstanding (they complete in order).
template <int kLoads>
__device__ __forceinline__ void wait_load_groups(uint32_t groups) {
    if (groups >= 3) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * kLoads) : "memory");
    else if (groups == 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * kLoads) : "memory");
    else if (groups == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoads) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// ---------------------------------------------------------------------------------------------------------------
// The multi-query map for tiles of up to 48 query columns: a loading wave and multiplying waves on each stream of
// KV tiles, all on one SIMD.
//
// A wave stands at a load until the memory pipeline takes it, and at a product until the matrix cores take it: one
// wave alone does the one or the other, and its time per tile is the sum (by the cycle counter, the K * Q^T phase of
// one column block took 1800 cycles with the tile's eight K loads in it and 200 without).  Here the waves p, p + 4,
// p + 8 of a workgroup (they share a SIMD) walk the tiles p, p + 4, ... of the row together through one set of LDS
// stages.  The last of them issues every load, announces each tile of K and of V in LDS as it lands and, in the
// one- and two-block forms, does nothing else; the others multiply, one column block each, and say in LDS when they
// have read a stage, so that it may be refilled.  While the loading wave stands at a load the others multiply.
// With three column blocks a fourth wave per SIMD would leave each 128 registers, less than a block's accumulators
// and operands take, so one wave multiplies two blocks and the loading wave takes the third (which costs: the same
// split at two blocks runs 10 % slower than the pure loader).  All of it is bounded: a wait on another wave's
// progress gives up after 65536 polls; the row is then stored as an empty state and the host is
// told through MapArgs::status, and no wave stays behind.
// ---------------------------------------------------------------------------------------------------------------
// Waves per stream of tiles: one that loads, and one that multiplies per column block; with three blocks (four waves
// of a SIMD would have 128 registers each, which a column block's 64 accumulators and its operands do not fit
// into) one multiplying wave takes two blocks and the loading wave the third.
constexpr int tiled_multiplying_waves(int column_blocks) { return column_blocks <= 2 ? column_blocks : 1; }
constexpr int tiled_paired_waves(int column_blocks) { return (tiled_multiplying_waves(column_blocks) + 1) * kTiledTileWaves; }

template <typename Tag, int D, int NB, bool kHalfPage>
__global__ __launch_bounds__(64 * tiled_paired_waves(NB), 1) void split_kv_tiled_paired_map(
    MapArgs a, const uint32_t* __restrict__ page_ids, const uint32_t* __restrict__ kv_splits,
    const uint32_t* __restrict__ req_slots, const uint16_t* __restrict__ q, const uint16_t* __restrict__ pages,
    const uint32_t* __restrict__ q_token_tiles, const uint32_t* __restrict__ flat_token_indices,
    const uint32_t* __restrict__ worker_cu) {
    resolve_active(a);
    constexpr int kPairs = kTiledTileWaves;
    constexpr int kWaves = tiled_paired_waves(NB);
    constexpr int kMultipliers = tiled_multiplying_waves(NB);   // multiplying waves per stream
    constexpr int kBlocksEach = NB <= 2 ? 1 : 2;                // column blocks of a multiplying wave
    constexpr int kBlocksLoader = NB - kMultipliers * kBlocksEach;  // and of the loading wave (0, or 1 of 3)
    constexpr int kKSteps = D / 32;             // MFMA k-steps of QK^T
    constexpr int kDimBlocks = D / 16;          // 16-dim output blocks of PV
    constexpr int kDQ = D / 64;                 // 128-byte lines per row
    constexpr int kTileLoads = 2 * kDQ;         // load instructions per tile of K (or of V)
    constexpr int kTileBytes = kTileTokens * D * 2;
    constexpr int kHalfBytes = kTileBytes / 2;
    constexpr int kPairBytes = 4 * kTileBytes;  // K stage 0, K stage 1, V stage 0, V stage 1
    constexpr int kCols = NB * 16;
    constexpr int kMergeStride = D + 4;         // floats per column row of the merge buffer
    constexpr int kStageBytes = kPairs * kPairBytes;
    constexpr int kQBytes = NB * kKSteps * 64 * 16;
    static_assert(kCols * kMergeStride * 4 <= kStageBytes, "the merge buffer reuses the tile stages");

    __shared__ __attribute__((aligned(1024))) unsigned char lds_union[kStageBytes + kQBytes];
    __shared__ float wave_max_lds[kPairs][kCols];
    __shared__ float col_max_lds[kCols];
    __shared__ float col_sum_lds[kCols];
    // tiles of the row so far, per pair: [K landed, V landed, K read by the first wave, V read by the first wave]
    __shared__ uint32_t progress[2 + 2 * kMultipliers][kPairs];
    __shared__ uint32_t row_failed;  // a wait of some wave ran out on the current row
    __shared__ uint32_t muted[2];    // see say_landed_k
    uint4* qb_lds = reinterpret_cast<uint4*>(lds_union + kStageBytes);  // [NB][kKSteps][64]
    float* merge = reinterpret_cast<float*>(lds_union);

    const uint32_t G = a.group;
    const uint32_t kv_head = blockIdx.x % a.walk.hkv;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t pair = wave % kPairs;
    const uint32_t role = wave / kPairs;  // 0 .. kMultipliers - 1: a multiplying wave; kMultipliers: the loading wave
    const bool second = role == (uint32_t)kMultipliers;
    unsigned char* my_stages = lds_union + pair * kPairBytes;
    const uint32_t my_stages_lds =
        (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char*)(lds_union) + pair * kPairBytes;
    // With three column blocks the words are addressed as LDS.  Through a generic pointer a volatile access becomes a
    // flat one, which counts as a global load too: waiting for its value then waits for every tile load the wave has
    // in flight, so that the loading wave drains its loads at each poll (449 against 482 us on the batch of 64 with
    // 8 new tokens).  With one and two blocks the generic form is kept on purpose: it measures 2.5 % faster there
    // (399 against 409 us and 414 against 425 us with 2 and 4 new tokens), and draining the loads by hand before each
    // new tile's loads recovers less than half of that.  Measured, not explained.
    typedef std::conditional_t<(NB <= 2), volatile uint32_t*, volatile __attribute__((address_space(3))) uint32_t*> LdsWord;
    auto word = [&](uint32_t which) { return (LdsWord)(&progress[which][pair]); };
    const LdsWord landed_k = word(0);
    const LdsWord landed_v = word(1);
    // what a multiplying wave reports; the loading wave waits for all of them
    const LdsWord read_k = word(2 + 2 * (second ? 0u : role));
    const LdsWord read_v = word(3 + 2 * (second ? 0u : role));
    // A wait that runs out marks the row as failed (it is then stored as an empty state and reported to the host)
    // and is this wave's last wait on the row: the wave walks on without waiting, so that the waves that wait for
    // its progress get through as well.
    bool gave_up = false;
    auto wait_until_above = [&](LdsWord counter, uint32_t value) __attribute__((always_inline)) {
        if (gave_up) return;
        uint32_t polls = 0;
        for (; *counter <= value && polls < kDefaultWaitPolls; ++polls) __builtin_amdgcn_s_sleep(1);
        if (polls == kDefaultWaitPolls) {
            gave_up = true;
            if ((threadIdx.x & 63) == 0) row_failed = 1u;  // the host is told when the row is stored
        }
        asm volatile("" ::: "memory");
    };
    // Where the loading wave says that a tile has landed.  A harness that wants to see waits run out
    // (MapArgs::mute_loaders) has the words written where no wave looks.
    const LdsWord say_landed_k = a.mute_loaders ? (LdsWord)(&muted[0]) : landed_k;
    const LdsWord say_landed_v = a.mute_loaders ? (LdsWord)(&muted[1]) : landed_v;

    uint32_t row_begin = blockIdx.x / a.walk.hkv, row_end = row_begin + 1;
    if (worker_cu != nullptr) {
        row_begin = worker_cu[blockIdx.x / a.walk.hkv];
        row_end = worker_cu[blockIdx.x / a.walk.hkv + 1];
    }
    const uint32_t log2p = 31 - __builtin_clz(a.walk.tokens_per_page);
    const uint32_t page_mask = a.walk.tokens_per_page - 1;
    const uint64_t v_region = (uint64_t)a.walk.hkv * a.walk.tokens_per_page * D;
    const uint32_t lane_id = threadIdx.x & 63;

    // What a wave must know of a row before it can start on it: a chain of four dependent reads (the row of the
    // split table, its query tile, the tile's request slot and token positions, the first page ids).
    struct RowStart {
        uint32_t step;                                 // links done
        uint32_t valid, kv_begin, kv_end, flat_begin, ncols, req_slot;
        uint32_t q_tile;
        uint32_t position[NB];                         // per lane: position of the query token of column 16 * nb + lane % 16
        TilePages page[3];                             // of this pair's first three tiles
    };
    auto page_of_tile = [&](const uint32_t* table_row, uint32_t tile, uint32_t kv_end_) -> TilePages {
        TilePages pg{0u, 0u};
        if (tile * kTileTokens < kv_end_) {
            const uint32_t first = (tile * kTileTokens) >> log2p;
            pg.a = table_row[first];
            if (kHalfPage) pg.b = table_row[min(first + 1, (kv_end_ - 1) >> log2p)];
        }
        return pg;
    };
    auto table_row_of = [&](uint32_t req_slot_) {
        return page_ids + ((uint64_t)req_slot_ * a.walk.num_layers + a.layer) * a.walk.num_blocks * a.walk.ids_per_block;
    };
    // One link of the chain for row `row`.
    auto advance = [&](RowStart& r, uint32_t row) __attribute__((always_inline)) {
        if (r.step == 0) {
            r.valid = row < row_end && row < a.num_active_kv_splits;
            if (r.valid) {
                r.q_tile = kv_splits[row * 3];
                r.kv_begin = kv_splits[row * 3 + 1];
                r.kv_end = kv_splits[row * 3 + 2];
                r.valid = r.q_tile < a.num_active_q_token_tiles;
            }
        } else if (r.step == 1) {
            if (r.valid) {
                uint32_t fb = q_token_tiles[r.q_tile * 2], fe = q_token_tiles[r.q_tile * 2 + 1];
                r.valid = !(fb >= a.num_active_tokens || fe > a.num_active_tokens || fe <= fb);
                r.flat_begin = fb;
                r.ncols = r.valid ? (fe - fb) * G : 0u;
            }
        } else if (r.step == 2) {
            if (r.valid) {
                r.req_slot = req_slots[r.flat_begin];
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) {
                    const uint32_t c = nb * 16 + (lane_id & 15);
                    r.position[nb] = c < r.ncols ? flat_token_indices[r.flat_begin + c / G] : 0xffffffffu;
                }
            }
        } else if (r.step == 3) {
            if (r.valid && r.ncols <= (uint32_t)kCols) {
                const uint32_t* table_row = table_row_of(r.req_slot);
                const uint32_t first = r.kv_begin / kTileTokens + pair;
#pragma unroll
                for (int j = 0; j < 3; ++j) {
                    r.page[j] = page_of_tile(table_row, first + j * kPairs, r.kv_end);
                }
            }
        }
        ++r.step;
    };
    bool lds_in_use = false;
    for (uint32_t split = row_begin; split < row_end; ++split) {
    if (split >= a.num_active_kv_splits) break;
    RowStart cur;
    cur.step = 0;
    while (cur.step < 4) advance(cur, split);
    if (!cur.valid) continue;  // sentinel padding or a tile outside the active ones
    const uint32_t kv_begin = cur.kv_begin, kv_end = cur.kv_end, flat_begin = cur.flat_begin, ncols = cur.ncols;
    if (ncols > (uint32_t)kCols) {
        // A tile wider than the launch was sized for (the caller's largest-tile bound was too small, e.g. a
        // capture made for two-token tiles replayed on a four-token batch).  The row cannot be computed here;
        // it is entered as an empty state, so that the combine merges nothing stale, and the tile's output is
        // then wrong in a visible way (zeros for a tile with no other row) rather than silently mixed.
        const uint32_t rows = a.rows_per_split_head;
        for (uint32_t idx = threadIdx.x; idx < ncols * (D / 4); idx += 64 * kWaves) {
            const uint32_t c = idx / (D / 4), d4 = idx % (D / 4);
            const uint64_t row = ((uint64_t)split * a.hq + (uint64_t)kv_head * G + c % G) * rows + c / G;
            *reinterpret_cast<float4*>(&a.part_acc[row * D + d4 * 4]) = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (d4 == 0) {
                a.part_max[row] = -INFINITY;
                a.part_sum[row] = 0.0f;
            }
        }
        continue;
    }
    if (lds_in_use) __syncthreads();  // the previous row's merge buffer has been read out
    lds_in_use = true;
    // Lane coordinates, re-derived per row from a value the optimiser cannot see through: nothing computed from
    // them is loop-invariant, so no per-lane address survives from one row into the next row's register budget.
    uint32_t tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const uint32_t lane = tid & 63;
    const uint32_t mt = lane & 15, mc = lane >> 4;

    // Keys below `open_until` are visible to every column in use (the unused ones are never stored).
    uint32_t open_until = kv_end;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
        if (cur.position[nb] != 0xffffffffu) open_until = min(open_until, cur.position[nb] + 1);
#pragma unroll
    for (int sh = 1; sh < 64; sh <<= 1) open_until = min(open_until, (uint32_t)__shfl_xor((int)open_until, sh, 64));
    open_until = __builtin_amdgcn_readfirstlane(open_until);

    const uint32_t* table_row = table_row_of(cur.req_slot);
    const uint32_t tile_begin = kv_begin / kTileTokens;
    const uint32_t tile_end = (kv_end + kTileTokens - 1) / kTileTokens;
    auto load_page_id = [&](uint32_t tile) -> TilePages { return page_of_tile(table_row, tile, kv_end); };
    // This lane's share of a load: chunk `lane / 8` of row `lane % 8` of the half tile.
    const uint32_t lane_elem = (lane & 7) * D + (lane >> 3) * 8;
    auto half_rows = [&](uint32_t tile, TilePages p, int half) -> const uint16_t* {
        if (kHalfPage)
            return pages + (uint64_t)(half ? p.b : p.a) * a.walk.page_elems +
                   (uint64_t)kv_head * a.walk.tokens_per_page * D + lane_elem;
        return pages + (uint64_t)p.a * a.walk.page_elems + (uint64_t)kv_head * a.walk.tokens_per_page * D +
               (((tile * kTileTokens) & page_mask) + half * 8) * D + lane_elem;
    };
    auto issue_k = [&](uint32_t tile, TilePages p, uint32_t stage) {
        dma_tile<kDQ, kHalfBytes>(my_stages_lds + stage * kTileBytes, half_rows(tile, p, 0), half_rows(tile, p, 1));
    };
    auto issue_v = [&](uint32_t tile, TilePages p, uint32_t stage) {
        dma_tile<kDQ, kHalfBytes>(my_stages_lds + (2 + stage) * kTileBytes, half_rows(tile, p, 0) + v_region,
                                  half_rows(tile, p, 1) + v_region);
    };
    const uint32_t first_tile = tile_begin + pair;
    const uint32_t my_tiles = first_tile < tile_end ? (tile_end - first_tile + kPairs - 1) / kPairs : 0u;
    // The row's first loads go out before anything else of it: the query columns are staged while they fly.
    if (second && my_tiles != 0) {
        issue_k(first_tile, cur.page[0], 0);
        issue_v(first_tile, cur.page[0], 0);
        if (my_tiles > 1) {
            issue_k(first_tile + kPairs, cur.page[1], 1);
            issue_v(first_tile + kPairs, cur.page[1], 1);
        }
    }

    // Query columns as MFMA B operands [nb][k-step][lane]; unused columns are zero.
    for (uint32_t nb = wave; nb < (uint32_t)NB; nb += kWaves) {
        const uint32_t c = nb * 16 + mt;
        const bool used = c < ncols;
        const uint32_t cc = used ? c : 0;
        const uint16_t* q_row =
            q + ((uint64_t)(flat_begin + cc / G) * a.hq + (uint64_t)kv_head * G + cc % G) * D + mc * 8;
#pragma unroll
        for (int i = 0; i < kKSteps; ++i) {
            const uint4 v = *reinterpret_cast<const uint4*>(q_row + i * 32);
            qb_lds[(nb * kKSteps + i) * 64 + lane] = used ? v : make_uint4(0, 0, 0, 0);
        }
    }
    if (tid < (2 + 2 * kMultipliers) * kPairs) (&progress[0][0])[tid] = 0;
    if (tid == 0) row_failed = 0u;
    gave_up = false;
    __syncthreads();

    // A operand of QK^T, k-step i: row mt, elements 32 * i + 8 * mc .. + 7 -> half mt / 8, line i / 2, chunk
    // 4 * (i % 2) + mc, row mt % 8: the k-steps lie 512 bytes apart.
    // B operand of PV, dim block db (tokens 4 * mc .. + 3 of dim 16 * db + mt) through the transposing read: the lane
    // hands in token 4 * mc + mt / 4, dims 16 * db + 4 * (mt % 4) .. + 3 -> half mc / 2, row 4 * (mc % 2) + mt / 4,
    // line db / 4, chunk 2 * (db % 4) + (mt % 4) / 2, its upper or lower 8 bytes: the dim blocks lie 256 bytes apart.
    const uint32_t k_read = (mt >> 3) * kHalfBytes + mc * 128 + (mt & 7) * 16;
    const uint32_t v_read =
        (mc >> 1) * kHalfBytes + (((mt & 3) >> 1) * 8 + (mc & 1) * 4 + (mt >> 2)) * 16 + (mt & 1) * 8;
    auto is_partial = [&](uint32_t t) { return t * kTileTokens < kv_begin || (t + 1) * kTileTokens > kv_end; };

    // The position of this lane's query token in column block `block` (values, not an indexed array: the block of
    // a wave is only known at run time, and an indexed array would live in memory).
    uint32_t position_of_block[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        position_of_block[b] = cur.position[b];
        asm volatile("" : "+v"(position_of_block[b]));
    }
    auto column_position = [&](uint32_t block) {
        uint32_t p = position_of_block[0];
#pragma unroll
        for (int b = 1; b < NB; ++b) p = block == (uint32_t)b ? position_of_block[b] : p;
        return p;
    };
    // One wave's part of the row: the column blocks kBlock0 .. + kBlocks - 1, and the loads if it is the second
    // wave of its pair.  Both instances pass the same workgroup barriers.
    auto walk_row = [&](auto blocks_tag, auto block0, auto loads_tag) __attribute__((always_inline)) {
        const uint32_t kBlock0 = block0;  // a constant where the wave's first column block is known at compile time
        constexpr int kBlocks = decltype(blocks_tag)::value;
        constexpr bool kLoads = decltype(loads_tag)::value;
        constexpr int kB = kBlocks > 0 ? kBlocks : 1;  // array extents

        uint32_t lim[kB];  // keys [kv_begin, lim) are visible to the column (0: column unused)
#pragma unroll
        for (int nb = 0; nb < kBlocks; ++nb) {
            const uint32_t position = column_position(kBlock0 + nb);
            lim[nb] = position != 0xffffffffu ? min(kv_end, position + 1) : 0u;
        }
        // A wave with one column block keeps its query operands in registers for the whole row.
        constexpr bool kQInRegs = kBlocks == 1;
        uint4 q_reg[kQInRegs ? kKSteps : 1];
        if (kQInRegs) {
#pragma unroll
            for (int ks = 0; ks < kKSteps; ++ks) q_reg[ks] = qb_lds[(kBlock0 * kKSteps + ks) * 64 + lane];
        }
        float run_max[kB], lane_sum[kB];
        f32x4_t o[kB][kDimBlocks];
#pragma unroll
        for (int nb = 0; nb < kB; ++nb) {
            run_max[nb] = -INFINITY;
            lane_sum[nb] = 0.0f;
#pragma unroll
            for (int db = 0; db < kDimBlocks; ++db) o[nb][db] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        }

        TilePages pid_ahead = cur.page[2];  // of tile i + 2
        for (uint32_t i = 0; i < my_tiles; ++i) {
            const uint32_t tile = first_tile + i * kPairs;
            const uint32_t stage = i & 1;
            const bool has1 = i + 1 < my_tiles, has2 = i + 2 < my_tiles;
            const TilePages pid2 = pid_ahead;
            if (kLoads) pid_ahead = load_page_id(tile + 3 * kPairs);
            const unsigned char* k_tile = my_stages + stage * kTileBytes;
            unsigned char* v_tile = my_stages + (2 + stage) * kTileBytes;

            // ---- K(i) is there: the loading wave sees its own loads return (they complete in order: K(i) has
            // landed once only V(i), K(i+1), V(i+1) are outstanding) and says so; the other wave reads that.
            if (kLoads) {
                wait_load_groups<kTileLoads>(has1 ? 3u : 1u);
                *say_landed_k = i + 1;
            } else {
                wait_until_above(landed_k, i);
            }
            // ---- logits S[token][column]
            f32x4_t s[kB];
            if constexpr (kBlocks > 0) {
#pragma unroll
                for (int nb = 0; nb < kBlocks; ++nb) s[nb] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int ks = 0; ks < kKSteps; ++ks) {
                    const uint4 ka = *reinterpret_cast<const uint4*>(k_tile + k_read + ks * 512);
#pragma unroll
                    for (int nb = 0; nb < kBlocks; ++nb)
                        s[nb] = mfma_16x16x32<Tag>(ka, kQInRegs ? q_reg[kQInRegs ? ks : 0]
                                                                : qb_lds[((kBlock0 + nb) * kKSteps + ks) * 64 + lane],
                                                   s[nb]);
                }
                wave_lds_fence();  // this wave has read the K stage
            }
            if (kLoads) {
                if (has2) {
#pragma unroll
                    for (int r = 0; r < kMultipliers; ++r) wait_until_above(word(2 + 2 * r), i);  // and so have the others
                    issue_k(tile + 2 * kPairs, pid2, stage);
                }
                // V(i) has landed once only K(i+1), V(i+1), K(i+2) are outstanding.  Rows outside the split have
                // probability 0, but their bytes may be NaN or Inf: they are zeroed before anyone multiplies.
                wait_load_groups<kTileLoads>((has1 ? 2u : 0u) + (has2 ? 1u : 0u));
                if (is_partial(tile)) {
                    for (uint32_t idx = lane; idx < kTileTokens * kDQ * 8; idx += 64) {
                        const uint32_t slot = idx & 63, block = idx >> 6;  // block = half * kDQ + line
                        const uint32_t vtoken = tile * kTileTokens + (block / kDQ) * 8 + (slot & 7);
                        if (vtoken < kv_begin || vtoken >= kv_end)
                            *reinterpret_cast<uint4*>(v_tile + idx * 16) = make_uint4(0, 0, 0, 0);
                    }
                    wave_lds_fence();
                }
                *say_landed_v = i + 1;
            } else {
                *read_k = i + 1;
            }

            if constexpr (kBlocks > 0) {
                // ---- online softmax per column over this lane's tokens 4*mc + r; nearly
                // every tile lies inside the range of every column and needs no mask
                ProbOperand<Tag> pa[kB];
                float alpha[kB];
                bool moved = false;
                auto softmax = [&](auto masked_tag) __attribute__((always_inline)) {
                    constexpr bool masked = decltype(masked_tag)::value;
#pragma unroll
                    for (int nb = 0; nb < kBlocks; ++nb) {
                        float v[4];
                        bool valid[4];
                        float m = -INFINITY;
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const uint32_t token = tile * kTileTokens + mc * 4 + r;
                            valid[r] = !masked || (token >= kv_begin && token < lim[nb]);
                            v[r] = valid[r] ? s[nb][r] * a.scale_log2 : -INFINITY;
                            m = fmaxf(m, v[r]);
                        }
                        m = quarter_wave_max(m);
                        const float next_max = m > run_max[nb] + kMaxSlack ? m : run_max[nb];
                        alpha[nb] = run_max[nb] > -INFINITY ? __builtin_amdgcn_exp2f(run_max[nb] - next_max) : 0.0f;
                        moved = moved || next_max != run_max[nb];
                        run_max[nb] = next_max;
                        float p[4], tile_sum = 0.0f;
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            p[r] = valid[r] ? __builtin_amdgcn_exp2f(v[r] - next_max) : 0.0f;
                            tile_sum += p[r];
                        }
                        lane_sum[nb] = lane_sum[nb] * alpha[nb] + tile_sum;
                        pa[nb].set(p);
                    }
                };
                if (tile * kTileTokens >= kv_begin && (tile + 1) * kTileTokens <= open_until) softmax(std::false_type());
                else softmax(std::true_type());
                if (__any(moved)) {
#pragma unroll
                    for (int nb = 0; nb < kBlocks; ++nb) {
                        float al[4];
#pragma unroll
                        for (int r = 0; r < 4; ++r) al[r] = __shfl(alpha[nb], mc * 4 + r, 64);
#pragma unroll
                        for (int db = 0; db < kDimBlocks; ++db)
#pragma unroll
                            for (int r = 0; r < 4; ++r) o[nb][db][r] *= al[r];
                    }
                }

                // ---- O[column][dim] += P^T V
                if (!kLoads) wait_until_above(landed_v, i);
#pragma unroll
                for (int db = 0; db < kDimBlocks; ++db) {
                    const uint2 b = lds_read_tr16_b64(v_tile + v_read + db * 256);
#pragma unroll
                    for (int nb = 0; nb < kBlocks; ++nb) {
#pragma unroll
                        for (int t = 0; t < ProbOperand<Tag>::kTerms; ++t)
                            o[nb][db] = mfma_16x16x16<Tag>(pa[nb].term[t], b, o[nb][db]);
                    }
                }
                wave_lds_fence();  // this wave has read the V stage
            } else if (!kLoads) {
                wait_until_above(landed_v, i);
            }
            if (kLoads) {
                if (has2) {
#pragma unroll
                    for (int r = 0; r < kMultipliers; ++r) wait_until_above(word(3 + 2 * r), i);
                    issue_v(tile + 2 * kPairs, pid2, stage);
                }
            } else {
                *read_v = i + 1;
            }
        }

        // ---- merge the states of the four waves that share these columns.  Column statistics live in the S layout
        // (lane <-> column mt), the accumulators in the MFMA output layout (lane <-> columns 4*mc + r, dim mt).
#pragma unroll
        for (int nb = 0; nb < kBlocks; ++nb) {
            lane_sum[nb] += __shfl_xor(lane_sum[nb], 16, 64);
            lane_sum[nb] += __shfl_xor(lane_sum[nb], 32, 64);
            if (mc == 0) wave_max_lds[pair][(kBlock0 + nb) * 16 + mt] = run_max[nb];
        }
        __syncthreads();  // every wave has left the tile loop: the stages may now be reused
#pragma unroll
        for (int nb = 0; nb < kBlocks; ++nb) {
            const uint32_t c = (kBlock0 + nb) * 16 + mt;
            float gm = wave_max_lds[0][c];
#pragma unroll
            for (int w = 1; w < kPairs; ++w) gm = fmaxf(gm, wave_max_lds[w][c]);
            const float f = run_max[nb] > -INFINITY ? __builtin_amdgcn_exp2f(run_max[nb] - gm) : 0.0f;
            lane_sum[nb] *= f;
            if (pair == 0 && mc == 0) col_max_lds[c] = gm;
            float fr[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) fr[r] = __shfl(f, mc * 4 + r, 64);
#pragma unroll
            for (int db = 0; db < kDimBlocks; ++db)
#pragma unroll
                for (int r = 0; r < 4; ++r) o[nb][db][r] *= fr[r];
        }
        for (uint32_t w = 0; w < (uint32_t)kPairs; ++w) {
            if (pair == w) {
#pragma unroll
                for (int nb = 0; nb < kBlocks; ++nb) {
                    if ((uint32_t)(kBlock0 + nb) * 16 < ncols) {
                        if (mc == 0) {
                            const uint32_t c = (kBlock0 + nb) * 16 + mt;
                            col_sum_lds[c] = (w == 0 ? 0.0f : col_sum_lds[c]) + lane_sum[nb];
                        }
#pragma unroll
                        for (int db = 0; db < kDimBlocks; ++db)
#pragma unroll
                            for (int r = 0; r < 4; ++r) {
                                float* dst =
                                    merge + ((kBlock0 + nb) * 16 + mc * 4 + r) * kMergeStride + db * 16 + mt;
                                *dst = (w == 0 ? 0.0f : *dst) + o[nb][db][r];
                            }
                    }
                }
            }
            __syncthreads();
        }
    };
    if (second)
        walk_row(std::integral_constant<int, kBlocksLoader>(), std::integral_constant<uint32_t, kMultipliers * kBlocksEach>(),
                 std::true_type());
    else if constexpr (kMultipliers == 1)
        walk_row(std::integral_constant<int, kBlocksEach>(), std::integral_constant<uint32_t, 0>(), std::false_type());
    else
        walk_row(std::integral_constant<int, kBlocksEach>(), role * kBlocksEach, std::false_type());

    // ---- emit: partial row of (split, q_head, token_in_tile); 1 KiB of contiguous f32 per wave store.  A row on
    // which a wait ran out is stored as an empty state.
    const bool failed = row_failed != 0u;  // written before the barriers of the merge
    if (failed && tid == 0) __hip_atomic_store(a.status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    const uint32_t rows = a.rows_per_split_head;
    for (uint32_t idx = tid; idx < ncols * (D / 4); idx += 64 * kWaves) {
        const uint32_t c = idx / (D / 4), d4 = idx % (D / 4);
        const uint64_t row = ((uint64_t)split * a.hq + (uint64_t)kv_head * G + c % G) * rows + c / G;
        float4 val = *reinterpret_cast<const float4*>(merge + c * kMergeStride + d4 * 4);
        if (failed) val = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        *reinterpret_cast<float4*>(&a.part_acc[row * D + d4 * 4]) = val;
    }
    if (tid < ncols) {
        const uint64_t row = ((uint64_t)split * a.hq + (uint64_t)kv_head * G + tid % G) * rows + tid / G;
        a.part_max[row] = failed ? -INFINITY : col_max_lds[tid];
        a.part_sum[row] = failed ? 0.0f : col_sum_lds[tid];
    }
    }  // rows of this workgroup
}

// Column blocks needed for tiles of up to `max_tile_tokens` query tokens and `group` heads per KV head.
inline int tiled_column_blocks(uint32_t max_tile_tokens, uint32_t group) { return (int)((max_tile_tokens * group + 15) / 16); }

template <typename Tag, int D>
inline int launch_tiled_map_typed(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a, uint32_t max_tile_tokens) {
    const int nb = tiled_column_blocks(max_tile_tokens, g.group);
    const dim3 grid((a.worker_cu ? a.num_workers : a.num_total_kv_splits) * g.hkv);
    const uint16_t* q = reinterpret_cast<const uint16_t*>(a.q);
    const uint16_t* pages = reinterpret_cast<const uint16_t*>(a.kv_pages);
#define PSI_TILED_PAIRED_LAUNCH(NB)                                                                                    \
    do {                                                                                                               \
        if (g.tokens_per_page == 8)                                                                                    \
            hipLaunchKernelGGL((split_kv_tiled_paired_map<Tag, D, NB, true>), grid, dim3(64 * tiled_paired_waves(NB)), 0, \
                               ctx->stream, a, a.walk.page_ids, a.kv_splits, a.req_slots, q, pages, a.q_token_tiles,   \
                               a.flat_token_indices, a.worker_cu);                                                     \
        else                                                                                                           \
            hipLaunchKernelGGL((split_kv_tiled_paired_map<Tag, D, NB, false>), grid, dim3(64 * tiled_paired_waves(NB)), 0, \
                               ctx->stream, a, a.walk.page_ids, a.kv_splits, a.req_slots, q, pages, a.q_token_tiles,   \
                               a.flat_token_indices, a.worker_cu);                                                     \
    } while (0)
    if (nb == 1) PSI_TILED_PAIRED_LAUNCH(1);
    else if (nb == 2) PSI_TILED_PAIRED_LAUNCH(2);
    else if (nb == 3) PSI_TILED_PAIRED_LAUNCH(3);
    else return PSI_HIP_ERR_UNSUPPORTED;  // (wider tiles: see launch_tiled_map_fast)
#undef PSI_TILED_PAIRED_LAUNCH
    return PSI_HIP_OK;
}

}  // namespace psi
