// gfx950 split-KV map for prefill chunks: many query tokens of one request against one KV range,
// 2-byte K/V (bf16 / f16), head_dim 256, pages of 16*2^k tokens.  Same results as the
// multi-query map (semantics of
// crates/inference-backend-metal/src/components/metal/gqa_split_kv_tiled_q.metal:49-319), other
// decomposition: here the matrix cores and the LDS are the bound, not HBM.
//
// Work decomposition
//   one workgroup (8 waves) = one (row group, kv_head [, half of the query heads]).  A row group is
//   a run of consecutive Q-token tiles of one request whose kv_split rows start at the same key
//   (the rows of one KV partition).  With more than 5 query heads per KV head the heads are dealt
//   to two workgroups.  The workgroup's query columns, column c = token_in_group * heads + head,
//   are dealt out 16 per wave: a wave keeps the online-softmax state and the accumulators of its
//   columns for the whole KV range, so wave states never merge.  The eight waves walk the KV range
//   together in tiles of 32 keys which they load once, together, into LDS (two buffers, one
//   barrier per tile; global loads run two tiles ahead in two register sets).
//
// Per 32-key tile and wave (16 columns)
//   QK^T  S[key][column] on v_mfma_f32_16x16x32 of the storage type: A = K rows from LDS (key 16 * b + i in row i of
//         key block b), B = the query columns, held in registers for the whole kernel.  A lane ends up with keys
//         16 * b + 4 * (lane / 16) + r, r = 0..3, b = 0, 1, of its column.
//   softmax  per column, in-lane over those 8 keys; masks only on tiles that touch the start of the range
//         or a column's causal limit.  The reference maximum of a column moves only when a tile
//         exceeds it by more than 2^8; a wave-wide vote guards the cross-lane maximum and the
//         rescaling of the accumulators, which therefore run a handful of times per range.
//         Probabilities stay below 2^8.
//   PV    O^T[dim][column] += V^T[dim][key] * P^T[key][column] on v_mfma_f32_16x16x32_f16: B = the probabilities,
//         rounded once to f16 (11 significant bits; one bf16 term alone, 8 bits, costs the whole output tolerance,
//         and two bf16 terms cost half as many matrix instructions again), A = V^T read straight out of the
//         row-major V tile with the transposing LDS read of gfx950 (ds_read_b64_tr_b16: the 16 lanes of a quarter
//         wave hand in 16 addresses of 4 elements each, a 16 x 4 block, and get it back transposed - lane 4a + c
//         receives element c of the addresses a, a + 4, a + 8, a + 12), so no instruction of the kernel
//         transposes V.  The V tile is kept as f16 in LDS: bf16 pages are converted once per tile on their way
//         from the load registers into LDS (exact for 6.1e-5 <= |v| <= 65504; smaller magnitudes lose bits or
//         flush to zero, larger ones saturate - neither occurs in a KV cache, and both stay far inside the output
//         tolerance for values that do).  The accumulators keep a column per lane, so rescaling needs no
//         cross-lane traffic.
//
// LDS layout per buffer
//   K    [32 keys][D] elements, 16-byte chunk index XOR (key % 16): the 16 lanes of an operand read (16 rows, one
//        chunk) then hit 16 different bank groups, and a row-wise store stays a permutation of its row.
//   V    [32 keys][D] f16, rows padded to D * 2 + 32 bytes: the four keys of a quarter wave's transposing read
//        (32 bytes each, 16 dims) then fall into different bank groups, and so do the eight keys of two quarters.
//   page IDs of up to 4096 pages of the range, refilled for longer ranges.
#pragma once
#include "split_kv_tiled_kernel.h"

namespace psi {

constexpr int kChunkKeys = 32;         // keys per KV tile
constexpr int kChunkWaves = 8;
constexpr int kChunkColBlocks = 1;     // 16-column blocks per wave
constexpr int kChunkWaveCols = 16 * kChunkColBlocks;
static_assert(kChunkWaves * kChunkWaveCols == kChunkCols, "128 query columns per workgroup");
constexpr uint32_t kNoRow = 0xffffffffu;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;  // 128-bit word that stays in registers

// Probabilities of 8 keys -> B operand of the 16x16x32 f16 contraction: one term, rounded to nearest.
__device__ __forceinline__ uint4 prob_operand_f16(const float (&p)[8]) {
    const f16x8_t h = {(_Float16)p[0], (_Float16)p[1], (_Float16)p[2], (_Float16)p[3],
                       (_Float16)p[4], (_Float16)p[5], (_Float16)p[6], (_Float16)p[7]};
    return __builtin_bit_cast(uint4, h);
}

// 8 elements of the storage type -> 8 f16.  bf16: widening is exact, the narrowing truncates (exact inside the
// f16 range, see the header).
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
        out[i] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo, hi));
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
    static constexpr int kIdCap = 4096;  // page IDs of a stretch of the KV range kept in LDS (+8: two tiles of look-ahead)
    static constexpr int bytes = 2 * (kKBytes + kVtBytes) + (kIdCap + 8) * 4;
};

template <typename Tag, int D>
__global__ __launch_bounds__(64 * kChunkWaves, 2) void split_kv_chunk_map(
    MapArgs a, const uint32_t* __restrict__ page_ids, const uint32_t* __restrict__ kv_splits,
    const uint32_t* __restrict__ req_slots, const uint16_t* __restrict__ q, const uint16_t* __restrict__ pages,
    const uint32_t* __restrict__ q_token_tiles, const uint32_t* __restrict__ flat_token_indices,
    const uint32_t* __restrict__ row_groups, uint32_t group_tiles, uint32_t num_groups, uint32_t head_subsets) {
    resolve_active(a);
    static_assert(D == 256, "the tile loaders are laid out for head_dim 256");
    constexpr int kKSteps = D / 32;              // MFMA k-steps of QK^T
    constexpr int kDimBlocks = D / 16;           // 16-dim output blocks of PV
    constexpr int kRowChunks = D / 8;            // 16-byte chunks per K row
    constexpr int kLoads = kChunkKeys * kRowChunks / (64 * kChunkWaves);  // 128-bit loads per thread and operand (2)
    constexpr int kKBytes = ChunkLds<D>::kKBytes;
    constexpr int kVtBytes = ChunkLds<D>::kVtBytes;
    constexpr int kVStride = ChunkLds<D>::kVStride;
    constexpr int kBufBytes = kKBytes + kVtBytes;
    constexpr int CB = kChunkColBlocks;
    constexpr float kSlack = 8.0f;
    constexpr int kIdCap = ChunkLds<D>::kIdCap;
    static_assert(kLoads == 2 && CB == 1, "loader and softmax are written for 8 waves of 16 columns");
    // Dynamic LDS (the launcher passes ChunkLds<D>::bytes): with a static size the compiler sees
    // that one workgroup fills the CU and lifts the register cap.
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const uint32_t TS = a.rows_per_split_head;  // Q tokens per tile
    // heads of the KV head served here: head_first + [0, G)
    const uint32_t subset = blockIdx.x % head_subsets;
    const uint32_t kv_head = (blockIdx.x / head_subsets) % a.walk.hkv;
    const uint32_t group = blockIdx.x / (head_subsets * a.walk.hkv);
    const uint32_t heads_per_subset = (a.group + head_subsets - 1) / head_subsets;
    const uint32_t head_first = kv_head * a.group + subset * heads_per_subset;
    const uint32_t G = min(heads_per_subset, a.group - subset * heads_per_subset);
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t mt = lane & 15, mc = lane >> 4;
    if (group >= num_groups) return;

    // ---- the group: rows[m] is the kv_split row of its m-th Q-token tile
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
    // wave-uniform by construction; said explicitly so that everything derived from it stays scalar
    const uint32_t kv_end_max = __builtin_amdgcn_readfirstlane(
        wave_max_u32(my_row_ok && lane < num_tiles ? kv_splits[my_row * 3 + 2] : 0u));
    const uint32_t flat_begin = q_token_tiles[q_tile0 * 2];
    const uint32_t flat_end = q_token_tiles[(q_tile0 + num_tiles - 1) * 2 + 1];
    if (flat_end <= flat_begin || flat_end > a.num_active_tokens || kv_end_max <= kv_begin) return;
    const uint32_t ncols = (flat_end - flat_begin) * G;
    if (ncols > (uint32_t)kChunkCols || flat_end - flat_begin > num_tiles * TS) return;  // the planner never builds such a group
    const uint32_t req_slot = req_slots[flat_begin];

    // ---- this lane's column c = 16 * wave + mt: visible range, partial-state row, query row as B
    // operands (dims 32 * ks + 8 * mc .. +8; zero for an unused column)
    const uint32_t c = wave * kChunkWaveCols + mt;
    const bool used = c < ncols;
    uint32_t lim = 0;        // keys [kv_begin, lim) are visible to the column; 0: column unused
    uint64_t part_row = 0;   // partial-state row of the column
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
    // Tiles at or beyond wave_hi hold no visible key for this wave; tiles inside [kv_begin, wave_lo)
    // need no mask.
    const uint32_t wave_lo = __builtin_amdgcn_readfirstlane(wave_min_u32(used ? lim : 0xffffffffu));
    const uint32_t wave_hi = __builtin_amdgcn_readfirstlane(wave_max_u32(lim));

    // ---- page walk.  The page IDs of a stretch of the KV range (kIdCap pages) sit in LDS, so the
    // per-tile path has no dependent global access; a tile's two IDs are read one step before they
    // are needed.
    const uint32_t log2p = 31 - __builtin_clz(a.walk.tokens_per_page);
    const uint32_t page_mask = a.walk.tokens_per_page - 1;
    const uint32_t* table_row = page_ids + ((uint64_t)req_slot * a.walk.num_layers + a.layer) *
                                                      a.walk.num_blocks * a.walk.ids_per_block;
    const uint32_t last_page = (kv_end_max - 1) >> log2p;
    const uint32_t key_base0 = kv_begin & ~(uint32_t)(kChunkKeys - 1);
    const uint32_t num_kv_tiles = (kv_end_max - key_base0 + kChunkKeys - 1) / kChunkKeys;
    const uint32_t stretch_tiles = ((uint32_t)kIdCap << log2p) / kChunkKeys;  // tiles per refill of the ID table
    uint32_t* id_lds = reinterpret_cast<uint32_t*>(lds + 2 * kBufBytes);
    uint32_t id_page0 = 0;  // page behind id_lds[0]
    auto refill_ids = [&](uint32_t first_tile) {
        id_page0 = (key_base0 + first_tile * kChunkKeys) >> log2p;
        // only the pages the range still has: every later lookup is clamped to last_page
        const uint32_t count = min((uint32_t)kIdCap + 8, last_page - id_page0 + 1);
        for (uint32_t i = tid; i < count; i += 64 * kChunkWaves) id_lds[i] = table_row[id_page0 + i];
    };
    struct TileIds {
        uint32_t a, b;  // page of keys 0..15 and of keys 16..31 of a tile (the same value in every lane)
    };
    // Tiles past the end of the range are clamped to the last one: loads and stores stay
    // unconditional, which keeps the compiler's count of outstanding loads exact.
    auto read_ids = [&](uint32_t t) -> TileIds {
        const uint32_t kb = key_base0 + min(t, num_kv_tiles - 1) * kChunkKeys;
        return TileIds{id_lds[min(kb >> log2p, last_page) - id_page0], id_lds[min((kb + 16) >> log2p, last_page) - id_page0]};
    };
    struct TileBases {
        const unsigned char* a;  // page of keys 0..15 of the tile, advanced to the tile's first token
        const unsigned char* b;  // page of keys 16..31
    };
    const uint64_t page_bytes = a.walk.page_elems * 2;
    auto tile_bases = [&](uint32_t t, TileIds ids) -> TileBases {
        const uint32_t kb = key_base0 + min(t, num_kv_tiles - 1) * kChunkKeys;
        const uint64_t in_page = (uint64_t)(kb & page_mask) * (D * 2);
        const unsigned char* base = reinterpret_cast<const unsigned char*>(pages);
        return TileBases{base + __builtin_amdgcn_readfirstlane(ids.a) * page_bytes + in_page,
                         base + __builtin_amdgcn_readfirstlane(ids.b) * page_bytes + in_page};
    };

    // ---- cooperative tile loaders: per-thread byte offsets inside a page are fixed for the kernel.  Thread
    // (ld_sub, ld_chunk) takes the 16-byte chunk ld_chunk of keys ld_sub and 16 + ld_sub, of K and of V.
    constexpr int kSubs = 64 * kChunkWaves / kRowChunks;  // 16
    const uint32_t ld_chunk = tid % kRowChunks;
    const uint32_t ld_sub = tid / kRowChunks;
    const uint32_t k_off = ((kv_head * a.walk.tokens_per_page + ld_sub) * D + ld_chunk * 8) * 2;
    const uint32_t v_off = (((a.walk.hkv + kv_head) * a.walk.tokens_per_page + ld_sub) * D + ld_chunk * 8) * 2;
    // keys 16..31 sit 16 rows further on in a page that holds the whole tile, and at the same offset of the next
    // page otherwise (tile_bases then points at that page)
    const uint32_t second_half = a.walk.tokens_per_page == 16 ? 0u : 16u * D * 2u;
    struct Staging {
        u32x4_t k[kLoads], v[kLoads];
    };
    auto issue_loads = [&](TileBases tb) __attribute__((always_inline)) -> Staging {
        Staging st;
        st.k[0] = *reinterpret_cast<const u32x4_t*>(tb.a + k_off);                // keys 0..15
        st.k[1] = *reinterpret_cast<const u32x4_t*>(tb.b + k_off + second_half);  // keys 16..31
        st.v[0] = *reinterpret_cast<const u32x4_t*>(tb.a + v_off);
        st.v[1] = *reinterpret_cast<const u32x4_t*>(tb.b + v_off + second_half);
        return st;
    };
    // Registers -> LDS buffer `buf`.  V rows outside [kv_begin, kv_end_max) are zeroed: their
    // probability is 0 but their bytes may be NaN / Inf.
    const uint32_t k_store0 = ld_sub * (D * 2) + ((ld_chunk ^ ld_sub) * 16);
    const uint32_t k_store1 = k_store0 + kSubs * (D * 2);
    const uint32_t v_store0 = ld_sub * kVStride + ld_chunk * 16;
    const uint32_t v_store1 = v_store0 + kSubs * kVStride;
    auto store_tile = [&](uint32_t it, uint32_t buf, const Staging& st) __attribute__((always_inline)) {
        unsigned char* kbuf = lds + buf * kBufBytes;
        unsigned char* vbuf = kbuf + kKBytes;
        const uint32_t kb = key_base0 + min(it, num_kv_tiles - 1) * kChunkKeys;
        *reinterpret_cast<u32x4_t*>(kbuf + k_store0) = st.k[0];
        *reinterpret_cast<u32x4_t*>(kbuf + k_store1) = st.k[1];
        u32x4_t w0 = to_f16x8<Tag>(st.v[0]), w1 = to_f16x8<Tag>(st.v[1]);
        if (kb < kv_begin || kb + kChunkKeys > kv_end_max) {  // first or last tile of the range
            const uint32_t token = kb + ld_sub;
            if (token < kv_begin || token >= kv_end_max) w0 = u32x4_t{0u, 0u, 0u, 0u};
            if (token + kSubs < kv_begin || token + kSubs >= kv_end_max) w1 = u32x4_t{0u, 0u, 0u, 0u};
        }
        *reinterpret_cast<u32x4_t*>(vbuf + v_store0) = w0;
        *reinterpret_cast<u32x4_t*>(vbuf + v_store1) = w1;
    };

    // ---- operand read addresses of this lane
    // K row of (block b, lane row mt): key 16 * b + mt, chunk (4 * ks + mc) ^ mt
    const uint32_t k_row0 = mt * (D * 2);
    // V^T operand of (dim block db, key block b): the lane hands in the address of key 16 * b + 4 * mc + mt / 4,
    // dims 16 * db + 4 * (mt % 4) .. + 3, and receives keys 16 * b + 4 * mc + 0..3 of dim 16 * db + mt
    const uint32_t vt_base = (4 * mc + (mt >> 2)) * kVStride + (mt & 3) * 8;

    float run_max = -INFINITY, lane_sum = 0.0f;
    f32x4_t o[kDimBlocks];
#pragma unroll
    for (int db = 0; db < kDimBlocks; ++db) o[db] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    const bool wave_has_cols = wave * kChunkWaveCols < ncols;

    // `masked`: the tile touches the start of the range or a causal limit of this wave (wave-uniform).
    auto compute_tile = [&](uint32_t it, uint32_t buf, bool masked) __attribute__((always_inline)) {
        const unsigned char* kbuf = lds + buf * kBufBytes;
        const unsigned char* vbuf = kbuf + kKBytes;
        const uint32_t kb = key_base0 + it * kChunkKeys;
        // ---- logits S[key][column]: two key blocks
        // The K operands are read kAhead k-steps before the products that take them, and the order is pinned: left
        // to itself the compiler keeps two operands in flight, and every product then waits out the LDS latency
        // (450 -> 441 us on the 2048-on-4096 chunk, side by side).  The same treatment of the V^T operands measures
        // slower than the compiler's own order (+3 %; +4 % with the first reads issued ahead of the softmax).
        f32x4_t s0 = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f}, s1 = s0;
        constexpr int kAhead = 4;
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
        // ---- online softmax; this lane holds keys kb + 16 * b + 4 * mc + r, j = 4 * b + r, of column mt.
        // Logits relative to the column's reference maximum; masked keys at -inf.
        float v[8];  // raw logits; masked keys at -inf
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = j < 4 ? s0[j] : s1[j - 4];
        if (masked) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t token = kb + 16 * (j >> 2) + 4 * mc + (j & 3);
                if (token < kv_begin || token >= lim) v[j] = -INFINITY;
            }
        }
        // scale > 0: the maximum of the scaled logits is the scaled maximum
        float m = fmaxf(fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3])), fmaxf(fmaxf(v[4], v[5]), fmaxf(v[6], v[7]))) * a.scale_log2;
        // The reference maximum moves only when some key exceeds it by more than kSlack (log2 domain):
        // rare after the first tiles, so the cross-lane maximum and the rescaling sit behind a
        // wave-wide test.  A column with no visible key so far keeps max = -inf, sum = 0, O = 0.
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
        // exp2(logit * scale - reference); a column that has seen no key at all (reference -inf) has
        // only masked keys here: -inf - 0 keeps them at probability 0
        const float neg_ref = run_max > -INFINITY ? -run_max : 0.0f;
        float p[8], tile_sum = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            p[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(v[j], a.scale_log2, neg_ref));
            tile_sum += p[j];
        }
        lane_sum += tile_sum;
        const uint4 pb = prob_operand_f16(p);
        // ---- O^T[dim][column] += V^T * P^T, four dim blocks at a time
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
    };

    // ---- main loop: tile `it` lives in LDS buffer it % 2.  Its global loads are issued two tiles
    // earlier into one of two register sets and parked in LDS one tile earlier, so a load has two
    // tile times to arrive.  The loop body is written twice so that the register sets keep their names.
    auto step = [&](uint32_t it, Staging& incoming, const Staging& parked, TileIds& ids) __attribute__((always_inline)) {
        incoming = issue_loads(tile_bases(it + 2, ids));
        ids = read_ids(it + 3);
        const uint32_t kb = key_base0 + it * kChunkKeys;
        if (it < num_kv_tiles && wave_has_cols && kb < wave_hi)
            compute_tile(it, it & 1, !(kb >= kv_begin && kb + kChunkKeys <= wave_lo));
        store_tile(it + 1, (it + 1) & 1, parked);
        __syncthreads();
    };
    refill_ids(0);
    __syncthreads();
    Staging st_a, st_b;
    st_a = issue_loads(tile_bases(0, read_ids(0)));
    store_tile(0, 0, st_a);
    st_a = issue_loads(tile_bases(1, read_ids(1)));
    TileIds ids = read_ids(2);
    uint32_t next_refill = stretch_tiles;
    __syncthreads();
    for (uint32_t it = 0; it < num_kv_tiles; it += 2) {
        if (it >= next_refill) {  // rare: the range is longer than the ID table
            refill_ids(it);
            next_refill += stretch_tiles;
            __syncthreads();
        }
        step(it, st_b, st_a, ids);
        step(it + 1, st_a, st_b, ids);
    }

    // ---- emit this wave's columns: un-normalised accumulators, log2-domain maximum, sum
    lane_sum += __shfl_xor(lane_sum, 16, 64);
    lane_sum += __shfl_xor(lane_sum, 32, 64);
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
    static const hipError_t lds_ok = hipFuncSetAttribute(reinterpret_cast<const void*>(&split_kv_chunk_map<Tag, D>),
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, ChunkLds<D>::bytes);
    if (lds_ok != hipSuccess) return PSI_HIP_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((split_kv_chunk_map<Tag, D>), grid, dim3(64 * kChunkWaves), ChunkLds<D>::bytes, ctx->stream, a, a.walk.page_ids,
                       a.kv_splits, a.req_slots, reinterpret_cast<const uint16_t*>(a.q),
                       reinterpret_cast<const uint16_t*>(a.kv_pages), a.q_token_tiles, a.flat_token_indices, row_groups,
                       group_tiles, num_groups, subsets);
    return PSI_HIP_OK;
}

}  // namespace psi
