// Multi-token attention over the fp16 KV cache for head size 128 on gfx950: the MFMA kernel.
//
// Replaces ggml's mul_mat / diag_mask_inf / add / soft_max / mul_mat nodes of chatglm.cpp:687-717
// for qlen > 1 without ever materialising the [kvs x qlen] score matrix.  A workgroup owns 128
// consecutive tokens of one query head (32 per wave; for a few tokens of a grouped-query model: 128
// (head, token) rows of one KV group) and walks the key sequence, or its share of it, in 64-key tiles
// that all four waves share through LDS.  Both products run on v_mfma_f32_32x32x16_f16 with keys (first
// product) and head dims (second product) on the rows and the wave's 32 tokens on the columns:
// S^T = K Q^T leaves every lane holding, for its token, exactly the keys that the B operand of
// O^T = V^T P^T needs from it, so probabilities never leave registers.  The cache layouts of the
// reference are already K-major for both products: k_cache rows are contiguous in d, v_cache rows
// are contiguous in the sequence.
#include "glm_attn_internal.h"

namespace glm_attn {

#ifdef GLM_ATTN_TIMELINE
// Instrumented build (csrc/Makefile, target `timeline`): every wave of prefill_kernel leaves 100 MHz clock
// readings here, 16 per wave: 0 start, 1 first copies issued, 2 first tiles landed, 3 first product done,
// 8 / 9 / 10 end of the group's 1st / 2nd / 4th tile, 4 end of the tile loop, 5 last second product done,
// 6 the two groups merged, 7 output stores issued.
__device__ unsigned long long g_prefill_timeline[kTimelineSlots * 16];
#define PTS(i)                                                                                                   \
    do {                                                                                                         \
        const int slot_ = (blockIdx.y * gridDim.x + blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6);        \
        if ((threadIdx.x & 63) == 0 && slot_ < kTimelineSlots) g_prefill_timeline[slot_ * 16 + (i)] = wall_clock64(); \
    } while (0)
// copies the readings of the launches since the last call to the host (a later launch overwrites an earlier
// one's) and clears them
extern "C" int glm_attn_debug_prefill_timeline(unsigned long long *host, size_t n) {
    if (n > (size_t)kTimelineSlots * 16) n = (size_t)kTimelineSlots * 16;
    hipError_t e = hipMemcpyFromSymbol(host, HIP_SYMBOL(g_prefill_timeline), n * sizeof(unsigned long long));
    void *at = nullptr;
    if (e == hipSuccess) e = hipGetSymbolAddress(&at, HIP_SYMBOL(g_prefill_timeline));
    if (e == hipSuccess) e = hipMemset(at, 0, sizeof(unsigned long long) * kTimelineSlots * 16);
    return (int)e;
}
#else
#define PTS(i) \
    do {       \
    } while (0)
#endif

namespace {

constexpr int D = kFastHeadSize;
constexpr int BM = kPrefillRows;      // tokens per workgroup
constexpr int BN = kPrefillTileKeys;  // keys per tile
constexpr int WAVES = 4;
constexpr int THREADS = WAVES * 64;
constexpr float LOG2E = 1.4426950408889634f;
constexpr int RING = 3;  // LDS fragments in flight ahead of the MFMAs (4 no longer fit the 256 registers)
constexpr float kLazy = 8.f / LOG2E;  // see the online softmax in the kernel: 8 in base-2 logarithm units

typedef _Float16 half2v __attribute__((ext_vector_type(2)));

// maximum / sum of a value over lane i and lane i ^ 32 (v_permlane32_swap: no trip through LDS)
__device__ inline float max_of_halves(float x) {
    const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
}
__device__ inline float sum_of_halves(float x) {
    const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
}

__device__ inline floatx16 mfma32(half8 a, half8 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

// Row i (0..31) of a 32-key block holds this key of the block, so that accumulator register
// r = 4b + r' of lane half c (rows 8b + 4c + r') is element 4 (b & 1) + r' of k-slice c of the
// 16-key step b >> 1 of the second product.
__device__ inline int block_key(int i) {
    const int b = i >> 3, cc = (i >> 2) & 1, r = i & 3;
    return 16 * (b >> 1) + 8 * cc + 4 * (b & 1) + r;
}

// LDS tiles are filled by global_load_lds_dwordx4: the 64 lanes of a wave drop their 16 bytes at
// consecutive LDS addresses, no registers and no ds_write in between.  That rules out row padding, so
// bank conflicts are avoided by a swizzle instead: 16-byte chunk c of row r is stored at position
// c ^ k_swz(r) (K rows, 16 chunks) or c ^ v_swz(r) (V rows, 8 chunks).  The lane that fills position p
// of row r therefore fetches chunk p ^ swz(r) from global memory.
__device__ inline int k_swz(int row) { return row & 15; }
__device__ inline int v_swz(int row) { return (row >> 1) & 7; }

// The copy of a 64-key tile (K rows key0.., V columns key0..) into an LDS buffer is 8 instructions per
// wave, four for K and four for V, each moving 1 KiB: the 64 lanes drop their 16 bytes at consecutive LDS
// addresses from M0 on.  Piece i of K is four rows (4 (4 i + w) ..), 16 lanes a row; piece i of V is eight
// rows (8 (4 i + w) ..), 8 lanes a row.  A lane's source within its piece is the same for every piece of
// its wave, because rows 16 (K) or 32 (V) apart share their swizzle: one offset per lane for K and one for V,
// and the piece's own offset is scalar.
//
// Written as assembly so that the compiler does not see a write to LDS that it would make every later LDS
// read wait for (it cannot tell the two tile buffers apart); the kernel waits for the copy itself, before
// the barrier that opens the next tile.  M0 is written without telling the compiler (it accepts no such
// clobber): nothing else in this file uses it, gfx9 LDS instructions take no M0 and no register array is
// indexed at run time.
__device__ inline void copy_piece(const void *src_base, uint32_t lane_offset, uint32_t lds_dst) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds_dst), "v"(lane_offset), "s"(src_base) : "memory");
}

struct TileCopy {
    uint32_t k, v;  // this lane's byte offsets within a K piece and within a V piece
};

__device__ inline TileCopy tile_copy_lanes(int L, int w, int lane) {
    TileCopy tc;
    tc.k = (uint32_t)((lane >> 4) * D + (((lane & 15) ^ k_swz(4 * w + (lane >> 4))) << 3)) * 2u;
    tc.v = (uint32_t)((lane >> 3) * L + (((lane & 7) ^ v_swz(8 * w + (lane >> 3))) << 3)) * 2u;
    return tc;
}

// Piece i (0..3: K, 4..7: V) of the copy of the tile that starts at key0, into the K buffer at LDS byte
// address ks and the V buffer at vs.  left = cache rows from key0 to the cache end (a multiple of 8): K rows
// and V columns past the end are masked later, but their addresses have to be legal, so a K piece past the
// end reads the tile's first rows instead (a piece is four rows, so it is past the end as a whole or not at
// all) and tcv is the V offset with the 8-key chunks past the end sent to the first one.
__device__ inline void fetch_piece(int i, const __half *Kg, const __half *Vg, int L, int key0, int left, int w,
                                   uint32_t tck, uint32_t tcv, uint32_t ks, uint32_t vs) {
    if (i < 4) {
        const int blk = i * WAVES + w;
        const int row = blk * 4 < left ? blk * 4 : 0;
        copy_piece(Kg + (int64_t)(key0 + row) * D, tck, ks + (uint32_t)(blk * 4 * D * 2));
    } else {
        const int blk = (i - 4) * WAVES + w;
        copy_piece(Vg + (int64_t)blk * 8 * L + key0, tcv, vs + (uint32_t)(blk * 8 * BN * 2));
    }
}

// tcv of fetch_piece for a tile with fewer than 64 rows left
__device__ inline uint32_t v_offset_clamped(int L, int w, int lane, int left) {
    const int chunk = (lane & 7) ^ v_swz(8 * w + (lane >> 3));
    return (uint32_t)((lane >> 3) * L + ((chunk * 8 < left ? chunk : 0) << 3)) * 2u;
}

// V columns of keys that do not exist (>= kvs) may hold anything, and 0 * NaN is NaN: zero them in LDS.
// (tid: 0..THREADS-1 within the four waves that own the buffer)
__device__ inline void zero_missing_columns(__half (*Vs)[BN], int key0, int kvs, int tid) {
    asm volatile("" : "+v"(tid));  // rare path: keeps its index arithmetic from being hoisted out of the tile loop
    for (int idx = tid; idx < D * BN; idx += THREADS) {
        const int row = idx / BN, col = idx % BN;  // col: position within the row, swizzled by 16-byte chunk
        const int key = key0 + (((col >> 3) ^ v_swz(row)) << 3) + (col & 7);
        if (key >= kvs) {
            Vs[row][col] = __float2half(0.f);
        }
    }
}

// Two waves per SIMD (at most 256 registers each).  Within a wave the work on consecutive tiles overlaps:
// an iteration runs the second product of tile T-1 with the row maxima of tile T in its shadow, then the
// first product of tile T+1 with the exponentials of tile T in its shadow, so that the vector ALU works
// while the matrix pipe does and the wave has no phase of vector work alone.  K tiles therefore run two
// ahead of V tiles: an iteration reads K(T+1) and V(T-1) and receives the copies of K(T+2) and V(T).
//
// order: how workgroup ids map to (token tile, head) items.  0: tile-major as they come (all items
// cost the same).  Causal items cost more the later their tile: 1 starts the longest first, which
// lets the dispatcher even the slots out; 2, for a grid that fills the chip exactly once with two workgroups
// per CU, also puts the i-th longest and the i-th shortest half a grid apart, which is where the two
// workgroups of a CU come from.
//
// GROUPS: 1, or 2 for a grid with too few workgroups to give every CU two of them (a prompt of a few thousand
// tokens or less).  Then a workgroup has eight waves in two groups of four that own the same 128 rows; each group
// is what a whole workgroup is otherwise, with its own tile buffers, and takes every other tile of the key range;
// the second group hands its (m, l, O) to the first through LDS at the end.  A CU then holds its eight waves on
// one item at a time: no tail in which the long item of a causal prompt runs alone at half the occupancy, and no
// pass over partial results in global memory.
template <int GROUPS>
__global__ __launch_bounds__(THREADS * GROUPS, 2 / GROUPS) void prefill_kernel(AttendArgs a, int n_qtiles, int order,
                                                                              int packed) {
    // per group: K tiles [2][BN][D], then V tiles [2][D][BN]; the k-th tile of a group lives in buffer k & 1
    constexpr int GROUP_HALFS = 2 * BN * D + 2 * D * BN;
    __shared__ __attribute__((aligned(1024))) __half smem_all[GROUPS * GROUP_HALFS];
    constexpr uint32_t TILE_BYTES = BN * D * 2;  // a K tile and a V tile are the same size
    constexpr uint32_t V_AT = 2 * TILE_BYTES;

    PTS(0);
    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // in a scalar register: LDS targets of the copy are per wave
    const int grp = GROUPS > 1 ? wv >> 2 : 0, w = wv & 3;
    const int tid = threadIdx.x & (THREADS - 1);  // within the group
    __half *const smem = smem_all + grp * GROUP_HALFS;
    const uint32_t smem_at = (uint32_t)reinterpret_cast<uintptr_t>(smem);  // LDS byte address
    const int n = lane & 31, c = lane >> 5;
    // A workgroup owns 128 rows of one unit.  Normally a unit is a query head and its rows are the tokens.
    // packed: a unit is a KV group and its rows are (head of the group, token) pairs, head-major, so that a
    // few tokens fill a tile with the group's heads and every K/V tile is copied once per group, not once per
    // head (q16 is [h][qlen][d]: the rows of a group are contiguous there).
    const int heads_per_unit = packed ? a.s.G : 1;
    const int units = a.s.h / heads_per_unit;
    const int rows = heads_per_unit * a.qlen;
    int item = blockIdx.x;
    if (order == 2 && item >= (int)gridDim.x / 2) {
        item = (int)gridDim.x - 1 - (item - (int)gridDim.x / 2);
    }
    const int qt = order ? n_qtiles - 1 - item / units : item / units;
    const int unit = item % units;
    const int g = packed ? unit : unit / a.s.G;
    const int L = a.s.L;
    const __half *Kg = a.k_cache + (int64_t)g * L * D;
    const __half *Vg = a.v_cache + (int64_t)g * D * L;

    const int row0 = qt * BM + w * 32;  // first row of this wave
    // this lane's row, token and query head, worked out afresh where they are needed (a division each): kept
    // in registers across the tile loop they would be three too many
    auto lane_row = [&](int lane_n) {
        const int r = row0 + lane_n;
        return r < rows ? r : rows - 1;
    };

    // first and last token among rows [first, first + count) of the unit: a range that crosses into the next
    // head holds them all
    auto token_range = [&](int first, int count, int &t_min, int &t_max) {
        int last = first + count - 1;
        last = last < rows ? last : rows - 1;
        first = first < rows ? first : rows - 1;
        if (first / a.qlen == last / a.qlen) {
            t_min = first % a.qlen;
            t_max = last % a.qlen;
        } else {
            t_min = 0;
            t_max = a.qlen - 1;
        }
    };
    int wg_t_min, wg_t_max, wave_t_min, wave_t_max;  // (the maxima of a wave and the minima of a workgroup go unused)
    token_range(qt * BM, BM, wg_t_min, wg_t_max);
    token_range(row0, 32, wave_t_min, wave_t_max);

    // keys this workgroup has to visit: everything for an unmasked call, up to the diagonal otherwise
    int kv_end = a.kvs;
    if (a.causal) {
        const int last = a.p0 + wg_t_max + 1;  // one past the last key visible to the last token of the tile
        kv_end = last < kv_end ? last : kv_end;
    }
    const int n_tiles = (kv_end + BN - 1) / BN;
    const int last_tile = n_tiles - 1;
    // With nsplit > 1 (few tokens against a long cache) workgroup (x, y) walks only share y of the tiles, an
    // even number of them from an even tile on, and leaves (m, l, O) for merge_splits_kernel.
    const int nsplit = gridDim.y, split = blockIdx.y;
    const int per_split = nsplit > 1 ? (((n_tiles + nsplit - 1) / nsplit + 1) & ~1) : n_tiles;
    const int t0 = split * per_split;
    const int t1 = t0 + per_split < n_tiles ? t0 + per_split : n_tiles;
    // where this lane's row of this share goes (worked out where it is needed: registers are short in the loop)
    auto part_row = [&]() { return ((int64_t)split * n_qtiles * BM + (row0 + n)) * units + unit; };
    auto part_ml = [&]() { return a.split_scratch + (int64_t)nsplit * n_qtiles * BM * units * D + part_row() * 2; };
    if (nsplit > 1 && t0 >= n_tiles) {  // nothing left for this share (a causal tile that ends early)
        if (c == 0) {
            float *ml = part_ml();
            ml[0] = -INFINITY;
            ml[1] = 0.f;
        }
        return;
    }
    // The loop below is written for two tiles per round (the two score accumulators swap roles), and every
    // group runs the same number of rounds (they meet at the same barriers): group g takes tiles t0 + g,
    // t0 + g + GROUPS, ...; what that reaches beyond the share are tiles whose keys are all masked (key >= kv_lim).
    // Copies of tiles past the last one read the last one again.
    const int n_iter = ((t1 - t0 + GROUPS - 1) / GROUPS + 1) & ~1;
    const int tg0 = t0 + grp;  // this group's first tile
    const int kv_lim = a.kvs < t1 * BN ? a.kvs : t1 * BN;

    const TileCopy tc = tile_copy_lanes(L, w, lane);
    // pieces 0..3 of the copy of K tile `tile` / V tile `tile` into buffer `buf`
    auto copy_k = [&](int tile, int i, int buf) {
        const int key0 = (tile < last_tile ? tile : last_tile) * BN;
        fetch_piece(i, Kg, Vg, L, key0, L - key0, w, tc.k, 0u, smem_at + buf * TILE_BYTES, 0u);
    };
    auto copy_v = [&](int tile, int i, int buf, uint32_t tcv) {
        const int key0 = (tile < last_tile ? tile : last_tile) * BN;
        fetch_piece(4 + i, Kg, Vg, L, key0, L - key0, w, 0u, tcv, 0u, smem_at + V_AT + buf * TILE_BYTES);
    };
    auto v_lanes = [&](int tile) {  // this lane's offset within a V piece of that tile
        const int left = L - (tile < last_tile ? tile : last_tile) * BN;
        return left < BN ? v_offset_clamped(L, w, lane, left) : tc.v;
    };

#pragma unroll
    for (int i = 0; i < 4; i++) {
        copy_k(tg0, i, 0);
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        copy_k(tg0 + GROUPS, i, 1);
    }
    // the second product of the first iteration stands for a tile -1: probabilities 0 times V buffer 1,
    // which must hold finite numbers for that
    for (int idx = tid; idx < D * BN / 8; idx += THREADS) {
        half8 z;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            z[e] = (_Float16)0.f;
        }
        reinterpret_cast<half8 *>(smem + 2 * BN * D + D * BN)[idx] = z;  // (the group's own buffer, its own threads)
    }

    // Q^T operand: token n, dims t*16 + c*8 .. +8, resident for the whole kernel
    half8 qf[8];
    {
        const int r_ld = lane_row(n);
        const int hh = unit * heads_per_unit + r_ld / a.qlen, t_abs = r_ld % a.qlen;
        const __half *qrow = a.q16 + ((int64_t)hh * a.qlen + t_abs) * D + c * 8;
#pragma unroll
        for (int t = 0; t < 8; t++) {
            qf[t] = *reinterpret_cast<const half8 *>(qrow + t * 16);
        }
    }

    floatx16 o[4];
#pragma unroll
    for (int db = 0; db < 4; db++) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            o[db][r] = 0.f;
        }
    }
    // Reference point of the exponentials for token n (in the scores' units, the same in both lane halves) and the sum of
    // the probabilities of this lane's keys (the two halves of a token are added up after the last tile).
    float m = -INFINITY, l = 0.f;
    floatx16 nb;  // -m in every register (0 while m is -inf): where the score sums start
#pragma unroll
    for (int r = 0; r < 16; r++) {
        nb[r] = 0.f;
    }
    half8 pf[4];  // probabilities of the tile whose second product comes next
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
#pragma unroll
        for (int e = 0; e < 8; e++) {
            pf[ks][e] = (_Float16)0.f;
        }
    }

    // LDS byte addresses of this lane's fragments in buffer 0.  K: row block_key(n), 16-dim slice t at ka[t]
    // (second key block: + 32 rows); V: row n, 16-key slice ks at va[ks] (dim blocks: + 32 rows each).  Rows
    // 32 apart share their swizzle.
    uint32_t ka[8], va[4];
    {
        const int krow = block_key(n);
#pragma unroll
        for (int t = 0; t < 8; t++) {
            ka[t] = smem_at + (uint32_t)((krow * D + (((2 * t + c) ^ k_swz(krow)) << 3)) * 2);
        }
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            va[ks] = smem_at + V_AT + (uint32_t)((n * BN + (((2 * ks + c) ^ v_swz(n)) << 3)) * 2);
        }
    }
    typedef const __attribute__((address_space(3))) half8 *lds_frag;
    auto kfrag = [&](int buf, int i) {  // step i of the first product: 16-dim slice i >> 1 of key block i & 1
        return *(lds_frag)(uintptr_t)(ka[i >> 1] + (uint32_t)(buf * TILE_BYTES + (i & 1) * 32 * D * 2));
    };
    auto vfrag = [&](int buf, int j) {  // step j of the second: 16-key slice j >> 2 of dim block j & 3
        return *(lds_frag)(uintptr_t)(va[j >> 2] + (uint32_t)(buf * TILE_BYTES + (j & 3) * 32 * BN * 2));
    };

    // S^T = K Q^T - m for the K tile in buffer buf: two 32-key blocks.  The 16 fragments come through a ring, so
    // that a read is issued RING MFMAs before its use.  between(i) runs after step i.  The sums start from
    // nb, which holds minus the reference point of the exponentials in all its registers (the lane's token is the
    // same for all of them): a score leaves the matrix pipe one multiplication (by log2 e) away from v_exp_f32.
    auto first_product = [&](int buf, floatx16 (&s)[2], auto between) __attribute__((always_inline)) {
        half8 fr[RING];
#pragma unroll
        for (int i = 0; i < RING; i++) {
            fr[i] = kfrag(buf, i);
        }
#pragma unroll
        for (int i = 0; i < 16; i++) {
            s[i & 1] = mfma32(fr[i % RING], qf[i >> 1], i < 2 ? nb : s[i & 1]);
            if (i + RING < 16) {
                fr[i % RING] = kfrag(buf, i + RING);
            }
            between(i);
        }
    };
    // O^T += V^T P^T for the V tile in buffer buf: four 16-key steps, four 32-dim blocks each
    auto second_product = [&](int buf, auto between) __attribute__((always_inline)) {
        half8 fr[RING];
#pragma unroll
        for (int j = 0; j < RING; j++) {
            fr[j] = vfrag(buf, j);
        }
#pragma unroll
        for (int j = 0; j < 16; j++) {
            o[j & 3] = mfma32(fr[j % RING], pf[j >> 2], o[j & 3]);
            if (j + RING < 16) {
                fr[j % RING] = vfrag(buf, j + RING);
            }
            between(j);
        }
    };

    floatx16 sa[2], sb[2];  // scores of the current and of the next tile, swapping roles every iteration

    // The wait is the builtin, not assembly: the compiler then knows that its own loads (the queries) are
    // over too and puts no waits for them between the MFMAs, where they would wait for the copies.
    PTS(1);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();
    PTS(2);
    first_product(0, sa, [](int) {});
    PTS(3);

    // One iteration: sc holds the scores of tile T (in the buffers of parity par), sn takes those of the group's
    // next tile.  In the comments T+1, T-1, ... count the group's own tiles (GROUPS apart in the key range).
    auto iteration = [&](const int T, const int par, floatx16 (&sc)[2], floatx16 (&sn)[2]) __attribute__((always_inline)) {
        const int key0 = T * BN;
        // K(T+1) and V(T-1) have landed for every wave, and nobody reads K(T) or V(T-2) any more
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        __syncthreads();
        // V(T-1) has columns past the end, in this group or in another one (all groups take the barrier)
        if (T != tg0 && (T - grp) * BN > a.kvs) {
            if ((T - GROUPS + 1) * BN > a.kvs) {
                zero_missing_columns(reinterpret_cast<__half (*)[BN]>(smem + 2 * BN * D + (par ^ 1) * D * BN),
                                     (T - GROUPS) * BN, a.kvs, tid);
            }
            __syncthreads();
        }
        const uint32_t tcv = v_lanes(T);

        // ---- mask
        const bool need_mask = (key0 + BN > kv_lim) || (a.causal && key0 + BN - 1 > a.p0 + wave_t_min) || a.mask;
        if (need_mask) {
            int nn = n;
            asm volatile("" : "+v"(nn));  // so that the token is not worked out before the loop and kept
            const int t_abs = lane_row(nn) % a.qlen;
#pragma unroll
            for (int kb = 0; kb < 2; kb++) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int b = r >> 2;
                    const int key = key0 + kb * 32 + 16 * (b >> 1) + 8 * c + 4 * (b & 1) + (r & 3);
                    float v = sc[kb][r];
                    if (a.mask && key < a.kvs) {
                        v += a.mask[(int64_t)t_abs * a.kvs + key];
                    }
                    if (key >= kv_lim || (a.causal && key > a.p0 + t_abs)) {
                        v = -INFINITY;
                    }
                    sc[kb][r] = v;
                    if ((r & 7) == 7) {
                        // keeps the loads of an additive mask from being gathered into one batch of 32,
                        // whose registers this kernel does not have
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        }

        // ---- second product of tile T-1, with the row maximum of tile T in its shadow and the copy of
        // K(T+2) between the MFMAs, one piece at a time (eight pieces issued in one go fill the memory
        // pipe's queue and hold the wave up).
        // Online softmax for token n (the two lane halves hold different keys of it): the reference point m
        // of the exponentials only moves when the running maximum has grown by more than kLazy (8 in log2
        // units): probabilities may then reach 2^8, which fp16 holds with full relative precision, and
        // the rescaling of the 64 accumulator registers becomes rare.
        float mx = -INFINITY;  // over the scores as they are: relative to m
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                mx = fmaxf(mx, sc[kb][r]);
            }
        }
        mx = max_of_halves(mx);
        const bool move = (mx > kLazy) || (m == -INFINITY && mx != -INFINITY);
        second_product(par ^ 1, [&](int j) {
            if ((j & 3) == 1) {
                copy_v(T, j >> 2, par, tcv);
            } else if ((j & 3) == 3) {
                copy_k(T + 2 * GROUPS, j >> 2, par);
            }
        });
        if (__builtin_amdgcn_ballot_w64(move) != 0) {
            // by how much the reference point rises (from 0 to the maximum for a token's first keys)
            const float d = (mx == -INFINITY) ? 0.f : (m == -INFINITY ? mx : fmaxf(mx, 0.f));
            const float alpha = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(-d * LOG2E);
#pragma unroll
            for (int db = 0; db < 4; db++) {
                o[db] *= alpha;
            }
            l *= alpha;
            if (mx != -INFINITY) {
                m = (m == -INFINITY) ? mx : m + d;
            }
            const float nm = (m == -INFINITY) ? 0.f : -m;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                sc[0][r] -= d;  // this tile's scores were taken relative to the old point
                sc[1][r] -= d;
                nb[r] = nm;
            }
        }

        // ---- first product of tile T+1, with the exponentials of tile T in its shadow and the copy of V(T)
        first_product(par ^ 1, sn, [](int) {});
        // two probabilities per conversion; the sum is taken over the rounded values, the ones the second
        // product multiplies (v_dot2_f32_f16 against ones: fp32 sums of pairs)
        const half2v ones = {(_Float16)1.f, (_Float16)1.f};
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
                const half2v h = {(_Float16)__builtin_amdgcn_exp2f(sc[kb][r] * LOG2E),
                                  (_Float16)__builtin_amdgcn_exp2f(sc[kb][r + 1] * LOG2E)};
                l = __builtin_amdgcn_fdot2(h, ones, l, false);
                const int b = r >> 2;
                pf[kb * 2 + (b >> 1)][4 * (b & 1) + (r & 3)] = h[0];
                pf[kb * 2 + (b >> 1)][4 * (b & 1) + (r & 3) + 1] = h[1];
            }
        }
    };

    for (int T = tg0; T < tg0 + n_iter * GROUPS; T += 2 * GROUPS) {
        iteration(T, 0, sa, sb);
        if (T == tg0) PTS(8);
        iteration(T + GROUPS, 1, sb, sa);
        if (T == tg0) PTS(9);
        if (T == tg0 + 2 * GROUPS) PTS(10);
    }
    PTS(4);

    // ---- second product of the last tile (n_iter is even: V buffer 1)
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();
    if ((t0 + n_iter * GROUPS) * BN > a.kvs) {  // in some group
        const int T_last = tg0 + (n_iter - 1) * GROUPS;
        if ((T_last + 1) * BN > a.kvs) {
            zero_missing_columns(reinterpret_cast<__half (*)[BN]>(smem + 2 * BN * D + D * BN), T_last * BN, a.kvs, tid);
        }
        __syncthreads();
    }
    second_product(1, [](int) {});
    PTS(5);

    l = sum_of_halves(l);
    m *= LOG2E;  // from here on in base-2 logarithm units, which is what the merges' exponentials take
    if (GROUPS > 1) {
        // ---- the second group's (m, l, O) into the first's: wave w of either holds the same rows in the same
        // lanes, so O goes through LDS register by register, 64 lanes side by side (the second group's own tile
        // buffers are exactly 4 waves x 64 registers x 64 lanes of fp32), m and l through the first group's.
        __syncthreads();  // every wave has read its last tile
        float *xo = reinterpret_cast<float *>(smem_all + GROUP_HALFS) + w * 64 * 64 + lane;
        float *xml = reinterpret_cast<float *>(smem_all) + w * 128 + lane;
        if (grp == 1) {
#pragma unroll
            for (int db = 0; db < 4; db++) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    xo[(db * 16 + r) * 64] = o[db][r];
                }
            }
            xml[0] = m;
            xml[64] = l;
        }
        __syncthreads();
        if (grp == 1) {
            return;
        }
        const float m1 = xml[0], l1 = xml[64];
        const float M = fmaxf(m, m1);
        const float a0 = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m - M);
        const float a1 = (m1 == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m1 - M);
#pragma unroll
        for (int db = 0; db < 4; db++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                o[db][r] = o[db][r] * a0 + xo[(db * 16 + r) * 64] * a1;
            }
        }
        l = l * a0 + l1 * a1;
        m = M;
    }
    PTS(6);
    // ---- out[t][head*128 + dim] = O / l, or this share's (m, l, O) as they are
    if (nsplit > 1 && c == 0) {
        float *ml = part_ml();
        ml[0] = m;
        ml[1] = l;
    }
    if (row0 + n < rows || nsplit > 1) {
        const float inv = nsplit > 1 ? 1.f : 1.f / l;
        const int r_ld = lane_row(n);
        const int hh_out = unit * heads_per_unit + r_ld / a.qlen, t_abs = r_ld % a.qlen;
        float *orow = nsplit > 1 ? a.split_scratch + part_row() * D : a.out + (int64_t)t_abs * (a.s.h * D) + hh_out * D;
#pragma unroll
        for (int db = 0; db < 4; db++) {
#pragma unroll
            for (int b = 0; b < 4; b++) {
                floatx4 v;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    v[r] = o[db][b * 4 + r] * inv;
                }
                *reinterpret_cast<floatx4 *>(orow + db * 32 + 8 * b + 4 * c) = v;
            }
        }
    }
    PTS(7);
}

// out[t][head] = sum_s O_s 2^(m_s - M) / sum_s l_s 2^(m_s - M) over the shares of the key range, M = max m_s.
// 32 threads of four dims each per (row, unit), eight of those per workgroup; a thread walks the shares itself.
__global__ __launch_bounds__(256) void merge_splits_kernel(AttendArgs a, int padded_rows, int nsplit, int packed) {
    const int heads_per_unit = packed ? a.s.G : 1;
    const int units = a.s.h / heads_per_unit;
    const int rows = heads_per_unit * a.qlen;
    const int64_t ru = (int64_t)blockIdx.x * 8 + (threadIdx.x >> 5);  // (row, unit) in the order of the partials
    if (ru >= (int64_t)rows * units) {
        return;
    }
    const int r = (int)(ru / units), unit = (int)(ru % units);
    const int t = r % a.qlen, hh = unit * heads_per_unit + r / a.qlen;
    const int d4 = threadIdx.x & 31;
    const float *ml = a.split_scratch + (int64_t)nsplit * padded_rows * units * D;
    auto prow = [&](int sp) { return ((int64_t)sp * padded_rows + r) * units + unit; };
    float M = -INFINITY;
    for (int sp = 0; sp < nsplit; sp++) {
        M = fmaxf(M, ml[prow(sp) * 2]);
    }
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
    float lsum = 0.f;
    for (int sp = 0; sp < nsplit; sp++) {
        const float *rec = ml + prow(sp) * 2;
        if (rec[1] == 0.f) {
            continue;  // a share without keys left its O unwritten
        }
        const float wgt = __builtin_amdgcn_exp2f(rec[0] - M);
        lsum += rec[1] * wgt;
        acc += *reinterpret_cast<const floatx4 *>(a.split_scratch + prow(sp) * D + d4 * 4) * wgt;
    }
    *reinterpret_cast<floatx4 *>(a.out + (int64_t)t * (a.s.h * D) + hh * D + d4 * 4) = acc * (1.f / lsum);
}

}  // namespace

hipError_t launch_prefill(const AttendArgs &a, int num_cus, hipStream_t stream) {
    // Measured on 2048 causal tokens of 32 heads (512 items, 2 to 32 tiles each): 58 us with two four-wave
    // workgroups per CU, 65 us with one of eight waves (nothing runs beside an item's first tiles and its last
    // stores); on 1024 tokens 29 us against 60 us for four-wave workgroups cut along the keys and merged by a
    // second kernel.
    const PrefillPlan pl = plan_prefill(a.qlen, a.p0, a.kvs, a.s.h, a.s.G, a.causal, a.split_scratch ? a.split_floats : 0,
                                        num_cus);
    // the partials of a cut launch must fit the scratch (a launch that does not would write past it: checked here
    // once more, whatever chose nsplit)
    if (pl.nsplit > 1 && (!a.split_scratch || pl.part_floats > a.split_floats)) {
        return hipErrorInvalidValue;
    }
    if (pl.two_groups) {
        hipLaunchKernelGGL(prefill_kernel<2>, dim3(pl.n_items, pl.nsplit), dim3(2 * THREADS), 0, stream, a, pl.n_qtiles,
                           pl.order, pl.packed);
    } else {
        hipLaunchKernelGGL(prefill_kernel<1>, dim3(pl.n_items, pl.nsplit), dim3(THREADS), 0, stream, a, pl.n_qtiles,
                           pl.order, pl.packed);
    }
    if (pl.nsplit > 1) {
        hipLaunchKernelGGL(merge_splits_kernel, dim3((unsigned)(((int64_t)pl.rows * pl.units + 7) / 8)), dim3(256), 0, stream,
                           a, pl.n_qtiles * BM, pl.nsplit, pl.packed);
    }
    return hipGetLastError();
}

}  // namespace glm_attn
