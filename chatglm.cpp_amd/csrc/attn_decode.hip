// Single-token attention over the fp16 KV cache for head size 128 on gfx950: a bandwidth kernel.
//
// One launch does rope(q, k), the K/V append and the attention of one layer (chatglm.cpp:655-717 for
// qlen == 1).  The cache sequence of each KV group is cut into 64-key tiles that are dealt out to
// nsplit workgroups, up to four tiles (256 keys) a round.  A workgroup is eight waves with two kinds of
// work: score wave w loads the K rows of tile w, prepares a quarter of the group's queries while they
// are on their way (rope, scale, fp16), computes S^T = K q^T for all heads of the group and, with the
// other score waves, the round's softmax, and leaves P in LDS; output wave w loads the V columns of 32
// output dims for all keys of the round and accumulates O^T = V^T P^T for those dims.  The up to 16
// query heads of the group are the 16 columns of v_mfma_f32_16x16x32_f16 tiles.  Waves hand over through
// counters in LDS (no workgroup barrier after the first), and O never leaves the registers of the
// output waves.
//
// Across workgroups the merge happens in the same launch: every workgroup leaves its partial in memory
// as self-validating 64-byte lines, one per (head, 16 output dims), stamped with the launch count, and
// the score waves of every workgroup then fold the lines of all splits for one slice of the output,
// polling them past the caches until they carry this launch's stamp.  The wait is bounded, and a slice
// whose wait ran out is redone by a later workgroup (decode_body).
//
// The new token's K and V never take part in a cache load of this launch: the first workgroup of each
// group ropes and appends them and attends to them from registers.
#include "glm_attn_internal.h"

namespace glm_attn {

#ifdef GLM_ATTN_TIMELINE
// Instrumented build (csrc/Makefile, target `timeline`): every wave leaves 100 MHz clock readings here,
// 16 per wave; DecodeTimelineStamp in glm_attn_internal.h names them.
__device__ unsigned long long g_decode_timeline[kTimelineSlots * 16];
#define TS(i)                                                                                                \
    do {                                                                                                     \
        const int slot_ = (blockIdx.y * gridDim.x + blockIdx.x) * 2 * kDecodeMaxWaves + (threadIdx.x >> 6);      \
        if ((threadIdx.x & 63) == 0 && slot_ < kTimelineSlots) g_decode_timeline[slot_ * 16 + (i)] = wall_clock64(); \
    } while (0)
#define TSCOUNT(i)                                                                                           \
    do {                                                                                                     \
        const int slot_ = (blockIdx.y * gridDim.x + blockIdx.x) * 2 * kDecodeMaxWaves + (threadIdx.x >> 6);  \
        if ((threadIdx.x & 63) == 0 && slot_ < kTimelineSlots) g_decode_timeline[slot_ * 16 + (i)] += 1;      \
    } while (0)
#else
#define TS(i) \
    do {      \
    } while (0)
#define TSCOUNT(i) \
    do {           \
    } while (0)
#endif

namespace {

constexpr int D = kFastHeadSize;
constexpr int TILE = kDecodeTileKeys;
constexpr int W = kDecodeMaxWaves;
constexpr int QUADS = D / 16;  // 16-dim slices of a head: one 64-byte line each in a split partial
static_assert(kDecodePartFloats == kMaxGroupHeads * QUADS * 16, "line layout");

typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------------------------------------------
// Lines of a split partial.  A line is four 16-byte pieces; a piece holds the launch's stamp, the fp32
// base-2 log-sum-exp max * log2(e) + log2(sum) of the (split, head) and four values of O / sum as fp16
// (O / sum is an average of fp16 V values: it cannot overflow, and the rounding is 2^-12 relative on a
// partial whose weight in the result is at most 1).  A 16-byte store is performed as one, so a piece that
// shows the stamp is complete with everything needed to fold it: the data is its own ready flag.
__device__ inline uintx4 pack_piece(unsigned int stamp, floatx4 v, unsigned int lse_bits) {
    const half2v a = {(_Float16)v[0], (_Float16)v[1]}, b = {(_Float16)v[2], (_Float16)v[3]};
    return uintx4{stamp, lse_bits, __builtin_bit_cast(unsigned int, a), __builtin_bit_cast(unsigned int, b)};
}

// Data that crosses workgroups inside one launch moves with relaxed device-scope accesses: they are
// performed at the device's coherence point, so neither side needs a device-scope fence (such fences
// write back or invalidate a whole L2 on this multi-die part and cost far more than the data).
// (The s_nop covers the wait state that the hardware wants between a store of more than 8 bytes and a
// write to the registers that hold its data: the compiler does not look into the assembly.)
__device__ inline void st_dev4(float *p, uintx4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(p), "v"(v) : "memory");
}
__device__ inline void wait_vm() { asm volatile("s_waitcnt vmcnt(0)" : : : "memory"); }

// 1, 2, 4 or 8 16-byte loads at device scope, all issued before the one wait.  Load i is done by the lanes
// whose bit is set in mask[i]; the other lanes keep what r[i] held.  One block of assembly, so that
// nothing can touch the destination registers between the loads and the wait.
#define GLM_LD_LINE(i) "s_and_b64 exec, %[sv], %[m" #i "]\n\tglobal_load_dwordx4 %[r" #i "], %[p" #i "], off sc1\n\t"
__device__ inline void ld_lines(const float *const (&p)[1], uintx4 (&r)[1], const unsigned long long (&m)[1]) {
    unsigned long long saved;
    asm volatile("s_mov_b64 %[sv], exec\n\t" GLM_LD_LINE(0) "s_mov_b64 exec, %[sv]\n\ts_waitcnt vmcnt(0)"
                 : [sv] "=&s"(saved), [r0] "+v"(r[0])
                 : [p0] "v"(p[0]), [m0] "s"(m[0])
                 : "memory", "scc");
}
__device__ inline void ld_lines(const float *const (&p)[2], uintx4 (&r)[2], const unsigned long long (&m)[2]) {
    unsigned long long saved;
    asm volatile("s_mov_b64 %[sv], exec\n\t" GLM_LD_LINE(0) GLM_LD_LINE(1) "s_mov_b64 exec, %[sv]\n\ts_waitcnt vmcnt(0)"
                 : [sv] "=&s"(saved), [r0] "+v"(r[0]), [r1] "+v"(r[1])
                 : [p0] "v"(p[0]), [p1] "v"(p[1]), [m0] "s"(m[0]), [m1] "s"(m[1])
                 : "memory", "scc");
}
__device__ inline void ld_lines(const float *const (&p)[4], uintx4 (&r)[4], const unsigned long long (&m)[4]) {
    unsigned long long saved;
    asm volatile("s_mov_b64 %[sv], exec\n\t" GLM_LD_LINE(0) GLM_LD_LINE(1) GLM_LD_LINE(2) GLM_LD_LINE(3)
                 "s_mov_b64 exec, %[sv]\n\ts_waitcnt vmcnt(0)"
                 : [sv] "=&s"(saved), [r0] "+v"(r[0]), [r1] "+v"(r[1]), [r2] "+v"(r[2]), [r3] "+v"(r[3])
                 : [p0] "v"(p[0]), [p1] "v"(p[1]), [p2] "v"(p[2]), [p3] "v"(p[3]), [m0] "s"(m[0]), [m1] "s"(m[1]),
                   [m2] "s"(m[2]), [m3] "s"(m[3])
                 : "memory", "scc");
}
__device__ inline void ld_lines(const float *const (&p)[8], uintx4 (&r)[8], const unsigned long long (&m)[8]) {
    unsigned long long saved;
    asm volatile("s_mov_b64 %[sv], exec\n\t" GLM_LD_LINE(0) GLM_LD_LINE(1) GLM_LD_LINE(2) GLM_LD_LINE(3) GLM_LD_LINE(4)
                 GLM_LD_LINE(5) GLM_LD_LINE(6) GLM_LD_LINE(7) "s_mov_b64 exec, %[sv]\n\ts_waitcnt vmcnt(0)"
                 : [sv] "=&s"(saved), [r0] "+v"(r[0]), [r1] "+v"(r[1]), [r2] "+v"(r[2]), [r3] "+v"(r[3]),
                   [r4] "+v"(r[4]), [r5] "+v"(r[5]), [r6] "+v"(r[6]), [r7] "+v"(r[7])
                 : [p0] "v"(p[0]), [p1] "v"(p[1]), [p2] "v"(p[2]), [p3] "v"(p[3]), [p4] "v"(p[4]), [p5] "v"(p[5]),
                   [p6] "v"(p[6]), [p7] "v"(p[7]), [m0] "s"(m[0]), [m1] "s"(m[1]), [m2] "s"(m[2]), [m3] "s"(m[3]),
                   [m4] "s"(m[4]), [m5] "s"(m[5]), [m6] "s"(m[6]), [m7] "s"(m[7])
                 : "memory", "scc");
}
#undef GLM_LD_LINE

__device__ inline floatx4 mfma16(half8 a, half8 b, floatx4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

// Row rho (0..15) of sub-block T (0..3) of a 64-key tile holds this key of the tile: accumulator row
// 4c + r of sub-block T is key (T >> 1) * 32 + c * 8 + (T & 1) * 4 + r, so that a lane's eight values
// of sub-blocks 2u and 2u + 1 are eight consecutive keys, one 16-byte piece of the P operand.
__device__ inline int tile_key(int T, int rho) { return (T >> 1) * 32 + (rho >> 2) * 8 + (T & 1) * 4 + (rho & 3); }

__device__ inline half8 ld_stream(const __half *p) { return *reinterpret_cast<const half8 *>(p); }

// K rows of one 64-key tile as MFMA A operands: lane (j, c) holds dims t*32 + c*8 .. of key tile_key(T, j).
__device__ inline void load_k_tile(const __half *Kg, int L, int key0, int lane, half8 (&kf)[4][4]) {
    const int j = lane & 15, c = lane >> 4;
#pragma unroll
    for (int T = 0; T < 4; T++) {
        int key = key0 + tile_key(T, j);
        key = key < L ? key : L - 1;  // rows past the cache end are masked later; keep the address legal
        const __half *row = Kg + (int64_t)key * D + c * 8;
#pragma unroll
        for (int t = 0; t < 4; t++) {
            kf[T][t] = ld_stream(row + t * 32);
        }
    }
}

// V columns of up to 256 keys (nk tiles from key0) for the 32 output dims of wave w, as MFMA A operands:
// lane (j, c) holds keys ks*32 + c*8 .. of dim w*32 + jb*16 + j.  Steps beyond the nk tiles read step 0
// again (the same lines, no extra memory traffic) and are not used.
template <int KS0, int KS1>
__device__ inline void load_v_dims(const __half *Vg, int L, int key0, int nk, int w, int lane, half8 (&vf)[2][8]) {
    const int j = lane & 15, c = lane >> 4;
#pragma unroll
    for (int jb = 0; jb < 2; jb++) {
        const __half *row = Vg + (int64_t)(w * 32 + jb * 16 + j) * L;
#pragma unroll
        for (int ks = KS0; ks < KS1; ks++) {
            int s0 = key0 + (ks < 2 * nk ? ks : 0) * 32 + c * 8;
            s0 = s0 <= L - 8 ? s0 : L - 8;
            vf[jb][ks] = ld_stream(row + s0);
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// A head's row in the registers of one lane, in the MFMA operand layout: lane (j, c) holds dims
// t*32 + c*8 + e, t = 0..3, e = 0..7.  For every rope type the partner of each of these 32 dims is
// one of them too, so a lane ropes its share on its own.  The cos/sin pairs it needs are contiguous in
// a table row and are fetched with 16-byte loads (two pairs each).
struct RowRegs {
    floatx4 x[4][2];
    floatx4 cs[8];
};

template <int TYPE>
__device__ inline void issue_row_loads(const float *head, int c, const int (&pos)[2], const RopeSpec &rope,
                                       RowRegs &r) {
#pragma unroll
    for (int t = 0; t < 4; t++) {
        r.x[t][0] = *reinterpret_cast<const floatx4 *>(head + t * 32 + c * 8);
        r.x[t][1] = *reinterpret_cast<const floatx4 *>(head + t * 32 + c * 8 + 4);
    }
    if (TYPE == GLM_ATTN_ROPE_GPTJ || TYPE == GLM_ATTN_ROPE_CHATGLM2) {
        // pair of dim d is d >> 1: four pairs per t, from t*16 + c*4
        constexpr int NT = (TYPE == GLM_ATTN_ROPE_GPTJ) ? 4 : 2;
        const float2 *row = rope.table + (int64_t)pos[0] * rope.pairs;
#pragma unroll
        for (int t = 0; t < NT; t++) {
            r.cs[t * 2 + 0] = *reinterpret_cast<const floatx4 *>(row + t * 16 + c * 4);
            r.cs[t * 2 + 1] = *reinterpret_cast<const floatx4 *>(row + t * 16 + c * 4 + 2);
        }
    } else if (TYPE == GLM_ATTN_ROPE_NEOX) {
        // pair of dim d is d % 64: eight pairs from (t & 1)*32 + c*8, shared by t and t + 2
        const float2 *row = rope.table + (int64_t)pos[0] * rope.pairs;
#pragma unroll
        for (int tt = 0; tt < 2; tt++) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                r.cs[tt * 4 + i] = *reinterpret_cast<const floatx4 *>(row + tt * 32 + c * 8 + i * 2);
            }
        }
    } else if (TYPE == GLM_ATTN_ROPE_CHATGLM) {
        // NEOX inside each half of the head: pair c*8 + e for both t of a half, positions per half
#pragma unroll
        for (int hf = 0; hf < 2; hf++) {
            const float2 *row = rope.table + (int64_t)pos[hf] * rope.pairs;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                r.cs[hf * 4 + i] = *reinterpret_cast<const floatx4 *>(row + c * 8 + i * 2);
            }
        }
    }
}

// rope (chatglm.cpp:523-618), then `* scale` in fp32 and the fp16 rounding of ggml's mat-mul operand
template <int TYPE>
__device__ inline void finish_row(const RowRegs &r, float scale, bool zero, half8 (&out)[4]) {
#pragma unroll
    for (int t = 0; t < 4; t++) {
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float self = r.x[t][e >> 2][e & 3];
            float x = self;
            if (TYPE == GLM_ATTN_ROPE_GPTJ || (TYPE == GLM_ATTN_ROPE_CHATGLM2 && t < 2)) {
                const float partner = r.x[t][e >> 2][(e & 3) ^ 1];
                const floatx4 cs = r.cs[t * 2 + (e >> 2)];
                const int k = (e >> 1) & 1;
                x = rope_rotate(self, partner, cs[2 * k], cs[2 * k + 1], !(e & 1));
            } else if (TYPE == GLM_ATTN_ROPE_NEOX) {
                const float partner = r.x[t ^ 2][e >> 2][e & 3];
                const floatx4 cs = r.cs[(t & 1) * 4 + (e >> 1)];
                x = rope_rotate(self, partner, cs[2 * (e & 1)], cs[2 * (e & 1) + 1], t < 2);
            } else if (TYPE == GLM_ATTN_ROPE_CHATGLM) {
                const float partner = r.x[t ^ 1][e >> 2][e & 3];
                const floatx4 cs = r.cs[(t >> 1) * 4 + (e >> 1)];
                x = rope_rotate(self, partner, cs[2 * (e & 1)], cs[2 * (e & 1) + 1], !(t & 1));
            }
            out[t][e] = zero ? (_Float16)0.f : (_Float16)__fmul_rn(x, scale);
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// The group's queries for the score waves: score wave w ropes, scales and rounds heads 4w .. 4w + 3
// (lane: head 4w + (lane >> 4), dims (lane & 15) * 8 .. + 7) and leaves them in LDS, where all four
// waves then pick up the whole operand.  Partners that are not among the lane's own eight dims (the
// NEOX pairings) are simply loaded as well.
constexpr int QPAD = D + 8;  // row pitch of the fp16 query tile in LDS (halfs): conflict-free b128 reads

struct QPart {
    floatx4 x[2], xp[2];
    floatx4 cs[4];
};

template <int TYPE>
__device__ inline void issue_q_part(const float *head, int d0, const int (&pos)[2], const RopeSpec &rope, QPart &r) {
    r.x[0] = *reinterpret_cast<const floatx4 *>(head + d0);
    r.x[1] = *reinterpret_cast<const floatx4 *>(head + d0 + 4);
    if (TYPE == GLM_ATTN_ROPE_GPTJ || TYPE == GLM_ATTN_ROPE_CHATGLM2) {
        // pair of dim d is d >> 1: four pairs from d0 / 2 (dims that are not rotated read the last four)
        int p0 = d0 >> 1;
        p0 = p0 <= rope.pairs - 4 ? p0 : rope.pairs - 4;
        const float2 *row = rope.table + (int64_t)pos[0] * rope.pairs + p0;
        r.cs[0] = *reinterpret_cast<const floatx4 *>(row);
        r.cs[1] = *reinterpret_cast<const floatx4 *>(row + 2);
    } else if (TYPE == GLM_ATTN_ROPE_NEOX) {
        // pairs (d, d + 64), pair index d % 64
        r.xp[0] = *reinterpret_cast<const floatx4 *>(head + (d0 ^ 64));
        r.xp[1] = *reinterpret_cast<const floatx4 *>(head + (d0 ^ 64) + 4);
        const float2 *row = rope.table + (int64_t)pos[0] * rope.pairs + (d0 & 63);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            r.cs[i] = *reinterpret_cast<const floatx4 *>(row + i * 2);
        }
    } else if (TYPE == GLM_ATTN_ROPE_CHATGLM) {
        // NEOX inside each half of the head: pairs (el, el + 32), pair index el % 32, positions per half
        r.xp[0] = *reinterpret_cast<const floatx4 *>(head + (d0 ^ 32));
        r.xp[1] = *reinterpret_cast<const floatx4 *>(head + (d0 ^ 32) + 4);
        const float2 *row = rope.table + (int64_t)pos[d0 >> 6] * rope.pairs + (d0 & 31);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            r.cs[i] = *reinterpret_cast<const floatx4 *>(row + i * 2);
        }
    }
}

// rope (chatglm.cpp:523-618), then `* scale` in fp32 (chatglm.cpp:686) and the fp16 rounding of ggml's
// mat-mul operand
template <int TYPE>
__device__ inline half8 finish_q_part(const QPart &r, int d0, float scale, bool zero) {
    half8 out;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const float self = r.x[e >> 2][e & 3];
        float x = self;
        if (TYPE == GLM_ATTN_ROPE_GPTJ || TYPE == GLM_ATTN_ROPE_CHATGLM2) {
            const float partner = r.x[e >> 2][(e & 3) ^ 1];
            const floatx4 cs = r.cs[e >> 2];
            const int k = (e >> 1) & 1;
            const float xr = rope_rotate(self, partner, cs[2 * k], cs[2 * k + 1], !(e & 1));
            x = (TYPE == GLM_ATTN_ROPE_GPTJ || d0 < D / 2) ? xr : self;
        } else if (TYPE == GLM_ATTN_ROPE_NEOX) {
            const floatx4 cs = r.cs[e >> 1];
            x = rope_rotate(self, r.xp[e >> 2][e & 3], cs[2 * (e & 1)], cs[2 * (e & 1) + 1], d0 < 64);
        } else if (TYPE == GLM_ATTN_ROPE_CHATGLM) {
            const floatx4 cs = r.cs[e >> 1];
            x = rope_rotate(self, r.xp[e >> 2][e & 3], cs[2 * (e & 1)], cs[2 * (e & 1) + 1], (d0 & 63) < 32);
        }
        out[e] = zero ? (_Float16)0.f : (_Float16)__fmul_rn(x, scale);
    }
    return out;
}

// ---------------------------------------------------------------------------------------------------
// Merge across workgroups: fold the lines of all splits for quads [q_begin, q_end) of KV group g (a quad
// is 16 output dims of one head, index head * QUADS + quad).  A wave works alone on its quads, no LDS:
// lane (s, quad slot, piece) takes piece `piece` of the lines of splits s, s + SL, ... of its quad, all
// lines of a block of quads are loaded at once, and the split lanes of a quad are summed with cross-lane
// operations.
struct MergeGeom {
    int nsplit, sl_log;  // SL = 1 << sl_log lanes per (quad, piece)
    int nl;              // lines per lane and quad: ceil(nsplit / SL)
    unsigned int stamp32;
    const float *part_g;    // lines of the group: [16 heads][QUADS][nsplit][16 floats], a slice's lines side by side
    float *out_g;           // [G][D]
    unsigned long long *gen_word;  // the group's launch count, and what it becomes when this launch is over
    unsigned long long gen_next;
};

// All-lanes reductions over the lanes that differ in the upper sl_log bits of the lane index, without
// LDS: the two row swaps of gfx950 for bits 5 and 4, rotations inside the rows of 16 lanes fused into
// the operation (DPP) for bits 3 and 2 (a rotation by 8 pairs lanes 8 apart; with all four bits in
// play, rotations by 4 and then 8 cover the four lanes 4 apart).
__device__ inline float rot_row(float x, int n) {
    return n == 4 ? __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x124, 0xf, 0xf, false))
                  : __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x128, 0xf, 0xf, false));
}
template <typename F>
__device__ inline float reduce_splits(float x, int sl_log, F op) {
    if (sl_log > 3) x = op(x, rot_row(x, 4));
    if (sl_log > 2) x = op(x, rot_row(x, 8));
    if (sl_log > 1) {
        auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
        x = op(__uint_as_float(a[0]), __uint_as_float(a[1]));
    }
    if (sl_log > 0) {
        auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
        x = op(__uint_as_float(b[0]), __uint_as_float(b[1]));
    }
    return x;
}

// (max, sum of weights, weighted O) of the lines a lane has folded, the weights relative to the max
struct Fold {
    float m, w;
    floatx4 o;
};

// One block of the merge: lines k0 .. k0 + NLP - 1 (line k is split k * SL + s) of the PC quads q[], all
// loaded at once and polled until every one carries the stamp, then folded into acc[] in the order of their
// index: the result does not depend on the order in which the lines showed up.  FIRST: acc[] is empty.
// Returns 1 when the wait ran out.
template <int NLP, int PC, bool FIRST>
__device__ inline int poll_block(const MergeGeom &mg, const int (&q)[PC], const bool (&qvalid)[PC], int k0, int s,
                                 int piece, unsigned long long t0, unsigned long long limit, Fold (&acc)[PC]) {
    constexpr int N = NLP * PC;
    uintx4 r[N];
    const float *p[N];
    bool need[N];
    unsigned long long pending[N];
#pragma unroll
    for (int pp = 0; pp < PC; pp++) {
#pragma unroll
        for (int k = 0; k < NLP; k++) {
            const int i = pp * NLP + k;
            const int sp = merge_split_of(k0 + k, mg.sl_log, s);
            r[i] = uintx4{0u, 0u, 0u, 0u};
            need[i] = qvalid[pp] && sp < mg.nsplit;
            p[i] = mg.part_g + merge_piece_offset(q[pp], mg.nsplit, sp < mg.nsplit ? sp : 0, piece);
            pending[i] = __ballot(need[i]);
        }
    }
    TS(13);
    while (true) {
        const unsigned long long now = wall_clock64();  // read while the loads are on their way
        ld_lines(p, r, pending);                        // only what has not arrived yet is loaded again
        TSCOUNT(14);
        TS(15);
        unsigned long long any = 0ull;
#pragma unroll
        for (int i = 0; i < N; i++) {
            if (pending[i] != 0ull) {
                pending[i] = __ballot(need[i] && r[i][0] != mg.stamp32);
                any |= pending[i];
            }
        }
        if (any == 0ull) {
            break;
        }
        if (now - t0 > limit) {
            return 1;
        }
        __builtin_amdgcn_s_sleep(1);
    }
    TS(12);
#pragma unroll
    for (int pp = 0; pp < PC; pp++) {
        float lse[NLP];
        float m_new = FIRST ? -INFINITY : acc[pp].m;
#pragma unroll
        for (int k = 0; k < NLP; k++) {
            lse[k] = need[pp * NLP + k] ? __uint_as_float(r[pp * NLP + k][1]) : -INFINITY;
            m_new = fmaxf(m_new, lse[k]);
        }
        const float m_ref = (m_new == -INFINITY) ? 0.f : m_new;  // nothing to fold: every weight below is 0
        Fold f;
        f.m = m_new;
        if (FIRST) {
            f.w = 0.f;
            f.o = floatx4{0.f, 0.f, 0.f, 0.f};
        } else {
            const float sc = __builtin_amdgcn_exp2f(acc[pp].m - m_ref);  // exp2(-inf) = 0
            f.w = acc[pp].w * sc;
            f.o = acc[pp].o * sc;
        }
#pragma unroll
        for (int k = 0; k < NLP; k++) {
            const uintx4 rr = r[pp * NLP + k];
            const float wgt = __builtin_amdgcn_exp2f(lse[k] - m_ref);  // 0 for lines that are not there
            // (copies first: a bit cast straight from a vector element reads the vector's first element)
            const unsigned int u0 = rr[2], u1 = rr[3];
            const half2v h0 = __builtin_bit_cast(half2v, u0), h1 = __builtin_bit_cast(half2v, u1);
            f.w += wgt;
            f.o[0] = __builtin_fmaf(wgt, (float)h0[0], f.o[0]);
            f.o[1] = __builtin_fmaf(wgt, (float)h0[1], f.o[1]);
            f.o[2] = __builtin_fmaf(wgt, (float)h1[0], f.o[2]);
            f.o[3] = __builtin_fmaf(wgt, (float)h1[1], f.o[3]);
        }
        acc[pp] = f;
    }
    return 0;
}

// What ends a quad: the (max, sum, O) of all lanes of a piece merged.
__device__ inline void reduce_fold(Fold &acc, int sl_log) {
    const float m_all = reduce_splits(acc.m, sl_log, [](float x, float y) { return fmaxf(x, y); });
    const float f = (acc.m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(acc.m - m_all);
    auto add = [](float x, float y) { return x + y; };
    acc.m = m_all;
    acc.w = reduce_splits(acc.w * f, sl_log, add);
#pragma unroll
    for (int e = 0; e < 4; e++) {
        acc.o[e] = reduce_splits(acc.o[e] * f, sl_log, add);
    }
}

// The quads of the calling wave (wave `wi` of `nw`), PC passes of its QW quad slots at a time, NLP lines per lane
// and block.
template <int NLP, int PC>
__device__ inline int merge_passes(const MergeGeom &mg, int q_begin, int q_end, int wi, int nw, int lane,
                                   unsigned long long t0, unsigned long long limit) {
    const int qw = 16 >> mg.sl_log;
    int piece, qslot, s;
    merge_lane(mg.sl_log, lane, &piece, &qslot, &s);
    for (int q0 = q_begin + wi * qw; q0 < q_end; q0 += PC * nw * qw) {
        int q[PC];
        bool qvalid[PC];
        Fold acc[PC];
#pragma unroll
        for (int pp = 0; pp < PC; pp++) {
            const int qq = merge_quad_of(q0, pp, nw, mg.sl_log, qslot);
            qvalid[pp] = qq < q_end;
            q[pp] = qvalid[pp] ? qq : q_end - 1;
        }
        if (poll_block<NLP, PC, true>(mg, q, qvalid, 0, s, piece, t0, limit, acc)) {
            return 1;
        }
        for (int k0 = NLP; k0 < mg.nl; k0 += NLP) {
            if (poll_block<NLP, PC, false>(mg, q, qvalid, k0, s, piece, t0, limit, acc)) {
                return 1;
            }
        }
#pragma unroll
        for (int pp = 0; pp < PC; pp++) {
            if (q0 + pp * nw * qw < q_end) {  // the same in every lane
                reduce_fold(acc[pp], mg.sl_log);
                if (qvalid[pp] && s == 0) {
                    // (1 / sum to one ulp, then a product: the values were rounded to fp16 on their way here)
                    *reinterpret_cast<floatx4 *>(mg.out_g + q[pp] * 16 + piece * 4) =
                        acc[pp].o * __builtin_amdgcn_rcpf(acc[pp].w);
                }
            }
        }
        TS(11);
    }
    return 0;
}

// Merges quads [q_begin, q_end) of KV group g, dealt out to the calling waves (wave `wi` of `nw`).  Returns 0 when
// every quad was written, 1 when the wait ran out (the quads of the block that was being waited for, and the wave's
// later ones, are not written).  Whoever completes a quad has seen a line of every workgroup of the group: all of
// them have read the launch count by then, and it may move on (`bump`: this caller is one of those that say so).
__device__ inline int merge_quads(const MergeGeom &mg, int q_begin, int q_end, int wi, int nw, int lane,
                                  unsigned long long t0, unsigned long long limit, bool bump) {
    // the code that runs is the one for the number of lines a lane really has: at 2.3 ns a vector instruction,
    // folding lines that are not there costs as much as folding lines that are
    // (the template arguments are merge_shape's nlp and pc, spelled as ranges of nl: within an instantiation the
    // compiler then knows how many blocks of lines there are)
    const int failed = mg.nl <= 1   ? merge_passes<1, 4>(mg, q_begin, q_end, wi, nw, lane, t0, limit)
                       : mg.nl <= 2 ? merge_passes<2, 2>(mg, q_begin, q_end, wi, nw, lane, t0, limit)
                       : mg.nl <= 4 ? merge_passes<4, 1>(mg, q_begin, q_end, wi, nw, lane, t0, limit)
                                    : merge_passes<8, 1>(mg, q_begin, q_end, wi, nw, lane, t0, limit);
    if (!failed && bump && lane == 0) {
        __hip_atomic_store(mg.gen_word, mg.gen_next, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return failed;
}

// Before its first look at the lines of the others a wave waits 0.7 us plus 0.12 us per 4096 keys of the group
// (see decode_body), in ticks of the 100 MHz clock.  Measured at 32767 keys: 1.0 us of waiting 11.7 us a layer,
// 1.6 to 1.9 us 11.3 us, 2.2 us 11.6 us; at 4095 keys 0.8 us is the best.
constexpr int kFirstLookTicks = 70;
constexpr int kFirstLookTicksPer64Tiles = 12;
constexpr int PPITCH = W * TILE + 8;  // row pitch of the P tile in LDS (halfs): conflict-free 16-byte accesses
constexpr int kBlock = 2 * W * 64;    // W score waves, then W output waves

struct DecodeShared {
    __attribute__((aligned(16))) __half p[16][PPITCH];  // P^T of the round: [head][key]
    float m[2][W][16];  // maxes of a round per score wave (rounds alternate between the two copies)
    float mrun[2][16];  // running max after a round
    float l[W][16];     // sums per score wave, at the final running max
    float pnew[16];     // probability of the new token
    __attribute__((aligned(16))) __half knew[D];  // its key, roped, fp16
    __attribute__((aligned(16))) __half q[16][QPAD];  // the group's queries, roped, scaled, fp16
    int k_issued;       // score waves whose first tile loads are in the memory pipeline
    int q_ready;        // score waves that have left their part of the queries
    int m_ready;        // score waves that have left their maxes, over all rounds
    int p_ready;        // score waves that have left their part of P, over all rounds
    int p_done;         // output waves that are through with P, over all rounds
    int stored;         // output waves whose line stores have been performed
};

// A wave waits for waves of its own workgroup (all resident by construction) through a counter in LDS.
// The wait is bounded all the same, so that a mistake in the hand-over could not hang the device: when
// it runs out the launch goes on with what it has and reports it.
__device__ inline void lds_wait_ge(int *ctr, int target, uint32_t *flags) {
    for (int i = 0; i < (1 << 20); i++) {
        if (__hip_atomic_load(ctr, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) >= target) {
            return;
        }
        __builtin_amdgcn_s_sleep(1);
    }
    atomicOr(flags, kFlagMergeIncomplete);
}
__device__ inline void lds_signal(int *ctr, int lane) {
    // the wave's LDS writes first, then the count
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    if (lane == 0) {
        __hip_atomic_fetch_add(ctr, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
}

__device__ inline float max_over_c(float x) {  // over the four lanes (j, c) of a head
    auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ inline float sum_over_c(float x) {
    auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// A slice that was left behind has been written after all: whoever takes the flag off takes it off the
// count of lost slices as well (once, however many redo it).
__device__ inline void slice_redone(unsigned long long *claim, unsigned long long stamp, unsigned int *lost, int lane) {
    if (lane == 0) {
        const unsigned long long old = __hip_atomic_exchange(claim, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (old == stamp) {
            __hip_atomic_fetch_add(lost, 0xffffffffu, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

struct Geom {
    int lane, w, j, c, g, split;
    int tb, te, rounds;
    bool owner_wg;
    unsigned long long t_start;
    unsigned long long gen_v;  // the launch count as loaded, in vector registers (see decode_body)
};

// A use of v that costs nothing: the load that produces v cannot be moved below this point, and the wave
// waits here for that load (and for no later one).
__device__ inline void pin_value(unsigned long long v) {
    const unsigned int lo = (unsigned int)v, hi = (unsigned int)(v >> 32);
    asm volatile("" : : "v"(lo), "v"(hi));
}

// ---- score waves: S^T = K q^T of one tile per round, the softmax across the workgroup's tiles, P to LDS
template <int TYPE>
__device__ inline void score_wave(const DecodeArgs &a, DecodeShared &sh, const Geom &ge) {
    const int lane = ge.lane, w = ge.w, j = ge.j, c = ge.c, g = ge.g;
    const int L = a.s.L, G = a.s.G;
    const __half *Kg = a.k_cache + (int64_t)g * L * D;
    const bool owner = ge.owner_wg && w == W - 1;
    TS(5);

    int pos[2] = {a.pos0, a.pos1};
    if (TYPE != GLM_ATTN_ROPE_DISABLED) {
        if (!a.pos_from_args) {
            pos[0] = a.position_ids[0];
            pos[1] = (TYPE == GLM_ATTN_ROPE_CHATGLM) ? a.position_ids[1] : 0;
        }
        pos[0] = clamp_position(pos[0], a.rope.table_positions, a.flags);
        pos[1] = clamp_position(pos[1], a.rope.table_positions, a.flags);
    }
    // loads of a wave return in order: the small rows first, so that the queries can be prepared while
    // the K tile is on its way.  (Left to the output waves, the queries come late: their loads queue up
    // behind the score waves' tiles in the CU's memory pipeline.)
    QPart qpart;
    const int q_hd = 4 * w + (lane >> 4), q_d0 = (lane & 15) * 8;
    {
        const int hd = q_hd < G ? q_hd : G - 1;  // rows beyond the group read a valid row and are zeroed below
        issue_q_part<TYPE>(a.qkv + a.lay.q_off + (int64_t)(g * G + hd) * a.lay.head_stride, q_d0, pos, a.rope, qpart);
    }
    QPart kpart;  // the new token's k: lane l (and l + 16, ...) takes dims (l & 15) * 8 ..
    if (owner) {
        issue_q_part<TYPE>(a.qkv + a.lay.k_off + (int64_t)g * a.lay.head_stride, q_d0, pos, a.rope, kpart);
    }
    int nk = ge.te - ge.tb < W ? ge.te - ge.tb : W;
    half8 kf[4][4];
    TS(8);
    load_k_tile(Kg, L, (ge.tb + (w < nk ? w : 0)) * TILE, lane, kf);
    if (lane == 0) {
        __hip_atomic_fetch_add(&sh.k_issued, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    TS(0);
    *reinterpret_cast<half8 *>(&sh.q[q_hd][q_d0]) = finish_q_part<TYPE>(qpart, q_d0, a.scale, q_hd >= G);
    pin_value(ge.gen_v);  // older than the query loads that have just been waited for
    lds_signal(&sh.q_ready, lane);
    lds_wait_ge(&sh.q_ready, W, a.flags);
    half8 qf[4];
#pragma unroll
    for (int t = 0; t < 4; t++) {
        qf[t] = *reinterpret_cast<const half8 *>(&sh.q[j][t * 32 + c * 8]);
    }
    float s_new = -INFINITY;  // score of the new token, in the wave that attends to it
    if (owner) {
        // chatglm.cpp:668-671: k (roped) of the new token goes to the cache as fp16
        const half8 k8 = finish_q_part<TYPE>(kpart, q_d0, 1.0f, false);
        if (lane < 16) {
            *reinterpret_cast<half8 *>(a.k_cache + ((int64_t)g * L + a.p0) * D + q_d0) = k8;
            *reinterpret_cast<half8 *>(&sh.knew[q_d0]) = k8;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
        const half8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
        floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const half8 kn = *reinterpret_cast<const half8 *>(&sh.knew[t * 32 + c * 8]);
            acc = mfma16(j == 0 ? kn : zero, qf[t], acc);  // row 0 of the product: the new key
        }
        s_new = __shfl(acc[0], j);
    }
    TS(1);

    float m_run = -INFINITY, l_run = 0.f;
    for (int r = 0; r < ge.rounds; r++) {
        const int rt0 = ge.tb + r * W;  // first tile of the round
        if (r > 0) {
            nk = ge.te - rt0 < W ? ge.te - rt0 : W;
            load_k_tile(Kg, L, (rt0 + (w < nk ? w : 0)) * TILE, lane, kf);
        }
        const bool has = w < nk;
        floatx4 s[4];
#pragma unroll
        for (int T = 0; T < 4; T++) {
            floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int t = 0; t < 4; t++) {
                acc = mfma16(kf[T][t], qf[t], acc);
            }
            s[T] = acc;
        }
        const int limit = has ? a.p0 - (rt0 + w) * TILE : 0;  // keys of the tile that exist
        if (limit < TILE) {
#pragma unroll
            for (int T = 0; T < 4; T++) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    if ((T >> 1) * 32 + c * 8 + (T & 1) * 4 + e >= limit) {
                        s[T][e] = -INFINITY;
                    }
                }
            }
        }
        float mx = fmaxf(fmaxf(s[0][0], s[0][1]), fmaxf(s[0][2], s[0][3]));
#pragma unroll
        for (int T = 1; T < 4; T++) {
            mx = fmaxf(mx, fmaxf(fmaxf(s[T][0], s[T][1]), fmaxf(s[T][2], s[T][3])));
        }
        mx = max_over_c(mx);
        if (r == 0) {
            mx = fmaxf(mx, s_new);
        }
        if (c == 0) {
            sh.m[r & 1][w][j] = mx;
        }
        lds_signal(&sh.m_ready, lane);
        TS(2);
        lds_wait_ge(&sh.m_ready, W * (r + 1), a.flags);
        float m_new = m_run;
#pragma unroll
        for (int ww = 0; ww < W; ww++) {
            m_new = fmaxf(m_new, sh.m[r & 1][ww][j]);
        }
        const float m_ref = (m_new == -INFINITY) ? 0.f : m_new;  // no visible key yet: every p below is 0
        const float alpha = (m_run == -INFINITY) ? 0.f : __expf(m_run - m_ref);
        float psum = 0.f;
        half8 pf[2];
#pragma unroll
        for (int T = 0; T < 4; T++) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float pv = __expf(s[T][e] - m_ref);  // exp(-inf) = 0 for masked keys
                psum += pv;
                pf[T >> 1][(T & 1) * 4 + e] = (_Float16)pv;
            }
        }
        psum = sum_over_c(psum);
        float pn = 0.f;
        if (r == 0 && s_new != -INFINITY) {
            pn = (float)(_Float16)__expf(s_new - m_ref);
            psum += pn;
        }
        l_run = l_run * alpha + psum;
        m_run = m_new;
        if (r > 0) {
            lds_wait_ge(&sh.p_done, W * r, a.flags);  // the output waves are through with the last round's P
        }
        *reinterpret_cast<half8 *>(&sh.p[j][w * TILE + c * 8]) = pf[0];
        *reinterpret_cast<half8 *>(&sh.p[j][w * TILE + 32 + c * 8]) = pf[1];
        if (c == 0) {
            sh.l[w][j] = l_run;
            if (w == 0) {
                sh.mrun[r & 1][j] = m_new;
            }
            if (r == 0 && owner) {
                sh.pnew[j] = pn;
            }
        }
        lds_signal(&sh.p_ready, lane);
    }
    TS(3);
}

// ---- output waves: O^T of 32 output dims over all keys of the workgroup.  Returns the lane's O (dims
// w*32 + jb*16 + c*4 .. of head j), the head's sum and running max.
// while_waiting(): work of the caller that needs the launch count but not the probabilities; it runs between the
// issue of the V loads and the wait for the first probabilities, when the wave has nothing else to do.
template <typename F>
__device__ inline void output_wave(const DecodeArgs &a, DecodeShared &sh, const Geom &ge, floatx4 (&o)[2],
                                   float &l_tot, float &m_fin, F while_waiting) {
    const int lane = ge.lane, w = ge.w, j = ge.j, c = ge.c, g = ge.g;
    const int L = a.s.L;
    const __half *Vg = a.v_cache + (int64_t)g * D * L;

    int nk = ge.te - ge.tb < W ? ge.te - ge.tb : W;
    half8 vf[2][8];
    // the new token's v, in the workgroup that appends it: asked for ahead of the V columns (loads of a
    // wave return in order, and two small loads behind them would be waited for one after the other)
    floatx4 vraw_new[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};
    if (ge.owner_wg) {
        const float *vhead = a.qkv + a.lay.v_off + (int64_t)g * a.lay.head_stride + w * 32;
        vraw_new[0] = *reinterpret_cast<const floatx4 *>(vhead + c * 4);
        vraw_new[1] = *reinterpret_cast<const floatx4 *>(vhead + 16 + c * 4);
    }
    // The K tiles go into the CU's memory pipeline first: the scores, the maxes and the probabilities are
    // all made from them while the V columns, which only the last step needs, are still on their way.
    lds_wait_ge(&sh.k_issued, W, a.flags);
    load_v_dims<0, 8>(Vg, L, ge.tb * TILE, nk, w, lane, vf);
    float vnew[2][4];
    if (ge.owner_wg) {
        // chatglm.cpp:672-675: v of the new token goes to the cache as fp16, and into this launch's output
#pragma unroll
        for (int jb = 0; jb < 2; jb++) {
            const floatx4 vraw = vraw_new[jb];
            _Float16 v16[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                v16[e] = (_Float16)vraw[e];
                vnew[jb][e] = (float)v16[e];
            }
            if (j < 4) {
                const _Float16 mine = j == 0 ? v16[0] : j == 1 ? v16[1] : j == 2 ? v16[2] : v16[3];
                *reinterpret_cast<_Float16 *>(a.v_cache + ((int64_t)g * D + w * 32 + jb * 16 + c * 4 + j) * L + a.p0) =
                    mine;
            }
        }
    }
    TS(0);
    pin_value(ge.gen_v);  // nothing to do before P anyway
    while_waiting();
    o[0] = floatx4{0.f, 0.f, 0.f, 0.f};
    o[1] = floatx4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY;
    for (int r = 0; r < ge.rounds; r++) {
        const int rt0 = ge.tb + r * W;
        if (r > 0) {
            nk = ge.te - rt0 < W ? ge.te - rt0 : W;
            load_v_dims<0, 8>(Vg, L, rt0 * TILE, nk, w, lane, vf);
        }
        lds_wait_ge(&sh.p_ready, W * (r + 1), a.flags);
        TS(3);
        const float m_new = sh.mrun[r & 1][j];
        const float alpha = (m_run == -INFINITY) ? 0.f : __expf(m_run - m_new);
        m_run = m_new;
        if ((rt0 + nk) * TILE > a.p0) {
            // V columns of keys that do not exist may hold anything (never written, or stale): zero them.
            // They can only be in the round's last tile.
#pragma unroll
            for (int ks = 0; ks < 8; ks++) {
                if (ks >= 2 * nk - 2 && ks < 2 * nk) {
                    const int nv = a.p0 - (rt0 * TILE + ks * 32 + c * 8);  // keys of this lane's eight that exist
                    uintx4 keep;
#pragma unroll
                    for (int dw = 0; dw < 4; dw++) {
                        keep[dw] = nv >= 2 * dw + 2 ? 0xffffffffu : nv == 2 * dw + 1 ? 0x0000ffffu : 0u;
                    }
#pragma unroll
                    for (int jb = 0; jb < 2; jb++) {
                        uintx4 bits = __builtin_bit_cast(uintx4, vf[jb][ks]);
                        bits &= keep;
                        vf[jb][ks] = __builtin_bit_cast(half8, bits);
                    }
                }
            }
        }
        o[0] *= alpha;
        o[1] *= alpha;
#pragma unroll
        for (int ks = 0; ks < 8; ks++) {
            if (ks < 2 * nk) {
                const half8 pb = *reinterpret_cast<const half8 *>(&sh.p[j][ks * 32 + c * 8]);
                o[0] = mfma16(vf[0][ks], pb, o[0]);
                o[1] = mfma16(vf[1][ks], pb, o[1]);
            }
        }
        if (r == 0 && ge.owner_wg) {
            const float pn = sh.pnew[j];
#pragma unroll
            for (int jb = 0; jb < 2; jb++) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    o[jb][e] = __builtin_fmaf(pn, vnew[jb][e], o[jb][e]);
                }
            }
        }
        if (r + 1 < ge.rounds) {
            lds_signal(&sh.p_done, lane);
        }
    }
    // the sums of the score waves are each at the final running max
    l_tot = 0.f;
#pragma unroll
    for (int ww = 0; ww < W; ww++) {
        l_tot += sh.l[ww][j];
    }
    m_fin = m_run;
    TS(4);
}

// Block = 8 waves: 4 score waves and 4 output waves, one of each per SIMD.  In a round the workgroup
// takes up to 4 consecutive tiles (256 keys).  Score wave w loads the K rows of tile w and computes its
// scores for all heads; the score waves agree on the maxes through LDS and leave their probabilities
// there.  Output wave w meanwhile loads the V columns of output dims [32 w, 32 w + 32) for all keys of
// the round (a wave that waits for room in the memory pipeline can do nothing else, which is why the two
// kinds of work are in different waves) and then accumulates those dims over all keys.  O never goes
// through LDS and ends up in the lanes in exactly the layout of the lines.
template <int TYPE>
__device__ inline void decode_body(const DecodeArgs &a, DecodeShared &sh) {
    Geom ge;
    ge.lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    ge.w = wave & (W - 1);
    const bool scores = wave < W;
    ge.t_start = wall_clock64();
    TS(10);
    ge.j = ge.lane & 15;
    ge.c = ge.lane >> 4;
    ge.g = blockIdx.y;
    ge.split = blockIdx.x;
    const int lane = ge.lane, w = ge.w, j = ge.j, c = ge.c, g = ge.g, split = ge.split;
    const int G = a.s.G;
    // tiles [tb, te) of the keys already in the cache are this workgroup's
    decode_tile_range(a.nsplit, a.tiles_q, a.tiles_r, split, &ge.tb, &ge.te);
    ge.rounds = ge.te - ge.tb > W ? (ge.te - ge.tb + W - 1) / W : 1;
    // The first workgroup also appends the new token and attends to it: every merge waits for its lines,
    // so it is the one that is dispatched first and never has the extra tile.
    ge.owner_wg = split == 0;

    // The launch count stamps this launch's lines.  Every lane reads it (no branch, one request per
    // wave) as its first load: no workgroup can have finished before that.  The load goes to the memory
    // side and takes about a microsecond: its value stays in vector registers, behind an address the
    // compiler cannot prove uniform, until the wave's tile loads have been issued and used (`resolve`),
    // or the wave would sit out that microsecond before it asks for its first tile.
    const unsigned long long *gen_at = &a.sync[g].gen;
    asm volatile("" : "+v"(gen_at));
    // (address space 1: a global load; a flat one would also stand in the way of every wait for LDS)
    const unsigned long long gen_v =
        __hip_atomic_load(reinterpret_cast<const __attribute__((address_space(1))) unsigned long long *>(
                              reinterpret_cast<uintptr_t>(gen_at)),
                          __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    ge.gen_v = gen_v;
    unsigned long long gen = 0ull, stamp = 0ull;
    unsigned int stamp32 = 0u;

    // What the exchange needs is worked out after the wave's own part (`resolve`): ahead of it, it would
    // stand between the start of the wave and its first loads.
    const int total_quads = G * QUADS;
    int qps = 0;  // quads per slice
    MergeGeom mg;
    DecodeGroupSync *sy = nullptr;
    unsigned long long *claim = nullptr;
    auto resolve = [&]() {
        qps = merge_quads_per_slice(total_quads, a.nsplit);
        mg.nsplit = a.nsplit;
        const MergeShape ms = merge_shape(a.nsplit);
        mg.sl_log = ms.sl_log;
        mg.nl = ms.nl;
        mg.part_g = a.part + (int64_t)g * a.nsplit * kDecodePartFloats;
        mg.out_g = a.out + (int64_t)g * G * D;
        mg.gen_word = &a.sync[g].gen;
        sy = a.sync + g;
        claim = a.claim + (int64_t)g * kDecodeMaxSplits;
        gen = ((unsigned long long)__builtin_amdgcn_readfirstlane((unsigned int)(gen_v >> 32)) << 32) |
              (unsigned long long)__builtin_amdgcn_readfirstlane((unsigned int)gen_v);
        stamp32 = a.stamp_groups ? decode_stamp_grouped(gen, g) : decode_stamp(gen);
        stamp = gen + 1ull;
        mg.stamp32 = stamp32;
        mg.gen_next = decode_next_gen(gen);
    };

    if (scores) {
        score_wave<TYPE>(a, sh, ge);
        if (a.nsplit == 1) {
            return;
        }
        resolve();
        // ---- grid-wide merge.  The score waves of every workgroup fold the quads of one slice of the
        // group's output from the lines of all splits, which they load past the caches and poll until
        // they carry this launch's stamp.  The poll is bounded: a wave whose wait runs out flags the
        // slice as left behind, looks once more and goes on to exit.  Every workgroup looks for such
        // flags once its own lines have been performed, and redoes the slices it finds flagged: the
        // workgroup whose lines are performed last finds every partial complete and every flag that
        // was raised before its look; a flag raised after that look is followed by a look that finds
        // every partial complete.  Two waves may merge the same slice; they then write identical values.
        const int q_begin = split * qps;
        const int q_end = (split + 1) * qps < total_quads ? (split + 1) * qps : total_quads;
        const int qw = 16 >> mg.sl_log;
        if (q_begin + w * qw >= q_end) {
            return;  // fewer quads in the slice than the score waves take in one pass
        }
        const unsigned long long t0 = wall_clock64();
        const unsigned long long limit = (unsigned long long)a.spin_ticks;
        // The lines are polled directly (a shared arrival counter would be one hot address for all the
        // workgroups of a group).  Other workgroups finish later than this one by a time that grows with
        // the bytes the launch moves, and a line takes a while to become visible: every look before the
        // last line is there loads the missing ones again, and those loads compete with the tiles that
        // slower workgroups are still waiting for.  So the first look waits.
        {
            const int n_tiles = a.tiles_q * a.nsplit + a.tiles_r;
            const unsigned long long wait_ticks =
                (unsigned long long)(kFirstLookTicks + n_tiles * kFirstLookTicksPer64Tiles / 64);
            while (wall_clock64() - t0 < wait_ticks && wait_ticks < limit) {
                __builtin_amdgcn_s_sleep(4);
            }
        }
        TS(6);
        // (the first slices' first waves move the launch count on: any of them is enough)
        const int failed = merge_quads(mg, q_begin, q_end, w, W, lane, t0, limit, split < 4 && w == 0);
        TS(7);
        if (failed) {
            // Flag the slice (its own word, then the group's), then look once more, on its own and at
            // the whole slice.  (The look starts after the flags are known to be in place.)
            if (lane == 0) {
                const unsigned long long old =
                    __hip_atomic_exchange(claim + split, stamp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (old != stamp) {
                    __hip_atomic_fetch_add(&sy->lost, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                __hip_atomic_store(&sy->flagged, stamp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            wait_vm();
            if (!merge_quads(mg, q_begin, q_end, 0, 1, lane, wall_clock64(), 0ull, split < 4)) {
                slice_redone(claim + split, stamp, &sy->lost, lane);
            }
        }
        return;
    }

    floatx4 o[2];
    float l_tot, m_fin;
    output_wave(a, sh, ge, o, l_tot, m_fin, resolve);
    if (a.nsplit == 1) {
        // a single workgroup saw every key of the group: normalise and finish
        if (j < G) {
#pragma unroll
            for (int jb = 0; jb < 2; jb++) {
                floatx4 ov;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    ov[e] = o[jb][e] / l_tot;
                }
                *reinterpret_cast<floatx4 *>(&a.out[(int64_t)(g * G + j) * D + w * 32 + jb * 16 + c * 4]) = ov;
            }
        }
        return;
    }
    // ---- the workgroup's partial as stamped lines: O / sum and the log-sum-exp per head.  Lane (j, c)
    // of output wave w holds piece c of quads 2 w and 2 w + 1 of head j.
    if (j < G) {
        float *pw = a.part + (int64_t)g * a.nsplit * kDecodePartFloats + split * 16;
        const float inv = l_tot > 0.f ? __builtin_amdgcn_rcpf(l_tot) : 0.f;
        const unsigned int lse =  // base 2: what the exponential instruction takes
            __float_as_uint(l_tot > 0.f ? __builtin_fmaf(m_fin, 1.44269504088896340736f, __log2f(l_tot)) : -INFINITY);
#pragma unroll
        for (int jb = 0; jb < 2; jb++) {
            st_dev4(pw + (int64_t)(j * QUADS + w * 2 + jb) * a.nsplit * 16 + c * 4,
                    pack_piece(stamp32, o[jb] * inv, lse));
        }
    }
    TS(5);
    // ---- once the lines of the whole workgroup have been performed: has anybody left a slice behind?
    wait_vm();  // this wave's line stores have been performed
    lds_signal(&sh.stored, lane);
    if (w != 0) {
        return;
    }
    lds_wait_ge(&sh.stored, W, a.flags);
    if (__hip_atomic_load(&sy->flagged, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != stamp) {
        return;  // normally
    }
    TS(8);
    const unsigned long long sweep_limit = a.spin_ticks > 10000 ? (unsigned long long)a.spin_ticks : 10000ull;
    const int n_slices = (total_quads + qps - 1) / qps;
    for (int sl0 = 0; sl0 < n_slices; sl0 += 64) {
        unsigned long long cl = 0;
        if (sl0 + lane < n_slices) {
            cl = __hip_atomic_load(claim + sl0 + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        unsigned long long left = __ballot(sl0 + lane < n_slices && cl == stamp);
        while (left) {
            const int sl = sl0 + __builtin_ctzll(left);
            left &= left - 1;
            const int qb = sl * qps;
            const int qe = (sl + 1) * qps < total_quads ? (sl + 1) * qps : total_quads;
            if (!merge_quads(mg, qb, qe, 0, 1, lane, wall_clock64(), sweep_limit, sl < 4)) {
                slice_redone(claim + sl, stamp, &sy->lost, lane);
            } else if (lane == 0) {
                atomicOr(a.flags, kFlagMergeIncomplete);  // even the long wait ran out: reported for good
            }
        }
    }
    TS(9);
}

__global__ __launch_bounds__(kBlock) void decode_kernel(DecodeArgs a) {
    __shared__ DecodeShared sh;
    if (threadIdx.x == 0) {
        sh.k_issued = 0;
        sh.q_ready = 0;
        sh.m_ready = 0;
        sh.p_ready = 0;
        sh.p_done = 0;
        sh.stored = 0;
    }
    __syncthreads();
    switch (a.rope.pairs > 0 ? a.rope.type : GLM_ATTN_ROPE_DISABLED) {
    case GLM_ATTN_ROPE_GPTJ:
        decode_body<GLM_ATTN_ROPE_GPTJ>(a, sh);
        break;
    case GLM_ATTN_ROPE_NEOX:
        decode_body<GLM_ATTN_ROPE_NEOX>(a, sh);
        break;
    case GLM_ATTN_ROPE_CHATGLM:
        decode_body<GLM_ATTN_ROPE_CHATGLM>(a, sh);
        break;
    case GLM_ATTN_ROPE_CHATGLM2:
        decode_body<GLM_ATTN_ROPE_CHATGLM2>(a, sh);
        break;
    default:
        decode_body<GLM_ATTN_ROPE_DISABLED>(a, sh);
        break;
    }
}

}  // namespace

#ifdef GLM_ATTN_TIMELINE
// Only in the instrumented build: copies the clock readings of the decode launches since the last call to the
// host (a later launch overwrites an earlier one's; the count at index 14 adds up) and clears them.
extern "C" int glm_attn_debug_decode_timeline(unsigned long long *host, size_t n) {
    if (n > (size_t)kTimelineSlots * 16) n = (size_t)kTimelineSlots * 16;
    hipError_t e = hipMemcpyFromSymbol(host, HIP_SYMBOL(g_decode_timeline), n * sizeof(unsigned long long));
    void *at = nullptr;
    if (e == hipSuccess) e = hipGetSymbolAddress(&at, HIP_SYMBOL(g_decode_timeline));
    if (e == hipSuccess) e = hipMemset(at, 0, sizeof(unsigned long long) * kTimelineSlots * 16);
    return (int)e;
}
#endif

hipError_t launch_decode(const DecodeArgs &a, hipStream_t stream) {
    if (a.nsplit < 1 || a.nsplit > kDecodeMaxSplits || a.tiles_q < 0 || a.tiles_r < 0 || a.tiles_r >= a.nsplit) {
        return hipErrorInvalidValue;
    }
    hipLaunchKernelGGL(decode_kernel, dim3(a.nsplit, a.s.kvh), dim3(kBlock), 0, stream, a);
    return hipGetLastError();
}

}  // namespace glm_attn
