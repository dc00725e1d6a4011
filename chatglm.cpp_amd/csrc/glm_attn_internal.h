// Internal declarations shared by the C-ABI layer and the gfx950 kernels of libglm_attn.so.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "glm_attn.h"

namespace glm_attn {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kFastHeadSize = 128;   // the MFMA kernels are written for d = 128
constexpr int kMaxGroupHeads = 16;   // q heads of one KV group fill the 16 columns of an MFMA tile
constexpr int kDecodeTileKeys = 64;  // keys one wave consumes per step of the decode kernel
constexpr int kDecodeMaxWaves = 4;   // tile waves per workgroup of the decode kernel
constexpr int kDecodeMaxSplits = 512;  // workgroups per KV group of the decode kernel
// floats of one (group, split) partial of the decode kernel: 16 heads x 8 lines of 64 bytes
constexpr int kDecodePartFloats = 16 * 8 * 16;
constexpr int kTimelineSlots = 4096;   // waves recorded by the instrumented build of the decode kernel
constexpr uint32_t kFlagPositionClamped = 1u;
constexpr uint32_t kFlagMergeIncomplete = 2u;  // a slice of a decode output was left unwritten

// Hand-over words of the decode kernel, one set per KV group (a 64-byte line of its own each).
struct DecodeGroupSync {
    unsigned long long gen;      // launches of this group completed so far (with more than one split)
    unsigned long long flagged;  // launch (gen + 1) in which a slice was last left behind by its owner
    unsigned int lost;           // slices left behind and not (yet) redone by anybody, over all launches
    unsigned int pad0;
    unsigned long long pad[5];
};
static_assert(sizeof(DecodeGroupSync) == 64, "one line per group");

// The 32-bit stamp of the lines written by the launch that follows `gen` completed ones.  It is never
// 0 (what a zero-filled exchange buffer holds): decode_next_gen skips the count whose stamp would be.
__host__ __device__ inline unsigned int decode_stamp(unsigned long long gen) { return (unsigned int)(gen + 1ull); }
// The same for exchange memory that contexts of different shapes share: the KV group is part of the stamp
// (5 bits), so that a line can only be taken for one of the group that wrote it, whatever region of the
// memory that group's lines occupied then; 27 bits of the launch count, never 0.
__host__ __device__ inline unsigned int decode_stamp_grouped(unsigned long long gen, int group) {
    return ((unsigned int)group << 27) | (unsigned int)(gen % 0x7ffffffull + 1ull);
}
__host__ __device__ inline unsigned long long decode_next_gen(unsigned long long gen) {
    const unsigned long long next = gen + 1ull;
    return decode_stamp(next) == 0u ? next + 1ull : next;
}

// Where q, k and v heads sit inside one token's row of the fused projection (chatglm.cpp:636-653).
struct QkvLayout {
    int64_t row_stride;  // floats between tokens
    int q_off, k_off, v_off;
    int head_stride;
};

struct RopeSpec {
    int type;             // glm_attn_rope_type
    int pairs;            // rotated pairs per table row (n_dims / 2), 0 when disabled
    int table_positions;  // rows of the table
    const float2 *table;  // [table_positions][pairs] (cos, sin), built on the host
};

struct Shape {
    int h, kvh, d, G, L;  // L = cache rows
};

// rope + append (+ fp16 query scratch); any head size
struct RopeAppendArgs {
    const float *qkv;
    QkvLayout lay;
    RopeSpec rope;
    Shape s;
    const int32_t *position_ids;  // device, [qlen] or [2 qlen]
    int qlen;
    int p0;  // nvt + n_past
    float scale;
    __half *q16;      // [h][qlen][d]
    __half *k_cache;  // [kvh][L][d]
    __half *v_cache;  // [kvh][d][L]
    uint32_t *flags;
};

struct AttendArgs {
    Shape s;
    const __half *q16;      // [h][qlen][d] roped, scaled
    const __half *k_cache;
    const __half *v_cache;
    const float *mask;      // additive [qlen][kvs] or null
    int causal;             // 1: key c masked for token t when c > p0 + t
    int qlen, p0, kvs;
    float *out;             // [qlen][h d]
    float *split_scratch;   // partials of a prefill cut along the keys: O [splits][rows][units][d], then (m, l)
    int64_t split_floats;   // [splits][rows][units][2]; room for this many floats in all.  Null: never cut.
};

struct DecodeArgs {
    const float *qkv;  // one token's row
    QkvLayout lay;
    RopeSpec rope;
    Shape s;
    const int32_t *position_ids;  // device or null
    int pos0, pos1;               // host-provided positions (pos1: block position of the 2-D rope)
    int pos_from_args;
    int p0;  // cache keys already present (nvt + n_past); the new key lands at p0
    float scale;
    __half *k_cache;
    __half *v_cache;
    int nsplit;     // workgroups per KV group
    int tiles_q, tiles_r;  // tiles of 64 cached keys per workgroup: tiles_q, one more in the first tiles_r
    float *part;    // [kvh][nsplit][kDecodePartFloats] split partials as stamped 64-byte lines
    float *out;     // [h d]
    uint32_t *flags;
    // grid-wide hand-over of the split partials
    DecodeGroupSync *sync;      // [kvh]
    unsigned long long *claim;  // [kvh][kDecodeMaxSplits] launch (gen + 1) that last left each slice behind
    long long spin_ticks;       // bound on the wait for the other workgroups, in 100 MHz ticks
    int stamp_groups;           // 1: stamps carry the KV group (exchange memory shared between contexts)
};

// activations of BasicMLP / BasicGLU (chatglm.cpp:444-454), shared by the elementwise kernel and the fused Linear
__device__ inline float silu_value(float x) { return x / (1.0f + expf(-x)); }

// the tanh approximation evaluated on the fp16 grid and rounded to fp16: what the table of ggml's CPU backend holds
__device__ inline float gelu_value(float x) {
    if (x <= -10.0f) return 0.0f;
    if (x >= 10.0f) return x;
    const float v = (float)(_Float16)x;
    const float g = 0.5f * v * (1.0f + tanhf(0.79788456080286535587989211986876f * v * (1.0f + 0.044715f * v * v)));
    return (float)(_Float16)g;
}

hipError_t launch_rope_append(const RopeAppendArgs &a, hipStream_t stream);
hipError_t launch_attend_generic(const AttendArgs &a, hipStream_t stream);
hipError_t launch_decode(const DecodeArgs &a, hipStream_t stream);
hipError_t launch_prefill(const AttendArgs &a, int num_cus, hipStream_t stream);
hipError_t launch_prefix_copy(const __half *past_kv, __half *k_cache, __half *v_cache, Shape s, int nvt,
                              hipStream_t stream);

// -------------------------------------------------------------------------------------------------
// rope of one element, shared by every kernel so that all of them produce the same bits

struct RopeElem {
    bool rot;     // element is rotated
    bool first;   // element is x0 of its pair (else x1)
    int pair;     // column of the cos/sin table
    int partner;  // index of the other element of the pair within the head
    int sel;      // 0: position_ids[t], 1: position_ids[qlen + t] (block position of the 2-D rope)
};

__host__ __device__ inline RopeElem rope_elem(int type, int d, int e) {
    RopeElem r;
    r.rot = false;
    r.first = true;
    r.pair = 0;
    r.partner = e;
    r.sel = 0;
    switch (type) {
    case GLM_ATTN_ROPE_GPTJ:  // pairs (2i, 2i+1) over the whole head
        r.rot = true;
        r.pair = e >> 1;
        r.partner = e ^ 1;
        r.first = !(e & 1);
        break;
    case GLM_ATTN_ROPE_NEOX: {  // pairs (i, i + d/2)
        const int n2 = d / 2;
        r.rot = true;
        r.pair = e % n2;
        r.partner = e < n2 ? e + n2 : e - n2;
        r.first = e < n2;
    } break;
    case GLM_ATTN_ROPE_CHATGLM2:  // adjacent pairs on dims [0, d/2), the rest passes through
        if (e < d / 2) {
            r.rot = true;
            r.pair = e >> 1;
            r.partner = e ^ 1;
            r.first = !(e & 1);
        }
        break;
    case GLM_ATTN_ROPE_CHATGLM: {  // NEOX inside each half; second half uses the block positions
        const int n = d / 2, n2 = n / 2;
        const int half = e / n, el = e % n;
        r.rot = true;
        r.pair = el % n2;
        r.partner = half * n + (el < n2 ? el + n2 : el - n2);
        r.first = el < n2;
        r.sel = half;
    } break;
    default:
        break;
    }
    return r;
}

// x0' = x0 cos - x1 sin, x1' = x0 sin + x1 cos with separately rounded products: the K cache has to
// match a CPU build of ggml's rope bit for bit, so no fused multiply-add here.
__device__ inline float rope_rotate(float self, float partner, float c, float s, bool first) {
    return first ? __fsub_rn(__fmul_rn(self, c), __fmul_rn(partner, s))
                 : __fadd_rn(__fmul_rn(partner, s), __fmul_rn(self, c));
}

__device__ inline int clamp_position(int pos, int table_positions, uint32_t *flags) {
    if (pos < 0 || pos >= table_positions) {
        atomicOr(flags, kFlagPositionClamped);
        pos = pos < 0 ? 0 : table_positions - 1;
    }
    return pos;
}

}  // namespace glm_attn
