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

// ---- launch geometry, worked out on the host (plain functions, so that a host test can walk the shapes and
// check every extent against what the launch is given)

// decode_kernel: the 64-key tiles of the keys already in the cache, dealt out to nsplit workgroups per KV group
// (tiles_q each, the last tiles_r one more).  max_parts: (group, split) partials the exchange memory holds.
struct DecodePlan {
    int n_tiles, nsplit, tiles_q, tiles_r;
};
inline DecodePlan plan_decode(int p0, int kvh, int num_cus, int max_splits, int max_parts) {
    DecodePlan pl;
    pl.n_tiles = (p0 + kDecodeTileKeys - 1) / kDecodeTileKeys;
    // spread over CUs first: that buys more load queues; a workgroup takes its tiles four at a time
    const int cu_share = num_cus / kvh > 0 ? num_cus / kvh : 1;
    int nsplit = pl.n_tiles < 1 ? 1 : pl.n_tiles;
    if (nsplit > cu_share) nsplit = cu_share;
    if (nsplit > max_splits) nsplit = max_splits;
    if (nsplit > kDecodeMaxSplits) nsplit = kDecodeMaxSplits;
    if (max_parts > 0 && nsplit > max_parts / kvh) nsplit = max_parts / kvh;
    // One round of tiles is over sooner in one workgroup than the exchange between several takes (a second
    // round in the same workgroup is not: it costs 3 us, the exchange 2).
    if (pl.n_tiles <= kDecodeMaxWaves) nsplit = 1;
    if (nsplit < 1) nsplit = 1;
    pl.nsplit = nsplit;
    pl.tiles_q = pl.n_tiles / nsplit;
    pl.tiles_r = pl.n_tiles % nsplit;
    return pl;
}

// tiles [*tb, *te) of workgroup `split`: the last tiles_r splits take one tile more (the first workgroup, which
// also appends the new token, never has the extra tile)
__host__ __device__ inline void decode_tile_range(int nsplit, int tiles_q, int tiles_r, int split, int *tb, int *te) {
    const int extra_from = nsplit - tiles_r;
    *tb = split * tiles_q + (split > extra_from ? split - extra_from : 0);
    *te = *tb + tiles_q + (split >= extra_from ? 1 : 0);
}

// decode_kernel, the fold of the split partials.  The partials of a KV group are lines of 64 bytes, one per
// (head, 16 output dims) = "quad" q = head * 8 + quad and split, laid out [q][split][16 floats]; a line is four
// 16-byte pieces.  The quads are dealt out in slices of qps to the group's workgroups, a slice's quads to the waves
// that fold (wave wi of nw).  Lane (s, quad slot, piece) of a wave takes piece `piece` of the lines of splits
// s, s + SL, ... (SL = 1 << sl_log, nl lines) of the quad in its slot; a wave loads the lines of pc passes of its
// 16 / SL quad slots, nlp lines each, in one block (nl > nlp: further blocks of nlp lines).
struct MergeShape {
    int sl_log, nl;  // split lanes per (quad, piece): 1 << sl_log; lines per lane and quad
    int nlp, pc;     // lines per lane, quad and block (1, 2, 4, 8); quads per lane and block (4, 2, 1, 1)
};
__host__ __device__ inline MergeShape merge_shape(int nsplit) {
    MergeShape m;
    m.sl_log = 0;
    while (m.sl_log < 4 && (1 << m.sl_log) < nsplit) {
        m.sl_log++;
    }
    m.nl = (nsplit + (1 << m.sl_log) - 1) >> m.sl_log;
    m.nlp = m.nl <= 1 ? 1 : m.nl <= 2 ? 2 : m.nl <= 4 ? 4 : 8;
    m.pc = m.nlp == 1 ? 4 : m.nlp == 2 ? 2 : 1;
    return m;
}
__host__ __device__ inline int merge_quads_per_slice(int total_quads, int nsplit) {
    return (total_quads + nsplit - 1) / nsplit;
}
__host__ __device__ inline void merge_lane(int sl_log, int lane, int *piece, int *qslot, int *s) {
    *piece = lane & 3;
    *qslot = (lane >> 2) & ((16 >> sl_log) - 1);
    *s = lane >> (6 - sl_log);  // in the upper bits of the lane index, where reductions are cheap
}
// the quad of pass pp of the block that starts at q0 (q0 = q_begin + wi * qw, then + pc * nw * qw per block)
__host__ __device__ inline int merge_quad_of(int q0, int pp, int nw, int sl_log, int qslot) {
    return q0 + pp * nw * (16 >> sl_log) + qslot;
}
__host__ __device__ inline int merge_split_of(int k, int sl_log, int s) { return (k << sl_log) + s; }
// where piece `piece` of the line of (quad q, split sp) starts, in floats from the group's first line
__host__ __device__ inline int64_t merge_piece_offset(int q, int nsplit, int sp, int piece) {
    return ((int64_t)q * nsplit + sp) * 16 + piece * 4;
}

// prefill_kernel: rows of 128 per item, items of one unit (a head, or a KV group when a few tokens are packed with
// the heads of their group), four-wave or eight-wave workgroups, and the cut along the keys with its partials.
constexpr int kPrefillRows = 128;        // rows (tokens) per workgroup
constexpr int kPrefillTileKeys = 64;     // keys per tile
constexpr int kPrefillMaxSplits = 128;   // shares of the key range
struct PrefillPlan {
    int packed, units, rows, n_qtiles, n_items;
    int two_groups, order, nsplit;
    int64_t part_floats;  // floats of the partials of a cut launch (0 when nsplit == 1)
};
inline PrefillPlan plan_prefill(int qlen, int p0, int kvs, int h, int G, int causal, int64_t split_floats, int num_cus) {
    PrefillPlan pl;
    const int D = kFastHeadSize, BM = kPrefillRows, BN = kPrefillTileKeys;
    // Up to 64 tokens of a grouped-query model are packed with the heads of their group: at least two heads then
    // share every K/V tile.
    pl.packed = (G > 1 && qlen <= BM / 2) ? 1 : 0;
    const int heads_per_unit = pl.packed ? G : 1;
    pl.units = h / heads_per_unit;
    pl.rows = heads_per_unit * qlen;
    pl.n_qtiles = (pl.rows + BM - 1) / BM;
    pl.n_items = pl.n_qtiles * pl.units;
    // Too few items to give every CU two workgroups: eight-wave workgroups, one per CU.
    pl.two_groups = pl.n_items < 2 * num_cus ? 1 : 0;
    const int slots = pl.two_groups ? num_cus : 2 * num_cus;
    pl.order = (!causal || pl.packed) ? 0 : (!pl.two_groups && pl.n_items == 2 * num_cus ? 2 : 1);
    // A few tokens against a long cache are a handful of workgroups with hundreds of tiles each: cut the key
    // range so that the chip is full once, as long as every share keeps at least four tiles per group of waves
    // and the partials fit the scratch.
    int nsplit = 1;
    if (split_floats > 0 && pl.n_items < slots) {
        int kv_end = kvs;
        const int t_max = pl.packed ? qlen : pl.n_qtiles * BM;  // one past the last token of the last tile (or beyond)
        if (causal && p0 + t_max < kv_end) kv_end = p0 + t_max;
        const int n_tiles = (kv_end + BN - 1) / BN;
        const int min_tiles = pl.two_groups ? 8 : 4;
        nsplit = (slots + pl.n_items - 1) / pl.n_items;
        if (nsplit > n_tiles / min_tiles) nsplit = n_tiles / min_tiles;
        if (nsplit > kPrefillMaxSplits) nsplit = kPrefillMaxSplits;
        while (nsplit > 1 && (int64_t)nsplit * pl.n_qtiles * BM * pl.units * (D + 2) > split_floats) nsplit--;
        if (nsplit < 2) nsplit = 1;
    }
    pl.nsplit = nsplit;
    pl.part_floats = nsplit > 1 ? (int64_t)nsplit * pl.n_qtiles * BM * pl.units * (D + 2) : 0;
    return pl;
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
    int tiles_q, tiles_r;  // tiles of 64 cached keys per workgroup: tiles_q, one more in the last tiles_r
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
