// Host-side check of the launch geometry of the decode and prefill kernels (csrc/glm_attn_internal.h: plan_decode,
// decode_tile_range, plan_prefill): the functions the launches use, walked over many shapes, with every extent
// that a launch derives from them checked against the memory the launch is given.  Built and run by
// tests/test_capi_cpu.py; no GPU.
#include <stdint.h>
#include <stdio.h>

#include <vector>

#include "glm_attn_internal.h"
#include "linear_plan.h"

using namespace glm_attn;

#define CHECK(cond)                                                                          \
    do {                                                                                     \
        if (!(cond)) {                                                                       \
            printf("FAILED line %d: %s  [%s]\n", __LINE__, #cond, what);                     \
            return 1;                                                                        \
        }                                                                                    \
    } while (0)

static int check_decode() {
    char what[160];
    const int cus[] = {256, 304, 64, 8};
    const int kvhs[] = {1, 2, 4, 8, 32, 64, 128};
    std::vector<int> p0s;
    for (int p = 0; p <= 1100; p++) p0s.push_back(p);
    for (int p = 1100; p <= 140000; p += 997) p0s.push_back(p);
    for (int p : {4095, 4096, 8191, 16383, 32767, 32768, 65535, 131071}) p0s.push_back(p);
    for (int num_cus : cus) {
        for (int kvh : kvhs) {
            int max_splits = num_cus / kvh > 0 ? num_cus / kvh : 1;  // what glm_attn_create sizes the partials for
            if (max_splits > kDecodeMaxSplits) max_splits = kDecodeMaxSplits;
            for (int max_parts : {0, 256}) {                          // 256: the static exchange memory (kvh <= 32)
                if (max_parts && kvh > 32) continue;
                for (int p0 : p0s) {
                    const DecodePlan pl = plan_decode(p0, kvh, num_cus, max_splits, max_parts);
                    snprintf(what, sizeof(what), "decode cus %d kvh %d parts %d p0 %d -> nsplit %d q %d r %d", num_cus, kvh,
                             max_parts, p0, pl.nsplit, pl.tiles_q, pl.tiles_r);
                    CHECK(pl.n_tiles * kDecodeTileKeys >= p0 && (pl.n_tiles - 1) * kDecodeTileKeys < p0 + (p0 == 0));
                    CHECK(pl.nsplit >= 1 && pl.nsplit <= max_splits && pl.nsplit <= kDecodeMaxSplits);  // partials, claims
                    CHECK(max_parts == 0 || pl.nsplit * kvh <= max_parts);
                    CHECK(pl.tiles_q >= 0 && pl.tiles_r >= 0 && pl.tiles_r < pl.nsplit);  // what launch_decode insists on
                    CHECK(pl.nsplit * pl.tiles_q + pl.tiles_r == pl.n_tiles);
                    CHECK(pl.nsplit == 1 || pl.tiles_q >= 1);  // no workgroup of an exchange without a tile
                    // the workgroups' ranges tile [0, n_tiles) in order, and the first never has the extra tile
                    int at = 0;
                    for (int s = 0; s < pl.nsplit; s++) {
                        int tb, te;
                        decode_tile_range(pl.nsplit, pl.tiles_q, pl.tiles_r, s, &tb, &te);
                        CHECK(tb == at && te >= tb && te - tb <= pl.tiles_q + 1);
                        CHECK(s != 0 || pl.nsplit == 1 || te - tb == pl.tiles_q);
                        at = te;
                    }
                    CHECK(at == pl.n_tiles);
                    // floats of the partials the launch writes against the buffer of kvh * max_splits partials
                    CHECK((int64_t)kvh * pl.nsplit * kDecodePartFloats <= (int64_t)kvh * max_splits * kDecodePartFloats);
                }
            }
        }
    }
    return 0;
}

// The fold of the split partials (merge_shape, merge_lane, merge_quad_of, merge_split_of, merge_piece_offset: what the
// score waves of decode_kernel use): for every split count and group size, walked the way the kernel walks it
// (slices of quads per workgroup, waves of a workgroup, blocks of passes, blocks of lines, 64 lanes), every piece
// of every line of every quad of the group is taken exactly once, by a lane that also writes that quad's output
// piece or has a lane beside it that does, and lies inside the lines the group's workgroups have written.
static int check_decode_merge() {
    char what[160];
    for (int G : {1, 2, 4, 16}) {
        for (int nsplit = 2; nsplit <= kDecodeMaxSplits; nsplit += (nsplit < 140 ? 1 : 31)) {
            for (int nw : {4, 1}) {  // the score waves of a workgroup, or one wave redoing a slice on its own
                const int total_quads = G * (kFastHeadSize / 16);
                const MergeShape ms = merge_shape(nsplit);
                const int qps = merge_quads_per_slice(total_quads, nsplit);
                const int SL = 1 << ms.sl_log, qw = 16 >> ms.sl_log;
                snprintf(what, sizeof(what), "merge G %d nsplit %d nw %d: sl_log %d nl %d nlp %d pc %d qps %d", G, nsplit, nw,
                         ms.sl_log, ms.nl, ms.nlp, ms.pc, qps);
                CHECK(SL * ms.nl >= nsplit && SL * (ms.nl - 1) < nsplit);  // the split lanes cover the splits, no line idle
                CHECK(ms.nlp >= 1 && ms.nlp <= 8 && ms.nlp * ms.pc <= 8);  // loads per lane and block: ld_lines has 1, 2, 4, 8
                CHECK(ms.nl <= ms.nlp || ms.nlp == 8);                      // only blocks of 8 lines repeat
                CHECK(qps >= 1 && (int64_t)qps * nsplit >= total_quads);
                const int64_t group_floats = (int64_t)nsplit * kDecodePartFloats;  // what the group's workgroups write
                std::vector<int> taken((size_t)total_quads * nsplit * 4, 0), written((size_t)total_quads * 4, 0);
                for (int split = 0; split < nsplit; split++) {
                    const int q_begin = split * qps;
                    const int q_end = (split + 1) * qps < total_quads ? (split + 1) * qps : total_quads;
                    for (int wi = 0; wi < nw; wi++) {
                        for (int q0 = q_begin + wi * qw; q0 < q_end; q0 += ms.pc * nw * qw) {
                            for (int k0 = 0; k0 < ms.nl; k0 += ms.nlp) {
                                for (int lane = 0; lane < 64; lane++) {
                                    int piece, qslot, sl;
                                    merge_lane(ms.sl_log, lane, &piece, &qslot, &sl);
                                    CHECK(piece >= 0 && piece < 4 && qslot >= 0 && qslot < qw && sl >= 0 && sl < SL);
                                    for (int pp = 0; pp < ms.pc; pp++) {
                                        const int q = merge_quad_of(q0, pp, nw, ms.sl_log, qslot);
                                        if (q >= q_end) continue;  // qvalid
                                        if (k0 == 0 && sl == 0) written[(size_t)q * 4 + piece]++;
                                        for (int k = 0; k < ms.nlp; k++) {
                                            const int sp = merge_split_of(k0 + k, ms.sl_log, sl);
                                            if (sp >= nsplit) continue;  // need
                                            const int64_t off = merge_piece_offset(q, nsplit, sp, piece);
                                            CHECK(off >= 0 && off + 4 <= group_floats);
                                            CHECK(off == ((int64_t)q * nsplit + sp) * 16 + piece * 4);
                                            taken[((size_t)q * nsplit + sp) * 4 + piece]++;
                                        }
                                    }
                                }
                            }
                        }
                    }
                }
                for (size_t i = 0; i < taken.size(); i++) CHECK(taken[i] == 1);
                for (size_t i = 0; i < written.size(); i++) CHECK(written[i] == 1);
                // the writer's side: lane (j, c) of output wave w stores piece c of quads 2 w, 2 w + 1 of head j
                for (int split = 0; split < nsplit; split += (nsplit > 8 ? nsplit - 1 : 1)) {
                    for (int j = 0; j < G; j++) {
                        for (int quad = 0; quad < 8; quad++) {
                            for (int c = 0; c < 4; c++) {
                                const int64_t off = (int64_t)(j * 8 + quad) * nsplit * 16 + split * 16 + c * 4;
                                CHECK(off == merge_piece_offset(j * 8 + quad, nsplit, split, c) && off + 4 <= group_floats);
                            }
                        }
                    }
                }
            }
        }
    }
    return 0;
}

static int check_prefill() {
    char what[200];
    const int D = kFastHeadSize;
    const int qlens[] = {2, 5, 20, 63, 64, 65, 127, 128, 129, 300, 512, 1000, 1024, 2048, 3000, 4096, 8192};
    const int p0s[] = {0, 1, 63, 100, 896, 8000, 24576, 32000};
    const int shapes[][2] = {{32, 16}, {32, 1}, {8, 4}, {64, 8}, {2, 2}};
    for (int num_cus : {256, 304, 64}) {
        for (auto &sh : shapes) {
            const int h = sh[0], G = sh[1];
            for (int qlen : qlens) {
                for (int p0 : p0s) {
                    for (int causal = 0; causal < 2; causal++) {
                        // the scratch glm_attn_create allocates, none, and a tiny one
                        for (int64_t split_floats : {(int64_t)2048 * ((int64_t)h * D + 2 * h), (int64_t)0, (int64_t)70000}) {
                            const int kvs = p0 + qlen;
                            const PrefillPlan pl = plan_prefill(qlen, p0, kvs, h, G, causal, split_floats, num_cus);
                            snprintf(what, sizeof(what),
                                     "prefill cus %d h %d G %d qlen %d p0 %d causal %d scratch %lld -> items %d groups %d nsplit %d",
                                     num_cus, h, G, qlen, p0, causal, (long long)split_floats, pl.n_items, pl.two_groups + 1,
                                     pl.nsplit);
                            const int hpu = pl.packed ? G : 1;
                            CHECK(pl.units * hpu == h && pl.rows == hpu * qlen);
                            CHECK(!pl.packed || (G > 1 && qlen <= kPrefillRows / 2));
                            CHECK(pl.n_qtiles * kPrefillRows >= pl.rows && (pl.n_qtiles - 1) * kPrefillRows < pl.rows);
                            CHECK(pl.n_items == pl.n_qtiles * pl.units && pl.n_items >= 1);
                            CHECK(pl.two_groups == (pl.n_items < 2 * num_cus));
                            CHECK(pl.order >= 0 && pl.order <= 2 && (pl.order == 0) == (!causal || pl.packed));
                            CHECK(pl.order != 2 || pl.n_items == 2 * num_cus);
                            CHECK(pl.nsplit >= 1 && pl.nsplit <= kPrefillMaxSplits && pl.nsplit <= 65535);
                            if (pl.nsplit > 1) {
                                // every float a workgroup of the cut launch writes lies inside the scratch: O of
                                // row (split, tile row, unit) at part_row * D, then (m, l) behind all the O
                                CHECK(pl.part_floats <= split_floats);
                                const int64_t last_row =
                                    ((int64_t)(pl.nsplit - 1) * pl.n_qtiles * kPrefillRows + (int64_t)pl.n_qtiles * kPrefillRows - 1) *
                                        pl.units + pl.units - 1;
                                const int64_t o_end = last_row * D + D;
                                const int64_t ml_at = (int64_t)pl.nsplit * pl.n_qtiles * kPrefillRows * pl.units * D;
                                CHECK(o_end <= ml_at && ml_at + last_row * 2 + 2 <= pl.part_floats);
                                // and every share keeps its minimum of tiles
                                int kv_end = kvs;
                                const int t_max = pl.packed ? qlen : pl.n_qtiles * kPrefillRows;
                                if (causal && p0 + t_max < kv_end) kv_end = p0 + t_max;
                                const int n_tiles = (kv_end + kPrefillTileKeys - 1) / kPrefillTileKeys;
                                CHECK(n_tiles / pl.nsplit >= (pl.two_groups ? 8 : 4));
                            } else {
                                CHECK(pl.part_floats == 0);
                            }
                        }
                    }
                }
            }
        }
    }
    return 0;
}

static int check_splitk() {
    char what[160];
    const int Ns[] = {4, 64, 128, 132, 4096, 4608, 13696, 27392, 32768, 151552};
    const int Ks[] = {64, 128, 256, 1408, 4096, 13696};
    for (int num_cus : {256, 304, 64}) {
        for (int N : Ns) {
            for (int K : Ks) {
                for (int rows : {1, 8, 9, 20, 64, 127, 128, 129, 300, 2048}) {
                    for (size_t scratch : {(size_t)0, (size_t)4096, sizeof(float) * kSplitKMax * 128 * (size_t)N}) {
                        const int ks = plan_splitk(rows, N, K, num_cus, scratch);
                        snprintf(what, sizeof(what), "splitk cus %d N %d K %d rows %d scratch %zu -> %d", num_cus, N, K, rows,
                                 scratch, ks);
                        CHECK(ks >= 1 && ks <= kSplitKMax && ks <= K / kGemmK);
                        CHECK(ks == 1 || (rows <= kGemmTile && sizeof(float) * (size_t)ks * rows * N <= scratch));
                        CHECK(ks <= 65535);  // gridDim.z
                        int at = 0;
                        for (int kz = 0; kz < ks; kz++) {
                            int s0, s1;
                            splitk_step_range(K, ks, kz, &s0, &s1);
                            CHECK(s0 == at && s1 > s0);  // in order, none empty
                            CHECK((int64_t)s1 * kGemmK <= K);  // the last fetch of a share ends inside a row
                            at = s1;
                        }
                        CHECK(at == K / kGemmK);
                    }
                }
            }
        }
    }
    return 0;
}

int main() {
    if (check_decode() || check_decode_merge() || check_prefill() || check_splitk()) return 1;
    printf("ok\n");
    return 0;
}
