/*
 * CPU oracle for the voxel scatter-reduction path (scatter_sum / scatter_mean /
 * scatter_max+argmax, forward and backward).
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the GPU kernels are
 * compared against; the product never calls it.
 *
 * Two families of functions live here:
 *
 *  1. "ref" functions restate the reference CUDA kernels lane by lane, so the
 *     fp32 rounding order and the arg-max tie rule are those of the reference:
 *       orc_up_2n            <- torchex/src/scatter/scatter_kernel.cu:14-24
 *       orc_block_width      <- scatter_kernel.cu:179,187 (launch geometry)
 *       orc_get_presum_ref   <- scatter_kernel.cu:85-100  (kernel getPreSum)
 *       orc_scatter_sum_ref  <- scatter_kernel.cu:26-39,102-129
 *       orc_scatter_max_ref  <- scatter_kernel.cu:41-83,131-171
 *     They need the reference's precondition: rows grouped by voxel (CSR
 *     offsets preSum), which is what ScatterData builds
 *     (torchex/operator_py/scatter_op.py:7-21).
 *
 *  2. "spec" functions state the same mathematics over an arbitrary (unsorted)
 *     unq_inv, with a double accumulator for sums and the first-occurrence
 *     (smallest row index) rule for arg-max.  The two arg-max rules give the
 *     same row whenever the maximum of a (voxel, channel) is unique; among
 *     equal maxima the reference's shuffle tree keeps the candidate whose lane
 *     index is smallest in bit-reversed order (and, per thread, the last row
 *     of its residue class), which is in general not the first row.
 *       orc_scatter_sum_f64, orc_scatter_max_first, orc_counts, orc_presum,
 *       orc_stable_perm
 *     plus the Python-level arithmetic of the reference wrappers:
 *       orc_mean_from_sum    <- scatter_op.py:69      (sum / unq_cnts)
 *       orc_sum_backward     <- scatter_op.py:47-50   (g[unq_inv])
 *       orc_mean_backward    <- scatter_op.py:74-78   ((g / unq_cnts)[unq_inv])
 *       orc_max_backward     <- scatter_op.py:106-111 (zeros.scatter_(0,arg,g))
 *
 * Pinning (what each function is checked against, all in tests/test_oracle.py):
 *   sum/mean/max/argmax "ref": closed forms of the reference's own test data
 *     (test/test_scatter.py:17-23: every group a permutation of 0..n-1, so
 *     sum = n(n-1)/2 exactly, mean = (n-1)/2, max = n-1, argmax = position of
 *     n-1), brute-force Python loops on tiny inputs, torch.scatter_reduce /
 *     index_add in fp64, invariants (sum of outputs == sum of inputs, all-ones
 *     features give the counts).
 *   arg-max tie rule "ref" (which row wins among equal maxima): restated from
 *     the kernel text only; the reference's tests hold no ties, so this one
 *     rule is PARITY UNPINNED by reference tests.  It is pinned here by
 *     hand-worked cases and by a closed form (bit-reversed lane priority)
 *     derived on paper from the shuffle tree and checked against the lane-exact
 *     emulation on random tie-heavy groups.
 *   getPreSum "ref": cumsum(bincount) on sorted input.
 */
#include <float.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_WARP 32
#define ORC_MAX_THREADS 1024

/* scatter_kernel.cu:14-24 */
int orc_up_2n(int n) {
    if (n == 1) return 1;
    int t = n - 1;
    t |= t >> 1;
    t |= t >> 2;
    t |= t >> 4;
    t |= t >> 8;
    t |= t >> 16;
    return t + 1;
}

/* blockDim.x chosen by the launchers, scatter_kernel.cu:179,187 */
int orc_block_width(int max_cnt) {
    int b = orc_up_2n(max_cnt);
    if (b > ORC_MAX_THREADS) b = ORC_MAX_THREADS;
    if (b < 32) b = 32;
    return b;
}

/* kernel getPreSum, scatter_kernel.cu:85-100: thread i writes
 * preSum[inv[i]+1] = i+1 when inv[i] != inv[i+1]; the last thread always
 * writes.  preSum must come in zero-filled with length inv[n-1]+2
 * (scatter_op.py:125-126).  On unsorted input the device writes race; here
 * they are applied in index order, which is one of the possible outcomes. */
void orc_get_presum_ref(const int32_t *inv, int64_t n, int32_t *preSum) {
    for (int64_t i = 0; i < n; ++i) {
        int differ = (i == n - 1) ? 1 : (inv[i] != inv[i + 1]);
        if (differ) preSum[inv[i] + 1] = (int32_t)(i + 1);
    }
}

/* __shfl_down_sync within a 32-lane warp: lanes whose source would fall
 * outside the warp keep their own value. */
static void shfl_down_f(const float *in, float *out, int delta) {
    for (int l = 0; l < ORC_WARP; ++l) out[l] = (l + delta < ORC_WARP) ? in[l + delta] : in[l];
}
static void shfl_down_i(const int *in, int *out, int delta) {
    for (int l = 0; l < ORC_WARP; ++l) out[l] = (l + delta < ORC_WARP) ? in[l + delta] : in[l];
}

/* warpReduceSum, scatter_kernel.cu:26-39; volatile keeps each add a separate
 * fp32 rounding (no contraction, no x87 excess precision on any -O level). */
static void warp_reduce_sum(float *s, int blockSize) {
    float t[ORC_WARP];
    for (int delta = 16; delta >= 1; delta >>= 1) {
        if (blockSize >= 2 * delta) {
            shfl_down_f(s, t, delta);
            for (int l = 0; l < ORC_WARP; ++l) {
                volatile float r = s[l] + t[l];
                s[l] = r;
            }
        }
    }
}

/* warpReduceMax, scatter_kernel.cu:41-83: strict '>' on the shuffled-in lane */
static void warp_reduce_max(float *m, int *idx, int blockSize) {
    float tm[ORC_WARP];
    int ti[ORC_WARP];
    for (int delta = 16; delta >= 1; delta >>= 1) {
        if (blockSize >= 2 * delta) {
            shfl_down_f(m, tm, delta);
            shfl_down_i(idx, ti, delta);
            for (int l = 0; l < ORC_WARP; ++l) {
                if (tm[l] > m[l]) {
                    m[l] = tm[l];
                    idx[l] = ti[l];
                }
            }
        }
    }
}

/* kernel scatter_sum, scatter_kernel.cu:102-129, one (voxel, channel) at a
 * time, in the thread/warp order of the device code. */
void orc_scatter_sum_ref(const float *feats, const int32_t *preSum, float *out,
                         int64_t C, int64_t U, int max_cnt) {
    const int B = orc_block_width(max_cnt);
    const int nvw = (B + ORC_WARP - 1) / ORC_WARP;
    float *thr = (float *)malloc(sizeof(float) * (size_t)B);
    float warpS[ORC_WARP];
    for (int64_t u = 0; u < U; ++u) {
        const int64_t begin = preSum[u], end = preSum[u + 1];
        for (int64_t c = 0; c < C; ++c) {
            /* threads past the group's size never enter the loop and hold +0;
             * a warp made only of such threads reduces to +0, so it is skipped */
            const int64_t live = (end - begin < B) ? (end - begin) : B;
            const int live_warps = (int)((live + ORC_WARP - 1) / ORC_WARP);
            for (int tid = 0; tid < live_warps * ORC_WARP; ++tid) {
                volatile float s = 0.0f;
                for (int64_t i = begin + tid; i < end; i += B) s = s + feats[i * C + c];
                thr[tid] = s;
            }
            for (int w = 0; w < ORC_WARP; ++w) warpS[w] = 0.0f;
            for (int w = 0; w < live_warps; ++w) {
                float lanes[ORC_WARP];
                memcpy(lanes, thr + w * ORC_WARP, sizeof(lanes));
                warp_reduce_sum(lanes, B);
                warpS[w] = lanes[0];
            }
            /* second stage: lanes >= nvw hold 0 (scatter_kernel.cu:123) */
            warp_reduce_sum(warpS, nvw);
            out[u * C + c] = warpS[0];
        }
    }
    free(thr);
}

/* kernel scatter_max, scatter_kernel.cu:131-171.  Init (-FLT_MAX, -1); '>='
 * inside a thread, strict '>' across lanes and warps. */
void orc_scatter_max_ref(const float *feats, const int32_t *preSum, float *out,
                         int32_t *arg, int64_t C, int64_t U, int max_cnt) {
    const int B = orc_block_width(max_cnt);
    const int nvw = (B + ORC_WARP - 1) / ORC_WARP;
    float *thr = (float *)malloc(sizeof(float) * (size_t)B);
    int *thi = (int *)malloc(sizeof(int) * (size_t)B);
    for (int64_t u = 0; u < U; ++u) {
        const int64_t begin = preSum[u], end = preSum[u + 1];
        for (int64_t c = 0; c < C; ++c) {
            const int64_t live = (end - begin < B) ? (end - begin) : B;
            int live_warps = (int)((live + ORC_WARP - 1) / ORC_WARP);
            if (live_warps < 1) live_warps = 1; /* warp 0 always feeds stage 2 */
            for (int tid = 0; tid < live_warps * ORC_WARP; ++tid) {
                float m = -FLT_MAX;
                int mi = -1;
                for (int64_t i = begin + tid; i < end; i += B) {
                    float v = feats[i * C + c];
                    if (v >= m) {
                        m = v;
                        mi = (int)i;
                    }
                }
                thr[tid] = m;
                thi[tid] = mi;
            }
            /* stage 1 per warp; stage 2 runs in warp 0, whose lanes >= nvw keep
             * their own stage-1 registers (scatter_kernel.cu:161-166) */
            float w0m[ORC_WARP], sm[ORC_WARP];
            int w0i[ORC_WARP], si[ORC_WARP];
            /* warps made only of idle threads reduce to the initial pair */
            for (int w = 0; w < ORC_WARP; ++w) {
                sm[w] = -FLT_MAX;
                si[w] = -1;
            }
            for (int w = 0; w < live_warps; ++w) {
                float lm[ORC_WARP];
                int li[ORC_WARP];
                memcpy(lm, thr + w * ORC_WARP, sizeof(lm));
                memcpy(li, thi + w * ORC_WARP, sizeof(li));
                warp_reduce_max(lm, li, B);
                sm[w] = lm[0];
                si[w] = li[0];
                if (w == 0) {
                    memcpy(w0m, lm, sizeof(lm));
                    memcpy(w0i, li, sizeof(li));
                }
            }
            for (int l = 0; l < nvw; ++l) {
                w0m[l] = sm[l];
                w0i[l] = si[l];
            }
            warp_reduce_max(w0m, w0i, nvw);
            out[u * C + c] = w0m[0];
            arg[u * C + c] = w0i[0];
        }
    }
    free(thr);
    free(thi);
}

/* ---- spec functions over an arbitrary unq_inv --------------------------- */

/* exact histogram of unq_inv; returns -1 if an id is outside [0, U) */
int orc_counts(const int32_t *inv, int64_t n, int64_t U, int64_t *cnt) {
    memset(cnt, 0, sizeof(int64_t) * (size_t)U);
    for (int64_t i = 0; i < n; ++i) {
        if (inv[i] < 0 || inv[i] >= U) return -1;
        cnt[inv[i]]++;
    }
    return 0;
}

/* preSum = [0, cumsum(cnt)]; equals orc_get_presum_ref on sorted input */
void orc_presum(const int64_t *cnt, int64_t U, int32_t *preSum) {
    int64_t s = 0;
    preSum[0] = 0;
    for (int64_t u = 0; u < U; ++u) {
        s += cnt[u];
        preSum[u + 1] = (int32_t)s;
    }
}

/* stable counting sort of row ids by voxel id: perm[preSum[u] + k] is the k-th
 * row (ascending) of voxel u */
void orc_stable_perm(const int32_t *inv, int64_t n, int64_t U, const int32_t *preSum,
                     int32_t *perm) {
    int64_t *cur = (int64_t *)malloc(sizeof(int64_t) * (size_t)(U > 0 ? U : 1));
    for (int64_t u = 0; u < U; ++u) cur[u] = preSum[u];
    for (int64_t i = 0; i < n; ++i) perm[cur[inv[i]]++] = (int32_t)i;
    free(cur);
}

/* out[u,c] = sum_{i: inv[i]==u} feats[i,c], accumulated in double in row
 * order (scatter_kernel.cu:114-116 with an exact accumulator) */
void orc_scatter_sum_f64(const float *feats, const int32_t *inv, int64_t n, int64_t C,
                         int64_t U, double *out) {
    memset(out, 0, sizeof(double) * (size_t)(U * C));
    for (int64_t i = 0; i < n; ++i) {
        double *o = out + (int64_t)inv[i] * C;
        const float *f = feats + i * C;
        for (int64_t c = 0; c < C; ++c) o[c] += (double)f[c];
    }
}

/* max with the first-occurrence rule: strict '>' scanning rows in ascending
 * order, NaN never wins (as in scatter_kernel.cu:148, where every comparison
 * with NaN is false), -0.0 and +0.0 tie, -inf is an ordinary value.  A voxel
 * with no non-NaN entry keeps the reference's initial pair (-FLT_MAX, -1)
 * (scatter_kernel.cu:139-140). */
void orc_scatter_max_first(const float *feats, const int32_t *inv, int64_t n, int64_t C,
                           int64_t U, float *out, int32_t *arg) {
    for (int64_t k = 0; k < U * C; ++k) {
        out[k] = -FLT_MAX;
        arg[k] = -1;
    }
    for (int64_t i = 0; i < n; ++i) {
        const int64_t u = inv[i];
        const float *f = feats + i * C;
        for (int64_t c = 0; c < C; ++c) {
            const float v = f[c];
            if (v != v) continue;
            if (arg[u * C + c] < 0 || v > out[u * C + c]) {
                out[u * C + c] = v;
                arg[u * C + c] = (int32_t)i;
            }
        }
    }
}

/* scatter_op.py:69: out = sum_value / unq_cnts, one correctly rounded fp32
 * division by the count converted to fp32 */
void orc_mean_from_sum(const float *sum, const int64_t *cnt, int64_t C, int64_t U, float *out) {
    for (int64_t u = 0; u < U; ++u) {
        volatile float d = (float)cnt[u];
        for (int64_t c = 0; c < C; ++c) {
            volatile float q = sum[u * C + c] / d;
            out[u * C + c] = q;
        }
    }
}

/* scatter_op.py:47-50 */
void orc_sum_backward(const float *g, const int32_t *inv, int64_t n, int64_t C, float *gin) {
    for (int64_t i = 0; i < n; ++i)
        memcpy(gin + i * C, g + (int64_t)inv[i] * C, sizeof(float) * (size_t)C);
}

/* scatter_op.py:74-78 */
void orc_mean_backward(const float *g, const int64_t *cnt, const int32_t *inv, int64_t n,
                       int64_t C, float *gin) {
    for (int64_t i = 0; i < n; ++i) {
        const int64_t u = inv[i];
        volatile float d = (float)cnt[u];
        for (int64_t c = 0; c < C; ++c) {
            volatile float q = g[u * C + c] / d;
            gin[i * C + c] = q;
        }
    }
}

/* scatter_op.py:106-111 as intended: gin = 0; gin[arg[u,c], c] = g[u,c].
 * Entries with arg < 0 (voxel without a winner) contribute nothing. */
void orc_max_backward(const float *g, const int32_t *arg, int64_t n, int64_t C, int64_t U,
                      float *gin) {
    memset(gin, 0, sizeof(float) * (size_t)(n * C));
    for (int64_t u = 0; u < U; ++u)
        for (int64_t c = 0; c < C; ++c) {
            const int32_t r = arg[u * C + c];
            if (r >= 0 && r < n) gin[(int64_t)r * C + c] = g[u * C + c];
        }
}

/* ---- callers on either side of the path -------------------------------- */

/* ingroup_inds_kernel (torchex/src/ingroup_inds/ingroup_inds_kernel.cu:17-30):
 * out[i] = atomicAdd(&counter[group[i]], 1).  The device hands the ranks of a
 * group out in whatever order its threads arrive; here the threads run in
 * index order, which is one of the possible outcomes and the one the HIP path
 * always produces.  counter must hold max_group_id + 1 zeroed ints
 * (ingroup_inds_kernel.cu:40-42). */
void orc_ingroup_inds(const int64_t *group, int64_t n, int64_t max_group_id, int64_t *out) {
    int32_t *counter = (int32_t *)calloc((size_t)(max_group_id + 1), sizeof(int32_t));
    for (int64_t i = 0; i < n; ++i) out[i] = counter[group[i]]++;
    free(counter);
}

/* c10::div_floor_floating<float> (what torch.div(a, b, rounding_mode='floor')
 * applies per element): Python's floor division. */
static float orc_div_floor(float a, float b) {
    if (b == 0.0f) return a / b;
    volatile float mod = fmodf(a, b);
    volatile float div = (a - mod) / b;
    if ((mod != 0.0f) && ((b < 0.0f) != (mod < 0.0f))) div = div - 1.0f;
    float fl;
    if (div != 0.0f) {
        fl = floorf(div);
        if (div - fl > 0.5f) fl += 1.0f;
    } else {
        fl = copysignf(0.0f, a / b);
    }
    return fl;
}

/* voxelize_single (test/test_incremental_mask.py:20-26):
 * torch.div(points[:, :3] - pc_range[:3], voxel_size, rounding_mode='floor').int()
 * and the x-major linear key of operator_py/incremental_points.py:18-19 */
void orc_voxelize(const float *points, int64_t n, int64_t stride, const float *lo, const float *vs,
                  const int32_t *dims, int32_t *coors, int32_t *keys) {
    for (int64_t i = 0; i < n; ++i) {
        int32_t c[3];
        for (int a = 0; a < 3; ++a) {
            volatile float d = points[i * stride + a] - lo[a];
            c[a] = (int32_t)orc_div_floor(d, vs[a]);
            coors[i * 3 + a] = c[a];
        }
        keys[i] = (c[0] * dims[1] + c[1]) * dims[2] + c[2];
    }
}

/* ---- dynamic point pool -------------------------------------------------
 * torchex/src/dynamic_point_pool/dynamic_point_pool_kernel.cu:22-170 (test and
 * 13 numbers per hit) and :280-310 (compaction), with the two atomic counters
 * (:108-113) advanced in (box, point) order -- the order the reference's own
 * wrapper comment calls the usual one.  Mixed float/double arithmetic as
 * written there; the rotation terms cos/sin(rz + pi/2) are evaluated in double
 * and rounded to float (the device's cosf/sinf is within an ulp of that).
 * rois_batch / pts_batch (both NULL, or both given): the sample every box and point
 * belongs to; a pair is tested only when they agree, as in
 * generate_pts_mask_for_box3d_mixed (dynamic_point_pool_kernel.cu:173-212).
 * Returns the number of entries written. */
int64_t orc_dynamic_point_pool_mixed(const float *rois, const int32_t *rois_batch, int64_t B,
                                     const float *pts, const int32_t *pts_batch, int64_t P,
                                     const float *extra_wlh, int max_pts, int64_t max_all,
                                     int64_t *out_pts_idx, int64_t *out_roi_idx, float *out_feats) {
    int64_t global = 0;
    for (int64_t b = 0; b < B; ++b) {
        const float *r = rois + b * 7;
        const float cx = r[0], cy = r[1], w = r[3], l = r[4], h = r[5];
        const float large_w = w + extra_wlh[0], large_l = l + extra_wlh[1], large_h = h + extra_wlh[2];
        const float cz = (float)((double)r[2] + (double)h / 2.0);
        const float rot = (float)((double)r[6] + 3.14159265358979323846 / 2); /* M_PI / 2 */
        const float cosa = (float)cos((double)rot), sina = (float)sin((double)rot);
        int in_box_counter = 0;
        for (int64_t p = 0; p < P; ++p) {
            if (rois_batch && pts_batch[p] != rois_batch[b]) continue;
            const float x = pts[p * 3], y = pts[p * 3 + 1], z = pts[p * 3 + 2];
            if ((double)fabsf(z - cz) > (double)large_h / 2.0) continue;
            volatile float sx = x - cx, sy = y - cy;
            volatile float t1 = sx * cosa, t2 = sy * (-sina), t3 = sx * sina, t4 = sy * cosa;
            volatile float local_x = t1 + t2, local_y = t3 + t4;
            const double lx = local_x, ly = local_y;
            const int in_flag = (lx > -(double)l / 2.0) & (lx < (double)l / 2.0) & (ly > -(double)w / 2.0) &
                                (ly < (double)w / 2.0) & ((double)fabsf(z - cz) < (double)h / 2.0);
            const int in_large = (lx > -(double)large_l / 2.0) & (lx < (double)large_l / 2.0) &
                                 (ly > -(double)large_w / 2.0) & (ly < (double)large_w / 2.0);
            const int flag = in_flag ? 2 : (in_large ? 1 : 0);
            if (!flag) continue;
            const int cnt = in_box_counter++;
            if (cnt >= max_pts) continue;
            const int64_t pos = global++;
            if (pos >= max_all) continue;
            volatile float local_z = (float)((double)z - ((double)r[2] + (double)h / 2.0));
            float *f = out_feats + pos * 13;
            out_pts_idx[pos] = p;
            out_roi_idx[pos] = b;
            f[0] = x; f[1] = y; f[2] = z;
            f[3] = local_x; f[4] = local_y; f[5] = local_z;
            { volatile float v = local_x + l / 2; f[6] = v; }
            { volatile float v = local_y + w / 2; f[7] = v; }
            { volatile float v = local_z + h / 2; f[8] = v; }
            { volatile float v = -local_x + l / 2; f[9] = v; }
            { volatile float v = -local_y + w / 2; f[10] = v; }
            { volatile float v = -local_z + h / 2; f[11] = v; }
            f[12] = flag == 1 ? 1.0f : 0.0f;
        }
    }
    return global < max_all ? global : max_all;
}
int64_t orc_dynamic_point_pool(const float *rois, int64_t B, const float *pts, int64_t P,
                               const float *extra_wlh, int max_pts, int64_t max_all,
                               int64_t *out_pts_idx, int64_t *out_roi_idx, float *out_feats) {
    return orc_dynamic_point_pool_mixed(rois, NULL, B, pts, NULL, P, extra_wlh, max_pts, max_all, out_pts_idx,
                                        out_roi_idx, out_feats);
}

/* ---- grid hash ------------------------------------------------------------
 * torchex/src/utils/functions.cuh:30-64 with the inserts applied in index
 * order.  table: int32 [table_size, 2], filled with -1 by the caller. */
static int orc_double_hash(long long key, int probe_i, int table_size) {
    return (int)((key % table_size + probe_i * (key * 2 + 1)) % table_size);
}
int orc_grid_hash_build(const int32_t *keys, const int32_t *values, int64_t n, int32_t *table,
                        int table_size) {
    for (int64_t k = 0; k < n; ++k) {
        int placed = 0;
        for (int i = 0; i < table_size && !placed; ++i) {
            const int s = orc_double_hash(keys[k], i, table_size);
            if (table[2 * s] == -1) {
                table[2 * s] = keys[k];
                table[2 * s + 1] = values[k];
                placed = 1;
            }
        }
        if (!placed) return -1;
    }
    return 0;
}
void orc_grid_hash_probe(const int32_t *keys, int64_t n, const int32_t *table, int table_size,
                         int32_t *out) {
    for (int64_t k = 0; k < n; ++k) {
        out[k] = -1;
        for (int i = 0; i < table_size; ++i) {
            const int s = orc_double_hash(keys[k], i, table_size);
            if (table[2 * s] == keys[k]) {
                out[k] = table[2 * s + 1];
                break;
            }
            /* functions.cuh:54-63 scans all table_size slots before returning -1;
             * an empty slot already proves absence (no deletions), same answer */
            if (table[2 * s] == -1) break;
        }
    }
}
