// The callers on either side of the scatter operators: voxel keys from points,
// the unique / inverse / counts triple (from an occupancy map of the key grid, or from
// the same sort the scatter plan uses),
// the rank of an element inside its group, points-in-boxes pooling, and the
// coordinate hash table.
//
// Reference behaviour being replaced: voxelize_single
// (test/test_incremental_mask.py:20-26), ingroup_inds
// (torchex/src/ingroup_inds/ingroup_inds_kernel.cu:17-30), dynamic_point_pool
// (torchex/src/dynamic_point_pool/dynamic_point_pool_kernel.cu:22-170,280-310),
// grid_hash (torchex/src/grid_hash/grid_hash_kernel.cu:19-49,
// torchex/src/utils/functions.cuh:30-64).

#include "txs_common.h"

namespace {

using txs_detail::exclusive_scan;
using txs_detail::scan_tiles;

__global__ void fill_i32_kernel(int *p, long n, int value) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = value;
}

// ------------------------------------------------ voxelization front-end --

// torch.div(a, b, rounding_mode='floor') for fp32 (c10::div_floor_floating,
// c10/util/generic_math.h): Python's floor division, not floor(a / b).
__device__ __forceinline__ float div_floor_f32(float a, float b) {
    if (b == 0.0f) return a / b;
    const float mod = fmodf(a, b);
    float div = (a - mod) / b;
    if ((mod != 0.0f) && ((b < 0.0f) != (mod < 0.0f))) div -= 1.0f;
    float fl;
    if (div != 0.0f) {
        fl = floorf(div);
        if (div - fl > 0.5f) fl += 1.0f;
    } else {
        fl = copysignf(0.0f, a / b);
    }
    return fl;
}

// coors = floor((p - lo) / voxel) per axis, key = (x * Y + y) * Z + z
// (test/test_incremental_mask.py:20-26, operator_py/incremental_points.py:18-19)
__global__ void voxel_keys_kernel(const float *__restrict__ pts, long n, int stride, float lo0,
                                  float lo1, float lo2, float v0, float v1, float v2, int d0, int d1,
                                  int d2, int *__restrict__ coors, int *__restrict__ keys,
                                  int *__restrict__ stats) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float *p = pts + i * stride;
    const int x = (int)div_floor_f32(p[0] - lo0, v0);
    const int y = (int)div_floor_f32(p[1] - lo1, v1);
    const int z = (int)div_floor_f32(p[2] - lo2, v2);
    if (coors) {
        coors[i * 3 + 0] = x;
        coors[i * 3 + 1] = y;
        coors[i * 3 + 2] = z;
    }
    const bool ok = (unsigned)x < (unsigned)d0 && (unsigned)y < (unsigned)d1 && (unsigned)z < (unsigned)d2;
    if (!ok) stats[TXS_STAT_OUT_OF_RANGE] = 1;
    keys[i] = ok ? (x * d1 + y) * d2 + z : 0;
}

// 1 where a new run of equal keys starts
__global__ void run_flags_kernel(const int *__restrict__ ks, long n, int *__restrict__ flags) {
    long j = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (j < n) flags[j] = (j == 0 || ks[j] != ks[j - 1]) ? 1 : 0;
}

// What torch.unique(keys, return_inverse=True, return_counts=True) returns,
// from the sorted keys and the exclusive scan `ex` of the run-start flags,
// plus the plan arrays: run index rid = ex[j] + flag - 1.
__global__ void unique_finish_kernel(const int *__restrict__ ks, const int *__restrict__ perm,
                                     const int *__restrict__ ex, long n, int *__restrict__ seg,
                                     int *__restrict__ inv, int *__restrict__ unq,
                                     int *__restrict__ preSum, int *__restrict__ stats) {
    long j = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= n) return;
    const bool flag = (j == 0 || ks[j] != ks[j - 1]);
    const int rid = ex[j] + (flag ? 1 : 0) - 1;
    const int row = stats[TXS_STAT_UNSORTED] ? perm[j] : (int)j;
    seg[j] = rid;
    if ((unsigned)row < (unsigned)n) inv[row] = rid;
    if (flag) {
        unq[rid] = ks[j];
        preSum[rid] = (int)j;
    }
    if (j == n - 1) {
        preSum[rid + 1] = (int)n;
        stats[TXS_STAT_NUM_UNQ] = rid + 1;
    }
}


// ---- unique by occupancy map (keys from a bounded grid) ----------------------
// One byte per possible key, set by plain stores (every writer stores the same 1, so no
// atomic is needed; device-scope atomics on a bitmap were measured at 220 us for 1M keys),
// then packed into one bit per key.  The dense id of a key is the number of occupied keys
// below it: the exclusive scan of the words' population counts plus the bits below the key
// inside its word.  That is the inverse torch.unique returns (ids ascend with the keys),
// found without sorting the keys.

__global__ void bytemap_clear_kernel(uint4 *__restrict__ map16, long n16) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n16) map16[i] = make_uint4(0u, 0u, 0u, 0u);
}

template <typename K>
__global__ void bytemap_mark_kernel(const K *__restrict__ keys, long n, long key_bound,
                                    unsigned char *__restrict__ map, int *__restrict__ stats) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const long k = (long)keys[i];
    if (k < 0 || k >= key_bound) {
        stats[TXS_STAT_OUT_OF_RANGE] = 1;
        return;
    }
    map[k] = 1;
}

// 32 map bytes (each 0 or 1) -> one bitmap word and its population count
__global__ void bytemap_pack_kernel(const uint4 *__restrict__ map16, long words, unsigned *__restrict__ bm,
                                    int *__restrict__ cnt) {
    const long w = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (w >= words) return;
    const uint4 lo = map16[2 * w], hi = map16[2 * w + 1];
    // bytes b0..b3 of a word, each 0 or 1 -> bits 0..3: (x * 0x10204080) >> 28 leaves b0 + 2 b1 + 4 b2 + 8 b3
    auto nib = [](unsigned x) -> unsigned { return ((x * 0x10204080u) >> 28) & 15u; };
    const unsigned word = nib(lo.x) | (nib(lo.y) << 4) | (nib(lo.z) << 8) | (nib(lo.w) << 12) | (nib(hi.x) << 16) |
                          (nib(hi.y) << 20) | (nib(hi.z) << 24) | (nib(hi.w) << 28);
    bm[w] = word;
    cnt[w] = __popc(word);
}

// base: exclusive scan of the population counts, words + 1 entries (the last is the total)
__global__ void bitmap_total_kernel(const int *__restrict__ base, long words, int *__restrict__ stats) {
    if (blockIdx.x == 0 && threadIdx.x == 0) stats[TXS_STAT_NUM_UNQ] = base[words];
}

template <typename K>
__global__ void bitmap_assign_kernel(const K *__restrict__ keys, long n, long key_bound,
                                     const unsigned *__restrict__ bm, const int *__restrict__ base,
                                     long words, int *__restrict__ inv, int *__restrict__ unq_keys) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const long k = (long)keys[i];
        int id = 0;
        if (k >= 0 && k < key_bound) id = base[k >> 5] + __popc(bm[k >> 5] & ((1u << (k & 31)) - 1u));
        inv[i] = id;
    }
    if (i < words) {
        unsigned m = bm[i];
        int r = base[i];
        while (m) {
            const int b = __builtin_ctz(m);
            if (r < n) unq_keys[r] = (int)(i * 32 + b);
            ++r;
            m &= m - 1u;
        }
    }
}

// counts of the voxels from their CSR offsets, as int64 (what torch.unique returns)
__global__ void counts_from_presum_kernel(const int *__restrict__ preSum, long U, long long *__restrict__ cnts) {
    const long u = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (u < U) cnts[u] = (long long)(preSum[u + 1] - preSum[u]);
}

// rank of every element inside its group (operator_py/ingroup_inds_op.py,
// src/ingroup_inds/ingroup_inds_kernel.cu:17-30): sorted position minus the
// group's first position; ascending with the element's index, where the
// reference's atomic counter hands ranks out in arbitrary order.
__global__ void ingroup_inds_kernel(const int *__restrict__ seg, const int *__restrict__ perm,
                                    const int *__restrict__ preSum, long n, int U,
                                    long long *__restrict__ out) {
    long j = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= n) return;
    const int u = seg[j] & kIdMask;
    const int row = perm ? perm[j] : (int)j;
    if ((unsigned)u < (unsigned)U && (unsigned)row < (unsigned)n) out[row] = (long long)(j - preSum[u]);
}

// the same from a plan whose order flag is still on the device: stats[UNSORTED] says whether
// perm was written (rows already in order leave it unwritten: position == row); a plan that
// was not completed (ids out of range, or handed to the general sequence) is left alone
__global__ void ingroup_inds_auto_kernel(const int *__restrict__ seg, const int *__restrict__ perm,
                                         const int *__restrict__ preSum, const int *__restrict__ stats,
                                         long n, int U, long long *__restrict__ out) {
    long j = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= n) return;
    if (stats[TXS_STAT_OUT_OF_RANGE] != 0 || stats[TXS_STAT_NEED_GENERAL] != 0) return;
    const int u = seg[j] & kIdMask;
    const int row = stats[TXS_STAT_UNSORTED] != 0 ? perm[j] : (int)j;
    if ((unsigned)u < (unsigned)U && (unsigned)row < (unsigned)n) out[row] = (long long)(j - preSum[u]);
}

// ------------------------------------------------------ dynamic point pool --
// Points inside (enlarged) rotated boxes, with 13 box-relative numbers per hit
// (torchex/src/dynamic_point_pool/dynamic_point_pool_kernel.cu:22-170,280-310).
// The reference compacts the hits with two atomic counters, so their order and,
// when a cap is hit, the surviving subset depend on thread timing.  Here the
// hits are counted per (box, tile of 256 points), scanned, and written in
// (box, point) order: the outcome the reference's own comment calls the usual
// one ("out_roi_idx is automatically sorted"), made deterministic.

constexpr int kDppInfo = 13;

struct DppBox {
    float cx, cy, czc, w, l, h, cosa, sina, large_w, large_l, large_h, cz_bottom;
    float r2;  // squared radius of a circle around (cx, cy) that contains the box and its margin
};

// per-box constants, computed once so both passes see identical numbers; the
// rotation terms are evaluated in double and rounded (within an ulp of any cosf)
__global__ void dpp_box_kernel(const float *__restrict__ rois, int B, float extra_w, float extra_l,
                               float extra_h, DppBox *__restrict__ boxes) {
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= B) return;
    const float *r = rois + (size_t)b * 7;
    DppBox bx;
    bx.cx = r[0];
    bx.cy = r[1];
    bx.cz_bottom = r[2];
    bx.w = r[3];
    bx.l = r[4];
    bx.h = r[5];
    bx.large_w = bx.w + extra_w;
    bx.large_l = bx.l + extra_l;
    bx.large_h = bx.h + extra_h;
    bx.czc = (float)((double)r[2] + (double)bx.h / 2.0);  // bottom centre -> centre (:46)
    const float rot = (float)((double)r[6] + 3.14159265358979323846 / 2);  // (:24)
    bx.cosa = (float)cos((double)rot);
    bx.sina = (float)sin((double)rot);
    // generous bound (0.1 % + 1 mm^2): a point outside this circle fails the exact
    // test whatever the rounding, so skipping it cannot change the result
    const float hl = 0.5f * fmaxf(fabsf(bx.l), fabsf(bx.large_l));
    const float hw = 0.5f * fmaxf(fabsf(bx.w), fabsf(bx.large_w));
    bx.r2 = (hl * hl + hw * hw) * 1.001f + 1e-6f;
    boxes[b] = bx;
}

// cheap conservative reject in the xy plane; most waves skip the exact test with it
__device__ __forceinline__ bool dpp_near(const DppBox &bx, float x, float y) {
    const float sx = x - bx.cx, sy = y - bx.cy;
    return sx * sx + sy * sy <= bx.r2;
}

// 0: outside the enlarged box, 1: in the margin, 2: inside the box (:33-71)
__device__ __forceinline__ int dpp_test(const DppBox &bx, float x, float y, float z, float &local_x,
                                        float &local_y) {
#pragma clang fp contract(off)
    if ((double)fabsf(z - bx.czc) > (double)bx.large_h / 2.0) return 0;
    const float sx = x - bx.cx, sy = y - bx.cy;
    local_x = sx * bx.cosa + sy * (-bx.sina);
    local_y = sx * bx.sina + sy * bx.cosa;
    const double lx = local_x, ly = local_y;
    const bool in_box = (lx > -(double)bx.l / 2.0) & (lx < (double)bx.l / 2.0) &
                        (ly > -(double)bx.w / 2.0) & (ly < (double)bx.w / 2.0) &
                        ((double)fabsf(z - bx.czc) < (double)bx.h / 2.0);
    const bool in_large = (lx > -(double)bx.large_l / 2.0) & (lx < (double)bx.large_l / 2.0) &
                          (ly > -(double)bx.large_w / 2.0) & (ly < (double)bx.large_w / 2.0);
    return in_box ? 2 : (in_large ? 1 : 0);
}

// A workgroup keeps its 256 points in registers and walks kDppBoxesPerWg boxes, so the
// points are read once per group of boxes and the box constants come through the
// scalar path.
constexpr int kDppBoxesPerWg = 8;

// hits per (box, tile); grid (tiles, groups of boxes)
// (pts_batch / rois_batch, both NULL or both given: a point meets only the boxes of its own
// sample, generate_pts_mask_for_box3d_mixed, dynamic_point_pool_kernel.cu:173-212)
__global__ __launch_bounds__(kThreads) void dpp_count_kernel(const float *__restrict__ pts, int P,
                                                             const DppBox *__restrict__ boxes, int B,
                                                             int n_tiles, int *__restrict__ counts,
                                                             unsigned short *__restrict__ flags16,
                                                             const int *__restrict__ pts_batch,
                                                             const int *__restrict__ rois_batch) {
    __shared__ int cnt[kDppBoxesPerWg];
    const int p = blockIdx.x * kThreads + threadIdx.x;
    const int b0 = blockIdx.y * kDppBoxesPerWg;
    if (threadIdx.x < kDppBoxesPerWg) cnt[threadIdx.x] = 0;
    __syncthreads();
    float x = 0.f, y = 0.f, z = 0.f;
    int sample = 0;
    if (p < P) {
        x = pts[(size_t)p * 3];
        y = pts[(size_t)p * 3 + 1];
        z = pts[(size_t)p * 3 + 2];
        if (pts_batch) sample = pts_batch[p];
    }
    // the result of every test (2 bits per box of the group) is kept for the second pass,
    // which so repeats the arithmetic only for the hits it writes
    unsigned flags = 0u;
    for (int bb = 0; bb < kDppBoxesPerWg && b0 + bb < B; ++bb) {
        const DppBox bx = boxes[b0 + bb];
        int flag = 0;
        if (p < P && (!rois_batch || rois_batch[b0 + bb] == sample) && dpp_near(bx, x, y)) {
            float lx, ly;
            flag = dpp_test(bx, x, y, z, lx, ly);
        }
        flags |= (unsigned)flag << (2 * bb);
        const int c = __popcll(__ballot(flag > 0));
        if (c && (threadIdx.x & 63) == 0) atomicAdd(&cnt[bb], c);
    }
    if (p < P) flags16[(size_t)blockIdx.y * P + p] = (unsigned short)flags;
    __syncthreads();
    if (threadIdx.x < kDppBoxesPerWg && b0 + (int)threadIdx.x < B)
        counts[(size_t)(b0 + threadIdx.x) * n_tiles + blockIdx.x] = cnt[threadIdx.x];
}

// per-box kept count = min(hits, cap), exclusive scan over boxes, total (one workgroup)
__global__ __launch_bounds__(kThreads) void dpp_box_base_kernel(const int *__restrict__ scanned,
                                                                int B, int n_tiles, int cap,
                                                                int max_all, int *__restrict__ box_base,
                                                                int *__restrict__ total_out) {
    int carry = 0;
    for (int base = 0; base < B; base += kThreads) {
        const int b = base + threadIdx.x;
        int kept = 0;
        if (b < B) kept = min(scanned[(size_t)(b + 1) * n_tiles] - scanned[(size_t)b * n_tiles], cap);
        int tot;
        const int ex = block_exclusive_scan(kept, &tot);
        if (b < B) box_base[b] = carry + ex;
        carry += tot;
    }
    if (threadIdx.x == 0) total_out[0] = min(carry, max_all);
}

// second pass: rank of every hit inside its box from the first pass's results, compact write
__global__ __launch_bounds__(kThreads) void dpp_write_kernel(
    const float *__restrict__ pts, int P, const DppBox *__restrict__ boxes, int B, int n_tiles,
    const int *__restrict__ scanned, const int *__restrict__ box_base, int cap, int max_all,
    const unsigned short *__restrict__ flags16, long long *__restrict__ out_pts_idx,
    long long *__restrict__ out_roi_idx, float *__restrict__ out_feats) {
#pragma clang fp contract(off)
    __shared__ int wsum[kDppBoxesPerWg][kThreads / 64];
    const int b0 = blockIdx.y * kDppBoxesPerWg;
    const int p = blockIdx.x * kThreads + threadIdx.x;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    // phase 1: the hits of each wave per box of the group
    const unsigned flags = p < P ? (unsigned)flags16[(size_t)blockIdx.y * P + p] : 0u;
    for (int bb = 0; bb < kDppBoxesPerWg && b0 + bb < B; ++bb) {
        const unsigned long long m = __ballot(((flags >> (2 * bb)) & 3u) != 0u);
        if (lane == 0) wsum[bb][w] = __popcll(m);
    }
    __syncthreads();
    if (flags == 0u) return;  // (no barrier follows)
    const float x = pts[(size_t)p * 3], y = pts[(size_t)p * 3 + 1], z = pts[(size_t)p * 3 + 2];
    // phase 2: rank of each hit inside its box, compact write (hits are rare)
    for (int bb = 0; bb < kDppBoxesPerWg && b0 + bb < B; ++bb) {
        const int flag = (int)((flags >> (2 * bb)) & 3u);
        const unsigned long long m = __ballot(flag > 0);
        if (flag == 0) continue;
        const int b = b0 + bb;
        int rank = __popcll(m & ((1ull << lane) - 1ull));
        for (int k = 0; k < w; ++k) rank += wsum[bb][k];
        rank += scanned[(size_t)b * n_tiles + blockIdx.x] - scanned[(size_t)b * n_tiles];
        if (rank >= cap) continue;
        const long pos = (long)box_base[b] + rank;
        if (pos >= max_all) continue;
        const DppBox bx = boxes[b];
        float lx, ly;
        dpp_test(bx, x, y, z, lx, ly);  // the same arithmetic as in phase 1
        const float local_z = (float)((double)z - ((double)bx.cz_bottom + (double)bx.h / 2.0));  // (:103)
        float *f = out_feats + pos * kDppInfo;
        out_pts_idx[pos] = p;
        out_roi_idx[pos] = b;
        f[0] = x;
        f[1] = y;
        f[2] = z;
        f[3] = lx;
        f[4] = ly;
        f[5] = local_z;
        f[6] = lx + bx.l / 2;
        f[7] = ly + bx.w / 2;
        f[8] = local_z + bx.h / 2;
        f[9] = -lx + bx.l / 2;
        f[10] = -ly + bx.w / 2;
        f[11] = -local_z + bx.h / 2;
        f[12] = flag == 1 ? 1.0f : 0.0f;
    }
}

// ------------------------------------------------------------- grid hash --
// Open-addressing table of (key, value) int32 pairs with the reference's probe
// sequence (torchex/src/utils/functions.cuh:30-64, double hashing with an odd
// step over a power-of-two table).  A slot is one 64-bit word (key in the low
// half, value in the high half, as the reference's [size, 2] int32 tensor lays
// them out) claimed with a single 64-bit compare-and-swap, so key and value
// appear together.

// (key % size + i * (2 * key + 1)) % size of the reference, for key >= 0 and a
// power-of-two size: both remainders are bit masks and the 64-bit sum cannot wrap
// (i < size <= 2^30, 2 * key + 1 < 2^32).
__device__ __forceinline__ int grid_hash_slot(int key, int probe_i, int table_size) {
    const unsigned long long mask = (unsigned long long)(table_size - 1);
    const unsigned long long k = (unsigned long long)(unsigned)key;
    return (int)(((k & mask) + (unsigned long long)probe_i * (k * 2ull + 1ull)) & mask);
}

__global__ void grid_hash_build_kernel(const int *__restrict__ keys, const int *__restrict__ values,
                                       unsigned long long *__restrict__ table, int table_size, long n,
                                       int *__restrict__ fail) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int key = keys[i];
    const unsigned long long word =
        ((unsigned long long)(unsigned)values[i] << 32) | (unsigned long long)(unsigned)key;
    const unsigned long long empty = ~0ull;  // (-1, -1)
    for (int t = 0; key >= 0 && t < table_size; ++t) {
        const int s = grid_hash_slot(key, t, table_size);
        if (atomicCAS(table + s, empty, word) == empty) return;
    }
    if (fail) fail[0] = 1;  // table full or key negative (the reference asserts)
}

__global__ void grid_hash_probe_kernel(const int *__restrict__ keys,
                                       const unsigned long long *__restrict__ table, int table_size,
                                       long n, int *__restrict__ out) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int key = keys[i];
    int v = -1;
    for (int t = 0; key >= 0 && t < table_size; ++t) {
        const int s = grid_hash_slot(key, t, table_size);
        const unsigned long long word = table[s];
        const int slot_key = (int)(unsigned)(word & 0xffffffffull);
        if (slot_key == key) {
            v = (int)(unsigned)(word >> 32);
            break;
        }
        // An empty slot on the probe sequence proves the key was never inserted
        // (no deletions).  The reference keeps scanning all table_size slots
        // before giving up (functions.cuh:54-63), with the same answer.
        if (slot_key == -1) break;
    }
    out[i] = v;
}

}  // namespace

extern "C" {

int txs_voxel_keys(const float *points, int64_t num_total, int64_t point_stride,
                   const float *range_lo, const float *voxel_size, const int32_t *dims,
                   int32_t *coors, int32_t *keys, int32_t *stats, void *stream) {
    if (!fits_i32(num_total) || point_stride < 3 || !range_lo || !voxel_size || !dims || !stats)
        return TXS_ERR_INVALID_ARG;
    const long long cells = (long long)dims[0] * dims[1] * dims[2];
    if (dims[0] <= 0 || dims[1] <= 0 || dims[2] <= 0 || !fits_i32(cells)) return TXS_ERR_INVALID_ARG;
    if (num_total == 0) return TXS_OK;
    if (!points || !keys) return TXS_ERR_INVALID_ARG;
    voxel_keys_kernel<<<dim3(blocks_for(num_total)), dim3(kThreads), 0, (hipStream_t)stream>>>(
        points, num_total, (int)point_stride, range_lo[0], range_lo[1], range_lo[2], voxel_size[0],
        voxel_size[1], voxel_size[2], dims[0], dims[1], dims[2], coors, keys, stats);
    return status_of(hipGetLastError());
}

int64_t txs_unique_bitmap_workspace_len(int64_t key_bound) {
    if (key_bound <= 0 || key_bound > (1LL << 31)) return -1;
    const int64_t words = (key_bound + 31) / 32;
    // byte map (32 bytes per word), bitmap, scanned counts, scan workspace
    return 8 * words + words + (words + 1) + scan_tiles(words + 1) + 17;
}

int txs_unique_bitmap_count(const void *keys, int key_is_int64, int64_t num_total, int64_t key_bound,
                            int32_t *bitmap_ws, int32_t *stats, void *stream) {
    if (!fits_i32(num_total) || key_bound <= 0 || key_bound > (1LL << 31) || !stats) return TXS_ERR_INVALID_ARG;
    if (num_total == 0) return TXS_OK;
    if (!keys || !bitmap_ws || ((uintptr_t)bitmap_ws & 15u) != 0) return TXS_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const long n = num_total;
    const long words = (long)((key_bound + 31) / 32);
    uint4 *map16 = reinterpret_cast<uint4 *>(bitmap_ws);
    unsigned char *map = reinterpret_cast<unsigned char *>(bitmap_ws);
    unsigned *bm = reinterpret_cast<unsigned *>(bitmap_ws + 8 * words);
    int *base = bitmap_ws + 9 * words;
    int *scan_ws = base + words + 1;
    bytemap_clear_kernel<<<dim3(blocks_for(2 * words)), dim3(kThreads), 0, st>>>(map16, 2 * words);
    if (key_is_int64)
        bytemap_mark_kernel<long long><<<dim3(blocks_for(n)), dim3(kThreads), 0, st>>>(
            static_cast<const long long *>(keys), n, (long)key_bound, map, stats);
    else
        bytemap_mark_kernel<int><<<dim3(blocks_for(n)), dim3(kThreads), 0, st>>>(
            static_cast<const int *>(keys), n, (long)key_bound, map, stats);
    bytemap_pack_kernel<<<dim3(blocks_for(words)), dim3(kThreads), 0, st>>>(map16, words, bm, base);
    if (exclusive_scan(base, words, base, words + 1, scan_ws, st) != hipSuccess) return TXS_ERR_LAUNCH;
    bitmap_total_kernel<<<dim3(1), dim3(64), 0, st>>>(base, words, stats);
    return status_of(hipGetLastError());
}

int txs_unique_bitmap_assign(const void *keys, int key_is_int64, int64_t num_total, int64_t key_bound,
                             const int32_t *bitmap_ws, int32_t *unq_inv, int32_t *unq_keys, void *stream) {
    if (!fits_i32(num_total) || key_bound <= 0 || key_bound > (1LL << 31)) return TXS_ERR_INVALID_ARG;
    if (num_total == 0) return TXS_OK;
    if (!keys || !bitmap_ws || !unq_inv || !unq_keys) return TXS_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const long n = num_total;
    const long words = (long)((key_bound + 31) / 32);
    const unsigned *bm = reinterpret_cast<const unsigned *>(bitmap_ws + 8 * words);
    const int *base = bitmap_ws + 9 * words;
    const long span = n > words ? n : words;
    if (key_is_int64)
        bitmap_assign_kernel<long long><<<dim3(blocks_for(span)), dim3(kThreads), 0, st>>>(
            static_cast<const long long *>(keys), n, (long)key_bound, bm, base, words, unq_inv, unq_keys);
    else
        bitmap_assign_kernel<int><<<dim3(blocks_for(span)), dim3(kThreads), 0, st>>>(
            static_cast<const int *>(keys), n, (long)key_bound, bm, base, words, unq_inv, unq_keys);
    return status_of(hipGetLastError());
}

int txs_counts_from_presum(const int32_t *preSum, int64_t num_unq, int64_t *unq_cnts, void *stream) {
    if (!fits_i32(num_unq)) return TXS_ERR_INVALID_ARG;
    if (num_unq == 0) return TXS_OK;
    if (!preSum || !unq_cnts) return TXS_ERR_INVALID_ARG;
    counts_from_presum_kernel<<<dim3(blocks_for(num_unq)), dim3(kThreads), 0, (hipStream_t)stream>>>(
        preSum, (long)num_unq, (long long *)unq_cnts);
    return status_of(hipGetLastError());
}

int64_t txs_unique_workspace_len(int64_t num_total) { return num_total + scan_tiles(num_total + 1) + 17; }

int txs_unique_runs(const int32_t *sorted_keys, const int32_t *perm, int64_t num_total,
                    int32_t *unique_ws, int32_t *seg, int32_t *unq_inv, int32_t *unq_keys,
                    int32_t *preSum, int32_t *stats, void *stream) {
    if (!fits_i32(num_total) || !stats || !preSum) return TXS_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    if (num_total == 0) {
        fill_i32_kernel<<<dim3(1), dim3(64), 0, st>>>(preSum, 1, 0);
        return status_of(hipGetLastError());
    }
    if (!sorted_keys || !perm || !unique_ws || !seg || !unq_inv || !unq_keys) return TXS_ERR_INVALID_ARG;
    const long n = num_total;
    int *flags = unique_ws;
    int *scan_ws = unique_ws + n;
    run_flags_kernel<<<dim3(blocks_for(n)), dim3(kThreads), 0, st>>>(sorted_keys, n, flags);
    if (exclusive_scan(flags, n, flags, n, scan_ws, st) != hipSuccess) return TXS_ERR_LAUNCH;
    unique_finish_kernel<<<dim3(blocks_for(n)), dim3(kThreads), 0, st>>>(sorted_keys, perm, flags, n, seg,
                                                                       unq_inv, unq_keys, preSum, stats);
    return status_of(hipGetLastError());
}

int txs_group_ranks(const int32_t *group_ids, int64_t num_total, int64_t num_groups, int32_t *plan_ws,
                    int32_t *perm, int32_t *seg, int32_t *preSum, int64_t *out, int32_t *stats, void *stream) {
    if (!fits_i32(num_total) || !fits_i32(num_groups) || !stats) return TXS_ERR_INVALID_ARG;
    if (num_total == 0) return TXS_OK;
    if (!group_ids || !plan_ws || !perm || !seg || !preSum || !out || num_groups <= 0) return TXS_ERR_INVALID_ARG;
    const int32_t heavy = txs_default_heavy_threshold();
    // the bucket kernels rank while they place; any other route leaves a plan to rank from
    const bool fused = txs_detail::plan_writes_ranks(num_total, num_groups);
    const int rc = txs_detail::plan_build(group_ids, num_total, num_groups, heavy, nullptr, plan_ws, perm, seg, preSum,
                                          nullptr, nullptr, stats, fused ? (long long *)out : nullptr, stream);
    if (rc != TXS_OK || fused) return rc;
    ingroup_inds_auto_kernel<<<dim3(blocks_for(num_total)), dim3(kThreads), 0, (hipStream_t)stream>>>(
        seg, perm, preSum, stats, num_total, (int)num_groups, (long long *)out);
    return status_of(hipGetLastError());
}

int txs_ingroup_inds(const int32_t *seg, const int32_t *perm, const int32_t *preSum,
                     int64_t num_total, int64_t num_unq, int64_t *out, void *stream) {
    if (!fits_i32(num_total) || !fits_i32(num_unq)) return TXS_ERR_INVALID_ARG;
    if (num_total == 0) return TXS_OK;
    if (!seg || !preSum || !out || num_unq <= 0) return TXS_ERR_INVALID_ARG;
    ingroup_inds_kernel<<<dim3(blocks_for(num_total)), dim3(kThreads), 0, (hipStream_t)stream>>>(
        seg, perm, preSum, num_total, (int)num_unq, (long long *)out);
    return status_of(hipGetLastError());
}

int64_t txs_dpp_workspace_len(int64_t num_pts, int64_t num_boxes) {
    const int64_t tiles = (num_pts + kThreads - 1) / kThreads;
    const int64_t cells = num_boxes * tiles + 1;
    // box constants, (box, tile) counts, scan workspace, box bases, and the first pass's test
    // results: 2 bits per (point, box), 16 bits per point and group of 8 boxes
    const int64_t groups = (num_boxes + kDppBoxesPerWg - 1) / kDppBoxesPerWg;
    return (int64_t)(sizeof(DppBox) / sizeof(int)) * num_boxes + cells + scan_tiles(cells + 2) + 1 +
           num_boxes + 16 + (groups * num_pts + 1) / 2;
}

int txs_dynamic_point_pool(const float *rois, const float *pts, int64_t num_boxes, int64_t num_pts,
                           const float *extra_wlh, int32_t max_pts_per_box, int64_t max_all_pts,
                           int32_t *workspace, int64_t *out_pts_idx, int64_t *out_roi_idx,
                           float *out_pts_feats, int32_t *num_out, void *stream) {
    return txs_dynamic_point_pool_mixed(rois, nullptr, pts, nullptr, num_boxes, num_pts, extra_wlh,
                                        max_pts_per_box, max_all_pts, workspace, out_pts_idx, out_roi_idx,
                                        out_pts_feats, num_out, stream);
}

int txs_dynamic_point_pool_mixed(const float *rois, const int32_t *rois_batch, const float *pts,
                                 const int32_t *pts_batch, int64_t num_boxes, int64_t num_pts,
                                 const float *extra_wlh, int32_t max_pts_per_box, int64_t max_all_pts,
                                 int32_t *workspace, int64_t *out_pts_idx, int64_t *out_roi_idx,
                                 float *out_pts_feats, int32_t *num_out, void *stream) {
    if (!fits_i32(num_boxes) || !fits_i32(num_pts) || !fits_i32(max_all_pts) || max_pts_per_box < 0 ||
        !extra_wlh || !num_out)
        return TXS_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    if (num_boxes == 0 || num_pts == 0) {
        fill_i32_kernel<<<dim3(1), dim3(64), 0, st>>>(num_out, 1, 0);
        return status_of(hipGetLastError());
    }
    if (!rois || !pts || !workspace || !out_pts_idx || !out_roi_idx || !out_pts_feats ||
        ((rois_batch == nullptr) != (pts_batch == nullptr)))
        return TXS_ERR_INVALID_ARG;
    const int B = (int)num_boxes, P = (int)num_pts;
    const int n_tiles = (P + kThreads - 1) / kThreads;
    const long cells = (long)B * n_tiles;
    if (!fits_i32(cells + 1) || B > 65535) return TXS_ERR_INVALID_ARG;
    DppBox *boxes = reinterpret_cast<DppBox *>(workspace);
    int *counts = workspace + (sizeof(DppBox) / sizeof(int)) * (size_t)B;
    int *scan_ws = counts + cells + 1;
    int *box_base = scan_ws + scan_tiles(cells + 2) + 1;
    unsigned short *flags16 = reinterpret_cast<unsigned short *>(box_base + B);
    dpp_box_kernel<<<dim3(blocks_for(B)), dim3(kThreads), 0, st>>>(rois, B, extra_wlh[0], extra_wlh[1],
                                                                 extra_wlh[2], boxes);
    const int box_groups = (B + kDppBoxesPerWg - 1) / kDppBoxesPerWg;
    dpp_count_kernel<<<dim3(n_tiles, box_groups), dim3(kThreads), 0, st>>>(pts, P, boxes, B, n_tiles, counts,
                                                                           flags16, pts_batch, rois_batch);
    if (exclusive_scan(counts, cells, counts, cells + 1, scan_ws, st) != hipSuccess) return TXS_ERR_LAUNCH;
    dpp_box_base_kernel<<<dim3(1), dim3(kThreads), 0, st>>>(counts, B, n_tiles, max_pts_per_box,
                                                           (int)max_all_pts, box_base, num_out);
    dpp_write_kernel<<<dim3(n_tiles, box_groups), dim3(kThreads), 0, st>>>(
        pts, P, boxes, B, n_tiles, counts, box_base, max_pts_per_box, (int)max_all_pts, flags16,
        (long long *)out_pts_idx, (long long *)out_roi_idx, out_pts_feats);
    return status_of(hipGetLastError());
}

int txs_grid_hash_build(const int32_t *keys, const int32_t *values, int64_t num_keys, int32_t *table,
                        int64_t table_size, int32_t *fail_flag, void *stream) {
    if (!fits_i32(num_keys) || !fits_i32(table_size) || table_size <= 0 || !table) return TXS_ERR_INVALID_ARG;
    if ((table_size & (table_size - 1)) != 0 || ((uintptr_t)table & 7) != 0) return TXS_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    fill_i32_kernel<<<dim3(blocks_for(2 * table_size)), dim3(kThreads), 0, st>>>(table, 2 * table_size, -1);
    if (num_keys > 0) {
        if (!keys || !values || num_keys > table_size) return TXS_ERR_INVALID_ARG;
        grid_hash_build_kernel<<<dim3(blocks_for(num_keys)), dim3(kThreads), 0, st>>>(
            keys, values, (unsigned long long *)table, (int)table_size, num_keys, fail_flag);
    }
    return status_of(hipGetLastError());
}

int txs_grid_hash_probe(const int32_t *keys, int64_t num_keys, const int32_t *table,
                        int64_t table_size, int32_t *out_values, void *stream) {
    if (!fits_i32(num_keys) || !fits_i32(table_size) || table_size <= 0 || !table) return TXS_ERR_INVALID_ARG;
    if ((table_size & (table_size - 1)) != 0 || ((uintptr_t)table & 7) != 0) return TXS_ERR_INVALID_ARG;
    if (num_keys == 0) return TXS_OK;
    if (!keys || !out_values) return TXS_ERR_INVALID_ARG;
    grid_hash_probe_kernel<<<dim3(blocks_for(num_keys)), dim3(kThreads), 0, (hipStream_t)stream>>>(
        keys, (const unsigned long long *)table, (int)table_size, num_keys, out_values);
    return status_of(hipGetLastError());
}

}  // extern "C"
