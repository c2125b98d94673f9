// Index preparation for the voxel scatter kernels (built once per ScatterData and
// reused by every forward/backward call): sortedness/range check, stable LSD radix
// sort of (voxel id, row), CSR offsets from run boundaries, table of special
// voxels, per-position voxel ids.  No histogram atomics on global memory and no
// inter-block spinning anywhere.
//
// Reference behaviour being replaced: ScatterData.__init__
// (torchex/operator_py/scatter_op.py:7-21) and getPreSum
// (torchex/src/scatter/scatter_kernel.cu:85-100).

#include "txs_common.h"

namespace {

// -------------------------------------------------------------- small utils --

// Reference getPreSum (scatter_kernel.cu:85-100) for sorted ids.
__global__ void get_presum_kernel(const int *__restrict__ inv, int *__restrict__ preSum, long n,
                                  long num_presum) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    int v = inv[i];
    bool boundary = (i == n - 1) || (inv[i + 1] != v);
    long slot = (long)v + 1;
    if (boundary && slot >= 0 && slot < num_presum) preSum[slot] = (int)(i + 1);
}

// Order and range flags of unq_inv (no histogram: counts come from the run
// boundaries of the sorted ids, which needs no atomics).
__global__ void plan_check_kernel(const int *__restrict__ inv, long n, int U,
                                  int *__restrict__ stats) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int v = inv[i];
    if ((unsigned)v >= (unsigned)U) stats[TXS_STAT_OUT_OF_RANGE] = 1;
    if (i + 1 < n && inv[i + 1] < v) stats[TXS_STAT_UNSORTED] = 1;
}

// ids that are already sorted are their own sorted keys
__global__ void copy_if_sorted_kernel(const int *__restrict__ inv, long n,
                                      const int *__restrict__ stats, int *__restrict__ keys) {
    if (stats[TXS_STAT_UNSORTED] != 0) return;
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) keys[i] = inv[i];
}

// CSR offsets from sorted keys: preSum[u] = first position whose key is >= u.
// Thread j owns the boundary in front of position j and fills the offsets of
// every id in (key[j-1], key[j]] (more than one only across empty voxels).
__global__ void presum_from_sorted_kernel(const int *__restrict__ keys, long n, int U,
                                          int *__restrict__ preSum) {
    long j = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (j > n) return;
    long lo = (j == 0) ? -1 : (long)(keys[j - 1] & kIdMask);
    long hi = (j == n) ? (long)U : (long)(keys[j] & kIdMask);
    if (hi > U) hi = U;
    for (long u = lo + 1; u <= hi; ++u)
        if (u >= 0) preSum[u] = (int)j;
}

// ------------------------------------------------------------ exclusive scan --
// out[i] = sum_{k<i} in[k] for i in [0, n_out), where in[k] = 0 for k >= n_in.
// Three launches, no inter-block waiting: tile sums, scan of tile sums by one
// workgroup, tile-local scan plus tile offset.

constexpr int kScanItems = 8;
constexpr int kScanTile = kThreads * kScanItems;
constexpr int kScanFusedTiles = 1024;  // up to this many tiles the apply kernel sums the tile totals itself

__global__ __launch_bounds__(kThreads) void scan_tile_sums_kernel(const int *__restrict__ in,
                                                                  long n_in,
                                                                  int *__restrict__ tile_sums) {
    long base = (long)blockIdx.x * kScanTile + (long)threadIdx.x * kScanItems;
    int s = 0;
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
        long i = base + k;
        if (i < n_in) s += in[i];
    }
    int tot;
    block_exclusive_scan(s, &tot);
    if (threadIdx.x == 0) tile_sums[blockIdx.x] = tot;
}

__global__ __launch_bounds__(kThreads) void scan_tile_offsets_kernel(int *__restrict__ tile_sums,
                                                                     long n_tiles) {
    int carry = 0;
    for (long base = 0; base < n_tiles; base += kThreads) {
        long i = base + threadIdx.x;
        int x = (i < n_tiles) ? tile_sums[i] : 0;
        int tot;
        int ex = block_exclusive_scan(x, &tot);
        if (i < n_tiles) tile_sums[i] = carry + ex;
        carry += tot;
    }
}

// in and out may be the same array: a thread reads its items before any write.
// With offsets_ready == 0, tile_offs still holds the plain tile sums and the
// workgroup adds up the ones in front of its own tile itself (cheaper than a
// launch of its own while there are few tiles).
__global__ __launch_bounds__(kThreads) void scan_apply_kernel(const int *in, long n_in, int *out,
                                                              long n_out, const int *tile_offs,
                                                              int offsets_ready) {
    long base = (long)blockIdx.x * kScanTile + (long)threadIdx.x * kScanItems;
    int x[kScanItems];
    int s = 0;
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
        long i = base + k;
        x[k] = (i < n_in) ? in[i] : 0;
        s += x[k];
    }
    int tile_off;
    if (offsets_ready) {
        tile_off = tile_offs[blockIdx.x];
    } else {
        int part = 0;
        for (int t = threadIdx.x; t < (int)blockIdx.x; t += kThreads) part += tile_offs[t];
        block_exclusive_scan(part, &tile_off);
    }
    int tot;
    int run = block_exclusive_scan(s, &tot) + tile_off;
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
        long i = base + k;
        if (i < n_out) out[i] = run;
        run += x[k];
    }
}

}  // namespace

namespace txs_detail {

long scan_tiles(long n_out) { return (n_out + kScanTile - 1) / kScanTile; }

hipError_t exclusive_scan(const int *in, long n_in, int *out, long n_out, int *ws,
                          hipStream_t st) {
    if (n_out <= 0) return hipSuccess;
    long tiles = scan_tiles(n_out);
    scan_tile_sums_kernel<<<dim3((unsigned)tiles), dim3(kThreads), 0, st>>>(in, n_in, ws);
    const int few = tiles <= kScanFusedTiles;
    if (!few) scan_tile_offsets_kernel<<<dim3(1), dim3(kThreads), 0, st>>>(ws, tiles);
    scan_apply_kernel<<<dim3((unsigned)tiles), dim3(kThreads), 0, st>>>(in, n_in, out, n_out, ws, !few);
    return hipGetLastError();
}

}  // namespace txs_detail

namespace {

using txs_detail::exclusive_scan;
using txs_detail::scan_tiles;

__device__ __forceinline__ int wave_max_i32(int x) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) x = max(x, __shfl_xor(x, d, 64));
    return x;
}

// Special-voxel table, max_cnt, and the check of the caller's counts against
// the histogram.  Launched with 1024-thread workgroups: the statistics are
// reduced across the workgroup first, because device-scope atomics on one
// address complete one after the other (~10 ns each) and one per wavefront
// would dominate the kernel.
constexpr int kSpecialThreads = 1024;
__global__ __launch_bounds__(kSpecialThreads) void plan_special_kernel(
    const int *__restrict__ preSum, int U_arg, int heavy_threshold,
    const long long *__restrict__ unq_cnts, int *__restrict__ slot_of,
    int *__restrict__ heavy_ids, int *__restrict__ stats, const int *__restrict__ num_unq_dev,
    long long *__restrict__ cnts_out) {
    __shared__ int s_max[kSpecialThreads / 64], s_bad[kSpecialThreads / 64];
    // the voxel count may only be known on the device (unique path): U_arg is then an upper bound
    const int U = num_unq_dev ? min(U_arg, *num_unq_dev) : U_arg;
    const int u = blockIdx.x * blockDim.x + threadIdx.x;
    const bool in = u < U;
    const int c = in ? preSum[u + 1] - preSum[u] : 0;
    const int wmax = wave_max_i32(c);
    const bool mismatch = in && unq_cnts && unq_cnts[u] != (long long)c;
    const int any_mismatch = __ballot(mismatch) != 0ull;
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) {
        s_max[w] = wmax;
        s_bad[w] = any_mismatch;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int m = 0, b = 0;
        for (int k = 0; k < kSpecialThreads / 64; ++k) {
            m = max(m, s_max[k]);
            b |= s_bad[k];
        }
        if (m > 0) atomicMax(&stats[TXS_STAT_MAX_CNT], m);
        if (b) stats[TXS_STAT_COUNT_MISMATCH] = 1;
    }
    if (in && cnts_out) cnts_out[u] = (long long)c;
    // Slots: heavy voxels fill heavy_ids from the front (their slot is also their row in
    // the scratch table), empty voxels from the back of the U-entry array (they own no
    // scratch).  One atomic per wave and kind hands out a contiguous range.
    const bool heavy = in && c > heavy_threshold;
    const bool empty = in && c == 0;
    const unsigned long long mh = __ballot(heavy), me = __ballot(empty);
    const int lane = threadIdx.x & 63;
    const unsigned long long below = (1ull << lane) - 1ull;
    int base_h = 0, base_e = 0;
    if (lane == 0) {
        if (mh) base_h = atomicAdd(&stats[TXS_STAT_NUM_HEAVY], __popcll(mh));
        if (me) base_e = atomicAdd(&stats[TXS_STAT_NUM_EMPTY], __popcll(me));
        if (mh | me) atomicAdd(&stats[TXS_STAT_NUM_SPECIAL], __popcll(mh) + __popcll(me));
    }
    base_h = __shfl(base_h, 0, 64);
    base_e = __shfl(base_e, 0, 64);
    if (!in) return;
    int slot = -1;
    if (heavy) {
        slot = base_h + __popcll(mh & below);
        if (slot < U_arg) heavy_ids[slot] = u;
    } else if (empty) {
        slot = U_arg - 1 - (base_e + __popcll(me & below));
        if (slot >= 0) heavy_ids[slot] = u;
    }
    slot_of[u] = slot;
}

// ----------------------------------------------------------- stable radix sort --
// One pass = per-tile digit histogram, exclusive scan of the digit-major
// histogram, stable scatter.  Inside a tile the order is (wave, item, lane),
// i.e. ascending input index, so each pass is stable.

constexpr int kSortItems = 8;
constexpr int kSortTile = kThreads * kSortItems;  // 2048 keys per workgroup
constexpr int kSortWaves = kThreads / 64;
constexpr int kSortWaveSpan = 64 * kSortItems;    // 512 consecutive keys per wave

__global__ __launch_bounds__(kThreads) void sort_hist_kernel(const int *__restrict__ keys, long n,
                                                             int shift, int rbits,
                                                             int *__restrict__ hist, int n_tiles,
                                                             const int *__restrict__ stats) {
    __shared__ int h[256];
    if (stats[TXS_STAT_UNSORTED] == 0) return;  // nothing to sort
    const int R = 1 << rbits;
    h[threadIdx.x] = 0;
    __syncthreads();
    long base = (long)blockIdx.x * kSortTile;
#pragma unroll
    for (int it = 0; it < kSortItems; ++it) {
        long i = base + (long)it * kThreads + threadIdx.x;
        if (i < n) atomicAdd(&h[(keys[i] >> shift) & (R - 1)], 1);
    }
    __syncthreads();
    if ((int)threadIdx.x < R) hist[(long)threadIdx.x * n_tiles + blockIdx.x] = h[threadIdx.x];
}

__global__ __launch_bounds__(kThreads) void sort_scatter_kernel(
    const int *__restrict__ keys_in, const int *__restrict__ vals_in, int *__restrict__ keys_out,
    int *__restrict__ vals_out, long n, int shift, int rbits, const int *__restrict__ hist_scanned,
    int n_tiles, const int *__restrict__ stats) {
    __shared__ int wcount[kSortWaves][256];
    if (stats[TXS_STAT_UNSORTED] == 0) return;  // nothing to sort
    __shared__ int woff[kSortWaves][256];
    const int R = 1 << rbits;
    const int w = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const unsigned long long lanes_below = (1ull << lane) - 1ull;
    for (int k = threadIdx.x; k < kSortWaves * 256; k += kThreads) (&wcount[0][0])[k] = 0;
    __syncthreads();

    const long base = (long)blockIdx.x * kSortTile + (long)w * kSortWaveSpan;
    int key[kSortItems], lrank[kSortItems];
    volatile int *wc = &wcount[w][0];
#pragma unroll
    for (int it = 0; it < kSortItems; ++it) {
        long i = base + (long)it * 64 + lane;
        bool valid = i < n;
        key[it] = valid ? keys_in[i] : 0;
        int digit = (key[it] >> shift) & (R - 1);
        unsigned long long mask = __ballot(valid);
        for (int b = 0; b < rbits; ++b) {
            bool bit = (digit >> b) & 1;
            unsigned long long bal = __ballot(bit);
            mask &= bit ? bal : ~bal;
        }
        int below = __popcll(mask & lanes_below);
        int prev = wc[digit];
        __builtin_amdgcn_wave_barrier();
        if (valid && below == 0) wc[digit] = prev + __popcll(mask);
        __builtin_amdgcn_wave_barrier();
        lrank[it] = prev + below;
    }
    __syncthreads();
    if ((int)threadIdx.x < R) {
        int run = hist_scanned[(long)threadIdx.x * n_tiles + blockIdx.x];
#pragma unroll
        for (int k = 0; k < kSortWaves; ++k) {
            woff[k][threadIdx.x] = run;
            run += wcount[k][threadIdx.x];
        }
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < kSortItems; ++it) {
        long i = base + (long)it * 64 + lane;
        if (i < n) {
            int digit = (key[it] >> shift) & (R - 1);
            long dst = (long)woff[w][digit] + lrank[it];
            if (dst >= 0 && dst < n) {
                keys_out[dst] = key[it];
                vals_out[dst] = vals_in ? vals_in[i] : (int)i;
            }
        }
    }
}

// seg[j] = id | special bit
__global__ void seg_flag_kernel(const int *ids, long n, int U, const int *__restrict__ slot_of,
                                int *seg) {
    long j = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= n) return;
    int u = ids[j] & kIdMask;
    int flag = ((unsigned)u < (unsigned)U && slot_of[u] >= 0) ? kSpecialBit : 0;
    seg[j] = u | flag;
}

// seg by binary search of each position in preSum (largest u with preSum[u] <= j)
__global__ void seg_from_presum_kernel(const int *__restrict__ preSum, long n, int U,
                                       const int *__restrict__ slot_of, int *__restrict__ seg) {
    long j = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= n) return;
    int lo = 0, hi = U;  // invariant: preSum[lo] <= j < preSum[hi]
    while (hi - lo > 1) {
        int mid = (lo + hi) >> 1;
        if ((long)preSum[mid] <= j) lo = mid; else hi = mid;
    }
    int flag = (slot_of[lo] >= 0) ? kSpecialBit : 0;
    seg[j] = lo | flag;
}

int radix_bits(int64_t U) {
    int bits = 1;
    while ((1LL << bits) < U) ++bits;
    return bits;
}

}  // namespace

extern "C" {

int txs_get_presum(const int32_t *unq_inv, int32_t *preSum, int64_t num_total, int64_t num_presum,
                   void *stream) {
    if (!fits_i32(num_total) || !fits_i32(num_presum)) return TXS_ERR_INVALID_ARG;
    if (num_total == 0) return TXS_OK;
    if (!unq_inv || !preSum) return TXS_ERR_INVALID_ARG;
    get_presum_kernel<<<dim3(blocks_for(num_total)), dim3(kThreads), 0, (hipStream_t)stream>>>(
        unq_inv, preSum, num_total, num_presum);
    return status_of(hipGetLastError());
}

int txs_plan_check(const int32_t *unq_inv, int64_t num_total, int64_t num_unq, int32_t *stats,
                   void *stream) {
    if (!fits_i32(num_total) || !fits_i32(num_unq) || !stats) return TXS_ERR_INVALID_ARG;
    if (num_total == 0) return TXS_OK;
    if (!unq_inv) return TXS_ERR_INVALID_ARG;
    plan_check_kernel<<<dim3(blocks_for(num_total)), dim3(kThreads), 0, (hipStream_t)stream>>>(
        unq_inv, num_total, (int)num_unq, stats);
    return status_of(hipGetLastError());
}

int64_t txs_sort_workspace_len(int64_t num_total, int64_t num_unq) {
    const int64_t tiles = (num_total + kSortTile - 1) / kSortTile;
    const int64_t hist = 256 * (tiles > 0 ? tiles : 1);
    (void)num_unq;
    // two ping-pong arrays, the digit-major histogram, and the scan workspace
    return 2 * num_total + hist + scan_tiles(hist + 1) + 17;
}

int txs_plan_sort(const int32_t *unq_inv, int64_t num_total, int64_t num_unq, const int32_t *stats,
                  int32_t *perm, int32_t *keys, int32_t *sort_ws, void *stream) {
    if (!fits_i32(num_total) || !fits_i32(num_unq)) return TXS_ERR_INVALID_ARG;
    if (num_total == 0) return TXS_OK;
    if (!unq_inv || !stats || !perm || !keys || !sort_ws || num_unq <= 0) return TXS_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const long n = num_total;
    const int n_tiles = (int)((n + kSortTile - 1) / kSortTile);
    const long hist_len = 256L * n_tiles;
    int *tmp_keys = sort_ws;
    int *tmp_vals = sort_ws + n;
    int *hist = sort_ws + 2 * n;
    int *scan_ws = hist + hist_len;

    copy_if_sorted_kernel<<<dim3(blocks_for(n)), dim3(kThreads), 0, st>>>(unq_inv, n, stats, keys);
    const int bits = radix_bits(num_unq);
    const int passes = (bits + 7) / 8;
    const int rbits = (bits + passes - 1) / passes;
    const int *kin = unq_inv;
    const int *vin = nullptr;  // identity
    for (int p = 0; p < passes; ++p) {
        const bool to_final = ((passes - 1 - p) % 2) == 0;
        int *kout = to_final ? keys : tmp_keys;
        int *vout = to_final ? perm : tmp_vals;
        const int shift = p * rbits;
        sort_hist_kernel<<<dim3(n_tiles), dim3(kThreads), 0, st>>>(kin, n, shift, rbits, hist, n_tiles,
                                                                  stats);
        const long used = (1L << rbits) * n_tiles;
        if (exclusive_scan(hist, used, hist, used, scan_ws, st) != hipSuccess) return TXS_ERR_LAUNCH;
        sort_scatter_kernel<<<dim3(n_tiles), dim3(kThreads), 0, st>>>(kin, vin, kout, vout, n, shift,
                                                                     rbits, hist, n_tiles, stats);
        kin = kout;
        vin = vout;
    }
    return status_of(hipGetLastError());
}

int txs_plan_presum(const int32_t *sorted_keys, int64_t num_total, int64_t num_unq, int32_t *preSum,
                    void *stream) {
    if (!fits_i32(num_total) || !fits_i32(num_unq) || !preSum) return TXS_ERR_INVALID_ARG;
    if (num_total > 0 && !sorted_keys) return TXS_ERR_INVALID_ARG;
    presum_from_sorted_kernel<<<dim3(blocks_for(num_total + 1)), dim3(kThreads), 0,
                                (hipStream_t)stream>>>(sorted_keys, num_total, (int)num_unq, preSum);
    return status_of(hipGetLastError());
}

int txs_plan_special(const int32_t *preSum, int64_t num_unq, int32_t heavy_threshold,
                     const int64_t *unq_cnts, int32_t *slot_of, int32_t *heavy_ids, int32_t *stats,
                     const int32_t *num_unq_dev, int64_t *cnts_out, void *stream) {
    if (!fits_i32(num_unq) || !preSum || !stats || heavy_threshold < kChunk) return TXS_ERR_INVALID_ARG;
    if (num_unq == 0) return TXS_OK;
    if (!slot_of || !heavy_ids) return TXS_ERR_INVALID_ARG;
    plan_special_kernel<<<dim3(blocks_for(num_unq, kSpecialThreads)), dim3(kSpecialThreads), 0,
                          (hipStream_t)stream>>>(
        preSum, (int)num_unq, heavy_threshold, (const long long *)unq_cnts, slot_of, heavy_ids, stats,
        num_unq_dev, (long long *)cnts_out);
    return status_of(hipGetLastError());
}

int txs_plan_seg_flag(int32_t *keys_to_seg, int64_t num_total, int64_t num_unq,
                      const int32_t *slot_of, void *stream) {
    if (!fits_i32(num_total) || !fits_i32(num_unq)) return TXS_ERR_INVALID_ARG;
    if (num_total == 0) return TXS_OK;
    if (!keys_to_seg || !slot_of) return TXS_ERR_INVALID_ARG;
    seg_flag_kernel<<<dim3(blocks_for(num_total)), dim3(kThreads), 0, (hipStream_t)stream>>>(
        keys_to_seg, num_total, (int)num_unq, slot_of, keys_to_seg);
    return status_of(hipGetLastError());
}

int txs_plan_seg_from_presum(const int32_t *preSum, int64_t num_total, int64_t num_unq,
                             const int32_t *slot_of, int32_t *seg, void *stream) {
    if (!fits_i32(num_total) || !fits_i32(num_unq)) return TXS_ERR_INVALID_ARG;
    if (num_total == 0) return TXS_OK;
    if (!preSum || !slot_of || !seg || num_unq <= 0) return TXS_ERR_INVALID_ARG;
    seg_from_presum_kernel<<<dim3(blocks_for(num_total)), dim3(kThreads), 0, (hipStream_t)stream>>>(
        preSum, num_total, (int)num_unq, slot_of, seg);
    return status_of(hipGetLastError());
}

}  // extern "C"
