// Voxel scatter-reduction kernels for MI355X (gfx950, wave64) and their C ABI.
//
// Design in one paragraph.  Index preparation sorts row ids by voxel id once
// (stable LSD radix sort) and stores, for every sorted position j, the row
// perm[j] and the voxel seg[j].  The forward pass is then a segmented reduction
// over sorted positions: a "lane group" (the lanes that together cover one
// feature row, each lane owning one 128-bit channel vector) walks a fixed-size
// chunk of positions, keeps the running sum / max of the current voxel in
// registers and writes a voxel's output row exactly once when its run of equal
// ids ends.  A run that starts in a chunk is finished by the same lane group
// even if it spills into the next chunk, so ordinary voxels never need an
// atomic.  Only voxels above the heavy threshold are split across lane groups;
// their per-chunk partials are first merged inside the workgroup through LDS,
// then meet in a scratch table through fp32 atomic adds (sum/mean) or a 64-bit
// atomic max on a packed (ordered value | ~row) word (max/argmax), and a small
// finalize kernel turns the table into output rows.  The backward pass is a
// gather over the same sorted positions: the upstream row of a voxel is read
// once per run and every row of the input gradient is written exactly once,
// with no zero-fill pass and no atomics.  The same sort also serves the callers
// on either side of the path: voxel keys from points, the unique/inverse/counts
// triple, and the rank of a point inside its voxel.
//
// Reference behaviour being replaced: torchex/src/scatter/scatter_kernel.cu
// (getPreSum :85-100, scatter_sum :102-129, scatter_max :131-171) and the
// tensor arithmetic of torchex/operator_py/scatter_op.py (:47-50, :69, :74-78,
// :106-111).

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "torchex_scatter.h"

namespace {

// Build-time tuning knobs (defaults are the values measured best on MI355X for
// 512-byte rows; a -D on the hipcc line overrides one for an experiment).
#ifndef TXS_CHUNK
#define TXS_CHUNK 16
#endif
#ifndef TXS_BATCH
#define TXS_BATCH 4
#endif
#ifndef TXS_NT_LOADS
#define TXS_NT_LOADS 1
#endif
#ifndef TXS_NT_STORES
#define TXS_NT_STORES 1
#endif

constexpr int kThreads = 256;        // 4 wavefronts per workgroup
constexpr int kChunk = TXS_CHUNK;    // sorted positions per lane group
constexpr int kBatch = TXS_BATCH;    // rows per load batch of a lane group (two batches in flight)
constexpr int kHeavyDefault = 64;    // voxels above this many rows use the atomic path
constexpr int kSpecialBit = (int)0x80000000;
constexpr int kIdMask = 0x7fffffff;

// ------------------------------------------------------------------ dtypes --

struct F32 {
    using raw = float;
    static __device__ __forceinline__ float to_f(raw x) { return x; }
    static __device__ __forceinline__ raw from_f(float x) { return x; }
    static __device__ __forceinline__ raw lowest() { return -3.402823466e+38f; }
    static __device__ __forceinline__ raw zero() { return 0.0f; }
};
struct F16 {
    using raw = _Float16;
    static __device__ __forceinline__ float to_f(raw x) { return (float)x; }
    static __device__ __forceinline__ raw from_f(float x) { return (_Float16)x; }  // RNE
    static __device__ __forceinline__ raw lowest() { return (_Float16)(-65504.0f); }
    static __device__ __forceinline__ raw zero() { return (_Float16)0.0f; }
};
struct BF16 {
    using raw = unsigned short;
    static __device__ __forceinline__ float to_f(raw x) {
        return __uint_as_float(((unsigned)x) << 16);
    }
    static __device__ __forceinline__ raw from_f(float x) {  // round to nearest even
        unsigned b = __float_as_uint(x);
        if ((b & 0x7fffffffu) > 0x7f800000u) return (raw)((b >> 16) | 0x0040u);
        b += 0x7fffu + ((b >> 16) & 1u);
        return (raw)(b >> 16);
    }
    static __device__ __forceinline__ raw lowest() { return (raw)0xff7f; }
    static __device__ __forceinline__ raw zero() { return (raw)0; }
};

// VEC consecutive elements moved by one lane with a single memory instruction.
template <typename T, int VEC>
struct alignas(sizeof(T) * VEC) Pack {
    T v[VEC];
};

template <typename T, int VEC>
__device__ __forceinline__ Pack<T, VEC> ld(const T *p) {
    return *reinterpret_cast<const Pack<T, VEC> *>(p);
}
template <typename T, int VEC>
__device__ __forceinline__ void st(T *p, const Pack<T, VEC> &x) {
    *reinterpret_cast<Pack<T, VEC> *>(p) = x;
}

// Streaming variants: data touched exactly once (feature rows on the way in,
// input-gradient rows on the way out) is moved with the non-temporal hint so it
// does not evict the index arrays and upstream-gradient rows that are re-read.
template <typename T, int VEC>
struct VecOf {
    typedef T type __attribute__((ext_vector_type(VEC)));
};
template <typename T>
struct VecOf<T, 1> {
    typedef T type;
};
template <typename T, int VEC>
__device__ __forceinline__ Pack<T, VEC> ld_stream(const T *p) {
#if TXS_NT_LOADS
    using V = typename VecOf<T, VEC>::type;
    V v = __builtin_nontemporal_load(reinterpret_cast<const V *>(p));
    Pack<T, VEC> r;
    __builtin_memcpy(&r, &v, sizeof(r));
    return r;
#else
    return ld<T, VEC>(p);
#endif
}
template <typename T, int VEC>
__device__ __forceinline__ void st_stream(T *p, const Pack<T, VEC> &x) {
#if TXS_NT_STORES
    using V = typename VecOf<T, VEC>::type;
    V v;
    __builtin_memcpy(&v, &x, sizeof(v));
    __builtin_nontemporal_store(v, reinterpret_cast<V *>(p));
#else
    st<T, VEC>(p, x);
#endif
}

// Workgroups are handed to the 8 XCDs round-robin.  Tiles are dealt to the XCDs
// in spans of kXcdSpan consecutive tiles so that neighbours (which share voxels
// and upstream-gradient rows) can meet in one L2.  Handing each XCD one long
// contiguous range instead was measured to be much slower on skewed data: bytes
// per position vary along the sorted order, so the XCDs finish at different times.
#ifndef TXS_XCD_SPAN
#define TXS_XCD_SPAN 1
#endif
constexpr int kXcdSpan = TXS_XCD_SPAN;  // gridDim.x is a multiple of 8 * kXcdSpan
__device__ __forceinline__ int xcd_block(int b, int nb) {
    (void)nb;
    if (kXcdSpan == 1) return b;
    const int xcd = b & 7, q = b >> 3;
    return (q / kXcdSpan) * (8 * kXcdSpan) + xcd * kXcdSpan + (q % kXcdSpan);
}

// Monotonic map from non-NaN floats to unsigned ints; -0.0 is folded into +0.0
// first so the two zeros tie, as they do under the reference's float compare.
__device__ __forceinline__ unsigned ordered_bits(float v) {
    unsigned b = __float_as_uint(v + 0.0f);
    return b ^ ((b >> 31) ? 0xffffffffu : 0x80000000u);
}

// -------------------------------------------------------------- small utils --

__global__ void fill_i32_kernel(int *p, long n, int value) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = value;
}

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

__device__ __forceinline__ int wave_inclusive_scan(int x) {
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        int y = __shfl_up(x, d, 64);
        if (lane >= d) x += y;
    }
    return x;
}

// exclusive scan of one int per thread across the 256-thread workgroup;
// *total receives the workgroup sum
__device__ __forceinline__ int block_exclusive_scan(int x, int *total) {
    __shared__ int wsum[kThreads / 64];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    int inc = wave_inclusive_scan(x);
    __syncthreads();  // wsum may still be read by a previous call
    if (lane == 63) wsum[w] = inc;
    __syncthreads();
    int off = 0, tot = 0;
#pragma unroll
    for (int k = 0; k < kThreads / 64; ++k) {
        int s = wsum[k];
        if (k < w) off += s;
        tot += s;
    }
    *total = tot;
    return off + inc - x;
}

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

// in and out may be the same array: a thread reads its items before any write
__global__ __launch_bounds__(kThreads) void scan_apply_kernel(const int *in, long n_in, int *out,
                                                              long n_out, const int *tile_offs) {
    long base = (long)blockIdx.x * kScanTile + (long)threadIdx.x * kScanItems;
    int x[kScanItems];
    int s = 0;
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
        long i = base + k;
        x[k] = (i < n_in) ? in[i] : 0;
        s += x[k];
    }
    int tot;
    int run = block_exclusive_scan(s, &tot) + tile_offs[blockIdx.x];
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
        long i = base + k;
        if (i < n_out) out[i] = run;
        run += x[k];
    }
}

long scan_tiles(long n_out) { return (n_out + kScanTile - 1) / kScanTile; }

hipError_t exclusive_scan(const int *in, long n_in, int *out, long n_out, int *ws,
                          hipStream_t st) {
    if (n_out <= 0) return hipSuccess;
    long tiles = scan_tiles(n_out);
    scan_tile_sums_kernel<<<dim3((unsigned)tiles), dim3(kThreads), 0, st>>>(in, n_in, ws);
    scan_tile_offsets_kernel<<<dim3(1), dim3(kThreads), 0, st>>>(ws, tiles);
    scan_apply_kernel<<<dim3((unsigned)tiles), dim3(kThreads), 0, st>>>(in, n_in, out, n_out, ws);
    return hipGetLastError();
}

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
    __shared__ int s_max[kSpecialThreads / 64], s_empty[kSpecialThreads / 64], s_bad[kSpecialThreads / 64];
    // the voxel count may only be known on the device (unique path): U_arg is then an upper bound
    const int U = num_unq_dev ? min(U_arg, *num_unq_dev) : U_arg;
    const int u = blockIdx.x * blockDim.x + threadIdx.x;
    const bool in = u < U;
    const int c = in ? preSum[u + 1] - preSum[u] : 0;
    const int wmax = wave_max_i32(c);
    const int n_empty = __popcll(__ballot(in && c == 0));
    const bool mismatch = in && unq_cnts && unq_cnts[u] != (long long)c;
    const int any_mismatch = __ballot(mismatch) != 0ull;
    const int w = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) {
        s_max[w] = wmax;
        s_empty[w] = n_empty;
        s_bad[w] = any_mismatch;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int m = 0, e = 0, b = 0;
        for (int k = 0; k < kSpecialThreads / 64; ++k) {
            m = max(m, s_max[k]);
            e += s_empty[k];
            b |= s_bad[k];
        }
        if (m > 0) atomicMax(&stats[TXS_STAT_MAX_CNT], m);
        if (e) atomicAdd(&stats[TXS_STAT_NUM_EMPTY], e);
        if (b) stats[TXS_STAT_COUNT_MISMATCH] = 1;
    }
    if (!in) return;
    if (cnts_out) cnts_out[u] = (long long)c;
    int slot = -1;
    if (c > heavy_threshold || c == 0) {
        slot = atomicAdd(&stats[TXS_STAT_NUM_SPECIAL], 1);
        if (slot < U) heavy_ids[slot] = u;
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
    boxes[b] = bx;
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

// hits per (box, tile); grid (tiles, boxes)
__global__ __launch_bounds__(kThreads) void dpp_count_kernel(const float *__restrict__ pts, int P,
                                                             const DppBox *__restrict__ boxes,
                                                             int n_tiles, int *__restrict__ counts) {
    __shared__ int wsum[kThreads / 64];
    const int p = blockIdx.x * kThreads + threadIdx.x;
    const DppBox bx = boxes[blockIdx.y];
    bool hit = false;
    if (p < P) {
        float lx, ly;
        hit = dpp_test(bx, pts[(size_t)p * 3], pts[(size_t)p * 3 + 1], pts[(size_t)p * 3 + 2], lx, ly) > 0;
    }
    const int c = __popcll(__ballot(hit));
    if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = c;
    __syncthreads();
    if (threadIdx.x == 0) {
        int t = 0;
        for (int k = 0; k < kThreads / 64; ++k) t += wsum[k];
        counts[(size_t)blockIdx.y * n_tiles + blockIdx.x] = t;
    }
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

// second pass: same test, rank of the hit inside its box, compact write
__global__ __launch_bounds__(kThreads) void dpp_write_kernel(
    const float *__restrict__ pts, int P, const DppBox *__restrict__ boxes, int n_tiles,
    const int *__restrict__ scanned, const int *__restrict__ box_base, int cap, int max_all,
    long long *__restrict__ out_pts_idx, long long *__restrict__ out_roi_idx,
    float *__restrict__ out_feats) {
#pragma clang fp contract(off)
    __shared__ int wsum[kThreads / 64];
    const int b = blockIdx.y;
    const int p = blockIdx.x * kThreads + threadIdx.x;
    const DppBox bx = boxes[b];
    int flag = 0;
    float x = 0.f, y = 0.f, z = 0.f, lx = 0.f, ly = 0.f;
    if (p < P) {
        x = pts[(size_t)p * 3];
        y = pts[(size_t)p * 3 + 1];
        z = pts[(size_t)p * 3 + 2];
        flag = dpp_test(bx, x, y, z, lx, ly);
    }
    const unsigned long long m = __ballot(flag > 0);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    if (lane == 0) wsum[w] = __popcll(m);
    __syncthreads();
    if (flag == 0) return;
    int rank = __popcll(m & ((1ull << lane) - 1ull));
    for (int k = 0; k < w; ++k) rank += wsum[k];
    rank += scanned[(size_t)b * n_tiles + blockIdx.x] - scanned[(size_t)b * n_tiles];
    if (rank >= cap) return;
    const long pos = (long)box_base[b] + rank;
    if (pos >= max_all) return;
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

// ------------------------------------------------------------- grid hash --
// Open-addressing table of (key, value) int32 pairs with the reference's probe
// sequence (torchex/src/utils/functions.cuh:30-64, double hashing with an odd
// step over a power-of-two table).  A slot is one 64-bit word (key in the low
// half, value in the high half, as the reference's [size, 2] int32 tensor lays
// them out) claimed with a single 64-bit compare-and-swap, so key and value
// appear together.

__device__ __forceinline__ int grid_hash_slot(long long key, int probe_i, int table_size) {
    return (int)((key % table_size + probe_i * (key * 2 + 1)) % table_size);
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
    for (int t = 0; t < table_size; ++t) {
        const int s = grid_hash_slot(key, t, table_size);
        if ((unsigned)s >= (unsigned)table_size) break;  // negative key
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
    for (int t = 0; t < table_size; ++t) {
        const int s = grid_hash_slot(key, t, table_size);
        if ((unsigned)s >= (unsigned)table_size) break;
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

// ----------------------------------------------------------------- forward --
//
// One workgroup owns a tile of G * kChunk consecutive sorted positions, where
// G = 256 / (lanes per row) lane groups each own kChunk of them.  The tile's seg
// and perm entries (plus one entry before and kMargin after) are staged in LDS
// by one coalesced load, so the row loads that follow never wait on an index
// load, and a lane group can look across its chunk borders for free.  Row loads
// are double-buffered: the next batch is in flight while the current one is
// reduced.

constexpr int kMargin = 64;           // staged entries past the tile's end
constexpr int kNoSeg = 0x7fffffff;    // never a valid seg value

// ---- the reference's winner among equal maxima (op TXS_MAX_REFTIE) ----------
// scatter_kernel.cu:131-171 runs B = clamp(up_2n(max_cnt), 32, 1024) threads per
// voxel; thread tid keeps the LAST maximal row of its residue class (rel % B ==
// tid, '>=' at :148) and the shuffle trees (:41-83, strict '>') let the
// candidate with the smallest bit-reversed lane index, then the smallest
// bit-reversed warp index, survive.  A row at offset `rel` inside its voxel
// therefore competes with the key below (smaller wins).
constexpr int kIterBits = 21;
constexpr unsigned kIterMask = (1u << kIterBits) - 1u;
__device__ __forceinline__ unsigned ref_prio(unsigned tid, int wbits) {
    const unsigned lane = __brev(tid & 31u) >> 27;
    const unsigned warp = wbits > 0 ? (__brev(tid >> 5) >> (32 - wbits)) : 0u;
    return (warp << 5) | lane;
}
__device__ __forceinline__ int ref_key(int rel, int blog2) {
    const unsigned tid = (unsigned)rel & ((1u << blog2) - 1u);
    const unsigned iter = ((unsigned)rel >> blog2) & kIterMask;
    return (int)((ref_prio(tid, blog2 - 5) << kIterBits) | (kIterMask - iter));
}
__device__ __forceinline__ int ref_rel(int key, int blog2) {  // inverse of ref_key
    const unsigned iter = kIterMask - ((unsigned)key & kIterMask);
    return (int)((iter << blog2) | ref_prio((unsigned)key >> kIterBits, blog2 - 5));
}

template <class TR, int VEC, int OP>
__global__ __launch_bounds__(kThreads) void scatter_fwd_kernel(
    const typename TR::raw *__restrict__ feats, const int *__restrict__ perm,
    const int *__restrict__ seg, const int *__restrict__ slot_of,
    typename TR::raw *__restrict__ out, int *__restrict__ arg,
    unsigned long long *__restrict__ scratch, const int *__restrict__ preSum, int N, int C, int U,
    int lpr_log2, int ref_log2) {
    using raw = typename TR::raw;
    constexpr bool kMax = OP == TXS_MAX || OP == TXS_MAX_REFTIE;
    constexpr bool kRef = OP == TXS_MAX_REFTIE;  // idx[] then holds ref_key, not a row
    extern __shared__ int lds[];
    const int G = kThreads >> lpr_log2;
    const int T = G * kChunk;
    const int n_seg_s = T + kMargin + 1;  // positions t0-1 .. t0+T+kMargin-1
    int *seg_s = lds;
    int *perm_s = lds + n_seg_s;          // positions t0 .. t0+T+kMargin-1
    // Partials of heavy voxels: two slots per lane group (a chunk can touch at
    // most two heavy runs, one at each end), combined across the workgroup
    // before anything goes to the global scratch table.
    using SlotT = typename std::conditional<kMax, unsigned long long, float>::type;
    int *slot_id = perm_s + (n_seg_s - 1);
    SlotT *slot_val = reinterpret_cast<SlotT *>(lds + ((2 * n_seg_s - 1 + 2 * G + 1) & ~1));
    const int W = VEC << lpr_log2;        // elements per slot
    const long t0l = (long)xcd_block(blockIdx.x, gridDim.x) * T;
    if (t0l >= N) return;  // uniform for the workgroup
    const int t0 = (int)t0l;
    bool saw_heavy = false;
    for (int e = threadIdx.x; e < n_seg_s; e += kThreads) {
        const long p = (long)t0 - 1 + e;
        const bool in = p >= 0 && p < N;
        const int sv = in ? seg[p] : kNoSeg;
        seg_s[e] = sv;
        saw_heavy |= (sv < 0) && e >= 1 && e <= T;  // special bit on a position of this tile
        if (e >= 1) perm_s[e - 1] = in ? (perm ? perm[p] : (int)p) : -1;
    }
    for (int e = threadIdx.x; e < 2 * G; e += kThreads) slot_id[e] = -1;
    // one barrier publishes the staged indices and tells the whole workgroup
    // whether the tile touches a heavy voxel (only then is there a merge phase)
    const bool tile_has_heavy = __syncthreads_or(saw_heavy);

    const int gi = (int)threadIdx.x >> lpr_log2;
    const int lane_in = (int)threadIdx.x & ((1 << lpr_log2) - 1);
    const int col = ((int)blockIdx.y << lpr_log2 | lane_in) * VEC;
    int n_heavy = 0;  // heavy partials this lane group has parked in LDS

    auto reduce_chunk = [&]() {
    if (col >= C) return;
    // l indexes seg_s (position t0 - 1 + l); entries past the staged range are
    // fetched from global memory (only an ordinary run longer than kMargin that
    // crosses the tile's end gets there)
    auto seg_at = [&](int l) -> int {
        if (l < n_seg_s) return seg_s[l];
        const long p = (long)t0 - 1 + l;
        return p < N ? seg[p] : kNoSeg;
    };
    auto row_at = [&](int l) -> int {
        if (l < n_seg_s) return perm_s[l - 1];
        const long p = (long)t0 - 1 + l;
        return p < N ? (perm ? perm[p] : (int)p) : -1;
    };

    // Range [la, lb) this lane group reduces: its chunk, minus the tail of an
    // ordinary run that began in an earlier chunk, plus the tail of an ordinary
    // run that begins here and ends later.
    int la = gi * kChunk + 1;
    const int lend = min(la + kChunk, N - t0 + 1);
    if (la >= lend) return;
    {
        const int s0 = seg_s[la];
        if (s0 >= 0 && seg_s[la - 1] == s0) {
            do ++la; while (la < lend && seg_s[la] == s0);
            if (la >= lend) return;
        }
    }
    int lb = lend;
    {
        const int sl = seg_s[lend - 1];
        if (sl >= 0)
            while (seg_at(lb) == sl) ++lb;  // ends at the latest at N (kNoSeg)
    }
    const int lb_fast = min(lb, n_seg_s);  // end of the part whose ids are staged in LDS

    // Start value of a running max: -inf, or in reference-tie mode the
    // reference's own -FLT_MAX (scatter_kernel.cu:139), which -inf never beats.
    const float acc0 = kRef ? TR::to_f(TR::lowest()) : (kMax ? -__builtin_inff() : 0.0f);
    // offset of position l inside its voxel, for the reference's tie key; an
    // ordinary run always starts inside the range, a heavy one may not
    auto rel_of_run_start = [&](int sg, int l) -> int {
        if (!kRef || sg >= 0) return 0;
        const int u = sg & kIdMask;
        return ((unsigned)u < (unsigned)U) ? (t0 - 1 + l) - preSum[u] : 0;
    };
    float acc[VEC];
    int idx[VEC];
    int cur = seg_s[la];
    int run_l0 = la;
    int rel0 = rel_of_run_start(cur, la);
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
        acc[k] = acc0;
        idx[k] = -1;
    }

    // Emit the finished run [run_l0, run_end) of voxel `cur`.
    auto flush = [&](int run_end) {
        const int u = cur & kIdMask;
        if ((unsigned)u >= (unsigned)U) return;
        if (kMax && !kRef) {
            bool missing = false;
#pragma unroll
            for (int k = 0; k < VEC; ++k) missing |= idx[k] < 0;
            if (__builtin_expect(missing, 0)) {
                // No value above -inf was seen in some channel: the run holds
                // only -inf and NaN there.  The first -inf row wins.
                for (int p = run_l0; p < run_end; ++p) {
                    const int row = row_at(p);
                    if ((unsigned)row >= (unsigned)N) continue;
                    Pack<raw, VEC> x = ld<raw, VEC>(feats + (size_t)row * C + col);
#pragma unroll
                    for (int k = 0; k < VEC; ++k)
                        if (idx[k] < 0 && TR::to_f(x.v[k]) == -__builtin_inff()) idx[k] = row;
                }
            }
        }
        if (cur >= 0) {  // ordinary voxel: the whole run was reduced here
            const size_t o = (size_t)u * C + col;
            Pack<raw, VEC> r;
            if (OP == TXS_SUM) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) r.v[k] = TR::from_f(acc[k]);
            } else if (OP == TXS_MEAN) {
                const float d = (float)(run_end - run_l0);
#pragma unroll
                for (int k = 0; k < VEC; ++k) r.v[k] = TR::from_f(acc[k] / d);
            } else {
                Pack<int, VEC> ai;
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    r.v[k] = idx[k] >= 0 ? TR::from_f(acc[k]) : TR::lowest();
                    ai.v[k] = idx[k];
                    if (kRef && idx[k] >= 0) ai.v[k] = row_at(run_l0 + ref_rel(idx[k], ref_log2) - rel0);
                }
                st_stream<int, VEC>(arg + o, ai);
            }
            st_stream<raw, VEC>(out + o, r);
        } else if (n_heavy < 2) {  // heavy voxel: park this chunk's partial in LDS
            const int sidx = 2 * gi + n_heavy;
            ++n_heavy;
            if (lane_in == 0) slot_id[sidx] = u;
            SlotT *sv = slot_val + (size_t)sidx * W + lane_in * VEC;
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                if constexpr (kMax) {
                    sv[k] = idx[k] >= 0 ? (((unsigned long long)ordered_bits(acc[k]) << 32) |
                                           (unsigned long long)(0xffffffffu - (unsigned)idx[k]))
                                        : 0ull;
                } else {
                    sv[k] = acc[k];
                }
            }
        }
        // (a third heavy partial in one chunk cannot occur: a heavy run is longer
        // than a chunk, so a chunk touches at most one at each end)
    };

    // Fold one loaded row (position l, voxel sg) into the running reduction.  With
    // kGate the row counts only when `valid` (a slot past the range in the last
    // batch of a chunk); the loaded registers are consumed on a straight-line path
    // either way so the compiler can count outstanding loads exactly.
    auto add_row = [&](auto gate, const Pack<raw, VEC> &v, int sg, int row, int l, bool valid) {
        constexpr bool kGate = decltype(gate)::value;
        if ((!kGate || valid) && sg != cur) {
            flush(l);
            cur = sg;
            run_l0 = l;
            rel0 = rel_of_run_start(sg, l);
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                acc[k] = acc0;
                idx[k] = -1;
            }
        }
        const int tag = kRef ? ref_key(rel0 + (l - run_l0), ref_log2) : row;
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            const float x = TR::to_f(v.v[k]);
            if (kMax) {
                // strict '>': the first row wins ties, NaN never wins.  Reference-tie
                // mode also takes an equal value whose key is smaller.
                bool take = x > acc[k];
                if (kRef) take |= (x == acc[k]) && ((unsigned)tag < (unsigned)idx[k]);
                if (kGate) take &= valid;
                acc[k] = take ? x : acc[k];
                idx[k] = take ? tag : idx[k];
            } else {
                acc[k] += (!kGate || valid) ? x : 0.0f;
            }
        }
    };

    // Row r of the feature matrix at this lane's columns: one 64-bit multiply-add.
    // A row index outside the matrix (only a corrupt plan has one) is clamped.
    const char *lane_base = reinterpret_cast<const char *>(feats) + (size_t)col * sizeof(raw);
    const unsigned row_bytes = (unsigned)C * (unsigned)sizeof(raw);
    const unsigned last_row = (unsigned)(N - 1);
    auto row_ptr = [&](int r) -> const raw * {
        const unsigned rc = min((unsigned)r, last_row);
        return reinterpret_cast<const raw *>(lane_base + (unsigned long long)rc * row_bytes);
    };

    // Every slot of a batch issues a load (slots past the range re-load the
    // range's last row, a cache hit) so that no load sits under a branch.
    struct Batch {
        int segs[kBatch], rows[kBatch];
        Pack<raw, VEC> v[kBatch];
    };
    auto issue = [&](Batch &bt, int l) {
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            const int lc = min(l + i, lb_fast - 1);
            bt.segs[i] = seg_s[lc];
            bt.rows[i] = perm_s[lc - 1];
            bt.v[i] = ld_stream<raw, VEC>(row_ptr(bt.rows[i]));
        }
    };
    // A batch that lies wholly inside the range needs no per-row gate; only the
    // last batch of a chunk can hold slots past the range.
    auto consume_full = [&](const Batch &bt, int l) {
#pragma unroll
        for (int i = 0; i < kBatch; ++i)
            add_row(std::false_type{}, bt.v[i], bt.segs[i], bt.rows[i], l + i, true);
    };
    auto consume_last = [&](const Batch &bt, int l) {
#pragma unroll
        for (int i = 0; i < kBatch; ++i)
            add_row(std::true_type{}, bt.v[i], bt.segs[i], bt.rows[i], l + i, l + i < lb_fast);
    };

    // Positions staged in LDS go through the double-buffered loop; the rare rest
    // (an ordinary run longer than kMargin crossing the tile's end) is walked
    // one row at a time with its ids fetched from global memory.
    // Each prefetch is unconditional on its path, so the count of loads in
    // flight is known at every use: a batch is reduced while the next one is
    // still arriving.
    Batch b0, b1;
    issue(b0, la);
    for (int l = la;;) {
        int ln = l + kBatch;
        if (ln >= lb_fast) {
            consume_last(b0, l);
            break;
        }
        issue(b1, ln);
        consume_full(b0, l);
        l = ln;
        ln = l + kBatch;
        if (ln >= lb_fast) {
            consume_last(b1, l);
            break;
        }
        issue(b0, ln);
        consume_full(b1, l);
        l = ln;
    }
    for (int l = lb_fast; l < lb; ++l) {
        const int r = row_at(l);
        if ((unsigned)r >= (unsigned)N) continue;
        add_row(std::false_type{}, ld_stream<raw, VEC>(row_ptr(r)), seg_at(l), r, l, true);
    }
    flush(lb);
    };  // reduce_chunk
    reduce_chunk();

    // Workgroup-level merge of the parked partials.  The used slots that carry
    // the same voxel id form one range (a heavy run is contiguous in sorted
    // order, so only unused slots can sit between them).  All 256 threads take
    // part: (A) mark the first slot of every range, (B) fold every other slot
    // into its range's first slot with LDS atomics, (C) send each range total to
    // the global table with one atomic per element.  Tiles without a heavy voxel
    // skip all of this and its barriers.
    if (!tile_has_heavy) return;
    __shared__ unsigned long long start_mask[(2 * kThreads) / 64];
    const int S = 2 * G;                       // slots in this workgroup
    const int w_log2 = lpr_log2 + (VEC == 8 ? 3 : VEC == 4 ? 2 : VEC == 2 ? 1 : 0);  // log2(W)
    __syncthreads();
    for (int base = 0; base < S; base += kThreads) {
        const int sl = base + (int)threadIdx.x;
        bool first = false;
        if (sl < S) {
            const int id = slot_id[sl];
            if (id >= 0) {
                int prev = sl - 1;
                while (prev >= 0 && slot_id[prev] < 0) --prev;
                first = prev < 0 || slot_id[prev] != id;
            }
        }
        const unsigned long long m = __ballot(first);
        if ((threadIdx.x & 63) == 0) start_mask[(base + (int)threadIdx.x) >> 6] = m;
    }
    __syncthreads();
    // first slot of the range that slot sl belongs to: nearest marked slot at or below sl
    auto range_start = [&](int sl) -> int {
        int wd = sl >> 6;
        unsigned long long m = start_mask[wd] & (~0ull >> (63 - (sl & 63)));
        while (m == 0ull && wd > 0) m = start_mask[--wd];
        return m ? (wd << 6) + 63 - __builtin_clzll(m) : sl;
    };
    for (int i = threadIdx.x; i < (S << w_log2); i += kThreads) {
        const int sl = i >> w_log2, e = i & (W - 1);
        if (slot_id[sl] < 0) continue;
        const int head = range_start(sl);
        if (head == sl) continue;
        const SlotT x = slot_val[i];
        SlotT *dst = slot_val + ((size_t)head << w_log2) + e;
        if constexpr (kMax) {
            if (x != 0ull) atomicMax(dst, x);
        } else {
            __hip_atomic_fetch_add(dst, x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < (S << w_log2); i += kThreads) {
        const int sl = i >> w_log2, e = i & (W - 1);
        if (!((start_mask[sl >> 6] >> (sl & 63)) & 1ull)) continue;
        const int c = (((int)blockIdx.y << lpr_log2) * VEC) + e;
        if (c >= C) continue;
        const int id = slot_id[sl];
        const int slot = ((unsigned)id < (unsigned)U) ? slot_of[id] : -1;
        if (slot < 0) continue;
        const SlotT tot = slot_val[i];
        const size_t o = (size_t)slot * C + c;
        if constexpr (kMax) {
            if (tot != 0ull) atomicMax(scratch + o, tot);
        } else {
            unsafeAtomicAdd(reinterpret_cast<float *>(scratch) + o, tot);
        }
    }
}

// Turn the scratch table of the special voxels into output rows and clear it.
template <class TR, int OP>
__global__ void scatter_finalize_kernel(const typename TR::raw *__restrict__ feats,
                                        const int *__restrict__ preSum,
                                        const int *__restrict__ heavy_ids,
                                        unsigned long long *__restrict__ scratch,
                                        typename TR::raw *__restrict__ out,
                                        int *__restrict__ arg, int n_special, int N, int C, int U,
                                        const int *__restrict__ perm, int ref_log2) {
    const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= (long)n_special * C) return;
    const int s = (int)(t / C), c = (int)(t - (long)s * C);
    const int u = heavy_ids[s];
    if ((unsigned)u >= (unsigned)U) return;
    const size_t o = (size_t)u * C + c;
    if (OP == TXS_MAX || OP == TXS_MAX_REFTIE) {
        const unsigned long long key = scratch[t];
        scratch[t] = 0ull;
        unsigned row = 0xffffffffu - (unsigned)(key & 0xffffffffull);
        if (OP == TXS_MAX_REFTIE && key != 0ull) {  // the low word holds a tie key, not a row
            const long pos = (long)preSum[u] + ref_rel((int)row, ref_log2);
            row = (pos >= 0 && pos < N) ? (unsigned)(perm ? perm[pos] : (int)pos) : 0xffffffffu;
        }
        if (key == 0ull || row >= (unsigned)N) {
            out[o] = TR::lowest();
            arg[o] = -1;
        } else {
            out[o] = feats[(size_t)row * C + c];  // exact bits of the winner
            arg[o] = (int)row;
        }
    } else {
        float *fs = reinterpret_cast<float *>(scratch);
        float s32 = fs[t];
        fs[t] = 0.0f;
        if (OP == TXS_MEAN) s32 = s32 / (float)(preSum[u + 1] - preSum[u]);
        out[o] = TR::from_f(s32);
    }
}

// ---------------------------------------------------------------- backward --
//
// Same tiling and LDS staging as the forward pass, no border logic: position j
// writes row perm[j] of the input gradient from the upstream row of voxel
// seg[j].  The upstream row (and arg row) is fetched once per run of equal ids
// inside a chunk, and the fetches of the next batch are in flight while the
// current batch is stored.

template <class TR, int VEC, int OP>
__global__ __launch_bounds__(kThreads) void scatter_bwd_kernel(
    const typename TR::raw *__restrict__ g, const int *__restrict__ arg,
    const int *__restrict__ perm, const int *__restrict__ seg, const int *__restrict__ preSum,
    typename TR::raw *__restrict__ gin, int N, int C, int U, int lpr_log2) {
    using raw = typename TR::raw;
    extern __shared__ int lds[];
    const int G = kThreads >> lpr_log2;
    const int T = G * kChunk;
    int *seg_s = lds;
    int *perm_s = lds + T;
    const long t0l = (long)xcd_block(blockIdx.x, gridDim.x) * T;
    if (t0l >= N) return;  // uniform for the workgroup
    const int t0 = (int)t0l;
    for (int e = threadIdx.x; e < T; e += kThreads) {
        const long p = (long)t0 + e;
        const bool in = p < N;
        const int u = in ? (seg[p] & kIdMask) : -1;
        const int r = in ? (perm ? perm[p] : (int)p) : -1;
        const bool good = (unsigned)u < (unsigned)U && (unsigned)r < (unsigned)N;
        seg_s[e] = good ? u : -1;
        perm_s[e] = good ? r : -1;
    }
    __syncthreads();

    const int col = ((int)blockIdx.y << lpr_log2 | ((int)threadIdx.x & ((1 << lpr_log2) - 1))) * VEC;
    if (col >= C) return;
    const int la = ((int)threadIdx.x >> lpr_log2) * kChunk;
    const int lb = min(la + kChunk, N - t0);
    if (la >= lb) return;

    // A batch keeps the fetched upstream rows and two bit masks; row ids are read
    // again from LDS when the batch is stored.  The upstream row (and arg row) is
    // fetched only where the voxel changes.
    struct Batch {
        Pack<raw, VEC> gv[kBatch];
        Pack<int, VEC> av[kBatch];
        int cnt[kBatch];
        unsigned valid, need;
    };
    auto issue = [&](Batch &bt, int l) {
        bt.valid = 0u;
        bt.need = 0u;
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            const int ll = l + i;
            if (ll >= lb) continue;
            const int u = seg_s[ll];
            if (perm_s[ll] < 0) continue;
            bt.valid |= 1u << i;
            // first position of the chunk, or the voxel changes here
            if (ll == la || seg_s[ll - 1] != u) {
                bt.need |= 1u << i;
                const size_t o = (size_t)u * C + col;
                // upstream rows are re-read by the neighbouring chunk when a run
                // straddles it (keep them cached); an arg row is consumed here and
                // nowhere else (stream it)
                bt.gv[i] = ld<raw, VEC>(g + o);
                if (OP == TXS_MAX) bt.av[i] = ld_stream<int, VEC>(arg + o);
                if (OP == TXS_MEAN) bt.cnt[i] = preSum[u + 1] - preSum[u];
            }
        }
    };
    Pack<raw, VEC> q;   // (scaled) upstream row of the current voxel
    Pack<int, VEC> aq;  // its arg row
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
        q.v[k] = TR::zero();
        aq.v[k] = -1;
    }
    auto consume = [&](const Batch &bt, int l) {
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            if (!(bt.valid & (1u << i))) continue;
            if (bt.need & (1u << i)) {
                if (OP == TXS_MEAN) {  // one division per run, not per row
                    const float d = (float)bt.cnt[i];
#pragma unroll
                    for (int k = 0; k < VEC; ++k) q.v[k] = TR::from_f(TR::to_f(bt.gv[i].v[k]) / d);
                } else {
                    q = bt.gv[i];
                }
                if (OP == TXS_MAX) aq = bt.av[i];
            }
            const int row = perm_s[l + i];
            Pack<raw, VEC> r = q;
            if (OP == TXS_MAX) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) r.v[k] = (aq.v[k] == row) ? q.v[k] : TR::zero();
            }
            st_stream<raw, VEC>(gin + (size_t)row * C + col, r);
        }
    };

    Batch b0, b1;
    issue(b0, la);
    for (int l = la;;) {
        int ln = l + kBatch;
        if (ln < lb) issue(b1, ln);
        consume(b0, l);
        if (ln >= lb) break;
        l = ln;
        ln = l + kBatch;
        if (ln < lb) issue(b0, ln);
        consume(b1, l);
        if (ln >= lb) break;
        l = ln;
    }
}

// ------------------------------------------------------------------ launch --

struct Geometry {
    int vec_bytes;  // bytes one lane moves per row
    int lpr_log2;   // log2(lanes that cover one row slice)
    int ytiles;     // column tiles when a row is wider than 64 lanes
    unsigned lds_fwd_idx, lds_slots, lds_bwd;  // dynamic LDS: fwd index part (bytes), fwd slot elements, bwd bytes
    dim3 grid;
};

bool aligned_to(const void *p, int bytes) { return p == nullptr || ((uintptr_t)p % (uintptr_t)bytes) == 0; }

Geometry make_geometry(long N, long C, int elem, const void *p0, const void *p1, const void *p2,
                       bool arg_used, const void *parg) {
    Geometry g;
    int vb = 16;
    while (vb > elem) {
        int vec = vb / elem;
        bool ok = (C * elem) % vb == 0 && aligned_to(p0, vb) && aligned_to(p1, vb) && aligned_to(p2, vb);
        if (arg_used) ok = ok && aligned_to(parg, vec * 4);
        if (ok) break;
        vb >>= 1;
    }
    g.vec_bytes = vb;
    const long vec = vb / elem;
    const long lanes = (C + vec - 1) / vec;
    int l2 = 0;
    while ((1L << l2) < lanes && l2 < 6) ++l2;
    g.lpr_log2 = l2;
    g.ytiles = (int)((lanes + (1L << l2) - 1) >> l2);
    const long tile = (long)(kThreads >> l2) * kChunk;  // sorted positions per workgroup
    long blocks = (N + tile - 1) / tile;
    blocks = (blocks + 8 * kXcdSpan - 1) / (8 * kXcdSpan) * (8 * kXcdSpan);
    g.lds_fwd_idx = (unsigned)((((2 * (tile + kMargin) + 1) + 2 * (kThreads >> l2) + 1) & ~1L) * sizeof(int));
    g.lds_slots = (unsigned)(2 * kThreads * vec);
    g.lds_bwd = (unsigned)(2 * tile * sizeof(int));
    g.grid = dim3((unsigned)blocks, (unsigned)g.ytiles, 1);
    return g;
}

template <class TR, int VEC>
hipError_t launch_fwd_op(int op, const Geometry &geo, hipStream_t st, const void *feats,
                         const int *perm, const int *seg, const int *preSum, const int *slot_of,
                         void *out, int *arg, void *scratch, int N, int C, int U, int ref_log2) {
    using raw = typename TR::raw;
    auto f = (const raw *)feats;
    auto o = (raw *)out;
    auto s = (unsigned long long *)scratch;
    dim3 blk(kThreads);
    const unsigned lds4 = geo.lds_fwd_idx + 4 * geo.lds_slots, lds8 = geo.lds_fwd_idx + 8 * geo.lds_slots;
    switch (op) {
        case TXS_SUM:
            scatter_fwd_kernel<TR, VEC, TXS_SUM><<<geo.grid, blk, lds4, st>>>(
                f, perm, seg, slot_of, o, arg, s, preSum, N, C, U, geo.lpr_log2, ref_log2);
            break;
        case TXS_MEAN:
            scatter_fwd_kernel<TR, VEC, TXS_MEAN><<<geo.grid, blk, lds4, st>>>(
                f, perm, seg, slot_of, o, arg, s, preSum, N, C, U, geo.lpr_log2, ref_log2);
            break;
        case TXS_MAX_REFTIE:
            scatter_fwd_kernel<TR, VEC, TXS_MAX_REFTIE><<<geo.grid, blk, lds8, st>>>(
                f, perm, seg, slot_of, o, arg, s, preSum, N, C, U, geo.lpr_log2, ref_log2);
            break;
        default:
            scatter_fwd_kernel<TR, VEC, TXS_MAX><<<geo.grid, blk, lds8, st>>>(
                f, perm, seg, slot_of, o, arg, s, preSum, N, C, U, geo.lpr_log2, ref_log2);
            break;
    }
    return hipGetLastError();
}

template <class TR>
hipError_t launch_fwd(int op, const Geometry &geo, hipStream_t st, const void *feats,
                      const int *perm, const int *seg, const int *preSum, const int *slot_of,
                      void *out, int *arg, void *scratch, int N, int C, int U, int ref_log2) {
    constexpr int e = (int)sizeof(typename TR::raw);
#define TXS_FWD(VB)                                                                              \
    if (geo.vec_bytes == VB)                                                                     \
        return launch_fwd_op<TR, (VB) / e>(op, geo, st, feats, perm, seg, preSum, slot_of, out,  \
                                           arg, scratch, N, C, U, ref_log2);
    TXS_FWD(16)
    TXS_FWD(8)
    TXS_FWD(4)
    if constexpr (e == 2) {
        TXS_FWD(2)
    }
#undef TXS_FWD
    return hipErrorInvalidValue;
}

template <class TR>
hipError_t launch_finalize(int op, hipStream_t st, const void *feats, const int *preSum,
                           const int *heavy_ids, void *scratch, void *out, int *arg,
                           long n_special, int N, int C, int U, const int *perm, int ref_log2) {
    using raw = typename TR::raw;
    const long total = n_special * C;
    if (total <= 0) return hipSuccess;
    dim3 grid((unsigned)((total + kThreads - 1) / kThreads)), blk(kThreads);
    auto f = (const raw *)feats;
    auto o = (raw *)out;
    auto s = (unsigned long long *)scratch;
    switch (op) {
        case TXS_SUM:
            scatter_finalize_kernel<TR, TXS_SUM><<<grid, blk, 0, st>>>(f, preSum, heavy_ids, s, o, arg,
                                                                      (int)n_special, N, C, U, perm, ref_log2);
            break;
        case TXS_MEAN:
            scatter_finalize_kernel<TR, TXS_MEAN><<<grid, blk, 0, st>>>(f, preSum, heavy_ids, s, o, arg,
                                                                       (int)n_special, N, C, U, perm, ref_log2);
            break;
        case TXS_MAX_REFTIE:
            scatter_finalize_kernel<TR, TXS_MAX_REFTIE><<<grid, blk, 0, st>>>(
                f, preSum, heavy_ids, s, o, arg, (int)n_special, N, C, U, perm, ref_log2);
            break;
        default:
            scatter_finalize_kernel<TR, TXS_MAX><<<grid, blk, 0, st>>>(f, preSum, heavy_ids, s, o, arg,
                                                                      (int)n_special, N, C, U, perm, ref_log2);
            break;
    }
    return hipGetLastError();
}

template <class TR, int VEC>
hipError_t launch_bwd_op(int op, const Geometry &geo, hipStream_t st, const void *g, const int *arg,
                         const int *perm, const int *seg, const int *preSum, void *gin, int N, int C,
                         int U) {
    using raw = typename TR::raw;
    auto gi = (const raw *)g;
    auto go = (raw *)gin;
    dim3 blk(kThreads);
    switch (op) {
        case TXS_SUM:
            scatter_bwd_kernel<TR, VEC, TXS_SUM><<<geo.grid, blk, geo.lds_bwd, st>>>(
                gi, arg, perm, seg, preSum, go, N, C, U, geo.lpr_log2);
            break;
        case TXS_MEAN:
            scatter_bwd_kernel<TR, VEC, TXS_MEAN><<<geo.grid, blk, geo.lds_bwd, st>>>(
                gi, arg, perm, seg, preSum, go, N, C, U, geo.lpr_log2);
            break;
        default:
            scatter_bwd_kernel<TR, VEC, TXS_MAX><<<geo.grid, blk, geo.lds_bwd, st>>>(
                gi, arg, perm, seg, preSum, go, N, C, U, geo.lpr_log2);
            break;
    }
    return hipGetLastError();
}

template <class TR>
hipError_t launch_bwd(int op, const Geometry &geo, hipStream_t st, const void *g, const int *arg,
                      const int *perm, const int *seg, const int *preSum, void *gin, int N, int C,
                      int U) {
    constexpr int e = (int)sizeof(typename TR::raw);
#define TXS_BWD(VB)                                                                               \
    if (geo.vec_bytes == VB)                                                                      \
        return launch_bwd_op<TR, (VB) / e>(op, geo, st, g, arg, perm, seg, preSum, gin, N, C, U);
    TXS_BWD(16)
    TXS_BWD(8)
    TXS_BWD(4)
    if constexpr (e == 2) {
        TXS_BWD(2)
    }
#undef TXS_BWD
    return hipErrorInvalidValue;
}

int status_of(hipError_t e) { return e == hipSuccess ? TXS_OK : TXS_ERR_LAUNCH; }

// extents are int32 on the device; the margin keeps chunk arithmetic from wrapping
bool fits_i32(int64_t x) { return x >= 0 && x < 2147483647LL - 4096; }

unsigned blocks_for(long n, int per = kThreads) { return (unsigned)((n + per - 1) / per); }

int radix_bits(int64_t U) {
    int bits = 1;
    while ((1LL << bits) < U) ++bits;
    return bits;
}

}  // namespace

// =================================================================== C ABI ==

extern "C" {

int txs_abi_version(void) { return 5; }

const char *txs_status_string(int status) {
    switch (status) {
        case TXS_OK: return "ok";
        case TXS_ERR_INVALID_ARG: return "invalid argument (null pointer, negative or oversized extent)";
        case TXS_ERR_LAUNCH: return "HIP kernel launch failed";
        case TXS_ERR_UNSUPPORTED: return "unsupported dtype or operator";
        default: return "unknown status";
    }
}

int txs_default_heavy_threshold(void) { return kHeavyDefault; }
int txs_chunk_rows(void) { return kChunk; }

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
    // box constants, (box, tile) counts, scan workspace, box bases
    return (int64_t)(sizeof(DppBox) / sizeof(int)) * num_boxes + cells + scan_tiles(cells + 1) + 1 +
           num_boxes + 16;
}

int txs_dynamic_point_pool(const float *rois, const float *pts, int64_t num_boxes, int64_t num_pts,
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
    if (!rois || !pts || !workspace || !out_pts_idx || !out_roi_idx || !out_pts_feats)
        return TXS_ERR_INVALID_ARG;
    const int B = (int)num_boxes, P = (int)num_pts;
    const int n_tiles = (P + kThreads - 1) / kThreads;
    const long cells = (long)B * n_tiles;
    if (!fits_i32(cells + 1) || B > 65535) return TXS_ERR_INVALID_ARG;
    DppBox *boxes = reinterpret_cast<DppBox *>(workspace);
    int *counts = workspace + (sizeof(DppBox) / sizeof(int)) * (size_t)B;
    int *scan_ws = counts + cells + 1;
    int *box_base = scan_ws + scan_tiles(cells + 2) + 1;
    dpp_box_kernel<<<dim3(blocks_for(B)), dim3(kThreads), 0, st>>>(rois, B, extra_wlh[0], extra_wlh[1],
                                                                 extra_wlh[2], boxes);
    dpp_count_kernel<<<dim3(n_tiles, B), dim3(kThreads), 0, st>>>(pts, P, boxes, n_tiles, counts);
    if (exclusive_scan(counts, cells, counts, cells + 1, scan_ws, st) != hipSuccess) return TXS_ERR_LAUNCH;
    dpp_box_base_kernel<<<dim3(1), dim3(kThreads), 0, st>>>(counts, B, n_tiles, max_pts_per_box,
                                                           (int)max_all_pts, box_base, num_out);
    dpp_write_kernel<<<dim3(n_tiles, B), dim3(kThreads), 0, st>>>(
        pts, P, boxes, n_tiles, counts, box_base, max_pts_per_box, (int)max_all_pts,
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

int txs_scatter_forward(int op, int dtype, const void *feats, const int32_t *perm,
                        const int32_t *seg, const int32_t *preSum, const int32_t *slot_of,
                        const int32_t *heavy_ids, int64_t num_special, void *scratch, void *out,
                        int32_t *arg, int64_t num_total, int64_t channel, int64_t num_unq,
                        int64_t max_cnt, void *stream) {
    if (op != TXS_SUM && op != TXS_MEAN && op != TXS_MAX && op != TXS_MAX_REFTIE)
        return TXS_ERR_UNSUPPORTED;
    if (dtype != TXS_F32 && dtype != TXS_F16 && dtype != TXS_BF16) return TXS_ERR_UNSUPPORTED;
    if (!fits_i32(num_total) || !fits_i32(num_unq) || !fits_i32(channel) || num_special < 0 ||
        num_special > num_unq)
        return TXS_ERR_INVALID_ARG;
    if (num_unq == 0 || channel == 0) return TXS_OK;
    const bool is_max = op == TXS_MAX || op == TXS_MAX_REFTIE;
    if (!out || !preSum || (is_max && !arg)) return TXS_ERR_INVALID_ARG;
    // block width the reference would launch for this max_cnt (scatter_kernel.cu:187)
    int ref_log2 = 5;
    while (ref_log2 < 10 && (1LL << ref_log2) < max_cnt) ++ref_log2;
    if (num_total > 0 && (!feats || !seg || !slot_of)) return TXS_ERR_INVALID_ARG;
    if (num_special > 0 && (!scratch || !heavy_ids)) return TXS_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const int N = (int)num_total, C = (int)channel, U = (int)num_unq;
    const int elem = dtype == TXS_F32 ? 4 : 2;
    hipError_t e = hipSuccess;
    if (N > 0) {
        Geometry geo = make_geometry(N, C, elem, feats, out, nullptr, is_max, arg);
        if (dtype == TXS_F32)
            e = launch_fwd<F32>(op, geo, st, feats, perm, seg, preSum, slot_of, out, arg, scratch, N, C, U, ref_log2);
        else if (dtype == TXS_F16)
            e = launch_fwd<F16>(op, geo, st, feats, perm, seg, preSum, slot_of, out, arg, scratch, N, C, U, ref_log2);
        else
            e = launch_fwd<BF16>(op, geo, st, feats, perm, seg, preSum, slot_of, out, arg, scratch, N, C, U, ref_log2);
        if (e != hipSuccess) return TXS_ERR_LAUNCH;
    }
    if (num_special > 0) {
        if (dtype == TXS_F32)
            e = launch_finalize<F32>(op, st, feats, preSum, heavy_ids, scratch, out, arg, num_special, N, C, U, perm, ref_log2);
        else if (dtype == TXS_F16)
            e = launch_finalize<F16>(op, st, feats, preSum, heavy_ids, scratch, out, arg, num_special, N, C, U, perm, ref_log2);
        else
            e = launch_finalize<BF16>(op, st, feats, preSum, heavy_ids, scratch, out, arg, num_special, N, C, U, perm, ref_log2);
    }
    return status_of(e);
}

int txs_scatter_backward(int op, int dtype, const void *grad_out, const int32_t *arg,
                         const int32_t *perm, const int32_t *seg, const int32_t *preSum,
                         void *grad_in, int64_t num_total, int64_t channel, int64_t num_unq,
                         void *stream) {
    if (op == TXS_MAX_REFTIE) op = TXS_MAX;  // the backward only reads arg
    if (op != TXS_SUM && op != TXS_MEAN && op != TXS_MAX) return TXS_ERR_UNSUPPORTED;
    if (dtype != TXS_F32 && dtype != TXS_F16 && dtype != TXS_BF16) return TXS_ERR_UNSUPPORTED;
    if (!fits_i32(num_total) || !fits_i32(num_unq) || !fits_i32(channel)) return TXS_ERR_INVALID_ARG;
    if (num_total == 0 || channel == 0) return TXS_OK;
    if (!grad_out || !seg || !grad_in || num_unq <= 0) return TXS_ERR_INVALID_ARG;
    if (op == TXS_MAX && !arg) return TXS_ERR_INVALID_ARG;
    if (op == TXS_MEAN && !preSum) return TXS_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const int N = (int)num_total, C = (int)channel, U = (int)num_unq;
    const int elem = dtype == TXS_F32 ? 4 : 2;
    Geometry geo = make_geometry(N, C, elem, grad_out, grad_in, nullptr, op == TXS_MAX, arg);
    hipError_t e;
    if (dtype == TXS_F32)
        e = launch_bwd<F32>(op, geo, st, grad_out, arg, perm, seg, preSum, grad_in, N, C, U);
    else if (dtype == TXS_F16)
        e = launch_bwd<F16>(op, geo, st, grad_out, arg, perm, seg, preSum, grad_in, N, C, U);
    else
        e = launch_bwd<BF16>(op, geo, st, grad_out, arg, perm, seg, preSum, grad_in, N, C, U);
    return status_of(e);
}

}  // extern "C"
