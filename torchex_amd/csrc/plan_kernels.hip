// Index preparation for the voxel scatter kernels (built once per ScatterData and
// reused by every forward/backward call): a two-level bucket sort of (voxel id, row) for up
// to 2^22 voxels that yields CSR offsets, the table of special voxels and the
// per-position voxel ids on the way; for anything else a general sequence of
// sortedness/range check, stable LSD radix sort, CSR offsets from run boundaries and the
// same tables.  No histogram atomics on global memory and no inter-block spinning anywhere.
//
// Reference behaviour being replaced: ScatterData.__init__
// (torchex/operator_py/scatter_op.py:7-21) and getPreSum
// (torchex/src/scatter/scatter_kernel.cu:85-100).

#include "txs_common.h"

#include <atomic>

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
// Thread j owns the boundary in front of position j, i.e. the ids in (key[j-1], key[j]]
// (more than one only across empty voxels).  A long run of empty voxels is not walked by
// its one owner: the aligned blocks of kGapBlock ids that lie wholly inside a gap are left to
// presum_gap_blocks_kernel, and the owner fills only the two ragged ends.
constexpr int kGapBlock = 256;
__global__ void presum_from_sorted_kernel(const int *__restrict__ keys, long n, int U,
                                          int *__restrict__ preSum) {
    long j = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (j > n) return;
    long lo = (j == 0) ? -1 : (long)(keys[j - 1] & kIdMask);
    long hi = (j == n) ? (long)U : (long)(keys[j] & kIdMask);
    if (hi > U) hi = U;
    // whole blocks [b0, b1) of ids inside (lo, hi]
    const long b0 = (lo + 1 + kGapBlock - 1) / kGapBlock * kGapBlock;
    const long b1 = (hi + 1) / kGapBlock * kGapBlock;
    if (b1 > b0) {
        for (long u = lo + 1; u < b0; ++u) preSum[u] = (int)j;
        for (long u = b1; u <= hi; ++u) preSum[u] = (int)j;
    } else {
        for (long u = lo + 1; u <= hi; ++u) preSum[u] = (int)j;
    }
}

// One workgroup per aligned block of kGapBlock ids: if no key falls inside the block (and
// none equals its last id's successor boundary), every id of it has the same offset, the
// first position whose key is at or above the block.
__global__ __launch_bounds__(kGapBlock) void presum_gap_blocks_kernel(const int *__restrict__ keys, long n, int U,
                                                                      int *__restrict__ preSum) {
    __shared__ long s_pos;
    const long bs = (long)blockIdx.x * kGapBlock, be = bs + kGapBlock;  // ids [bs, be)
    if (be - 1 > (long)U) return;                                       // not wholly inside [0, U]
    if (threadIdx.x == 0) {
        long a = 0, b = n;  // first position whose key is >= bs
        while (a < b) {
            const long m = (a + b) >> 1;
            if ((long)(keys[m] & kIdMask) < bs) a = m + 1; else b = m;
        }
        // the block lies wholly inside one gap iff the key at that position (or the end of
        // the ids, U) is at or beyond the block's last id
        const long next = a < n ? (long)(keys[a] & kIdMask) : (long)U;
        s_pos = next >= be - 1 ? a : -1;
    }
    __syncthreads();
    const long pos = s_pos;
    if (pos >= 0) preSum[bs + threadIdx.x] = (int)pos;
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

// ------------------------------------------------ two-level plan (bucket sort) --
//
// For up to 2^22 voxels the whole index preparation is four kernels and a scan:
//   (1) bucket_hist_kernel: per tile of 2048 - 8192 rows, the histogram of the HIGH digit of the
//       voxel id (the "bucket") and the tile's order / range flags;
//   (2) exclusive scan of the digit-major histogram;
//   (3) bucket_scatter_kernel: flags of the whole input, bucket boundaries, and the stable
//       scatter of (id, row) pairs by bucket (wave-ballot ranking);
//   (4) bucket_count_kernel: a bucket is cut into slices of 2048 rows (at most 64, longer ones
//       beyond), one workgroup per slice; each counts its slice's rows per voxel (LOW digit,
//       <= 11 bits) in LDS and writes the counts out;
//   (5) bucket_plan_kernel: the same workgroups add up the counts of their bucket's slices
//       (a voxel's count, and its rows in the slices in front), which at the same time yields
//       the bucket's share of everything else the plan holds: CSR offsets, per-voxel counts
//       (checked against the caller's), the special-voxel table and its slots, max_cnt; then
//       each places its slice by the low digit, stably, writing the flagged per-position ids
//       next to the permutation.
// (Measured against one kernel in which every workgroup of a bucket counted the whole bucket:
// 1M ids of a voxelised sweep 67 -> 63 us, of its pillars 64 -> 57 us, 200k ids 38 -> 41 us
// (one launch more), and 1.25M ids of which 250k fall into 900 neighbouring voxels 198 -> 101 us.)
// Ids of at most 11 bits need no low digit: (3) already gives the final order, and the
// elementwise kernels used by the general sequence finish the plan.
// Measured alternatives (1M ids of 19 bits, 0.13 ms per plan as built): an 11-bit bucket digit
// makes the scatter write 16-byte runs and costs 30 us instead of 20; folding the scan into
// the scatter (every workgroup adding up the tile histograms itself) saves two launches but
// costs more than it saves from about 100 tiles on; per-voxel instead of per-row offset
// bookkeeping in (5) makes no difference.

#ifndef TXS_BUCKET_HIGH_BITS
#define TXS_BUCKET_HIGH_BITS 9
#endif
constexpr int kBucketHighBits = TXS_BUCKET_HIGH_BITS;
constexpr int kBucketLowBitsMax = 11;   // also the largest high digit
constexpr int kBucketBitsMax = 22;
constexpr int kHistThreads = 512;
// rows per tile of the histogram and scatter kernels: 512 * {4, 8, 16}, the largest that still
// gives every compute unit a tile
int hist_items_for(long n) {
    return n >= 256L * kHistThreads * 16 ? 16 : (n >= 256L * kHistThreads * 8 ? 8 : 4);
}
constexpr int kHistWaves = kHistThreads / 64;
#ifndef TXS_BKT_ITEMS
#define TXS_BKT_ITEMS 8
#endif
#ifndef TXS_BKT_SLICE_CHUNKS
#define TXS_BKT_SLICE_CHUNKS 1
#endif
constexpr int kBktItems = TXS_BKT_ITEMS;
constexpr int kBktChunk = kThreads * kBktItems;        // 4096 rows per placement round
constexpr int kBktWaves = kThreads / 64;
constexpr int kBktSlice = TXS_BKT_SLICE_CHUNKS * kBktChunk;  // rows one workgroup places
#ifndef TXS_BKT_MAX_SLICES
#define TXS_BKT_MAX_SLICES 64
#endif
constexpr int kBktMaxSlices = TXS_BKT_MAX_SLICES;      // workgroups per bucket at most
constexpr long kBktGiant = 262144;                     // rows in one bucket beyond which the general sequence runs
constexpr int kFlagUnsorted = 1, kFlagOutOfRange = 2;

// hist: [high_bins][n_tiles] digit-major (the order its exclusive scan needs); tile_flags: [n_tiles]
template <int ITEMS>
__global__ __launch_bounds__(kHistThreads) void bucket_hist_kernel(
    const int *__restrict__ inv, long n, int U, int low_bits, int high_bins, int *__restrict__ hist,
    int *__restrict__ tile_flags, int n_tiles) {
    __shared__ int h[1 << kBucketLowBitsMax];
    __shared__ int s_flags;
    for (int d = threadIdx.x; d < high_bins; d += kHistThreads) h[d] = 0;
    if (threadIdx.x == 0) s_flags = 0;
    __syncthreads();
    const long base = (long)blockIdx.x * (kHistThreads * ITEMS);
    int v[ITEMS];
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
        const long i = base + (long)it * kHistThreads + threadIdx.x;
        v[it] = i < n ? inv[i] : 0x7fffffff;
    }
    bool bad_range = false, bad_order = false;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
        const long i = base + (long)it * kHistThreads + threadIdx.x;
        if (i >= n) continue;
        if ((unsigned)v[it] >= (unsigned)U) {
            bad_range = true;
        } else {
            atomicAdd(&h[v[it] >> low_bits], 1);
        }
        // neighbour in memory = the next thread's element of the same round
        int nb = __shfl_down(v[it], 1, 64);
        if ((threadIdx.x & 63) == 63) nb = (i + 1 < n) ? inv[i + 1] : 0x7fffffff;
        if (i + 1 < n && nb < v[it]) bad_order = true;
    }
    const int f = (__ballot(bad_order) != 0ull ? kFlagUnsorted : 0) | (__ballot(bad_range) != 0ull ? kFlagOutOfRange : 0);
    if (f && (threadIdx.x & 63) == 0) atomicOr(&s_flags, f);
    __syncthreads();
    for (int d = threadIdx.x; d < high_bins; d += kHistThreads) hist[(long)d * n_tiles + blockIdx.x] = h[d];
    if (threadIdx.x == 0) tile_flags[blockIdx.x] = s_flags;
}

// id at position i: of unq_inv itself (rows in order) or of the (id, row) pairs the bucket scatter wrote
__device__ __forceinline__ int kread(const int *keys, long i, bool packed) {
    return packed ? keys[2 * i] : keys[i];
}

// Stable scatter by the high digit.  hist: the exclusive scan of the digit-major tile histograms.
//   bucket_start [high_bins + 1] (written by workgroup 0): first position of every bucket.
//   stats: zero-filled here (workgroup 0), then UNSORTED / OUT_OF_RANGE of the whole input
//   and NEED_GENERAL (a bucket above `giant` rows: the bucket kernels step aside).
// Rows already in order are not moved: out_keys (if given) receives a copy of the ids, and
// the next kernel reads unq_inv itself.  out_pairs: (id, row) per position, one 8-byte
// store; or out_keys / out_rows as two arrays when the order is already final.
template <int ITEMS>
__global__ __launch_bounds__(kHistThreads) void bucket_scatter_kernel(
    const int *__restrict__ inv, long n, int U, int low_bits, int high_bits,
    const int *__restrict__ hist, const int *__restrict__ tile_flags, int n_tiles, long giant,
    int *__restrict__ bucket_start, int *__restrict__ stats, int *__restrict__ out_keys,
    int *__restrict__ out_rows, int2 *__restrict__ out_pairs) {
    extern __shared__ int wcount[];  // [kHistWaves][bins], then base[bins]
    __shared__ int s_flags;
    const int bins = 1 << high_bits;
    int *base_s = wcount + kHistWaves * bins;  // first destination of this tile's rows, per digit
    const int w = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const unsigned long long lanes_below = (1ull << lane) - 1ull;
    if (threadIdx.x == 0) s_flags = 0;
    for (int k = threadIdx.x; k < kHistWaves * bins; k += kHistThreads) wcount[k] = 0;
    __syncthreads();

    // ---- flags of the whole input
    int f = 0;
    for (int t = threadIdx.x; t < n_tiles; t += kHistThreads) f |= tile_flags[t];
    if (f) atomicOr(&s_flags, f);

    // ---- first destination of this tile's rows per digit (from the scanned histogram), the
    // bucket boundaries (workgroup 0 publishes them) and the test for an overfull bucket
    for (int d = threadIdx.x; d < bins; d += kHistThreads) {
        const int first = hist[(long)d * n_tiles];
        const int next = hist[(long)(d + 1) * n_tiles];  // the entry after the last bucket holds the total
        base_s[d] = hist[(long)d * n_tiles + blockIdx.x];
        if (blockIdx.x == 0) {
            bucket_start[d] = first;
            if (d == bins - 1) bucket_start[bins] = next;
        }
        if ((long)next - first > giant) atomicOr(&s_flags, 4);
    }
    __syncthreads();
    const int flags = s_flags;
    if (blockIdx.x == 0) {
        for (int k = threadIdx.x; k < TXS_STATS_LEN; k += kHistThreads) {
            int val = 0;
            if (k == TXS_STAT_UNSORTED) val = (flags & kFlagUnsorted) ? 1 : 0;
            if (k == TXS_STAT_OUT_OF_RANGE) val = (flags & kFlagOutOfRange) ? 1 : 0;
            if (k == TXS_STAT_NEED_GENERAL) val = (flags & 4) ? 1 : 0;
            stats[k] = val;
        }
    }
    if (flags & 4) return;  // the caller re-plans with the general sequence
    const long tile0 = (long)blockIdx.x * (kHistThreads * ITEMS);
    if (!(flags & kFlagUnsorted)) {
        if (out_keys)
            for (int it = 0; it < ITEMS; ++it) {
                const long i = tile0 + (long)it * kHistThreads + threadIdx.x;
                if (i < n) out_keys[i] = inv[i];
            }
        return;
    }

    // ---- stable ranking inside the tile and the scatter
    const long wbase = tile0 + (long)w * (64 * ITEMS);
    int key[ITEMS], lrank[ITEMS];
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
        const long i = wbase + (long)it * 64 + lane;
        const int v = i < n ? inv[i] : -1;
        key[it] = (unsigned)v < (unsigned)U ? v : -1;  // out-of-range ids are dropped (and flagged)
    }
    volatile int *wc = wcount + w * bins;
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
        const bool valid = key[it] >= 0;
        const int digit = valid ? (key[it] >> low_bits) : 0;
        unsigned long long mask = __ballot(valid);
        for (int b = 0; b < high_bits; ++b) {
            const bool bit = (digit >> b) & 1;
            const unsigned long long bal = __ballot(bit);
            mask &= bit ? bal : ~bal;
        }
        const int below = __popcll(mask & lanes_below);
        const int prev = wc[digit];
        __builtin_amdgcn_wave_barrier();
        if (valid && below == 0) wc[digit] = prev + __popcll(mask);
        __builtin_amdgcn_wave_barrier();
        lrank[it] = prev + below;
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
        if (key[it] < 0) continue;
        const long i = wbase + (long)it * 64 + lane;
        const int dg = key[it] >> low_bits;
        int before = base_s[dg];
        for (int k = 0; k < w; ++k) before += wcount[k * bins + dg];
        const long dst = (long)before + lrank[it];
        if (dst >= 0 && dst < n) {
            if (out_pairs) {
                out_pairs[dst] = make_int2(key[it], (int)i);
            } else {
                out_keys[dst] = key[it];
                out_rows[dst] = (int)i;
            }
        }
    }
}

// Rows of bucket b that slice j of it covers.  A bucket is cut into slices of kBktSlice rows,
// at most kBktMaxSlices of them (longer slices beyond that).
struct BucketSlice {
    long s, e;        // the bucket's rows [s, e) in bucket order
    long my_s, my_e;  // the slice's rows
    int nsl;          // slices of the bucket
};
__device__ __forceinline__ int slices_of(long cnt_b) {
    return (int)min((long)kBktMaxSlices, max(1L, (cnt_b + kBktSlice - 1) / kBktSlice));
}
__device__ __forceinline__ BucketSlice bucket_slice(long s, long e, int j) {
    BucketSlice r;
    r.s = s;
    r.e = e;
    const long nb = r.e - r.s;
    r.nsl = slices_of(nb);
    long slice = kBktSlice;
    if (nb > (long)kBktMaxSlices * kBktSlice)
        slice = ((nb + kBktMaxSlices - 1) / kBktMaxSlices + kBktChunk - 1) / kBktChunk * kBktChunk;
    r.my_s = r.s + (long)j * slice;
    r.my_e = min(r.e, r.my_s + slice);
    return r;
}

// Workgroup g serves slice j of bucket b; (b, j) follows from the bucket sizes and is kept with
// the bucket's bounds in wg_pick[g] = (b, j, start, end) (b = -1: no work) for the kernel that
// follows, which so learns its work from one load.  Each workgroup
// counts the rows of ITS slice per voxel (low digit) and writes the counts to part_hist[g][*]:
// the slices of a bucket sit in consecutive workgroups, so the next kernel gets a voxel's count in
// the whole bucket, and in the slices in front of its own, from at most kBktMaxSlices short
// reads instead of every workgroup of a crowded bucket counting all of its rows.
__global__ __launch_bounds__(kThreads) void bucket_count_kernel(
    const int *__restrict__ inv, const int *__restrict__ pairs1, long n, int U, int low_bits, int high_bins,
    const int *__restrict__ bucket_start, const int *__restrict__ stats, int4 *__restrict__ wg_pick,
    int *__restrict__ part_hist) {
    extern __shared__ int cnt_s[];  // [low_bins]
    __shared__ int s_pick[2];
    const int low_bins = 1 << low_bits;
    if (stats[TXS_STAT_NEED_GENERAL] != 0) return;
    {
        if (threadIdx.x == 0) s_pick[0] = -1;
        int carried = 0;
        for (int bb0 = 0; bb0 < high_bins; bb0 += kThreads) {
            const int bb = bb0 + (int)threadIdx.x;
            int nsl = 0;
            if (bb < high_bins && ((long)bb << low_bits) < (long)U)
                nsl = slices_of((long)bucket_start[bb + 1] - bucket_start[bb]);
            int total;
            const int first = carried + block_exclusive_scan(nsl, &total);  // (synchronises the workgroup)
            if ((int)blockIdx.x >= first && (int)blockIdx.x < first + nsl) {
                s_pick[0] = bb;
                s_pick[1] = (int)blockIdx.x - first;
            }
            carried += total;
        }
        __syncthreads();
    }
    const int b = s_pick[0], j = s_pick[1];
    if (b < 0) {
        if (threadIdx.x == 0) wg_pick[blockIdx.x] = make_int4(-1, 0, 0, 0);
        return;
    }
    const int u_lo = b << low_bits;
    const bool packed = stats[TXS_STAT_UNSORTED] != 0;
    const int *keys = packed ? pairs1 : inv;
    const BucketSlice sl = bucket_slice(bucket_start[b], bucket_start[b + 1], j);
    if (threadIdx.x == 0) wg_pick[blockIdx.x] = make_int4(b, j, (int)sl.s, (int)sl.e);
    for (int k = threadIdx.x; k < low_bins; k += kThreads) cnt_s[k] = 0;
    __syncthreads();
    for (long i0 = sl.my_s; i0 < sl.my_e; i0 += (long)kThreads * kBktItems) {
        int v[kBktItems];
#pragma unroll
        for (int it = 0; it < kBktItems; ++it) {
            const long i = i0 + (long)it * kThreads + threadIdx.x;
            v[it] = i < sl.my_e ? kread(keys, i, packed) : -1;
        }
#pragma unroll
        for (int it = 0; it < kBktItems; ++it) {
            const int d = v[it] - u_lo;
            if (v[it] >= 0 && (unsigned)d < (unsigned)low_bins) atomicAdd(&cnt_s[d], 1);
        }
    }
    __syncthreads();
    int *mine = part_hist + (long)blockIdx.x * low_bins;
    for (int k = threadIdx.x; k < low_bins; k += kThreads) mine[k] = cnt_s[k];
}

__global__ __launch_bounds__(kThreads) void bucket_plan_kernel(
    const int *__restrict__ inv, const int *__restrict__ pairs1, long n, int U,
    int low_bits, int high_bins, const int *__restrict__ bucket_start, int heavy_threshold,
    const long long *__restrict__ unq_cnts, int *__restrict__ perm, int *__restrict__ seg,
    int *__restrict__ preSum, int *__restrict__ slot_of, int *__restrict__ heavy_ids,
    int *__restrict__ stats, const int4 *__restrict__ wg_pick, const int *__restrict__ part_hist,
    long long *__restrict__ ranks) {
    // ranks != NULL: the caller wants the rank of every row inside its voxel and nothing else
    // (ingroup_inds): off[] then counts from the voxel's first row instead of the bucket's,
    // and the placement writes ranks[row] in place of the permutation and the ids
    const bool rank_mode = ranks != nullptr;
    extern __shared__ int wc[];  // [kBktWaves][low_bins], tot[low_bins], off[low_bins]
    __shared__ int s_red[kBktWaves], s_bad[kBktWaves];
    const int low_bins = 1 << low_bits;
    int *tot = wc + kBktWaves * low_bins;
    int *off = tot + low_bins;
    const int w = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const unsigned long long lanes_below = (1ull << lane) - 1ull;
    if (stats[TXS_STAT_NEED_GENERAL] != 0) return;
    (void)high_bins;
    const int4 pick = wg_pick[blockIdx.x];
    const int b = pick.x, j = pick.y;
    if (b < 0) return;
    const int u_lo = b << low_bits;
    const int u_hi = min(U, u_lo + low_bins);
    const bool unsorted = stats[TXS_STAT_UNSORTED] != 0;
    const bool packed = unsorted;
    const BucketSlice sl = bucket_slice(pick.z, pick.w, j);
    const long s = sl.s, e = sl.e, my_s = sl.my_s, my_e = sl.my_e;

    // Everything the workgroup reads from memory is requested here, in one go: the first
    // round of the slice's rows, the caller's counts of this bucket's voxels (first slice
    // only; compared once the kernel's own counts are complete), and the per-slice counts.
    auto load_round = [&](long c0, int (&key)[kBktItems], int (&row)[kBktItems]) {
        const long wbase = c0 + (long)w * (64 * kBktItems);
#pragma unroll
        for (int it = 0; it < kBktItems; ++it) {
            const long i = wbase + (long)it * 64 + lane;
            int v = -1;
            row[it] = (int)i;
            if (i < my_e) {
                if (packed) {
                    const int2 kr = reinterpret_cast<const int2 *>(pairs1)[i];
                    v = kr.x;
                    row[it] = kr.y;
                } else {
                    v = inv[i];
                }
            }
            key[it] = (i < my_e && (unsigned)(v - u_lo) < (unsigned)low_bins) ? v : -1;
        }
    };
    int key0[kBktItems], row0[kBktItems];
    load_round(my_s, key0, row0);
    constexpr int kCntPer = (1 << kBucketLowBitsMax) / kThreads;
    long long given[kCntPer];
    const bool check_counts = j == 0 && unq_cnts != nullptr;
    if (check_counts) {
#pragma unroll
        for (int k = 0; k < kCntPer; ++k) {
            const int d = k * kThreads + (int)threadIdx.x;
            given[k] = (d < low_bins && u_lo + d < u_hi) ? unq_cnts[u_lo + d] : -1;
        }
    }
    // ---- counts of the bucket's voxels, and of the rows in front of this slice: sums over the
    // per-slice counts of the bucket's workgroups (blockIdx.x - j is the bucket's first), eight
    // loads in flight per thread
    for (int k = threadIdx.x; k < (kBktWaves + 2) * low_bins; k += kThreads) wc[k] = 0;
    __syncthreads();
    {
        const int *first = part_hist + ((long)blockIdx.x - j) * low_bins;
        const int total = sl.nsl << low_bits;
        constexpr int kGather = 8;
        for (int i0 = threadIdx.x; i0 < total; i0 += kThreads * kGather) {
            int c[kGather];
#pragma unroll
            for (int q = 0; q < kGather; ++q) {
                const int i = i0 + q * kThreads;
                c[q] = i < total ? first[i] : 0;
            }
#pragma unroll
            for (int q = 0; q < kGather; ++q) {
                const int i = i0 + q * kThreads;
                if (c[q] == 0) continue;
                const int d = i & (low_bins - 1), k = i >> low_bits;
                atomicAdd(&tot[d], c[q]);
                if (k < j) atomicAdd(&off[d], c[q]);
            }
        }
    }
    __syncthreads();
    // ---- exclusive scan over the voxels of the bucket: a run of consecutive voxels per thread
    const int per = (low_bins + kThreads - 1) / kThreads;
    const int d0 = threadIdx.x * per;
    int mine = 0;
    for (int k = 0; k < per; ++k)
        if (d0 + k < low_bins) mine += tot[d0 + k];
    int total;
    int run = block_exclusive_scan(mine, &total);
    // off[d] becomes the bucket-relative position of the slice's first row of voxel d
    for (int k = 0; k < per; ++k) {
        const int d = d0 + k;
        if (d >= low_bins) break;
        const int c = tot[d];
        const int excl = run;
        run += c;
        if (!rank_mode) off[d] += excl;
        if (j == 0 && u_lo + d < u_hi) {
            preSum[u_lo + d] = (int)s + excl;
            if (u_lo + d == U - 1) preSum[U] = (int)n;
        }
    }
    __syncthreads();
    // ---- statistics, special voxels and their slots (first slice only; as plan_special_kernel)
    if (j == 0 && slot_of != nullptr) {
        int vmax = 0;
        bool mismatch = false;
        if (check_counts) {
#pragma unroll
            for (int k = 0; k < kCntPer; ++k) {
                const int d = k * kThreads + (int)threadIdx.x;
                if (d < low_bins && u_lo + d < u_hi) mismatch |= given[k] != (long long)tot[d];
            }
        }
        for (int dd = 0; dd < low_bins; dd += kThreads) {
            const int d = dd + (int)threadIdx.x;
            const int u = u_lo + d;
            const bool in = d < low_bins && u < u_hi;
            const int cnt = in ? tot[d] : 0;
            vmax = max(vmax, cnt);
            const bool heavy = in && cnt > heavy_threshold;
            const bool empty = in && cnt == 0;
            const unsigned long long mh = __ballot(heavy), me = __ballot(empty);
            int base_h = 0, base_e = 0;
            if (lane == 0) {
                if (mh) base_h = atomicAdd(&stats[TXS_STAT_NUM_HEAVY], __popcll(mh));
                if (me) base_e = atomicAdd(&stats[TXS_STAT_NUM_EMPTY], __popcll(me));
                if (mh | me) atomicAdd(&stats[TXS_STAT_NUM_SPECIAL], __popcll(mh) + __popcll(me));
            }
            base_h = __shfl(base_h, 0, 64);
            base_e = __shfl(base_e, 0, 64);
            if (in) {
                int slot = -1;
                if (heavy) {
                    slot = base_h + __popcll(mh & lanes_below);
                    if (slot < U) heavy_ids[slot] = u;
                } else if (empty) {
                    slot = U - 1 - (base_e + __popcll(me & lanes_below));
                    if (slot >= 0) heavy_ids[slot] = u;
                }
                slot_of[u] = slot;
            }
        }
        const int wmax = wave_max_i32(vmax);
        const bool any_mismatch = __ballot(mismatch) != 0ull;
        if (lane == 0) {
            s_red[w] = wmax;
            s_bad[w] = any_mismatch;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            int m = 0, bad = 0;
            for (int k = 0; k < kBktWaves; ++k) {
                m = max(m, s_red[k]);
                bad |= s_bad[k];
            }
            if (m > 0) atomicMax(&stats[TXS_STAT_MAX_CNT], m);
            if (bad) stats[TXS_STAT_COUNT_MISMATCH] = 1;
        }
    }

    // ---- stable placement of the slice by the low digit, round after round
    for (long c0 = my_s; c0 < my_e; c0 += kBktChunk) {
        int key[kBktItems], row[kBktItems], lrank[kBktItems];
        volatile int *mywc = wc + w * low_bins;
        if (c0 == my_s) {
#pragma unroll
            for (int it = 0; it < kBktItems; ++it) {
                key[it] = key0[it];
                row[it] = row0[it];
            }
        } else {
            load_round(c0, key, row);
        }
#pragma unroll
        for (int it = 0; it < kBktItems; ++it) {
            const bool valid = key[it] >= 0;
            const int digit = valid ? key[it] - u_lo : 0;
            unsigned long long mask = __ballot(valid);
            for (int bb = 0; bb < low_bits; ++bb) {
                const bool bit = (digit >> bb) & 1;
                const unsigned long long bal = __ballot(bit);
                mask &= bit ? bal : ~bal;
            }
            const int below = __popcll(mask & lanes_below);
            const int prev = mywc[digit];
            __builtin_amdgcn_wave_barrier();
            if (valid && below == 0) mywc[digit] = prev + __popcll(mask);
            __builtin_amdgcn_wave_barrier();
            lrank[it] = prev + below;
        }
        __syncthreads();
        // destination = slice-start position of the voxel + rows of the voxel that the waves
        // in front of this one hold in this pass + rank inside the wave; the per-voxel
        // bookkeeping is done per ROW (a few LDS operations each), never per voxel: a pass
        // has fewer rows than a bucket can have voxel-times-wave counters
        long dst[kBktItems];
#pragma unroll
        for (int it = 0; it < kBktItems; ++it) {
            dst[it] = -1;
            if (key[it] < 0) continue;
            const int dg = key[it] - u_lo;
            int before = off[dg];
            for (int k = 0; k < w; ++k) before += wc[k * low_bins + dg];
            dst[it] = s + before + lrank[it];
        }
        __syncthreads();
#pragma unroll
        for (int it = 0; it < kBktItems; ++it) {
            if (key[it] < 0) continue;
            const int dg = key[it] - u_lo;
            atomicAdd(&off[dg], 1);       // the next pass starts behind this pass's rows
            wc[w * low_bins + dg] = 0;    // (every row of the group stores the same zero)
            if (rank_mode) {
                if ((unsigned)row[it] < (unsigned)n) ranks[row[it]] = (long long)(dst[it] - s);
            } else if (dst[it] >= s && dst[it] < e) {
                const int c = tot[dg];
                seg[dst[it]] = key[it] | (c > heavy_threshold ? kSpecialBit : 0);
                if (unsorted) perm[dst[it]] = row[it];
            }
        }
        __syncthreads();
    }
}

__global__ void stats_clear_kernel(int *__restrict__ stats) {
    if (threadIdx.x < TXS_STATS_LEN) stats[threadIdx.x] = 0;
}

// Heavy voxel number blockIdx.x of the list becomes an ordinary one again: the special bit
// comes off its positions and it gives up its slot.
__global__ void demote_heavy_kernel(const int *__restrict__ preSum, int *__restrict__ seg,
                                    int *__restrict__ slot_of, const int *__restrict__ heavy_ids,
                                    int N, int U, int *__restrict__ stats) {
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        stats[TXS_STAT_NUM_HEAVY] = 0;
        stats[TXS_STAT_NUM_SPECIAL] = stats[TXS_STAT_NUM_EMPTY];
    }
    const int u = heavy_ids[blockIdx.x];
    if ((unsigned)u >= (unsigned)U) return;
    const int lo = max(preSum[u], 0), hi = min(preSum[u + 1], N);
    for (int p = lo + (int)threadIdx.x; p < hi; p += (int)blockDim.x) seg[p] &= kIdMask;
    if (threadIdx.x == 0) slot_of[u] = -1;
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
    // long runs of empty voxels, one workgroup per 256 ids (only where there can be any)
    if (num_unq + 1 >= kGapBlock)
        presum_gap_blocks_kernel<<<dim3((unsigned)((num_unq + 1) / kGapBlock)), dim3(kGapBlock), 0,
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

int txs_plan_demote_heavy(const int32_t *preSum, int32_t *seg, int32_t *slot_of, const int32_t *heavy_ids,
                          int64_t num_heavy, int64_t num_total, int64_t num_unq, int32_t *stats, void *stream) {
    if (!fits_i32(num_total) || !fits_i32(num_unq) || num_heavy < 0 || num_heavy > num_unq)
        return TXS_ERR_INVALID_ARG;
    if (num_heavy == 0) return TXS_OK;
    if (!preSum || !seg || !slot_of || !heavy_ids || !stats) return TXS_ERR_INVALID_ARG;
    demote_heavy_kernel<<<dim3((unsigned)num_heavy), dim3(128), 0, (hipStream_t)stream>>>(
        preSum, seg, slot_of, heavy_ids, (int)num_total, (int)num_unq, stats);
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

int64_t txs_plan_workspace_len(int64_t num_total, int64_t num_unq) {
    if (!fits_i32(num_total) || !fits_i32(num_unq)) return -1;
    const int64_t general = txs_sort_workspace_len(num_total, num_unq);
    const int64_t tile = (int64_t)kHistThreads * hist_items_for(num_total);
    const int64_t tiles = (num_total + tile - 1) / tile;
    const int64_t bins = (int64_t)1 << kBucketLowBitsMax;
    // (id, row) pairs after the bucket scatter, the digit-major histogram, tile flags, bucket
    // boundaries, the scan workspace
    const int64_t hist = bins * (tiles > 0 ? tiles : 1) + 1;
    // per-slice voxel counts of the bucket kernels: (slices + buckets) * voxels per bucket, for
    // the digit split txs_plan_build uses
    const int ubits = radix_bits(num_unq > 1 ? num_unq : 1);
    int low_bits = ubits <= kBucketLowBitsMax ? 0 : ubits - kBucketHighBits;
    if (low_bits > kBucketLowBitsMax) low_bits = kBucketLowBitsMax;
    int64_t counts = 0;
    if (low_bits > 0 && ubits <= kBucketBitsMax) {
        const int64_t groups = num_total / kBktSlice + ((int64_t)1 << (ubits - low_bits));
        counts = 4 + 4 * groups + groups * ((int64_t)1 << low_bits);
    }
    const int64_t bucket = 2 * num_total + hist + tiles + bins + 1 + scan_tiles(hist + 1) + 17 + counts;
    return general > bucket ? general : bucket;
}

int txs_plan_build_general(const int32_t *unq_inv, int64_t num_total, int64_t num_unq, int32_t heavy_threshold,
                           const int64_t *unq_cnts, int32_t *plan_ws, int32_t *perm, int32_t *seg,
                           int32_t *preSum, int32_t *slot_of, int32_t *heavy_ids, int32_t *stats, void *stream) {
    if (!fits_i32(num_total) || !fits_i32(num_unq) || !stats || !preSum || heavy_threshold < kChunk)
        return TXS_ERR_INVALID_ARG;
    const long n = num_total;
    const int U = (int)num_unq;
    if (n > 0 && (!unq_inv || !plan_ws || !perm || !seg)) return TXS_ERR_INVALID_ARG;
    if (U > 0 && ((slot_of == nullptr) != (heavy_ids == nullptr))) return TXS_ERR_INVALID_ARG;
    // order/range flags, three-kernel radix passes, CSR offsets, special table, flags
    int rc = txs_plan_check(unq_inv, n, U, stats, stream);
    if (rc == TXS_OK && n > 0 && U > 0) rc = txs_plan_sort(unq_inv, n, U, stats, perm, seg, plan_ws, stream);
    if (rc == TXS_OK) rc = txs_plan_presum(seg, U > 0 ? n : 0, U, preSum, stream);
    if (slot_of == nullptr) return rc;  // order and offsets only
    if (rc == TXS_OK)
        rc = txs_plan_special(preSum, U, heavy_threshold, unq_cnts, slot_of, heavy_ids, stats, nullptr, nullptr,
                              stream);
    if (rc == TXS_OK) rc = txs_plan_seg_flag(seg, U > 0 ? n : 0, U, slot_of, stream);
    return rc;
}

int txs_plan_build(const int32_t *unq_inv, int64_t num_total, int64_t num_unq, int32_t heavy_threshold,
                   const int64_t *unq_cnts, int32_t *plan_ws, int32_t *perm, int32_t *seg, int32_t *preSum,
                   int32_t *slot_of, int32_t *heavy_ids, int32_t *stats, void *stream) {
    return txs_detail::plan_build(unq_inv, num_total, num_unq, heavy_threshold, unq_cnts, plan_ws, perm, seg, preSum,
                                  slot_of, heavy_ids, stats, nullptr, stream);
}

}  // extern "C"

// txs_plan_build, or with `ranks` the in-voxel rank of every row and no special-voxel table.
// Ranks are written by the bucket kernels only: txs_detail::plan_writes_ranks tells a caller
// whether they apply to the extents (otherwise it ranks from the plan this call leaves).
bool txs_detail::plan_writes_ranks(long num_total, long num_unq) {
    const int bits = radix_bits(num_unq > 1 ? num_unq : 1);
    return num_total > 0 && num_unq > 0 && bits <= kBucketBitsMax && bits > kBucketLowBitsMax;
}

int txs_detail::plan_build(const int32_t *unq_inv, int64_t num_total, int64_t num_unq, int32_t heavy_threshold,
                           const int64_t *unq_cnts, int32_t *plan_ws, int32_t *perm, int32_t *seg,
                           int32_t *preSum, int32_t *slot_of, int32_t *heavy_ids, int32_t *stats,
                           long long *ranks, void *stream) {
    if (!fits_i32(num_total) || !fits_i32(num_unq) || !stats || !preSum || heavy_threshold < kChunk)
        return TXS_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const long n = num_total;
    const int U = (int)num_unq;
    if (n > 0 && (!unq_inv || !plan_ws || !perm || !seg)) return TXS_ERR_INVALID_ARG;
    if (U > 0 && ((slot_of == nullptr) != (heavy_ids == nullptr))) return TXS_ERR_INVALID_ARG;
    if (((uintptr_t)plan_ws & 7u) != 0) return TXS_ERR_INVALID_ARG;
    if (slot_of == nullptr) heavy_threshold = 0x7fffffff;  // no special voxels: no flag bit in seg
    const int bits = radix_bits(U > 1 ? U : 1);
    if (n == 0 || U == 0) {
        // nothing to sort: the general sequence only writes the offsets and the table of
        // (empty) voxels; it adds to `stats`, which this call promises to initialise itself
        stats_clear_kernel<<<dim3(1), dim3(64), 0, st>>>(stats);
        if (hipGetLastError() != hipSuccess) return TXS_ERR_LAUNCH;
    }
    if (n == 0 || U == 0 || bits > kBucketBitsMax)
        return txs_plan_build_general(unq_inv, num_total, num_unq, heavy_threshold, unq_cnts, plan_ws, perm, seg,
                                      preSum, slot_of, heavy_ids, stats, stream);
    // ids of up to 11 bits are sorted by the bucket pass alone; beyond that the bucket digit has
    // 9 bits (narrower, and the buckets of a spatially sorted id space get too uneven: a
    // bucket's workgroups each count the whole bucket; wider, and a tile sends too few rows to
    // a bucket for the scatter to write whole cache lines) and the low digit takes the rest,
    // at most 11
    const int low_bits = bits <= kBucketLowBitsMax ? 0 : min(bits - kBucketHighBits, kBucketLowBitsMax);
    const int high_bits = bits - low_bits;
    const int high_bins = 1 << high_bits;
    const int items = hist_items_for(n);
    const long tile = (long)kHistThreads * items;
    const int n_tiles = (int)((n + tile - 1) / tile);
    int *pairs1 = plan_ws;  // (id, row) after the bucket scatter, 8-byte aligned
    int *hist = plan_ws + 2 * n;
    const long used = (long)high_bins * n_tiles;
    int *tile_flags = hist + used + 1;
    int *bucket_start = tile_flags + n_tiles;
    int *scan_ws = bucket_start + high_bins + 1;
    // an upper bound of the (bucket, slice) pairs; workgroups beyond the last pair return at once
    const long groups = n / kBktSlice + high_bins;
    int *wg_pick = reinterpret_cast<int *>(  // 16-byte records
        ((uintptr_t)(scan_ws + scan_tiles(used + 1) + 17) + 15u) & ~(uintptr_t)15u);
    int *part_hist = wg_pick + 4 * groups;
    // (the attribute belongs to the current device's copy of a kernel: once per device)
    constexpr int kMaxDevices = 64;
    static std::atomic<bool> lds_allowed[kMaxDevices];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return TXS_ERR_LAUNCH;
    if (!lds_allowed[dev].load(std::memory_order_acquire)) {
        for (const void *k : {reinterpret_cast<const void *>(bucket_scatter_kernel<4>),
                              reinterpret_cast<const void *>(bucket_scatter_kernel<8>),
                              reinterpret_cast<const void *>(bucket_scatter_kernel<16>)})
            if (hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024) != hipSuccess)
                return TXS_ERR_LAUNCH;
        lds_allowed[dev].store(true, std::memory_order_release);
    }
    auto hist_kernel = items == 16 ? bucket_hist_kernel<16> : (items == 8 ? bucket_hist_kernel<8> : bucket_hist_kernel<4>);
    auto scatter_kernel =
        items == 16 ? bucket_scatter_kernel<16> : (items == 8 ? bucket_scatter_kernel<8> : bucket_scatter_kernel<4>);
    hist_kernel<<<dim3(n_tiles), dim3(kHistThreads), 0, st>>>(unq_inv, n, U, low_bits, high_bins, hist, tile_flags,
                                                              n_tiles);
    // one entry more than the histogram: it receives the total, the end of the last bucket
    if (exclusive_scan(hist, used, hist, used + 1, scan_ws, st) != hipSuccess) return TXS_ERR_LAUNCH;
    const size_t lds_scatter = (size_t)(kHistWaves + 1) * high_bins * sizeof(int);
    if (low_bits == 0) {
        // a bucket is a voxel: the scatter already gives the final order
        scatter_kernel<<<dim3(n_tiles), dim3(kHistThreads), lds_scatter, st>>>(
            unq_inv, n, U, low_bits, high_bits, hist, tile_flags, n_tiles, n + 1, bucket_start, stats, seg, perm,
            nullptr);
        int rc = txs_plan_presum(seg, n, U, preSum, stream);
        if (slot_of == nullptr) return rc;
        if (rc == TXS_OK)
            rc = txs_plan_special(preSum, U, heavy_threshold, unq_cnts, slot_of, heavy_ids, stats, nullptr, nullptr,
                                  stream);
        if (rc == TXS_OK) rc = txs_plan_seg_flag(seg, n, U, slot_of, stream);
        return rc;
    }
    // a bucket so full that its workgroups would run long after all others have finished
    // (only a few voxels holding most of the rows do that) sends the call to the general sequence
    const long giant = kBktGiant;
    scatter_kernel<<<dim3(n_tiles), dim3(kHistThreads), lds_scatter, st>>>(
        unq_inv, n, U, low_bits, high_bits, hist, tile_flags, n_tiles, giant, bucket_start, stats, nullptr,
        nullptr, reinterpret_cast<int2 *>(pairs1));
    const int low_bins = 1 << low_bits;
    const size_t lds = (size_t)(kBktWaves + 2) * low_bins * sizeof(int);
    bucket_count_kernel<<<dim3((unsigned)groups), dim3(kThreads), (size_t)low_bins * sizeof(int), st>>>(
        unq_inv, pairs1, n, U, low_bits, high_bins, bucket_start, stats, reinterpret_cast<int4 *>(wg_pick), part_hist);
    bucket_plan_kernel<<<dim3((unsigned)groups), dim3(kThreads), lds, st>>>(
        unq_inv, pairs1, n, U, low_bits, high_bins, bucket_start, heavy_threshold,
        (const long long *)unq_cnts, perm, seg, preSum, slot_of, heavy_ids, stats,
        reinterpret_cast<const int4 *>(wg_pick), part_hist, ranks);
    return status_of(hipGetLastError());
}
