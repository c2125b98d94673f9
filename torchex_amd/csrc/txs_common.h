// Shared pieces of the voxel scatter library for MI355X (gfx950, wave64): build
// knobs, dtype traits, 128-bit lane vectors, workgroup scan, host-side helpers.
// Included by every translation unit of libtorchex_scatter.so; everything in the
// unnamed namespace is private to the unit that includes it.
#pragma once

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
#ifndef TXS_CHUNK_BWD_SHORT
#define TXS_CHUNK_BWD_SHORT 8
#endif
#ifndef TXS_BATCH
#define TXS_BATCH 4
#endif
#ifndef TXS_BATCH_BWD
#define TXS_BATCH_BWD TXS_BATCH
#endif
#ifndef TXS_BATCH_HALF
#define TXS_BATCH_HALF TXS_BATCH
#endif
#ifndef TXS_BATCH_BWD_HALF
#define TXS_BATCH_BWD_HALF 8
#endif
#ifndef TXS_HALF_VEC_BYTES
#define TXS_HALF_VEC_BYTES 8
#endif
#ifndef TXS_F16_NATIVE_MAX
#define TXS_F16_NATIVE_MAX 1
#endif
#ifndef TXS_F16_FMA_MIX
#define TXS_F16_FMA_MIX 1
#endif
#ifndef TXS_BATCH_HALF_MAX
#define TXS_BATCH_HALF_MAX 4
#endif
#ifndef TXS_BATCH_BF16_MAX
#define TXS_BATCH_BF16_MAX 8
#endif
#ifndef TXS_FAST_DIV_HALF
#define TXS_FAST_DIV_HALF 1
#endif
#ifndef TXS_NT_LOADS
#define TXS_NT_LOADS 1
#endif
#ifndef TXS_NT_STORES
#define TXS_NT_STORES 1
#endif

constexpr int kThreads = 256;        // 4 wavefronts per workgroup
constexpr int kChunk = TXS_CHUNK;    // sorted positions per lane group (forward)
constexpr int kChunkLong = 2 * TXS_CHUNK;  // the same when runs are long on average
constexpr int kChunkShort = TXS_CHUNK / 2;  // ... and for short runs of 4-byte elements
constexpr int kChunkBwdShort = TXS_CHUNK_BWD_SHORT;  // backward kernel, mean run shorter than kChunkBwdLong
constexpr int kChunkBwdLong = TXS_CHUNK;             // backward kernel, longer runs
constexpr int kBatchBwd = TXS_BATCH_BWD;
constexpr int kBatch = TXS_BATCH;    // rows per load batch of a lane group (two batches in flight)
constexpr int kBatchHalf = TXS_BATCH_HALF;         // the same for the 2-byte types
constexpr int kBatchBwdHalf = TXS_BATCH_BWD_HALF;
constexpr int kBatchHalfMax = TXS_BATCH_HALF_MAX;  // forward max of fp16
constexpr int kBatchBf16Max = TXS_BATCH_BF16_MAX;  // forward max of bf16
constexpr int kHalfVecBytes = TXS_HALF_VEC_BYTES;  // bytes one lane moves per row for fp16 / bf16
constexpr int kHeavyDefault = 64;    // voxels above this many rows use the atomic path
constexpr int kTableMinRowsPerVoxel = 512;  // table mode needs at least this many rows per voxel on average
constexpr int kSpecialBit = (int)0x80000000;
constexpr int kIdMask = 0x7fffffff;

// ------------------------------------------------------------------ dtypes --

struct F32 {
    using raw = float;
    static __device__ __forceinline__ float to_f(raw x) { return x; }
    static __device__ __forceinline__ raw from_f(float x) { return x; }
    static __device__ __forceinline__ raw lowest() { return -3.402823466e+38f; }
    static __device__ __forceinline__ raw zero() { return 0.0f; }
    // type a running max is kept and compared in (exact for every value of raw)
    using max_t = float;
    static __device__ __forceinline__ max_t to_m(raw x) { return x; }
    static __device__ __forceinline__ raw from_m(max_t x) { return x; }
};
struct F16 {
    using raw = _Float16;
    static __device__ __forceinline__ float to_f(raw x) { return (float)x; }
    static __device__ __forceinline__ raw from_f(float x) { return (_Float16)x; }  // RNE
    static __device__ __forceinline__ raw lowest() { return (_Float16)(-65504.0f); }
    static __device__ __forceinline__ raw zero() { return (_Float16)0.0f; }
#if TXS_F16_NATIVE_MAX
    using max_t = _Float16;  // compared with the 16-bit compare instructions, no widening
    static __device__ __forceinline__ max_t to_m(raw x) { return x; }
    static __device__ __forceinline__ raw from_m(max_t x) { return x; }
#else
    using max_t = float;
    static __device__ __forceinline__ max_t to_m(raw x) { return (float)x; }
    static __device__ __forceinline__ raw from_m(max_t x) { return (_Float16)x; }
#endif
};
struct BF16 {
    using raw = unsigned short;
    static __device__ __forceinline__ float to_f(raw x) {
        return __uint_as_float(((unsigned)x) << 16);
    }
    static __device__ __forceinline__ raw from_f(float x) {
        // round to nearest even in hardware (v_cvt_pk_bf16_f32 on gfx950); NaN stays NaN
        return __builtin_bit_cast(unsigned short, (__bf16)x);
    }
    static __device__ __forceinline__ raw lowest() { return (raw)0xff7f; }
    static __device__ __forceinline__ raw zero() { return (raw)0; }
    using max_t = float;
    static __device__ __forceinline__ max_t to_m(raw x) { return to_f(x); }
    static __device__ __forceinline__ raw from_m(max_t x) { return from_f(x); }
};

// acc + (float)half taken from the low / high 16 bits of a packed word, in one instruction
// (the mixed-precision FMA: half operand times 1.0f plus an fp32 accumulator; the product is
// exact, so the result is the correctly rounded fp32 sum, as a widening followed by an add)
__device__ __forceinline__ float add_f16_lo(float acc, unsigned packed) {
    float r;
    asm("v_fma_mix_f32 %0, %1, 1.0, %2 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "=v"(r) : "v"(packed), "v"(acc));
    return r;
}
__device__ __forceinline__ float add_f16_hi(float acc, unsigned packed) {
    float r;
    asm("v_fma_mix_f32 %0, %1, 1.0, %2 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(r) : "v"(packed), "v"(acc));
    return r;
}

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

// inverse of ordered_bits (a zero comes back as +0.0)
__device__ __forceinline__ float from_ordered_bits(unsigned r) {
    return __uint_as_float((r & 0x80000000u) ? (r ^ 0x80000000u) : ~r);
}

// ----------------------------------------------------------- workgroup scan --

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

// ------------------------------------------------------------- host helpers --

int status_of(hipError_t e) { return e == hipSuccess ? TXS_OK : TXS_ERR_LAUNCH; }

// extents are int32 on the device; the margin (more than the largest tile, 256 lane groups
// of 32 positions, plus its look-ahead) keeps position arithmetic from wrapping
bool fits_i32(int64_t x) { return x >= 0 && x < 2147483647LL - 32768; }

unsigned blocks_for(long n, int per = kThreads) { return (unsigned)((n + per - 1) / per); }

}  // namespace

// Functions one translation unit provides to the others (defined in plan_kernels.hip).
namespace txs_detail {

// Number of int32 workspace entries exclusive_scan needs for n_out outputs.
long scan_tiles(long n_out);

// out[i] = sum_{k<i} in[k] for i in [0, n_out), where in[k] = 0 for k >= n_in; in
// and out may alias.  Three launches on `st`, no inter-block waiting.
hipError_t exclusive_scan(const int *in, long n_in, int *out, long n_out, int *ws, hipStream_t st);


// txs_plan_build with one more output (plan_kernels.hip): ranks != NULL asks for the rank of
// every row inside its voxel instead of the permutation and the per-position ids; only the
// bucket kernels write it, which plan_writes_ranks() predicts from the extents.
int plan_build(const int32_t *unq_inv, int64_t num_total, int64_t num_unq, int32_t heavy_threshold,
               const int64_t *unq_cnts, int32_t *plan_ws, int32_t *perm, int32_t *seg, int32_t *preSum,
               int32_t *slot_of, int32_t *heavy_ids, int32_t *stats, long long *ranks, void *stream);
bool plan_writes_ranks(long num_total, long num_unq);

// Row-order "table mode" for inputs with few voxels (table_kernels.hip): whether it
// applies to a call and with which launch geometry.
struct TablePlan {
    bool use;            // false: the call takes the voxel-order kernels
    int vec_bytes;       // bytes one lane moves per row
    int lpr_log2;        // log2(lanes per row)
    int stride;          // cells (forward) or elements (backward) per table row in LDS
    unsigned lds_bytes;  // dynamic LDS per workgroup
    int workgroups, rows_per_wg;
    long partial_cells;  // 8-byte cells of workspace the forward needs for its partial tables
};
// `align`: alignment in bytes shared by every tensor of the call (a power of two).
TablePlan table_plan(bool backward, int op, int dtype, long N, long C, long U, long align);
// Workspace (8-byte cells) that lets any operator / dtype of these extents run in table mode; 0 if none can.
long table_partial_cells(long N, long C, long U);
hipError_t table_forward(const TablePlan &tp, int op, int dtype, hipStream_t st, const void *feats,
                         const int *inv, const int *preSum, void *partials, void *out, int *arg, int N,
                         int C, int U);
hipError_t table_backward(const TablePlan &tp, int op, int dtype, hipStream_t st, const void *g,
                          const int *arg, const int *inv, const int *preSum, void *gin, int N, int C, int U);

}  // namespace txs_detail
