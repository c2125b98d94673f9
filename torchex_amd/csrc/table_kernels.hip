// Row-order kernels for inputs with few voxels ("table mode").
//
// When the whole [U, C] result fits in the LDS of one compute unit, the rows need not be
// visited in voxel order at all.  Forward: every workgroup streams a contiguous span of
// feature rows in the order they lie in memory (fully coalesced, no permutation, which
// matters most for rows narrower than a cache line), reduces them into a private [U, C]
// table in LDS with LDS atomics (fp64 add; 64-bit max on ordered(value)<<32 | ~row, so the
// smallest row wins ties), and stores its table as one partial; a second small kernel
// combines the partials of all workgroups in a fixed order and writes out / arg.  No
// global atomics, and nothing has to be zero on entry.  Backward: the upstream rows (and
// arg rows) are staged in LDS once per workgroup and every input-gradient row is produced
// in row order, so the large tensor is written sequentially.
//
// Replaces, for such inputs, the same reference code as the voxel-order kernels:
// torchex/src/scatter/scatter_kernel.cu:102-171 and the backward arithmetic of
// torchex/operator_py/scatter_op.py:47-50,74-78,106-111.

#include "txs_common.h"

#include <atomic>

namespace {

constexpr int kTableThreads = 1024;          // one workgroup per compute unit
constexpr int kTableLdsBudget = 144 * 1024;  // bytes of LDS a table may take (160 KB per CU on gfx950)
#ifndef TXS_TABLE_MAX_WGS
#define TXS_TABLE_MAX_WGS 1024
#endif
#ifndef TXS_TABLE_NT_LOADS
#define TXS_TABLE_NT_LOADS 1
#endif
#ifndef TXS_TABLE_NT_STORES
#define TXS_TABLE_NT_STORES 0
#endif
#ifndef TXS_TABLE_UNROLL
#define TXS_TABLE_UNROLL 2
#endif
#ifndef TXS_TABLE_HALF_SUM_VB
#define TXS_TABLE_HALF_SUM_VB 4
#endif
#ifndef TXS_TABLE_MAX_PREFILTER
#define TXS_TABLE_MAX_PREFILTER 1
#endif
constexpr int kTableUnroll = TXS_TABLE_UNROLL;  // rows per lane in flight (twice as many for lanes of 4 bytes or less in the forward)
constexpr int kReduceThreads = 1024;
constexpr int kReduceSplit = 32;             // lanes that share the partials of one output cell
#ifndef TXS_REDUCE_LOADS
#define TXS_REDUCE_LOADS 4
#endif
constexpr int kReduceLoads = TXS_REDUCE_LOADS;  // partials each of them has in flight

// ------------------------------------------------------------------ forward --
//
// LDS cells are 8 bytes for every operator: a packed (ordered value, ~row) word for max,
// a double for sum / mean.  The fp64 cell is a matter of speed, not of accuracy: on this
// part an LDS fp32 atomic add retires about one lane every three cycles, whatever the
// addresses, while fp64 and integer LDS atomics run seven times faster (2M rows of 16
// channels into 1024 voxels: 164 us with fp32 cells, 26 us with fp64 cells, 20 us for the
// load stream alone).  A workgroup's partial is stored as fp32 (sum / mean) or, for max, as
// two 4-byte cells in separate planes: the ordered value and the winner's row.

template <class TR, int VEC, int OP>
__global__ __launch_bounds__(kTableThreads) void table_fwd_kernel(
    const typename TR::raw *__restrict__ feats, const int *__restrict__ inv,
    void *__restrict__ partials, int N, int C, int U, int lpr_log2, int stride, int rows_per_wg) {
    using raw = typename TR::raw;
    constexpr bool kMax = OP == TXS_MAX;
    constexpr int kRows = sizeof(raw) * VEC <= 4 ? 2 * kTableUnroll : kTableUnroll;  // rows per lane in flight
    extern __shared__ unsigned long long table_lds[];
    unsigned long long *tkey = table_lds;
    double *tsum = reinterpret_cast<double *>(table_lds);
    const int cells = U * stride;

    const int lane_in = (int)threadIdx.x & ((1 << lpr_log2) - 1);
    const int g = (int)threadIdx.x >> lpr_log2;
    const int G = kTableThreads >> lpr_log2;
    const int col = lane_in * VEC;
    const long r0 = (long)blockIdx.x * rows_per_wg;
    const int r_end = (int)min((long)N, r0 + rows_per_wg);
    {
        // Two batches of kRows rows per lane: the next one is on its way from memory
        // while the current one goes into the table.
        struct Batch {
            int u[kRows];
            Pack<raw, VEC> v[kRows];
        };
        const int step = G * kRows;
        auto issue = [&](Batch &b, int rb) {
#pragma unroll
            for (int k = 0; k < kRows; ++k) {
                const int r = min(rb + k * G, r_end - 1);  // slots past the span re-load its last row
                b.u[k] = inv[r] & kIdMask;
                b.v[k] = TXS_TABLE_NT_LOADS ? ld_stream<raw, VEC>(feats + (size_t)r * C + col) : ld<raw, VEC>(feats + (size_t)r * C + col);
            }
        };
        auto consume = [&](const Batch &b, int rb) {
#pragma unroll
            for (int k = 0; k < kRows; ++k) {
                const int r = rb + k * G;
                if (r >= r_end || (unsigned)b.u[k] >= (unsigned)U) continue;
                const int cell = b.u[k] * stride + col;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float x = TR::to_f(b.v[k].v[e]);
                    if constexpr (kMax) {
                        // A cell only ever grows, so a key that does not beat a plain (possibly
                        // stale) read of it cannot change it: after a voxel's first few rows
                        // almost every row stops at the read, which costs a fraction of the atomic.
                        const unsigned long long key = ((unsigned long long)ordered_bits(x) << 32) |
                                                       (unsigned long long)(0xffffffffu - (unsigned)r);
                        const bool beats = !(TXS_TABLE_MAX_PREFILTER && sizeof(raw) == 2) ||
                            key > __hip_atomic_load(tkey + cell + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                        if (x == x && beats)  // NaN never wins
                            __hip_atomic_fetch_max(tkey + cell + e, key, __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_WORKGROUP);
                    } else {
                        __hip_atomic_fetch_add(tsum + cell + e, (double)x, __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_WORKGROUP);
                    }
                }
            }
        };
        int rb = (int)r0 + g;
        const bool act = col < C && rb < r_end;
        Batch b0, b1;
        if (act) issue(b0, rb);  // the first rows are on their way while the table is cleared
        for (int i = threadIdx.x; i < cells; i += kTableThreads) tkey[i] = 0ull;  // +0.0 as a double
        __syncthreads();
        if (act) {
            for (;;) {
                if (rb + step >= r_end) {
                    consume(b0, rb);
                    break;
                }
                issue(b1, rb + step);
                consume(b0, rb);
                rb += step;
                if (rb + step >= r_end) {
                    consume(b1, rb);
                    break;
                }
                issue(b0, rb + step);
                consume(b1, rb);
                rb += step;
            }
        }
    }
    __syncthreads();
    // this workgroup's partial: [U, C], dense; four cells per lane and store where the row
    // length and the partial's address allow 16-byte stores
    const int total = U * C;
    const bool wide = (C & 3) == 0 && (reinterpret_cast<size_t>(partials) & 15) == 0;
    if constexpr (kMax) {
        // two planes of 4-byte cells: the ordered values of all workgroups first (all that the
        // second kernel reads to find the winning partial), the winners' rows behind them
        unsigned *pval = reinterpret_cast<unsigned *>(partials) + (size_t)blockIdx.x * total;
        unsigned *prow = reinterpret_cast<unsigned *>(partials) + ((size_t)gridDim.x + blockIdx.x) * total;
        if (wide) {
            for (int i = (int)threadIdx.x * 4; i < total; i += kTableThreads * 4) {
                const int uu = i / C;
                const unsigned long long *t = tkey + uu * stride + (i - uu * C);
                Pack<unsigned, 4> v, r;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v.v[e] = (unsigned)(t[e] >> 32);
                    r.v[e] = 0xffffffffu - (unsigned)(t[e] & 0xffffffffull);
                }
                st<unsigned, 4>(pval + i, v);
                st<unsigned, 4>(prow + i, r);
            }
        } else {
            for (int i = threadIdx.x; i < total; i += kTableThreads) {
                const int uu = i / C;
                const unsigned long long key = tkey[uu * stride + (i - uu * C)];
                pval[i] = (unsigned)(key >> 32);
                prow[i] = 0xffffffffu - (unsigned)(key & 0xffffffffull);
            }
        }
    } else {
        float *part = reinterpret_cast<float *>(partials) + (size_t)blockIdx.x * total;
        if (wide) {
            for (int i = (int)threadIdx.x * 4; i < total; i += kTableThreads * 4) {
                const int uu = i / C;
                const double *t = tsum + uu * stride + (i - uu * C);
                Pack<float, 4> v;
#pragma unroll
                for (int e = 0; e < 4; ++e) v.v[e] = (float)t[e];
                st<float, 4>(part + i, v);
            }
        } else {
            for (int i = threadIdx.x; i < total; i += kTableThreads) {
                const int uu = i / C;
                part[i] = (float)tsum[uu * stride + (i - uu * C)];
            }
        }
    }
}

// out / arg from the partial tables: one output cell per group of kReduceSplit lanes, the
// partials combined in workgroup order (a fixed order: for a given launch geometry only
// the order of the atomic adds inside a workgroup varies from run to run).
template <class TR, int OP>
__global__ __launch_bounds__(kReduceThreads) void table_reduce_kernel(
    const typename TR::raw *__restrict__ feats, const void *__restrict__ partials,
    const int *__restrict__ preSum, typename TR::raw *__restrict__ out, int *__restrict__ arg,
    int num_parts, int N, int C, int U) {
    constexpr bool kMax = OP == TXS_MAX;
    using Cell = typename std::conditional<kMax, unsigned, float>::type;  // as the forward stored it
    // max: (ordered value) << 32 | ~workgroup: the largest value wins, among equal values the
    // first workgroup, whose rows all come before those of the workgroups behind it
    using Acc = typename std::conditional<kMax, unsigned long long, double>::type;
    constexpr int kSplit = kReduceSplit;  // a wave reads whole 128-byte lines of a partial: 32 cells
    constexpr int kCellsPerWg = kReduceThreads / kSplit;
    __shared__ Acc part_s[kSplit][kCellsPerWg];
    const int cl = (int)threadIdx.x % kCellsPerWg, wl = (int)threadIdx.x / kCellsPerWg;
    const long cell = (long)blockIdx.x * kCellsPerWg + cl;
    const long total = (long)U * C;
    const Cell *p = reinterpret_cast<const Cell *>(partials);
    Acc acc = Acc(0);
    if (cell < total) {
        // kReduceLoads independent loads in flight per lane
        for (int w0 = wl; w0 < num_parts; w0 += kSplit * kReduceLoads) {
            Cell x[kReduceLoads];
#pragma unroll
            for (int k = 0; k < kReduceLoads; ++k) {
                const int w = w0 + k * kSplit;
                x[k] = w < num_parts ? p[(size_t)w * total + cell] : Cell(0);
            }
#pragma unroll
            for (int k = 0; k < kReduceLoads; ++k) {
                if constexpr (kMax) {
                    const Acc key = ((Acc)x[k] << 32) | (Acc)(0xffffffffu - (unsigned)(w0 + k * kSplit));
                    acc = key > acc ? key : acc;
                } else {
                    acc += (Acc)x[k];
                }
            }
        }
    }
    part_s[wl][cl] = acc;
    __syncthreads();
    // second level in a fixed order: lanes 0..7 of a cell each fold an eighth of the values, lane 0 folds those
    constexpr int kFold = kSplit / 8;
    if (wl < 8) {
        acc = part_s[wl * kFold][cl];
#pragma unroll
        for (int k = 1; k < kFold; ++k) {
            const Acc x = part_s[wl * kFold + k][cl];
            if constexpr (kMax) acc = x > acc ? x : acc; else acc += x;
        }
    }
    __syncthreads();
    if (wl < 8) part_s[wl][cl] = acc;
    __syncthreads();
    if (wl != 0 || cell >= total) return;
#pragma unroll
    for (int k = 1; k < 8; ++k) {
        const Acc x = part_s[k][cl];
        if constexpr (kMax) acc = x > acc ? x : acc; else acc += x;
    }
    const int u = (int)(cell / C), c = (int)(cell - (long)u * C);
    if constexpr (kMax) {
        const unsigned val = (unsigned)(acc >> 32);  // 0: no partial holds a value for this cell
        const unsigned w = 0xffffffffu - (unsigned)(acc & 0xffffffffull);
        const unsigned row = (val != 0u && w < (unsigned)num_parts)
                                 ? reinterpret_cast<const unsigned *>(partials)[((size_t)num_parts + w) * total + cell]
                                 : 0xffffffffu;
        if (row >= (unsigned)N) {  // no rows, or only NaN: the reference's init pair
            out[cell] = TR::lowest();
            arg[cell] = -1;
        } else {
            // the key carries the winning value; only the sign of a zero is read back from the winner
            const float x = from_ordered_bits((unsigned)(acc >> 32));
            out[cell] = x == 0.0f ? feats[(size_t)row * C + c] : TR::from_f(x);
            arg[cell] = (int)row;
        }
    } else {
        float s = (float)acc;
        if (OP == TXS_MEAN) s = s / (float)(preSum[u + 1] - preSum[u]);  // 0/0 for an empty voxel, as the reference
        out[cell] = TR::from_f(s);
    }
}

// ----------------------------------------------------------------- backward --

template <class TR, int VEC, int OP>
__global__ __launch_bounds__(kTableThreads) void table_bwd_kernel(
    const typename TR::raw *__restrict__ g, const int *__restrict__ arg, const int *__restrict__ inv,
    const int *__restrict__ preSum, typename TR::raw *__restrict__ gin, int N, int C, int U,
    int lpr_log2, int stride, int rows_per_wg) {
    using raw = typename TR::raw;
    extern __shared__ unsigned long long table_lds[];
    raw *gt = reinterpret_cast<raw *>(table_lds);
    // arg rows follow the upstream rows, 32-byte aligned
    int *at = reinterpret_cast<int *>(reinterpret_cast<char *>(table_lds) +
                                      (((size_t)U * stride * sizeof(raw) + 31) & ~(size_t)31));
    const int lane_in = (int)threadIdx.x & ((1 << lpr_log2) - 1);
    const int grp = (int)threadIdx.x >> lpr_log2;
    const int G = kTableThreads >> lpr_log2;
    const int col = lane_in * VEC;
    const long r0 = (long)blockIdx.x * rows_per_wg;
    const int r_end = (int)min((long)N, r0 + rows_per_wg);
    // the voxel ids of the next batch of rows are fetched while the current batch is written
    // (and those of the first batch while the tables are staged)
    const int step = G * kTableUnroll;
    auto issue = [&](int (&u)[kTableUnroll], int rb) {
#pragma unroll
        for (int k = 0; k < kTableUnroll; ++k) u[k] = inv[min(rb + k * G, r_end - 1)] & kIdMask;
    };
    int rb = (int)r0 + grp;
    const bool act = col < C && rb < r_end;
    int u0[kTableUnroll], u1[kTableUnroll];
    if (act) issue(u0, rb);

    const int total = U * C;
    constexpr int kStage = 4;  // independent loads per lane while the tables are staged
    // one cell of the staged tables: upstream value (mean: divided by the voxel's count, one
    // division per output cell as (g / unq_cnts) in the reference) and, for max, the winner
    auto staged = [&](raw x, int cnt) -> raw {
        return OP == TXS_MEAN ? TR::from_f(TR::to_f(x) / (float)cnt) : x;
    };
    if constexpr (VEC * sizeof(raw) >= 4) {
        // VEC cells per lane and load (C is a multiple of VEC and every tensor is aligned to
        // the lane's bytes; arg rows, 4 bytes per cell, go in pieces of that many bytes)
        constexpr int kArgPiece = VEC * (int)sizeof(raw) / 4;  // ints per piece
        constexpr int kArgPieces = VEC / kArgPiece;
        for (int i0 = (int)threadIdx.x * VEC; i0 < total; i0 += kTableThreads * VEC * kStage) {
            Pack<raw, VEC> x[kStage];
            Pack<int, kArgPiece> a[kStage][kArgPieces];
            int cnt[kStage], uu[kStage];
#pragma unroll
            for (int k = 0; k < kStage; ++k) {
                const int i = min(i0 + k * kTableThreads * VEC, total - VEC);
                uu[k] = i / C;
                x[k] = ld<raw, VEC>(g + i);
                if (OP == TXS_MEAN) cnt[k] = preSum[uu[k] + 1] - preSum[uu[k]];
                if (OP == TXS_MAX) {
#pragma unroll
                    for (int q = 0; q < kArgPieces; ++q) a[k][q] = ld<int, kArgPiece>(arg + i + q * kArgPiece);
                }
            }
#pragma unroll
            for (int k = 0; k < kStage; ++k) {
                const int i = i0 + k * kTableThreads * VEC;
                if (i >= total) break;
                const int cell = uu[k] * stride + (i - uu[k] * C);
#pragma unroll
                for (int e = 0; e < VEC; ++e) x[k].v[e] = staged(x[k].v[e], OP == TXS_MEAN ? cnt[k] : 1);
                st<raw, VEC>(gt + cell, x[k]);
                if (OP == TXS_MAX) {
#pragma unroll
                    for (int q = 0; q < kArgPieces; ++q) st<int, kArgPiece>(at + cell + q * kArgPiece, a[k][q]);
                }
            }
        }
    } else {
        for (int i0 = threadIdx.x; i0 < total; i0 += kTableThreads * kStage) {
            raw x[kStage];
            int a[kStage], cnt[kStage], uu[kStage];
#pragma unroll
            for (int k = 0; k < kStage; ++k) {
                const int i = min(i0 + k * kTableThreads, total - 1);
                uu[k] = i / C;
                x[k] = g[i];
                if (OP == TXS_MEAN) cnt[k] = preSum[uu[k] + 1] - preSum[uu[k]];
                if (OP == TXS_MAX) a[k] = arg[i];
            }
#pragma unroll
            for (int k = 0; k < kStage; ++k) {
                const int i = i0 + k * kTableThreads;
                if (i >= total) break;
                const int c = i - uu[k] * C;
                gt[uu[k] * stride + c] = staged(x[k], OP == TXS_MEAN ? cnt[k] : 1);
                if (OP == TXS_MAX) at[uu[k] * stride + c] = a[k];
            }
        }
    }
    __syncthreads();

    if (!act) return;
    auto emit = [&](const int (&u)[kTableUnroll], int rb) {
#pragma unroll
        for (int k = 0; k < kTableUnroll; ++k) {
            const int r = rb + k * G;
            if (r >= r_end) continue;
            Pack<raw, VEC> o;
            if ((unsigned)u[k] < (unsigned)U) {
                o = *reinterpret_cast<const Pack<raw, VEC> *>(gt + u[k] * stride + col);
                if (OP == TXS_MAX) {
                    const Pack<int, VEC> a = *reinterpret_cast<const Pack<int, VEC> *>(at + u[k] * stride + col);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) o.v[e] = (a.v[e] == r) ? o.v[e] : TR::zero();
                }
            } else {
#pragma unroll
                for (int e = 0; e < VEC; ++e) o.v[e] = TR::zero();
            }
            if (TXS_TABLE_NT_STORES) st_stream<raw, VEC>(gin + (size_t)r * C + col, o); else st<raw, VEC>(gin + (size_t)r * C + col, o);
        }
    };
    for (;;) {
        if (rb + step >= r_end) {
            emit(u0, rb);
            break;
        }
        issue(u1, rb + step);
        emit(u0, rb);
        rb += step;
        if (rb + step >= r_end) {
            emit(u1, rb);
            break;
        }
        issue(u0, rb + step);
        emit(u1, rb);
        rb += step;
    }
}

// ------------------------------------------------------------------- launch --

// Compute units of the current device (looked up once per device and kept: the only state
// this translation unit holds besides the per-kernel "large LDS allowed" flags).
constexpr int kMaxDevices = 64;
int compute_units() {
    static std::atomic<int> cus[kMaxDevices];  // 0 = not asked yet
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
    int n = cus[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cus[dev].store(n, std::memory_order_relaxed);  // every thread that races here stores the same value
    }
    return n;
}

int table_workgroups(long N) {
    const int cus = compute_units();
    // at least 4096 rows per workgroup: a partial table costs as much as its rows otherwise
    long w = (N + 4095) / 4096;
    const long most = cus < TXS_TABLE_MAX_WGS ? cus : TXS_TABLE_MAX_WGS;
    return (int)(w < 1 ? 1 : (w > most ? most : w));
}

// Tables above 64 KB need the kernel's dynamic-LDS limit raised; the attribute belongs to the
// current device's copy of the kernel, so it is set once per (instantiation, device).
template <class K>
hipError_t allow_lds(K kernel, std::atomic<bool> (&done)[kMaxDevices]) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    if (done[dev].load(std::memory_order_acquire)) return hipSuccess;
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, kTableLdsBudget);
    if (e == hipSuccess) done[dev].store(true, std::memory_order_release);
    return e;
}

template <class TR, int VEC, int OP>
hipError_t launch_table_fwd(const txs_detail::TablePlan &tp, hipStream_t st, const void *feats,
                            const int *inv, const int *preSum, void *partials, void *out, int *arg,
                            int N, int C, int U) {
    using raw = typename TR::raw;
    auto kernel = table_fwd_kernel<TR, VEC, OP>;
    static std::atomic<bool> lds_allowed[kMaxDevices];  // per instantiation and device
    if (allow_lds(kernel, lds_allowed) != hipSuccess) return hipErrorInvalidValue;
    kernel<<<dim3(tp.workgroups), dim3(kTableThreads), tp.lds_bytes, st>>>(
        (const raw *)feats, inv, partials, N, C, U, tp.lpr_log2, tp.stride, tp.rows_per_wg);
    const long total = (long)U * C;
    constexpr int kCellsPerWg = kReduceThreads / kReduceSplit;
    table_reduce_kernel<TR, OP><<<dim3((unsigned)((total + kCellsPerWg - 1) / kCellsPerWg)), dim3(kReduceThreads), 0, st>>>(
        (const raw *)feats, partials, preSum, (raw *)out, arg, tp.workgroups, N, C, U);
    return hipGetLastError();
}

template <class TR, int VEC>
hipError_t launch_table_fwd_op(int op, const txs_detail::TablePlan &tp, hipStream_t st, const void *feats,
                               const int *inv, const int *preSum, void *partials, void *out, int *arg,
                               int N, int C, int U) {
    switch (op) {
        case TXS_SUM: return launch_table_fwd<TR, VEC, TXS_SUM>(tp, st, feats, inv, preSum, partials, out, arg, N, C, U);
        case TXS_MEAN: return launch_table_fwd<TR, VEC, TXS_MEAN>(tp, st, feats, inv, preSum, partials, out, arg, N, C, U);
        default: return launch_table_fwd<TR, VEC, TXS_MAX>(tp, st, feats, inv, preSum, partials, out, arg, N, C, U);
    }
}

template <class TR, int VEC, int OP>
hipError_t launch_table_bwd(const txs_detail::TablePlan &tp, hipStream_t st, const void *g, const int *arg,
                            const int *inv, const int *preSum, void *gin, int N, int C, int U) {
    using raw = typename TR::raw;
    auto kernel = table_bwd_kernel<TR, VEC, OP>;
    static std::atomic<bool> lds_allowed[kMaxDevices];
    if (allow_lds(kernel, lds_allowed) != hipSuccess) return hipErrorInvalidValue;
    kernel<<<dim3(tp.workgroups), dim3(kTableThreads), tp.lds_bytes, st>>>(
        (const raw *)g, arg, inv, preSum, (raw *)gin, N, C, U, tp.lpr_log2, tp.stride, tp.rows_per_wg);
    return hipGetLastError();
}

template <class TR, int VEC>
hipError_t launch_table_bwd_op(int op, const txs_detail::TablePlan &tp, hipStream_t st, const void *g,
                               const int *arg, const int *inv, const int *preSum, void *gin, int N, int C,
                               int U) {
    switch (op) {
        case TXS_SUM: return launch_table_bwd<TR, VEC, TXS_SUM>(tp, st, g, arg, inv, preSum, gin, N, C, U);
        case TXS_MEAN: return launch_table_bwd<TR, VEC, TXS_MEAN>(tp, st, g, arg, inv, preSum, gin, N, C, U);
        default: return launch_table_bwd<TR, VEC, TXS_MAX>(tp, st, g, arg, inv, preSum, gin, N, C, U);
    }
}

// elements per lane: the widest vector (16 bytes at most) that divides a row and fits the
// alignment of every tensor involved
int table_vec_bytes(long C, int elem, long align) {
    int vb = 16;
    while (vb > elem && ((C * elem) % vb != 0 || align % vb != 0)) vb >>= 1;
    return vb;
}

}  // namespace

namespace txs_detail {

TablePlan table_plan(bool backward, int op, int dtype, long N, long C, long U, long align) {
    TablePlan tp{};
    if (op == TXS_MAX_REFTIE && !backward) return tp;  // the reference's tie key needs voxel order
    if (op == TXS_MAX_REFTIE) op = TXS_MAX;
    if (N <= 0 || C <= 0 || U <= 0) return tp;
    if (N > 0x7fffffffL - (1L << 16)) return tp;  // the row loops step past the end in 32-bit arithmetic
    // few voxels, many rows each: a partial table per workgroup must stay small next to its rows
    if (N < (long)kTableMinRowsPerVoxel * U || N < 16384) return tp;
    const int elem = dtype == TXS_F32 ? 4 : 2;
    int vb = table_vec_bytes(C, elem, align);
    // 2-byte sum / mean: 4-byte lanes.  Wide lanes put many rows into one LDS atomic instruction,
    // and rows of one voxel in the same instruction are served one after the other (2M rows of
    // 16 channels into 1024 Zipf-distributed voxels: 42 us with 16-byte lanes, 35 with 8, 29
    // with 4); fp32 rows, which take twice as long to stream, gain nothing from narrower lanes.
    if (!backward && op != TXS_MAX && elem == 2)
        while (vb > TXS_TABLE_HALF_SUM_VB && C * elem / (vb / 2) <= 64) vb /= 2;
    const int vec = vb / elem;
    const long lanes = (C + vec - 1) / vec;
    if (lanes > 64) return tp;
    int l2 = 0;
    while ((1L << l2) < lanes) ++l2;
    long bytes, stride;
    if (!backward) {
        const long cell = 8;  // every operator keeps 8-byte cells in LDS
        stride = C + 1;  // odd number of cells per table row: lanes of different rows spread over the banks
        bytes = U * stride * cell;
        if (bytes > kTableLdsBudget) {
            stride = C;
            bytes = U * stride * cell;
        }
    } else {
        stride = C + vec;  // keeps every row's vectors aligned
        bytes = ((U * stride * elem + 31) & ~31L) + (op == TXS_MAX ? U * stride * 4 : 0);
        if (bytes > kTableLdsBudget) {
            stride = C;
            bytes = ((U * stride * elem + 31) & ~31L) + (op == TXS_MAX ? U * stride * 4 : 0);
        }
    }
    if (bytes > kTableLdsBudget) return tp;
    tp.use = true;
    tp.vec_bytes = vb;
    tp.lpr_log2 = l2;
    tp.stride = (int)stride;
    tp.lds_bytes = (unsigned)((bytes + 15) & ~15L);
    tp.workgroups = table_workgroups(N);
    tp.rows_per_wg = (int)((N + tp.workgroups - 1) / tp.workgroups);
    tp.partial_cells = backward ? 0 : (long)tp.workgroups * U * C;
    return tp;
}

long table_partial_cells(long N, long C, long U) {
    // capacity for whichever operator and dtype asks for the most (8-byte cells either way)
    long most = 0;
    for (int op = TXS_SUM; op <= TXS_MAX; ++op)
        for (int dt = TXS_F32; dt <= TXS_BF16; ++dt) {
            const TablePlan tp = table_plan(false, op, dt, N, C, U, 16);
            if (tp.use && tp.partial_cells > most) most = tp.partial_cells;
        }
    return most;
}

hipError_t table_forward(const TablePlan &tp, int op, int dtype, hipStream_t st, const void *feats,
                         const int *inv, const int *preSum, void *partials, void *out, int *arg, int N,
                         int C, int U) {
#define TXS_TAB(TR, VB)                                                                                  \
    if (tp.vec_bytes == VB)                                                                              \
        return launch_table_fwd_op<TR, (VB) / (int)sizeof(typename TR::raw)>(op, tp, st, feats, inv, preSum, \
                                                                             partials, out, arg, N, C, U);
    if (dtype == TXS_F32) {
        TXS_TAB(F32, 16) TXS_TAB(F32, 8) TXS_TAB(F32, 4)
    } else if (dtype == TXS_F16) {
        TXS_TAB(F16, 16) TXS_TAB(F16, 8) TXS_TAB(F16, 4) TXS_TAB(F16, 2)
    } else {
        TXS_TAB(BF16, 16) TXS_TAB(BF16, 8) TXS_TAB(BF16, 4) TXS_TAB(BF16, 2)
    }
#undef TXS_TAB
    return hipErrorInvalidValue;
}

hipError_t table_backward(const TablePlan &tp, int op, int dtype, hipStream_t st, const void *g,
                          const int *arg, const int *inv, const int *preSum, void *gin, int N, int C, int U) {
#define TXS_TAB(TR, VB)                                                                                  \
    if (tp.vec_bytes == VB)                                                                              \
        return launch_table_bwd_op<TR, (VB) / (int)sizeof(typename TR::raw)>(op, tp, st, g, arg, inv, preSum, \
                                                                             gin, N, C, U);
    if (dtype == TXS_F32) {
        TXS_TAB(F32, 16) TXS_TAB(F32, 8) TXS_TAB(F32, 4)
    } else if (dtype == TXS_F16) {
        TXS_TAB(F16, 16) TXS_TAB(F16, 8) TXS_TAB(F16, 4) TXS_TAB(F16, 2)
    } else {
        TXS_TAB(BF16, 16) TXS_TAB(BF16, 8) TXS_TAB(BF16, 4) TXS_TAB(BF16, 2)
    }
#undef TXS_TAB
    return hipErrorInvalidValue;
}

}  // namespace txs_detail
