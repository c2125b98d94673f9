// Voxel scatter-reduction kernels for MI355X (gfx950, wave64) and their C ABI.
//
// Design in one paragraph.  Index preparation sorts row ids by voxel id once
// and stores, for every sorted position j, the row perm[j] and the voxel seg[j].
// The forward pass is then a segmented reduction over sorted positions: a "lane
// group" (the lanes that together cover one feature row, each lane owning one
// 128-bit channel vector) keeps the running sum / max of the current voxel in
// registers and writes a voxel's output row exactly once when its run of equal
// ids ends.  A workgroup owns a tile of positions whose borders are moved to the
// next run start, so that an ordinary voxel lies in one tile, and deals the tile's
// rows evenly to its lane groups: all lane groups of a wavefront walk the same
// number of rows.  A run that crosses the border between two lane groups is
// completed after one barrier: the earlier group leaves its part in LDS, the group
// that holds the run's end adds it.  Only voxels above the heavy threshold are
// split across tiles; their per-tile partials meet in a scratch table through one
// fp32 atomic add (sum/mean) or one 64-bit atomic max on a packed (ordered value |
// ~row) word (max/argmax) per element and tile, and a small finalize kernel turns
// the table into output rows.  The backward pass is a gather over the same sorted
// positions: the upstream row of a voxel is read once per run and every row of the
// input gradient is written exactly once, with no zero-fill pass and no atomics.
// The same sort also serves the callers on either side of the path: voxel keys
// from points, the unique/inverse/counts triple, and the rank of a point inside
// its voxel.
//
// Reference behaviour being replaced: torchex/src/scatter/scatter_kernel.cu
// (getPreSum :85-100, scatter_sum :102-129, scatter_max :131-171) and the
// tensor arithmetic of torchex/operator_py/scatter_op.py (:47-50, :69, :74-78,
// :106-111).

#include "txs_common.h"

#include <stdio.h>

#include <initializer_list>
#include <mutex>

// Heavy-voxel table that lives in the library's own device image, for callers that cannot
// allocate device memory (code under HIP graph capture, tight serving loops): one copy
// per GPU, 8 MiB each, held until the process ends.  Host code never passes this name to
// a kernel: the device address is looked up once per GPU (resident_table() below) and
// that pointer is what kernels and the clearing launch receive.
constexpr long long kResidentCells = 1LL << 20;
static __device__ __align__(256) unsigned long long static_scratch[kResidentCells];

namespace {

// ----------------------------------------------------------------- forward --
//
// One workgroup owns a tile of G * chunk consecutive sorted positions (G = 256 /
// (lanes per row) lane groups).  The tile's seg and perm entries (plus one entry
// before and kMargin after) are staged in LDS by one coalesced load, so the row
// loads that follow never wait on an index load.  The tile's own range runs from
// the first run start at or after its first position to the first run start at or
// after the next tile's first position (a heavy run is cut anywhere): it is dealt
// to the lane groups in shares that differ by one row at most.  Measured on the
// LiDAR sweep before this: chunks of a fixed 16 positions whose owner skipped the
// tail of a run begun earlier and finished the run open at its end gave the lane
// groups 16 +- 9.7 rows, and a wavefront walked 39 % more rows than it reduced.
// Row loads are double-buffered: the next batch is in flight while the current one
// is reduced.

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

// Waves per SIMD the compiler has to make room for: the fp16 max/argmax kernel comes out at 84
// registers (allocated in eights: 5 waves) and is the one forward kernel that gains from a
// sixth (80 registers and three spilled dwords; pillar binning: 76-79 -> 73-75 us); asked of
// the fp32 max it spills in earnest (152 -> 202 us), so it is asked of that kernel only.
template <class TR, int OP>
constexpr int fwd_min_waves() {
    return (std::is_same<TR, F16>::value && OP == TXS_MAX) ? 6 : 1;
}

template <class TR, int VEC, int OP>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(fwd_min_waves<TR, OP>(), 8)))
void scatter_fwd_kernel(
    const typename TR::raw *__restrict__ feats, const int *__restrict__ perm,
    const int *__restrict__ seg, const int *__restrict__ slot_of,
    typename TR::raw *__restrict__ out, int *__restrict__ arg,
    unsigned long long *__restrict__ scratch, const int *__restrict__ preSum, int N, int C, int U,
    int lpr_log2, int ref_log2, int chunk) {
    using raw = typename TR::raw;
    constexpr bool kMax = OP == TXS_MAX || OP == TXS_MAX_REFTIE;
    constexpr bool kRef = OP == TXS_MAX_REFTIE;  // idx[] then holds the winner's staged position, not its row
    // rows per load batch (two batches in flight); measured per dtype and operator
    constexpr int kBatch = sizeof(raw) == 2
                               ? (kMax ? (std::is_same<TR, F16>::value ? kBatchHalfMax : kBatchBf16Max) : kBatchHalf)
                               : ::kBatch;
    using AccT = typename std::conditional<kMax, typename TR::max_t, float>::type;
    constexpr int kEndBit = kSpecialBit;
    extern __shared__ int lds[];
    const int g_log2 = 8 - lpr_log2;      // kThreads == 256
    const int G = 1 << g_log2;
    const int T = G * chunk;              // `chunk` positions per lane group on average
    const int n_seg_s = T + kMargin + 1;  // positions t0-1 .. t0+T+kMargin-1
    int *seg_s = lds;                     // seg_s[l]: voxel (bit 31: special) at position t0 - 1 + l
    int *pk_s = lds + n_seg_s;            // pk_s[l - 1]: row at position t0 - 1 + l, bit 31 = last row of its run
    int *bnd_s = lds + 2 * n_seg_s - 1;   // [0]: first l of the tile's own range, [1]: one past its last l
    // what a lane group hands to the next one: the reduction of the run that is still open at
    // the end of its share (4-byte cells: a value per element, and for max the winner's tag)
    float *carry_v = reinterpret_cast<float *>(lds + ((2 * n_seg_s + 1 + 3) & ~3));
    int *carry_i = reinterpret_cast<int *>(carry_v) + kThreads * VEC;
    const long t0l = (long)xcd_block(blockIdx.x, gridDim.x) * T;
    if (t0l >= N) return;  // uniform for the workgroup
    const int t0 = (int)t0l;
    const unsigned last_row = (unsigned)(N - 1);

    // Stage the tile's ids.  The tile's own range [b_lo, b_hi) starts at the first position
    // at or after the tile's first one where a run starts (or that lies in a heavy run, which
    // is split anywhere) and ends at the first such position at or after the next tile's first
    // one: an ordinary run belongs, whole, to the tile it starts in.  Both are found among the
    // kMargin positions behind each border with one wave ballot.
    for (int e0 = 0; e0 < n_seg_s; e0 += kThreads) {
        const int e = e0 + (int)threadIdx.x;
        const long p = (long)t0 - 1 + e;
        const bool in = e < n_seg_s && p >= 0 && p < N;
        const int sv = in ? seg[p] : kNoSeg;
        const int sn = (e < n_seg_s && p + 1 < N) ? seg[p + 1] : kNoSeg;
        if (e < n_seg_s) {
            seg_s[e] = sv;
            if (e >= 1) {
                // a row index outside the matrix (only a corrupt plan has one) is clamped
                const int r = in ? (int)min((unsigned)(perm ? perm[p] : (int)p), last_row) : 0;
                pk_s[e - 1] = r | ((in && sn != sv) ? kEndBit : 0);
            }
        }
        // position p + 1 (l = e + 1) can open a range: a run starts there, or it is heavy
        const int eb = e0 + ((int)threadIdx.x & ~63);  // first entry of this wave in this pass of the loop
        if (eb == 0 || eb == T) {
            const unsigned long long m = __ballot(e < n_seg_s && (sn != sv || (sn < 0)));
            if (((int)threadIdx.x & 63) == 0)
                bnd_s[eb == 0 ? 0 : 1] = m ? eb + 1 + (int)__builtin_ctzll(m) : -1;
        }
    }
    __syncthreads();
    int b_lo = bnd_s[0], b_hi = bnd_s[1];
    const int l_staged_end = n_seg_s;  // one past the last staged l
    if (b_lo < 0) {
        // an ordinary run of more than kMargin rows covers the tile's first positions (a plan
        // with a heavy threshold above kMargin has such runs, and so has one whose few voxels
        // just above the threshold were made ordinary again): look for its end one by one
        b_lo = kMargin + 1;
        while (b_lo < l_staged_end && seg_s[b_lo] == seg_s[b_lo - 1] && seg_s[b_lo] >= 0) ++b_lo;
    }
    // no border found behind the tile's end: the range ends with the staged ids, and the last
    // lane group walks on from there, one row at a time
    const bool long_tail = b_hi < 0;
    if (long_tail) b_hi = l_staged_end;
    if (b_lo > b_hi) b_lo = b_hi;
    const int Tp = b_hi - b_lo;  // rows of the tile's own range: dealt evenly to the lane groups
    if (Tp <= 0) return;         // uniform for the workgroup

    const int gi = (int)threadIdx.x >> lpr_log2;
    const int lane_in = (int)threadIdx.x & ((1 << lpr_log2) - 1);
    const int col = ((int)blockIdx.y << lpr_log2 | lane_in) * VEC;
    const bool live = col < C;
    auto share_begin = [&](int k) -> int { return b_lo + (int)(((long)k * Tp) >> g_log2); };
    const int c0 = share_begin(gi), c_end = share_begin(gi + 1);  // this lane group's positions (l)
    const int ch = (Tp + G - 1) >> g_log2;                          // the largest share

    // ids / rows past the staged range are fetched from global memory (only an ordinary run
    // longer than kMargin that crosses the tile's end gets there)
    auto seg_at = [&](int l) -> int {
        if (l < n_seg_s) return seg_s[l];
        const long p = (long)t0 - 1 + l;
        return p < N ? seg[p] : kNoSeg;
    };
    auto pk_at = [&](int l) -> int {
        if (l < n_seg_s) return pk_s[l - 1];
        const long p = (long)t0 - 1 + l;
        if (p >= N) return 0;
        const int r = (int)min((unsigned)(perm ? perm[p] : (int)p), last_row);
        const int sn = p + 1 < N ? seg[p + 1] : kNoSeg;
        return r | (sn != seg[p] ? kEndBit : 0);
    };

    // Start value of a running max: -inf, or in reference-tie mode the
    // reference's own -FLT_MAX (scatter_kernel.cu:139), which -inf never beats.
    const AccT acc0 = kRef ? (AccT)TR::to_m(TR::lowest()) : (AccT)(kMax ? -__builtin_inff() : 0.0f);
    AccT acc[VEC], hacc[VEC];
    int idx[VEC], hidx[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
        acc[k] = acc0;
        idx[k] = -1;
        hacc[k] = acc0;
        hidx[k] = -1;
    }
    int run_l0 = c0;  // first position (of this lane group) of the run being reduced
    // The first run end in the share closes a run that began in an earlier share unless a run
    // starts exactly at the share's first position: its reduction is kept (`hacc`) until the
    // earlier lane groups have published theirs.
    bool pend_head = c0 < c_end && seg_s[c0 - 1] == seg_s[c0];
    int head_seg = kNoSeg;  // voxel (with its special bit) of the kept head, kNoSeg: none
    int head_l = 0;         // its last position

    const char *lane_base = reinterpret_cast<const char *>(feats) + (size_t)col * sizeof(raw);
    const unsigned row_bytes = (unsigned)C * (unsigned)sizeof(raw);
    auto row_ptr = [&](int r) -> const raw * {
        return reinterpret_cast<const raw *>(lane_base + (unsigned long long)(unsigned)r * row_bytes);
    };

    // tie key of the reference for the row at position l (as staged) of voxel u (reference-tie mode)
    auto ref_key_at = [&](int l, int u) -> unsigned {
        return (unsigned)ref_key((t0 - 1 + l) - preSum[u], ref_log2);
    };
    // What competes in the low word of a heavy voxel's packed key (smaller wins): the row, or in
    // reference-tie mode the reference's tie key of the winner's offset inside its voxel.
    auto low_word = [&](int id, int u) -> unsigned { return kRef ? ref_key_at(id, u) : (unsigned)id; };

    // Write out the finished reduction (a, ix) of voxel sgv: an output row for an ordinary voxel
    // (cnt rows, all of them reduced here), one atomic per element into the table for a heavy one
    // (rows [p_lo, p_hi) of the sorted order went into it).  `staged`: every position involved
    // has its ids in LDS (so no value that the common path uses comes from a global load, which
    // would make the path wait for every row still on its way).
    auto emit = [&](auto staged, int sgv, AccT(&a)[VEC], int(&ix)[VEC], int cnt, long p_lo, long p_hi) {
        constexpr bool kStaged = decltype(staged)::value;
        const int u = sgv & kIdMask;
        if ((unsigned)u >= (unsigned)U) return;
        if (kMax && !kRef) {
            bool missing = false;
#pragma unroll
            for (int k = 0; k < VEC; ++k) missing |= ix[k] < 0;
            if (__builtin_expect(missing, 0)) {
                // No value above -inf was seen in some channel: the rows hold only -inf and NaN
                // there.  The first -inf row wins.
                // (an ordinary voxel: all its rows; a heavy one: its rows inside [p_lo, p_hi))
                long lo = preSum[u], hi = preSum[u + 1];
                if (sgv < 0) {
                    lo = lo > p_lo ? lo : p_lo;
                    hi = hi < p_hi ? hi : p_hi;
                }
                for (long p = lo; p < hi; ++p) {
                    const int row = perm ? perm[p] : (int)p;
                    if ((unsigned)row >= (unsigned)N) continue;
                    Pack<raw, VEC> x = ld<raw, VEC>(feats + (size_t)row * C + col);
#pragma unroll
                    for (int k = 0; k < VEC; ++k)
                        if (ix[k] < 0 && TR::to_f(x.v[k]) == -__builtin_inff()) ix[k] = row;
                }
            }
        }
        if (sgv >= 0) {
            const size_t o = (size_t)u * C + col;
            Pack<raw, VEC> r;
            if (OP == TXS_SUM) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) r.v[k] = TR::from_f((float)a[k]);
            } else if (OP == TXS_MEAN) {
                const float d = (float)cnt;
                if constexpr (TXS_FAST_DIV_HALF && sizeof(raw) == 2) {
                    // 2-byte outputs: the fp32 quotient is rounded to 8 or 11 bits right away, so
                    // the hardware reciprocal (1 ulp) and one multiply stand in for the division
                    // (a dozen instructions per element, in a kernel bound by instruction issue)
                    // (the instruction is spelled out: left to itself the compiler takes a different
                    // reciprocal instruction where it sees the count come straight from an integer,
                    // and the two do not always agree in the last bit)
                    float rd;
                    asm("v_rcp_f32 %0, %1" : "=v"(rd) : "v"(d));
#pragma unroll
                    for (int k = 0; k < VEC; ++k) {
                        // (the fp32 product is pinned in a register: where the compiler may fuse the
                        // multiply with the conversion it rounds once instead of twice, and a sum on
                        // a rounding boundary would come out differently from one code path to the next)
                        float q = (float)a[k] * rd;
                        asm("" : "+v"(q));
                        r.v[k] = TR::from_f(q);
                    }
                } else {
#pragma unroll
                    for (int k = 0; k < VEC; ++k) r.v[k] = TR::from_f((float)a[k] / d);
                }
            } else {
                Pack<int, VEC> ai;
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    r.v[k] = ix[k] >= 0 ? TR::from_m((typename TR::max_t)a[k]) : TR::lowest();
                    ai.v[k] = ix[k];
                    if (kRef && ix[k] >= 0) ai.v[k] = (kStaged ? pk_s[ix[k] - 1] : pk_at(ix[k])) & kIdMask;
                }
                st_stream<int, VEC>(arg + o, ai);
            }
            st_stream<raw, VEC>(out + o, r);
        } else {
            const int slot = slot_of[u];
            if (slot < 0) return;
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                const size_t o = (size_t)slot * C + col + k;
                if constexpr (kMax) {
                    if (ix[k] >= 0)
                        atomicMax(scratch + o, ((unsigned long long)ordered_bits((float)a[k]) << 32) |
                                                   (unsigned long long)(0xffffffffu - low_word(ix[k], u)));
                } else {
                    unsafeAtomicAdd(reinterpret_cast<float *>(scratch) + o, (float)a[k]);
                }
            }
        }
    };

    // Fold the reduction (b, bi) of EARLIER rows of the same voxel into (a, ix).
    auto fold_earlier = [&](AccT(&a)[VEC], int(&ix)[VEC], const AccT(&b)[VEC], const int(&bi)[VEC], int u) {
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            if constexpr (!kMax) {
                a[k] += b[k];
            } else {
                bool take = b[k] > a[k];
                if (bi[k] >= 0 && b[k] == a[k]) {
                    // equal values: the earlier row wins, or the smaller tie key of the reference
                    take = ix[k] < 0 || !kRef || ref_key_at(bi[k], u) < ref_key_at(ix[k], u);
                }
                if (take) {
                    a[k] = b[k];
                    ix[k] = bi[k];
                }
            }
        }
    };

    // A run ends at position l.
    auto on_end = [&](auto staged, int l) {
        constexpr bool kStaged = decltype(staged)::value;
        const int sgv = kStaged ? seg_s[l] : seg_at(l);
        if (pend_head) {
            pend_head = false;
            head_seg = sgv;
            head_l = l;
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                hacc[k] = acc[k];
                hidx[k] = idx[k];
            }
        } else {
            emit(staged, sgv, acc, idx, l + 1 - run_l0, (long)t0 - 1 + run_l0, (long)t0 + l);
        }
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            acc[k] = acc0;
            idx[k] = -1;
        }
        run_l0 = l + 1;
    };

    // Fold one loaded row (position l, staged word pk) into the running reduction.
    auto add_row = [&](auto staged, const Pack<raw, VEC> &v, int l, int pk) {
        constexpr bool kStaged = decltype(staged)::value;
        const int tag = kRef ? l : (pk & kIdMask);
        if constexpr (!kMax && TXS_F16_FMA_MIX && std::is_same<TR, F16>::value && VEC % 2 == 0) {
            unsigned w[VEC / 2 > 0 ? VEC / 2 : 1];
            __builtin_memcpy(w, &v, sizeof(unsigned) * (VEC / 2));
#pragma unroll
            for (int k = 0; k < VEC / 2; ++k) {
                acc[2 * k] = add_f16_lo(acc[2 * k], w[k]);
                acc[2 * k + 1] = add_f16_hi(acc[2 * k + 1], w[k]);
            }
            return;
        }
        if constexpr (kRef) {
            // Reference-tie mode also takes an equal value whose tie key is smaller.  Equal
            // values are rare, so the keys are only worked out where a lane meets one.
            bool tie = false;
#pragma unroll
            for (int k = 0; k < VEC; ++k) tie |= TR::to_m(v.v[k]) == acc[k];
            if (__builtin_expect(tie, 0)) {
                const int u = (kStaged ? seg_s[l] : seg_at(l)) & kIdMask;
                if ((unsigned)u < (unsigned)U) {
                    const unsigned kn = ref_key_at(l, u);
#pragma unroll
                    for (int k = 0; k < VEC; ++k) {
                        if (!(TR::to_m(v.v[k]) == acc[k])) continue;
                        const unsigned ko = idx[k] < 0 ? 0xffffffffu : ref_key_at(idx[k], u);
                        if (kn < ko) {  // the value's bits follow the winner (a zero's sign)
                            idx[k] = tag;
                            acc[k] = TR::to_m(v.v[k]);
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            if constexpr (kMax) {
                const AccT x = TR::to_m(v.v[k]);
                // strict '>': the first row wins ties, NaN never wins
                const bool take = x > acc[k];
                acc[k] = take ? x : acc[k];
                idx[k] = take ? tag : idx[k];
            } else {
                acc[k] += TR::to_f(v.v[k]);
            }
        }
    };

    if (live) {
        // Every lane group walks `ch` steps (the last one empty for those with a row less), so
        // the lane groups of a wavefront stay in step.  Row loads are double-buffered, every
        // load is issued on a straight-line path (slots past the share re-load its last row, a
        // cache hit) and the prefetch loop is peeled, so that the counts of loads in flight
        // are known where a batch is reduced.
        struct Batch {
            Pack<raw, VEC> v[kBatch];
        };
        const int l_stop = c0 + ch;  // the same distance for every lane group
        const int l_clamp = max(c_end - 1, c0);
        auto issue = [&](Batch &bt, int l) {
#pragma unroll
            for (int i = 0; i < kBatch; ++i) bt.v[i] = ld_stream<raw, VEC>(row_ptr(pk_s[min(l + i, l_clamp) - 1] & kIdMask));
        };
        auto consume_full = [&](const Batch &bt, int l) {
#pragma unroll
            for (int i = 0; i < kBatch; ++i) {
                const int pk = pk_s[l + i - 1];
                add_row(std::true_type{}, bt.v[i], l + i, pk);
                if (pk < 0) on_end(std::true_type{}, l + i);
            }
        };
        auto consume_last = [&](const Batch &bt, int l) {
#pragma unroll
            for (int i = 0; i < kBatch; ++i) {
                if (l + i < c_end) {
                    const int pk = pk_s[l + i - 1];
                    add_row(std::true_type{}, bt.v[i], l + i, pk);
                    if (pk < 0) on_end(std::true_type{}, l + i);
                }
            }
        };
        Batch b0, b1;
        issue(b0, c0);
        for (int l = c0;;) {
            int ln = l + kBatch;
            if (ln >= l_stop) {
                consume_last(b0, l);
                break;
            }
            issue(b1, ln);
            consume_full(b0, l);
            l = ln;
            ln = l + kBatch;
            if (ln >= l_stop) {
                consume_last(b1, l);
                break;
            }
            issue(b0, ln);
            consume_full(b1, l);
            l = ln;
        }
        if (c0 < c_end) {
            const int l_last = c_end - 1;
            const int sg_last = seg_s[l_last];
            const bool open = pk_s[l_last - 1] >= 0 && sg_last != kNoSeg;
            if (open && c_end == b_hi) {
                if (sg_last >= 0 && long_tail) {
                    // (rare) the range ends inside an ordinary run whose end lies beyond the
                    // staged ids: walk on to it
                    for (int l = c_end;; ++l) {
                        const int pk = pk_at(l);
                        if (seg_at(l) == kNoSeg) break;
                        add_row(std::false_type{}, ld_stream<raw, VEC>(row_ptr(pk & kIdMask)), l, pk);
                        if (pk < 0) {
                            on_end(std::false_type{}, l);
                            break;
                        }
                    }
                } else if (sg_last < 0) {
                    // the range ends inside a heavy run: its rows in this tile are complete here
                    on_end(std::true_type{}, l_last);
                }
            } else if (open) {
                float *cv = carry_v + (size_t)threadIdx.x * VEC;
                int *ci = carry_i + (size_t)threadIdx.x * VEC;
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    cv[k] = (float)acc[k];
                    if (kMax) ci[k] = idx[k];
                }
            }
        }
    }
    __syncthreads();
    if (!live || head_seg == kNoSeg) return;
    // The kept head: add what the lane groups before this one reduced of the same run (a
    // heavy run can cover many shares), then write it out.  An ordinary run always starts inside
    // the tile's range; a heavy one that began in an earlier tile leaves its rows of this tile.
    int first_l = c0;
    for (int k = gi - 1; k >= 0; --k) {
        const int k0 = share_begin(k);
        if (k0 == share_begin(k + 1)) continue;  // a lane group without rows
        const float *cv = carry_v + ((size_t)(k << lpr_log2) + lane_in) * VEC;
        const int *ci = carry_i + ((size_t)(k << lpr_log2) + lane_in) * VEC;
        AccT b[VEC];
        int bi[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            b[e] = (AccT)cv[e];
            bi[e] = kMax ? ci[e] : 0;
        }
        fold_earlier(hacc, hidx, b, bi, head_seg & kIdMask);
        first_l = k0;
        if (seg_s[k0 - 1] != head_seg) break;  // the run starts in this share
    }
    const int u = head_seg & kIdMask;
    const int cnt = ((unsigned)u < (unsigned)U && head_seg >= 0) ? preSum[u + 1] - preSum[u] : 1;
    emit(std::false_type{}, head_seg, hacc, hidx, cnt, (long)t0 - 1 + first_l, (long)t0 + head_l);
}

// Turn the scratch table of the special voxels into output rows and clear it.  The first
// n_heavy entries of heavy_ids are the heavy voxels (entry s owns table row s), the rest are
// empty voxels, which own no row: a cell's table word does not depend on the voxel's id, so
// it is requested together with the id, and only the mean goes on to the voxel's count.
template <class TR, int OP>
__global__ void scatter_finalize_kernel(const typename TR::raw *__restrict__ feats,
                                        const int *__restrict__ preSum,
                                        const int *__restrict__ heavy_ids,
                                        unsigned long long *__restrict__ scratch,
                                        typename TR::raw *__restrict__ out,
                                        int *__restrict__ arg, int n_special, int n_heavy, int N, int C,
                                        int U, const int *__restrict__ perm, int ref_log2) {
    constexpr bool kMaxOp = OP == TXS_MAX || OP == TXS_MAX_REFTIE;
    const long t = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= (long)n_special * C) return;
    const int s = (int)(t / C), c = (int)(t - (long)s * C);
    const bool heavy = s < n_heavy;
    unsigned long long key = 0ull;
    float s32 = 0.0f;
    if (heavy) {
        if (kMaxOp) {
            key = scratch[t];
            scratch[t] = 0ull;
        } else {
            float *fs = reinterpret_cast<float *>(scratch);
            s32 = fs[t];
            fs[t] = 0.0f;
        }
    }
    const int u = heavy_ids[s];
    if ((unsigned)u >= (unsigned)U) return;
    const size_t o = (size_t)u * C + c;
    if (!heavy) {  // empty voxel
        if (kMaxOp) {
            out[o] = TR::lowest();
            arg[o] = -1;
        } else {
            out[o] = TR::from_f(OP == TXS_MEAN ? __builtin_nanf("") : 0.0f);  // mean: 0/0 as in the reference
        }
        return;
    }
    if (kMaxOp) {
        unsigned row = 0xffffffffu - (unsigned)(key & 0xffffffffull);
        if (OP == TXS_MAX_REFTIE && key != 0ull) {  // the low word holds a tie key, not a row
            const long pos = (long)preSum[u] + ref_rel((int)row, ref_log2);
            row = (pos >= 0 && pos < N) ? (unsigned)(perm ? perm[pos] : (int)pos) : 0xffffffffu;
        }
        if (key == 0ull || row >= (unsigned)N) {
            out[o] = TR::lowest();
            arg[o] = -1;
        } else {
            // the key carries the winning value itself (exactly: it came from the dtype);
            // only the sign of a zero was folded away and is read back from the winner
            const float x = from_ordered_bits((unsigned)(key >> 32));
            out[o] = x == 0.0f ? feats[(size_t)row * C + c] : TR::from_f(x);
            arg[o] = (int)row;
        }
    } else {
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
// current batch is stored.  CHUNK (positions per lane group) is 8 when runs are
// short (measured 1-5 % faster on LiDAR-like occupancy) and 16 when they are long
// (fewer re-fetches of the same upstream row at chunk borders).

template <class TR, int VEC, int OP, int CHUNK>
__global__ __launch_bounds__(kThreads) void scatter_bwd_kernel(
    const typename TR::raw *__restrict__ g, const int *__restrict__ arg,
    const int *__restrict__ perm, const int *__restrict__ seg, const int *__restrict__ preSum,
    typename TR::raw *__restrict__ gin, int N, int C, int U, int lpr_log2) {
    using raw = typename TR::raw;
    constexpr int kBatchBwd = sizeof(raw) == 2 ? kBatchBwdHalf : ::kBatchBwd;
    extern __shared__ int lds[];
    const int G = kThreads >> lpr_log2;
    const int T = G * CHUNK;
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
    const int la = ((int)threadIdx.x >> lpr_log2) * CHUNK;
    const int lb = min(la + CHUNK, N - t0);
    if (la >= lb) return;

    // A batch keeps the fetched upstream rows and two bit masks; row ids are read
    // again from LDS when the batch is stored.  The upstream row (and arg row) is
    // fetched only where the voxel changes.
    struct Batch {
        Pack<raw, VEC> gv[kBatchBwd];
        Pack<int, VEC> av[kBatchBwd];
        int cnt[kBatchBwd];
        unsigned valid, need;
    };
    auto issue = [&](Batch &bt, int l) {
        bt.valid = 0u;
        bt.need = 0u;
#pragma unroll
        for (int i = 0; i < kBatchBwd; ++i) {
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
        for (int i = 0; i < kBatchBwd; ++i) {
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
        int ln = l + kBatchBwd;
        if (ln < lb) issue(b1, ln);
        consume(b0, l);
        if (ln >= lb) break;
        l = ln;
        ln = l + kBatchBwd;
        if (ln < lb) issue(b0, ln);
        consume(b1, l);
        if (ln >= lb) break;
        l = ln;
    }
}

// ------------------------------------------------------------------ launch --

// Sorted positions per lane group of the forward kernel (on average: a tile's range is dealt
// evenly).  Long runs (64 rows per voxel and more) are reduced fastest in tiles of 32 positions
// per lane group (fewer tile borders for a run to cross, one atomic row per tile and heavy
// voxel); short runs of 4-byte elements in tiles of 8 (twice the workgroups, shorter dependent
// walks: 4 % on the LiDAR sweep, 8 % on 200k rows); everything else in tiles of 16.
int fwd_chunk_for(long N, long U, int op, int elem) {
#ifdef TXS_FORCE_FWD_CHUNK
    return TXS_FORCE_FWD_CHUNK;
#endif
    (void)op;
    if (N >= 64 * U) return kChunkLong;
    return (elem == 4 && N < 8 * U) ? kChunkShort : kChunk;
}

struct Geometry {
    int vec_bytes;  // bytes one lane moves per row
    int lpr_log2;   // log2(lanes that cover one row slice)
    int ytiles;     // column tiles when a row is wider than 64 lanes
    int chunk;      // sorted positions per lane group
    unsigned lds_fwd_idx, lds_slots, lds_bwd;  // dynamic LDS: fwd index part (bytes), fwd slot elements, bwd bytes
    dim3 grid;
};

bool aligned_to(const void *p, int bytes) { return p == nullptr || ((uintptr_t)p % (uintptr_t)bytes) == 0; }

Geometry make_geometry(long N, long C, int elem, const void *p0, const void *p1, const void *p2,
                       bool arg_used, const void *parg, int chunk, bool forward = false) {
    Geometry g;
    // bytes per lane and row: 16 for fp32; 8 for the 2-byte types, whose kernels carry
    // twice the registers per byte (measured 4-12 % faster than 16 on fp16 / bf16)
    int vb = elem == 2 ? kHalfVecBytes : 16;
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
    // a tile (lane groups x chunk positions) is a whole number of wavefronts' worth of staged
    // ids: the forward kernel finds the borders of a tile's range with one ballot each
    // (forward) a small input gets smaller tiles while that gives the chip more workgroups
    // (below eight per compute unit a tile's fixed costs show: 3-5 % on 200k rows of 256 bytes)
    while (forward && chunk > 4 && N / ((long)(kThreads >> l2) * chunk) < 2048) chunk /= 2;
    while (forward && ((long)(kThreads >> l2) * chunk) % 64 != 0) chunk *= 2;
    g.chunk = chunk;
    g.ytiles = (int)((lanes + (1L << l2) - 1) >> l2);
    const long tile = (long)(kThreads >> l2) * chunk;  // sorted positions per workgroup
    long blocks = (N + tile - 1) / tile;
    blocks = (blocks + 8 * kXcdSpan - 1) / (8 * kXcdSpan) * (8 * kXcdSpan);
    g.lds_fwd_idx = (unsigned)(((2 * (tile + kMargin + 1) + 1 + 3) & ~3L) * sizeof(int));
    g.lds_slots = (unsigned)(2 * kThreads * vec);  // carry cells: a value and a tag per element
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
    const unsigned lds8 = geo.lds_fwd_idx + 4 * geo.lds_slots;  // staged ids, then 4-byte carry cells
#define TXS_FWD_OP(OPC)                                                            \
    scatter_fwd_kernel<TR, VEC, OPC><<<geo.grid, blk, lds8, st>>>(                 \
        f, perm, seg, slot_of, o, arg, s, preSum, N, C, U, geo.lpr_log2, ref_log2, geo.chunk);
    switch (op) {
        case TXS_SUM: TXS_FWD_OP(TXS_SUM) break;
        case TXS_MEAN: TXS_FWD_OP(TXS_MEAN) break;
        case TXS_MAX_REFTIE: TXS_FWD_OP(TXS_MAX_REFTIE) break;
        default: TXS_FWD_OP(TXS_MAX) break;
    }
#undef TXS_FWD_OP
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
    if constexpr (e == 4 || kHalfVecBytes == 16) {
        TXS_FWD(16)
    }
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
                           long n_special, long n_heavy, int N, int C, int U, const int *perm, int ref_log2) {
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
                                                                      (int)n_special, (int)n_heavy, N, C, U, perm, ref_log2);
            break;
        case TXS_MEAN:
            scatter_finalize_kernel<TR, TXS_MEAN><<<grid, blk, 0, st>>>(f, preSum, heavy_ids, s, o, arg,
                                                                       (int)n_special, (int)n_heavy, N, C, U, perm, ref_log2);
            break;
        case TXS_MAX_REFTIE:
            scatter_finalize_kernel<TR, TXS_MAX_REFTIE><<<grid, blk, 0, st>>>(
                f, preSum, heavy_ids, s, o, arg, (int)n_special, (int)n_heavy, N, C, U, perm, ref_log2);
            break;
        default:
            scatter_finalize_kernel<TR, TXS_MAX><<<grid, blk, 0, st>>>(f, preSum, heavy_ids, s, o, arg,
                                                                      (int)n_special, (int)n_heavy, N, C, U, perm, ref_log2);
            break;
    }
    return hipGetLastError();
}

template <class TR, int VEC, int CHUNK>
hipError_t launch_bwd_chunk(int op, const Geometry &geo, hipStream_t st, const void *g, const int *arg,
                            const int *perm, const int *seg, const int *preSum, void *gin, int N,
                            int C, int U) {
    using raw = typename TR::raw;
    auto gi = (const raw *)g;
    auto go = (raw *)gin;
    dim3 blk(kThreads);
    switch (op) {
        case TXS_SUM:
            scatter_bwd_kernel<TR, VEC, TXS_SUM, CHUNK><<<geo.grid, blk, geo.lds_bwd, st>>>(
                gi, arg, perm, seg, preSum, go, N, C, U, geo.lpr_log2);
            break;
        case TXS_MEAN:
            scatter_bwd_kernel<TR, VEC, TXS_MEAN, CHUNK><<<geo.grid, blk, geo.lds_bwd, st>>>(
                gi, arg, perm, seg, preSum, go, N, C, U, geo.lpr_log2);
            break;
        default:
            scatter_bwd_kernel<TR, VEC, TXS_MAX, CHUNK><<<geo.grid, blk, geo.lds_bwd, st>>>(
                gi, arg, perm, seg, preSum, go, N, C, U, geo.lpr_log2);
            break;
    }
    return hipGetLastError();
}

template <class TR, int VEC>
hipError_t launch_bwd_op(int op, const Geometry &geo, hipStream_t st, const void *g, const int *arg,
                         const int *perm, const int *seg, const int *preSum, void *gin, int N, int C,
                         int U) {
    if (geo.chunk == kChunkBwdShort)
        return launch_bwd_chunk<TR, VEC, kChunkBwdShort>(op, geo, st, g, arg, perm, seg, preSum, gin, N, C, U);
    return launch_bwd_chunk<TR, VEC, kChunkBwdLong>(op, geo, st, g, arg, perm, seg, preSum, gin, N, C, U);
}

template <class TR>
hipError_t launch_bwd(int op, const Geometry &geo, hipStream_t st, const void *g, const int *arg,
                      const int *perm, const int *seg, const int *preSum, void *gin, int N, int C,
                      int U) {
    constexpr int e = (int)sizeof(typename TR::raw);
#define TXS_BWD(VB)                                                                               \
    if (geo.vec_bytes == VB)                                                                      \
        return launch_bwd_op<TR, (VB) / e>(op, geo, st, g, arg, perm, seg, preSum, gin, N, C, U);
    if constexpr (e == 4 || kHalfVecBytes == 16) {
        TXS_BWD(16)
    }
    TXS_BWD(8)
    TXS_BWD(4)
    if constexpr (e == 2) {
        TXS_BWD(2)
    }
#undef TXS_BWD
    return hipErrorInvalidValue;
}

// Largest power of two (up to 16) that divides every given address.
long common_alignment(std::initializer_list<const void *> ptrs) {
    uintptr_t bits = 16;
    for (const void *p : ptrs) bits |= (uintptr_t)p;
    return (long)(bits & (~bits + 1));
}

// Row-order ids for the table kernels: unq_inv itself, or for grouped rows (no perm) the
// per-position ids, whose bit 31 the kernels mask off.
const int32_t *row_order_ids(const int32_t *unq_inv, const int32_t *perm, const int32_t *seg) {
    return unq_inv ? unq_inv : (perm == nullptr ? seg : nullptr);
}

__global__ void clear_cells_kernel(unsigned long long *__restrict__ cells, long n) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) cells[i] = 0ull;
}

// Argument checks, the choice between the row-order table kernels and the voxel-order
// kernels, and the launches, behind txs_scatter_forward and txs_scatter_forward_resident.
// clear_heavy_cells: the heavy voxels' cells of `scratch` may hold anything on entry (the
// library-resident table); they are cleared by a kernel once the arguments have passed
// every check and only if the voxel-order kernels, which use them, are the ones that run.
int scatter_forward_impl(int op, int dtype, const void *feats, const int32_t *unq_inv, const int32_t *perm,
                         const int32_t *seg, const int32_t *preSum, const int32_t *slot_of,
                         const int32_t *heavy_ids, int64_t num_special, int64_t num_heavy, void *scratch,
                         int64_t scratch_cells, void *out, int32_t *arg, int64_t num_total, int64_t channel,
                         int64_t num_unq, int64_t max_cnt, int path, void *stream,
                         bool clear_heavy_cells = false) {
    if (op != TXS_SUM && op != TXS_MEAN && op != TXS_MAX && op != TXS_MAX_REFTIE)
        return TXS_ERR_UNSUPPORTED;
    if (dtype != TXS_F32 && dtype != TXS_F16 && dtype != TXS_BF16) return TXS_ERR_UNSUPPORTED;
    if (path != TXS_PATH_AUTO && path != TXS_PATH_VOXEL_ORDER && path != TXS_PATH_TABLE) return TXS_ERR_UNSUPPORTED;
    if (!fits_i32(num_total) || !fits_i32(num_unq) || !fits_i32(channel) || num_special < 0 ||
        num_special > num_unq || num_heavy < 0 || num_heavy > num_special || scratch_cells < 0)
        return TXS_ERR_INVALID_ARG;
    if (num_unq == 0 || channel == 0) return TXS_OK;
    const bool is_max = op == TXS_MAX || op == TXS_MAX_REFTIE;
    if (!out || !preSum || (is_max && !arg)) return TXS_ERR_INVALID_ARG;
    const int64_t heavy_cells = num_heavy * channel;  // both below 2^31
    if (heavy_cells > scratch_cells || (scratch_cells > 0 && !scratch)) return TXS_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const int N = (int)num_total, C = (int)channel, U = (int)num_unq;

    // few voxels: reduce in row order into per-workgroup LDS tables (the partial tables
    // go behind the heavy-voxel table in `scratch`)
    const int32_t *ids = row_order_ids(unq_inv, perm, seg);
    if (path != TXS_PATH_VOXEL_ORDER && ids && feats) {
        const txs_detail::TablePlan tp = txs_detail::table_plan(
            false, op, dtype, N, C, U, common_alignment({feats, out}));
        if (tp.use && heavy_cells + tp.partial_cells <= scratch_cells) {
            unsigned long long *partials = static_cast<unsigned long long *>(scratch) + heavy_cells;
            return status_of(txs_detail::table_forward(tp, op, dtype, st, feats, ids, preSum, partials, out,
                                                       arg, N, C, U));
        }
    }
    if (path == TXS_PATH_TABLE) return TXS_ERR_UNSUPPORTED;

    // block width the reference would launch for this max_cnt (scatter_kernel.cu:187)
    int ref_log2 = 5;
    while (ref_log2 < 10 && (1LL << ref_log2) < max_cnt) ++ref_log2;
    if (num_total > 0 && (!feats || !seg || !slot_of)) return TXS_ERR_INVALID_ARG;
    if (num_special > 0 && !heavy_ids) return TXS_ERR_INVALID_ARG;
    const int elem = dtype == TXS_F32 ? 4 : 2;
    hipError_t e = hipSuccess;
    if (clear_heavy_cells && heavy_cells > 0) {
        clear_cells_kernel<<<dim3(blocks_for(heavy_cells)), dim3(kThreads), 0, st>>>(
            static_cast<unsigned long long *>(scratch), heavy_cells);
        if (hipGetLastError() != hipSuccess) return TXS_ERR_LAUNCH;
    }
    if (N > 0) {
        Geometry geo = make_geometry(N, C, elem, feats, out, nullptr, is_max, arg, fwd_chunk_for(N, U, op, elem), true);
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
            e = launch_finalize<F32>(op, st, feats, preSum, heavy_ids, scratch, out, arg, num_special, num_heavy, N, C, U, perm, ref_log2);
        else if (dtype == TXS_F16)
            e = launch_finalize<F16>(op, st, feats, preSum, heavy_ids, scratch, out, arg, num_special, num_heavy, N, C, U, perm, ref_log2);
        else
            e = launch_finalize<BF16>(op, st, feats, preSum, heavy_ids, scratch, out, arg, num_special, num_heavy, N, C, U, perm, ref_log2);
    }
    return status_of(e);
}

}  // namespace

// =================================================================== C ABI ==

extern "C" {

int txs_abi_version(void) { return 9; }

const char *txs_status_string(int status) {
    switch (status) {
        case TXS_OK: return "ok";
        case TXS_ERR_INVALID_ARG: return "invalid argument (null pointer, negative or oversized extent)";
        case TXS_ERR_LAUNCH: return "HIP kernel launch failed";
        case TXS_ERR_UNSUPPORTED: return "unsupported dtype or operator";
        case TXS_ERR_TOO_LARGE:
            return "heavy-voxel table (num_heavy * channel cells) exceeds the library's resident table";
        default: return "unknown status";
    }
}

int txs_kernel_name(int backward, int op, int dtype, int64_t num_total, int64_t channel,
                    int64_t num_unq, int64_t pointer_alignment, int table_allowed, char *buf,
                    int64_t buf_len) {
    if (!buf || buf_len < 48) return TXS_ERR_INVALID_ARG;
    if (op < TXS_SUM || op > TXS_MAX_REFTIE || dtype < TXS_F32 || dtype > TXS_BF16) return TXS_ERR_UNSUPPORTED;
    if (!fits_i32(num_total) || !fits_i32(channel) || !fits_i32(num_unq) || channel < 1 || num_unq < 1 ||
        pointer_alignment < 1)
        return TXS_ERR_INVALID_ARG;
    static const char *const kOps[] = {"SUM", "MEAN", "MAX", "MAX_REFTIE"};
    static const char *const kTypes[] = {"F32", "F16", "BF16"};
    const int elem = dtype == TXS_F32 ? 4 : 2;
    const void *p = (const void *)(uintptr_t)pointer_alignment;  // stands for the least aligned tensor
    if (backward && op == TXS_MAX_REFTIE) op = TXS_MAX;
    if (table_allowed) {
        const txs_detail::TablePlan tp = txs_detail::table_plan(backward != 0, op, dtype, num_total, channel,
                                                                num_unq, common_alignment({p}));
        if (tp.use) {
            snprintf(buf, (size_t)buf_len, "table_%s_kernel<%s,%d,%s>", backward ? "bwd" : "fwd", kTypes[dtype],
                     tp.vec_bytes / elem, kOps[op]);
            return TXS_OK;
        }
    }
    if (backward) {
        const int chunk = (num_total < (int64_t)kChunkBwdLong * num_unq) ? kChunkBwdShort : kChunkBwdLong;
        const Geometry geo = make_geometry(num_total, channel, elem, p, p, nullptr, op == TXS_MAX, p, chunk);
        snprintf(buf, (size_t)buf_len, "scatter_bwd_kernel<%s,%d,%s,%d>", kTypes[dtype], geo.vec_bytes / elem,
                 kOps[op], chunk);
    } else {
        const bool is_max = op == TXS_MAX || op == TXS_MAX_REFTIE;
        const Geometry geo = make_geometry(num_total, channel, elem, p, p, nullptr, is_max, p,
                                           fwd_chunk_for(num_total, num_unq, op, elem), true);
        snprintf(buf, (size_t)buf_len, "scatter_fwd_kernel<%s,%d,%s>", kTypes[dtype], geo.vec_bytes / elem, kOps[op]);
    }
    return TXS_OK;
}

int txs_default_heavy_threshold(void) { return kHeavyDefault; }
int txs_chunk_rows(void) { return kChunk; }

int64_t txs_scatter_scratch_cells(int64_t num_total, int64_t channel, int64_t num_unq, int64_t num_heavy) {
    if (!fits_i32(num_total) || !fits_i32(channel) || !fits_i32(num_unq) || num_heavy < 0 || num_heavy > num_unq)
        return -1;
    return num_heavy * channel + txs_detail::table_partial_cells(num_total, channel, num_unq);
}

int txs_scatter_forward(int op, int dtype, const void *feats, const int32_t *unq_inv, const int32_t *perm,
                        const int32_t *seg, const int32_t *preSum, const int32_t *slot_of,
                        const int32_t *heavy_ids, int64_t num_special, int64_t num_heavy, void *scratch,
                        int64_t scratch_cells, void *out, int32_t *arg, int64_t num_total, int64_t channel,
                        int64_t num_unq, int64_t max_cnt, int path, void *stream) {
    return scatter_forward_impl(op, dtype, feats, unq_inv, perm, seg, preSum, slot_of, heavy_ids, num_special,
                                num_heavy, scratch, scratch_cells, out, arg, num_total, channel, num_unq,
                                max_cnt, path, stream);
}

int txs_scatter_backward(int op, int dtype, const void *grad_out, const int32_t *arg, const int32_t *unq_inv,
                         const int32_t *perm, const int32_t *seg, const int32_t *preSum, void *grad_in,
                         int64_t num_total, int64_t channel, int64_t num_unq, int path, void *stream) {
    if (op == TXS_MAX_REFTIE) op = TXS_MAX;  // the backward only reads arg
    if (op != TXS_SUM && op != TXS_MEAN && op != TXS_MAX) return TXS_ERR_UNSUPPORTED;
    if (dtype != TXS_F32 && dtype != TXS_F16 && dtype != TXS_BF16) return TXS_ERR_UNSUPPORTED;
    if (path != TXS_PATH_AUTO && path != TXS_PATH_VOXEL_ORDER && path != TXS_PATH_TABLE) return TXS_ERR_UNSUPPORTED;
    if (!fits_i32(num_total) || !fits_i32(num_unq) || !fits_i32(channel)) return TXS_ERR_INVALID_ARG;
    if (num_total == 0 || channel == 0) return TXS_OK;
    if (!grad_out || !seg || !grad_in || num_unq <= 0) return TXS_ERR_INVALID_ARG;
    if (op == TXS_MAX && !arg) return TXS_ERR_INVALID_ARG;
    if (op == TXS_MEAN && !preSum) return TXS_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const int N = (int)num_total, C = (int)channel, U = (int)num_unq;
    const int32_t *ids = row_order_ids(unq_inv, perm, seg);
    if (path != TXS_PATH_VOXEL_ORDER && ids) {
        // few voxels: upstream rows staged in LDS, input gradient written in row order
        const txs_detail::TablePlan tp = txs_detail::table_plan(
            true, op, dtype, N, C, U, common_alignment({grad_out, grad_in, op == TXS_MAX ? (const void *)arg : nullptr}));
        if (tp.use)
            return status_of(txs_detail::table_backward(tp, op, dtype, st, grad_out, arg, ids, preSum, grad_in, N, C, U));
    }
    if (path == TXS_PATH_TABLE) return TXS_ERR_UNSUPPORTED;
    const int elem = dtype == TXS_F32 ? 4 : 2;
    // short runs on average -> the short chunk; long runs -> the long one
    const int chunk = ((long)N < (long)kChunkBwdLong * U) ? kChunkBwdShort : kChunkBwdLong;
    Geometry geo = make_geometry(N, C, elem, grad_out, grad_in, nullptr, op == TXS_MAX, arg, chunk);
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

// ------------------------------------------------ library-resident heavy table --

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_resident_mu;
unsigned long long *g_resident_ptr[kMaxDevices];  // device address of static_scratch on each GPU

// Address of the current GPU's copy of static_scratch, looked up on first use.
int resident_table(unsigned long long **table) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return TXS_ERR_LAUNCH;
    std::lock_guard<std::mutex> lock(g_resident_mu);
    if (g_resident_ptr[dev] == nullptr) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(static_scratch)) != hipSuccess || p == nullptr)
            return TXS_ERR_LAUNCH;
        g_resident_ptr[dev] = static_cast<unsigned long long *>(p);
    }
    *table = g_resident_ptr[dev];
    return TXS_OK;
}

}  // namespace

extern "C" {

int64_t txs_resident_table_cells(void) { return kResidentCells; }

int txs_resident_table_init(void) {
    unsigned long long *table = nullptr;
    return resident_table(&table);
}

int txs_scatter_forward_resident(int op, int dtype, const void *feats, const int32_t *unq_inv,
                                 const int32_t *perm, const int32_t *seg, const int32_t *preSum,
                                 const int32_t *slot_of, const int32_t *heavy_ids, int64_t num_special,
                                 int64_t num_heavy, void *out, int32_t *arg, int64_t num_total, int64_t channel,
                                 int64_t num_unq, int64_t max_cnt, int path, void *stream) {
    if (!fits_i32(channel) || !fits_i32(num_unq) || num_heavy < 0 || num_heavy > num_special ||
        num_special > num_unq)
        return TXS_ERR_INVALID_ARG;
    const int64_t cells = num_heavy * channel;  // both below 2^31: no overflow
    if (cells > kResidentCells) return TXS_ERR_TOO_LARGE;
    unsigned long long *table = nullptr;
    const int rc = resident_table(&table);
    if (rc != TXS_OK) return rc;
    // the table is shared by every call on this GPU and keeps what the last one left: the
    // part the heavy voxels use is cleared (by a kernel, so that the call can be captured)
    // after the argument checks, and only when the kernels that use it are launched
    return scatter_forward_impl(op, dtype, feats, unq_inv, perm, seg, preSum, slot_of, heavy_ids, num_special,
                                num_heavy, table, kResidentCells, out, arg, num_total, channel, num_unq,
                                max_cnt, path, stream, /*clear_heavy_cells=*/true);
}

}  // extern "C"
