// Histogram statistics of the histogram observer (aimet_torch/quantization/encoding_analyzer.py:121-338).
//
// One ahq_hist_update() call folds a batch into the running per-encoding histogram:
//   1. finite min/max of the batch                     (ahq_minmax with finite_only, reduce.hip)
//   2. hist_prepare_kernel (one workgroup per slot):   bin edges of the batch's own histogram, the updated range
//      clamped to the growth limit, and the running counts re-binned onto that range (same fp32 operations in the
//      same order as the reference, encoding_analyzer.py:221-310)
//   3. hist_bin_kernel:                                one pass over the batch that bins every element against BOTH
//      ranges (the batch's own and the updated one) into wave-private LDS sub-histograms, merged per workgroup
//   4. hist_finish_kernel:                             integer counts -> fp32, plus carried counts and the
//      below/above-range counts, in the reference's order of additions (encoding_analyzer.py:198-207, 313-323)
//
// Bin index formula = torch.histc on CPU:  pos = int64(((x - lo) * B) / (hi - lo)) in fp32, the top edge belongs to the
// last bin, values outside [lo, hi] and NaN are not counted.


#include <algorithm>
#include <atomic>

#include "ahq_device.h"
#include "ahq_host.h"
#include "layout.h"
#include "tiling.h"

extern "C" int ahq_minmax(int32_t dtype, const ahq_layout* layout, const void* x, void* out_min, void* out_max,
                          void* run_min, void* run_max, int finite_only, void* workspace, size_t workspace_bytes,
                          void* stream);
extern "C" size_t ahq_minmax_workspace_bytes(const ahq_layout* layout);
extern "C" int ahq_minmax_finite_partials(int32_t dtype, const ahq_layout* layout, const void* x, void* out_min,
                                          void* out_max, void* workspace, size_t workspace_bytes, void* stream,
                                          const float** part_min, const float** part_max, int64_t* nparts);

namespace ahq {

constexpr int kHistBlocksMax = 1536;  // persistent workgroups of the binning pass (6 per CU)
constexpr int kRng = 8;               // floats per slot in `ranges`
constexpr int kPartBins = 8;          // entries per block of the single-slot partial counts
constexpr int kHistBinU = 1;          // 16-byte vectors per lane and tile of the single-slot binning pass

// ranges[slot]: lo1, hi1, thr_lo1, thr_hi1 (batch's own range), lo2, hi2, thr_lo2, thr_hi2 (updated range).
// thr_* are the edges rounded to the tensor dtype: the reference compares `x < edge` in the tensor's dtype.

template <typename IO>
__device__ __forceinline__ float round_io(float v) { return load_f32(store_cast<IO>(v)); }

struct PrepArgs {
    int32_t num_slots, num_bins, first;
    float growth;
    const void* bmin;  // [S] io dtype
    const void* bmax;
    const float* part_min;  // single slot: per-workgroup partial extrema of the batch, folded here when nparts > 0
    const float* part_max;
    int64_t nparts;
    float* hist;       // [S][B] running
    float* edges;      // [S][B+1]
    float* minmax;     // [S][2] stored min / max
    float* limits;     // [S][2]
    float* new_edges;  // [S][B+1]
    float* new_minmax; // [S][2]
    float* carried;    // [S][B]
    float* upd_edges;  // [S][B+1]
    float* ranges;     // [S][8]
    int32_t* scratch;  // [S][2][B] destination indices
    int32_t* rebin;    // optional [S]: set to 1 when the running range changed (the batch has to be binned again)
};

// _create_bin_edges (encoding_analyzer.py:221-229).  `lo`/`hi` already hold the min==max adjustment.
__device__ __forceinline__ float edge_at(float lo, float step, int i) { return (float)i * step + lo; }

// Fold of the per-workgroup partial extrema of the min/max pass by one workgroup (saves that pass's own finishing
// launch); min and max are exact and order-independent, and the partials already are values of the tensor's dtype.
__device__ __forceinline__ void fold_partial_extrema(const PrepArgs& a, float& mn, float& mx) {
    __shared__ float red_mn[16], red_mx[16];
    mn = __builtin_inff();
    mx = -__builtin_inff();
    for (int64_t q = threadIdx.x; q < a.nparts; q += blockDim.x) {
        mn = fminf(mn, a.part_min[q]);
        mx = fmaxf(mx, a.part_max[q]);
    }
#pragma unroll
    for (int m = kWave / 2; m >= 1; m >>= 1) {
        mn = fminf(mn, __shfl_xor(mn, m, kWave));
        mx = fmaxf(mx, __shfl_xor(mx, m, kWave));
    }
    if ((threadIdx.x & (kWave - 1)) == 0) {
        red_mn[threadIdx.x / kWave] = mn;
        red_mx[threadIdx.x / kWave] = mx;
    }
    __syncthreads();
    const int nw = (blockDim.x + kWave - 1) / kWave;
    mn = red_mn[0];
    mx = red_mx[0];
    for (int w = 1; w < nw; ++w) {
        mn = fminf(mn, red_mn[w]);
        mx = fmaxf(mx, red_mx[w]);
    }
}

// The running range after a batch with extrema (mn, mx) (encoding_analyzer.py:266-270): clamp(min=left, max=edge0) ==
// min(max(x, left), edge0).  Returns whether it equals the range the state holds.
struct RunningRange {
    float first_edge, last_edge, limit_lo, limit_hi, min, max;
};

__device__ __forceinline__ RunningRange load_running_range(const PrepArgs& a, int s) {
    const float* ce = a.edges + (size_t)s * (a.num_bins + 1);
    const float* lim = a.limits + (size_t)s * 2;
    const float* mmx = a.minmax + (size_t)s * 2;
    return RunningRange{ce[0], ce[a.num_bins], lim[0], lim[1], mmx[0], mmx[1]};
}

__device__ __forceinline__ bool updated_range(const RunningRange& r, float mn, float mx, float& umin, float& umax) {
    umin = fminf(fmaxf(mn, r.limit_lo), r.first_edge);
    umax = fminf(fmaxf(mx, r.last_edge), r.limit_hi);
    return (umin == r.min) && (umax == r.max);
}

// Everything between the extrema of a batch and its binning pass, for slot `s`, by one workgroup.  `keep_minmax`: the
// new running range goes to `ranges` only and the state's min / max stay as they are (other workgroups of the same
// launch still compare against them; the launch that finishes the update stores them).
template <typename IO>
__device__ void prepare_slot(const PrepArgs& a, const int s, const float mn, const float mx, const bool keep_minmax) {
    const int B = a.num_bins;
    const float Bf = (float)B;
    // the batch's own bin edges; "min - 0.5" happens in the tensor dtype before the cast to float
    const bool eq = mn == mx;
    const float lo1 = eq ? round_io<IO>(mn - 0.5f) : mn;
    const float hi1 = eq ? round_io<IO>(mx + 0.5f) : mx;
    const float step1 = (hi1 - lo1) / Bf;
    if (a.new_edges) {
        float* ne = a.new_edges + (size_t)s * (B + 1);
        for (int i = threadIdx.x; i <= B; i += blockDim.x) ne[i] = edge_at(lo1, step1, i);
    }
    const float e1_first = edge_at(lo1, step1, 0), e1_last = edge_at(lo1, step1, B);
    float* rg = a.ranges + (size_t)s * kRng;
    float* mmx = a.minmax + (size_t)s * 2;
    float* lim = a.limits + (size_t)s * 2;
    if (threadIdx.x == 0) {
        if (a.new_minmax) {
            a.new_minmax[2 * s] = mn;
            a.new_minmax[2 * s + 1] = mx;
        }
        rg[0] = e1_first;
        rg[1] = e1_last;
        rg[2] = round_io<IO>(e1_first);
        rg[3] = round_io<IO>(e1_last);
    }
    if (a.first) {
        // the first batch becomes the running statistics; the growth limit is fixed from its edge range
        if (threadIdx.x == 0) {
            const float range = e1_last - e1_first;
            lim[0] = e1_first - (range * a.growth) / 2.0f;
            lim[1] = e1_last + (range * a.growth) / 2.0f;
            mmx[0] = mn;
            mmx[1] = mx;
            rg[4] = rg[0];
            rg[5] = rg[1];
            rg[6] = rg[2];
            rg[7] = rg[3];
        }
        float* ue = a.upd_edges + (size_t)s * (B + 1);
        for (int i = threadIdx.x; i <= B; i += blockDim.x) ue[i] = edge_at(lo1, step1, i);
        return;
    }
    const float* ce = a.edges + (size_t)s * (B + 1);
    const float* ch = a.hist + (size_t)s * B;
    float* carried = a.carried + (size_t)s * B;
    float umin, umax;
    const bool same = updated_range(load_running_range(a, s), mn, mx, umin, umax);
    if (a.rebin && threadIdx.x == 0) a.rebin[s] = same ? 0 : 1;
    if (same) {
        for (int i = threadIdx.x; i < B; i += blockDim.x) carried[i] = ch[i];
    } else {
        const float dst_w = (umax - umin) / Bf;
        const float src_w = ce[1] - ce[0];
        int32_t* di = a.scratch + (size_t)s * 2 * B;
        int32_t* oi = di + B;
        for (int i = threadIdx.x; i < B; i += blockDim.x) {
            const float start = ce[i];
            int d = (int)((start - umin) / dst_w);
            di[i] = d < B - 1 ? d : B - 1;
            int o = (int)(((start + dst_w) - umin) / dst_w);
            oi[i] = o < B - 1 ? o : B - 1;
        }
        __syncthreads();
        // index_add_ runs over the source bins in order.  Both index arrays are non-decreasing, so the sources of a
        // destination bin form one contiguous run: find it by bisection and add it up in source order.
        for (int d = threadIdx.x; d < B; d += blockDim.x) {
            float acc = 0.f;
            for (int pass = 0; pass < 2; ++pass) {
                const int32_t* idx = pass == 0 ? di : oi;
                int lo = 0, hi = B;
                while (lo < hi) {  // first i with idx[i] >= d
                    const int mid = (lo + hi) >> 1;
                    if (idx[mid] < d) lo = mid + 1;
                    else hi = mid;
                }
                for (int i = lo; i < B && idx[i] == d; ++i) {
                    const float start = ce[i];
                    const float dst_end = umin + dst_w * (float)(di[i] + 1);
                    const float part = __builtin_rintf(((dst_end - start) / src_w) * ch[i]);
                    const float first = fminf(part, ch[i]);
                    if (pass == 0) acc += first;
                    else if (first < ch[i]) acc += ch[i] - first;
                }
            }
            carried[d] = acc;
        }
    }
    // bin edges of the updated range (with the min == max adjustment, in fp32 here)
    const bool ueq = umin == umax;
    const float lo2 = ueq ? umin - 0.5f : umin;
    const float hi2 = ueq ? umax + 0.5f : umax;
    const float step2 = (hi2 - lo2) / Bf;
    float* ue = a.upd_edges + (size_t)s * (B + 1);
    for (int i = threadIdx.x; i <= B; i += blockDim.x) ue[i] = edge_at(lo2, step2, i);
    __syncthreads();
    if (threadIdx.x == 0) {
        rg[4] = umin;
        rg[5] = umax;
        rg[6] = round_io<IO>(umin);
        rg[7] = round_io<IO>(umax);
        if (!keep_minmax) {
            mmx[0] = umin;
            mmx[1] = umax;
        }
    }
}

template <typename IO>
__global__ void hist_prepare_kernel(const PrepArgs a) {
    const int s = blockIdx.x;
    float mn, mx;
    if (a.nparts > 0) {
        fold_partial_extrema(a, mn, mx);
    } else {
        mn = load_f32(static_cast<const IO*>(a.bmin)[s]);
        mx = load_f32(static_cast<const IO*>(a.bmax)[s]);
    }
    prepare_slot<IO>(a, s, mn, mx, false);
}

// ------------------------------------------------------------------------------------------------ binning pass --
struct BinArgs : Geom {
    const void* x;
    const float* ranges;   // [S][8]
    uint32_t* partials;    // single slot: [NH][blocks of kPartBins entries][nblocks][kPartBins]  (bins, below, above)
    uint32_t* counts;      // several slots: [S][NH][B + 2], zero-initialised
    int32_t num_bins;
    int32_t nhist;
    int32_t copies;        // interleaved LDS copies of each histogram (power of two, 1..8)
    int32_t copy_shift;    // log2(copies)
    int64_t ntiles;
    // speculative pass (see hist_bin_kernel): the running range as the state holds it, and where the batch's extrema go
    const float* state_minmax;
    const float* state_edges;  // running bin edges [B + 1]
    float* part_min;       // [nblocks]
    float* part_max;
    const int32_t* rebin;  // second pass: leave at once unless *rebin != 0
};

struct RangeC {
    float lo, hi, width, rwidth, thr_lo, thr_hi;
};

__device__ __forceinline__ RangeC load_range(const float* rg, int h) {
    RangeC r;
    r.lo = rg[4 * h];
    r.hi = rg[4 * h + 1];
    // torch.histc widens an empty range by one on each side
    if (r.lo == r.hi) {
        r.lo -= 1.f;
        r.hi += 1.f;
    }
    r.width = r.hi - r.lo;
    r.rwidth = 1.0f / r.width;
    r.thr_lo = rg[4 * h + 2];
    r.thr_hi = rg[4 * h + 3];
    return r;
}

// Reference bin index: trunc(((v - lo) * B) / width) with a correctly rounded fp32 division, capped at B - 1.
__device__ __forceinline__ int bin_exact(float v, const RangeC& r, float Bf, int B) {
    const int p = (int)(((v - r.lo) * Bf) / r.width);
    return p > B - 1 ? B - 1 : p;
}

// Division-free estimate of the same index.  q1 = q0 + (t - q0*w) * (1/w) with fused multiply-adds differs from the
// correctly rounded quotient by at most one unit in the last place (the residual is evaluated without rounding of
// the product, so q0 + e/w is the true quotient to ~2^-46 and rounds to the quotient or to its neighbour).  The two
// can only truncate differently when q1 is an integer or the float just below one.  `fast` is true when
//   * q1 is +0, or is not within q1 * 2^-23 (>= one ulp) of an integer, and
//   * 0 <= q1 < B - 4 ulp, tested on the bit pattern (negative values, -0, NaN and +inf all compare above the limit).
// v < lo gives q1 <= 0 with the sign bit set; v > hi gives a quotient of at least B - 2 ulp; so a `fast` element is
// inside the range and its truncated estimate is the reference bin.  Everything else is redone with bin_exact().
__device__ __forceinline__ int bin_estimate(float v, const RangeC& r, float Bf, uint32_t limit_bits, bool& fast) {
    const float t = (v - r.lo) * Bf;
    const float q0 = t * r.rwidth;
    const float e = __builtin_fmaf(-q0, r.width, t);
    const float q1 = __builtin_fmaf(e, r.rwidth, q0);
    // ">=": an estimate of exactly +0 (v == lo, which is every zero of a rectified activation whose minimum is 0) is
    // safe -- the quotient is exactly 0; for every other q1 equality needs q1 a power of two, where the left side is 0
    const bool safe = __builtin_fabsf(__builtin_rintf(q1) - q1) >= q1 * 1.1920929e-7f;
    fast = safe & (f32_to_bits(q1) < limit_bits);
    return (int)q1;
}

// Single-slot fast path: persistent workgroups, lane-interleaved LDS sub-histograms, one partial per workgroup.
// The kernel is bound by instruction issue, not by LDS or HBM, so the per-element path is kept free of branches:
// elements that need the exact division or lie outside the range are only flagged, and one wave-uniform branch per
// tile revisits them.
//
// SPEC (one histogram): the speculative pass of a batch after the first, for a caller that wants the running
// statistics only.  Most batches of a calibration stay inside the running range, and then the reference bins them on
// exactly that range; so the batch is binned on the running range as the state holds it.  The reference clamps the
// batch's extrema with the outermost bin edges (updated_max = clamp(new.max, bin_edges[-1], limit),
// encoding_analyzer.py:266-270), so the batch's own minimum / maximum matters only beyond those edges.  When the edges
// coincide with the running range or lie outside it, such elements are outside the running range too and already take
// the kernel's rare element-by-element path: their extrema are collected there at no cost to the others
// (per-workgroup partials that the prepare kernel folds; +-inf when there are none, which the clamp turns into the
// edge).  The last edge B * RN(width / B) + min can also round to a value BELOW the running maximum; a batch whose
// maximum lies between the two (a repeated batch, a saturating activation) must then report it, so in that case the
// kernel follows the extrema of every finite element (`track_all`, kernel-uniform).  If the prepare kernel then finds
// the range unchanged, these counts are the batch's contribution and the second read of the batch is skipped (the
// ordinary pass is launched with `rebin` and leaves at once); if the range moved, the ordinary pass bins again on the
// new range and overwrites the partial histograms.  A running range of zero width is binned on a widened one, so then
// every element is looked at.
template <typename IO, int VEC, int NH, bool SPEC = false>
__global__ __launch_bounds__(kBlock, 6) void hist_bin_kernel(const BinArgs a) {
    extern __shared__ uint32_t lds[];  // [NH][B][copies]: lane l adds to copy l % copies, neighbouring copies sit in neighbouring banks
    __shared__ uint32_t cnt_smem[kBlock / kWave][NH][2];
    __shared__ float ext_smem[kBlock / kWave][2];
    if (!SPEC && a.rebin && *a.rebin == 0) return;
    const int B = a.num_bins;
    const float Bf = (float)B;
    const int copies = a.copies;
    for (int i = threadIdx.x; i < copies * NH * B; i += kBlock) lds[i] = 0;
    RangeC r[NH];
    float run_lo = 0.f, run_hi = 0.f;  // SPEC: the running range itself
    if (SPEC) {
        run_lo = a.state_minmax[0];
        run_hi = a.state_minmax[1];
        const float rg[4] = {run_lo, run_hi, round_io<IO>(run_lo), round_io<IO>(run_hi)};
        r[0] = load_range(rg, 0);
    } else {
#pragma unroll
        for (int h = 0; h < NH; ++h) r[h] = load_range(a.ranges, h);
    }
    float ext_min = __builtin_inff(), ext_max = -__builtin_inff();  // SPEC: finite extrema of this lane's elements
    // thresholds beyond which the batch's own extrema reach the reference's clamp
    float thr_min = run_lo, thr_max = run_hi;
    bool track_all = false;
    if (SPEC) {
        const float c_first = a.state_edges[0], c_last = a.state_edges[B];
        thr_min = c_first;
        thr_max = c_last;
        // every element has to be followed when an edge lies strictly inside the running range (or the range is empty)
        track_all = (run_lo == run_hi) | (c_last < run_hi) | (c_first > run_lo);
    }
    auto track = [&](float v) {  // finite elements beyond the outermost edges
        if (SPEC) {
            const bool fin = __builtin_fabsf(v) < __builtin_inff();
            ext_min = fminf(ext_min, (fin & (v < thr_min)) ? v : __builtin_inff());
            ext_max = fmaxf(ext_max, (fin & (v > thr_max)) ? v : -__builtin_inff());
        }
    };
    __syncthreads();
    const int wave = threadIdx.x / kWave;
    const int cshift = a.copy_shift;  // copies == 1 << cshift
    const int bshift = cshift + 2;    // bin index -> byte offset inside one histogram
    const uint32_t limit_bits = f32_to_bits(Bf) - 4u;
    uint32_t* mine[NH];
#pragma unroll
    for (int h = 0; h < NH; ++h) mine[h] = lds + (size_t)h * B * copies + (threadIdx.x & (copies - 1));
    const IO* __restrict__ x = static_cast<const IO*>(a.x);
    uint32_t below[NH], above[NH], zeros[NH];
#pragma unroll
    for (int h = 0; h < NH; ++h) below[h] = above[h] = zeros[h] = 0;

    // every element, exactly (ragged tile, tail elements and the revisit of flagged elements)
    auto bin_slow = [&](float v, bool only_flagged) {
        track(v);
#pragma unroll
        for (int h = 0; h < NH; ++h) {
            const bool inr = (v >= r[h].lo) & (v <= r[h].hi);
            bool fast = false;
            if (only_flagged) (void)bin_estimate(v, r[h], Bf, limit_bits, fast);
            if (inr & !fast) atomicAdd(&mine[h][bin_exact(v, r[h], Bf, B) << cshift], 1u);
            // values below/above the edges (rounded to the tensor dtype) are necessarily outside the fp32 range
            if (!inr) {
                below[h] += v < r[h].thr_lo ? 1u : 0u;
                above[h] += v > r[h].thr_hi ? 1u : 0u;
            }
        }
    };

    // Tiles of kBinU vectors per lane and two register buffers used alternately: a tile's load is issued one round
    // ahead of its binning.  The shape is an empirical optimum, measured on one device back to back (16-batch stream of
    // 268 MB batches): four vectors per lane loaded and binned in a plain loop 1.21 ms, one vector per lane in a
    // plain loop 1.205 ms, this form with two vectors per buffer 1.17 ms, with one 1.15 ms, and the same with the
    // compiler made to wait for the older load only (two loads per lane truly overlapping the binning) 1.19 ms -- as
    // compiled, the branch between the two kinds of load below makes it wait for both.  Fewer bytes in flight per
    // wave are answered sooner on this memory system; the quantize-dequantize kernels show the same.  Past the end
    // the prefetch reads the tensor's first tile with ordinary loads (cache hits after the first workgroup) and the
    // data is dropped.
    constexpr int kBinU = kHistBinU;
    constexpr int kBinVec = kBlock * kBinU;
    const int64_t full_tiles = a.nvec / kBinVec;
    auto load_tile = [&](Pack<IO, VEC>* buf, int64_t t, bool real) {
        if (real) {
#pragma unroll
            for (int u = 0; u < kBinU; ++u) buf[u] = load_pack_stream<IO, VEC>(x + (t * kBinVec + u * kBlock + threadIdx.x) * VEC);
        } else {
#pragma unroll
            for (int u = 0; u < kBinU; ++u) buf[u] = load_pack<IO, VEC>(x + (u * kBlock + threadIdx.x) * VEC);
        }
    };
    auto bin_tile = [&](const Pack<IO, VEC>* in) {
        if (track_all) {
            // (the empty asm keeps the elements' comparisons inside this rarely taken branch: hoisted above it they
            // cost three instructions per element on every tile and spill the masks)
            for (int u = 0; u < kBinU; ++u)
                for (int k = 0; k < VEC; ++k) {
                    float v = load_f32(in[u].v[k]);
                    asm volatile("" : "+v"(v));
                    track(v);
                }
        }
        uint32_t binned = 0;  // this lane's elements that took the fast path
#pragma unroll
        for (int u = 0; u < kBinU; ++u) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                const float v = load_f32(in[u].v[k]);
                // exact zeros (half of a rectified activation) would all add to one LDS word, which serialises the
                // wave's atomics (161 instead of 126 us per batch on such data); they are counted in a register and
                // added to their bin once, at the end.  Costs 4 % on data without zeros.
                const bool zero = v == 0.f;
#pragma unroll
                for (int h = 0; h < NH; ++h) {
                    bool fast;
                    const int b = bin_estimate(v, r[h], Bf, limit_bits, fast);
                    if (fast) {
                        ++binned;
                        if (zero) ++zeros[h];
                        else atomicAdd(reinterpret_cast<uint32_t*>(reinterpret_cast<char*>(mine[h]) + ((uint32_t)b << bshift)), 1u);
                    }
                }
            }
        }
        if (__builtin_amdgcn_ballot_w64(binned != (uint32_t)(kBinU * VEC * NH)) != 0) {
            for (int u = 0; u < kBinU; ++u)
                for (int k = 0; k < VEC; ++k) bin_slow(load_f32(in[u].v[k]), true);
        }
    };
    {
        Pack<IO, VEC> bufa[kBinU], bufb[kBinU];
        const int64_t step = gridDim.x;
        int64_t tile = blockIdx.x;
        if (tile < full_tiles) load_tile(bufa, tile, true);
        while (tile < full_tiles) {
            load_tile(bufb, tile + step, tile + step < full_tiles);
            bin_tile(bufa);
            tile += step;
            if (tile >= full_tiles) break;
            load_tile(bufa, tile + step, tile + step < full_tiles);
            bin_tile(bufb);
            tile += step;
        }
    }
    // the ragged last tile
    if (blockIdx.x == 0 && full_tiles * kBinVec < a.nvec) {
        const int64_t v0 = full_tiles * kBinVec;
        const int nv = (int)(a.nvec - v0);
        for (int u = 0; u < kBinU; ++u) {
            const int lv = u * kBlock + threadIdx.x;
            if (lv < nv) {
                const Pack<IO, VEC> pk = load_pack_stream<IO, VEC>(x + (v0 + lv) * VEC);
                for (int k = 0; k < VEC; ++k) bin_slow(load_f32(pk.v[k]), false);
            }
        }
    }
    if (VEC > 1 && blockIdx.x == 0) {  // elements past the last full vector
        const int64_t i = a.nvec * VEC + threadIdx.x;
        if (i < a.numel) bin_slow(load_f32(x[i]), false);
    }
    // the zeros counted in registers (a non-zero count means zero took the fast path, so it lies inside the range
    // and its estimated bin is the exact one)
#pragma unroll
    for (int h = 0; h < NH; ++h)
        if (zeros[h] != 0) atomicAdd(&mine[h][bin_exact(0.f, r[h], Bf, B) << cshift], zeros[h]);
    // below / above: wave reduce, then across waves
#pragma unroll
    for (int h = 0; h < NH; ++h) {
        uint32_t bl = below[h], ab = above[h];
#pragma unroll
        for (int m = kWave / 2; m >= 1; m >>= 1) {
            bl += __shfl_xor(bl, m, kWave);
            ab += __shfl_xor(ab, m, kWave);
        }
        if ((threadIdx.x & (kWave - 1)) == 0) {
            cnt_smem[wave][h][0] = bl;
            cnt_smem[wave][h][1] = ab;
        }
    }
    if (SPEC) {
#pragma unroll
        for (int m = kWave / 2; m >= 1; m >>= 1) {
            ext_min = fminf(ext_min, __shfl_xor(ext_min, m, kWave));
            ext_max = fmaxf(ext_max, __shfl_xor(ext_max, m, kWave));
        }
        if ((threadIdx.x & (kWave - 1)) == 0) {
            ext_smem[wave][0] = ext_min;
            ext_smem[wave][1] = ext_max;
        }
    }
    __syncthreads();
    if (SPEC && threadIdx.x == 0) {
        float mn = ext_smem[0][0], mx = ext_smem[0][1];
        for (int wv = 1; wv < kBlock / kWave; ++wv) {
            mn = fminf(mn, ext_smem[wv][0]);
            mx = fmaxf(mx, ext_smem[wv][1]);
        }
        a.part_min[blockIdx.x] = mn;
        a.part_max[blockIdx.x] = mx;
    }
    // partial counts in blocks of kPartBins entries (an entry: a bin, or one of the two edge counters behind the bins):
    // [NH][blocks][gridDim.x][kPartBins] -- a workgroup stores 32-byte pieces, and the launch that folds the partials
    // reads all workgroups' counts of a block as one contiguous run
    const size_t np = gridDim.x;
    const int nblk = (B + 2 + kPartBins - 1) / kPartBins;
    auto slot = [&](int h, int entry) {
        return a.partials + (((size_t)h * nblk + entry / kPartBins) * np + blockIdx.x) * kPartBins + entry % kPartBins;
    };
    for (int i = threadIdx.x; i < NH * B; i += kBlock) {
        const int h = i / B, b = i - h * B;
        uint32_t c = 0;
        for (int cp = 0; cp < copies; ++cp) c += lds[(size_t)i * copies + cp];
        *slot(h, b) = c;
    }
    if (threadIdx.x < NH * 2) {
        const int h = threadIdx.x / 2, w = threadIdx.x & 1;
        uint32_t c = 0;
        for (int wv = 0; wv < kBlock / kWave; ++wv) c += cnt_smem[wv][h][w];
        *slot(h, B + w) = c;
    }
}

// Single slot, 16-bit tensors, one histogram: binning through a table.  A 16-bit element has 65536 possible bit
// patterns, and the bin of a pattern is the same for the whole batch, so each workgroup first fills a table in LDS --
// pattern -> bin, or one of three further entries: below the range, above it, neither (NaN, or outside the float
// range but not beyond the thresholds) -- with the exact reference arithmetic (128 KB of the compute unit's 160 KB),
// and an element then costs one table read and one LDS add instead of the thirteen vector instructions of
// hist_bin_kernel, which is what binds that kernel on 16-bit tensors (twice the elements per byte).  Workgroups of
// 1024 threads, one per compute unit; partial counts leave in the layout of hist_bin_kernel.  SPEC as there: the
// elements the table sends outside the range leave their finite extrema, looked at one by one (they are rare).
constexpr int kLutThreads = 1024;
constexpr int kLutEntries = 65536;
constexpr size_t kLutBytes = (size_t)kLutEntries * 2;
constexpr size_t kLdsMax = 160 * 1024;
// Filling the table costs a workgroup as much as binning 64K elements, and a launch has up to 256 of them: below this
// many elements the table does not pay for itself (measured on bf16: 20.8 us against 26.1 at 4M elements, 39.1
// against 42.9 at 32M, 70.9 against 62.3 at 64M).
std::atomic<int64_t> g_table_min_numel{(int64_t)48 << 20};

constexpr int kLutU = 2;  // 16-byte vectors per lane and round of the aligned form

template <typename IO, int VEC, bool SPEC>
__global__ __launch_bounds__(kLutThreads) void hist_bin16_kernel(const BinArgs a) {
    extern __shared__ uint32_t lds[];
    __shared__ float ext_smem[kLutThreads / kWave][2];
    __shared__ uint16_t chunk_entry[kLutEntries / 64];
    if (!SPEC && a.rebin && *a.rebin == 0) return;
    uint16_t* lut = reinterpret_cast<uint16_t*>(lds);
    uint32_t* cnt = lds + kLutBytes / 4;  // [B + 3][copies], lane l adds to copy l % copies
    const int B = a.num_bins;
    const float Bf = (float)B;
    const int copies = a.copies, cshift = a.copy_shift;
    // behind the counters: one word per thread for its exact zeros (see below)
    uint32_t* zero_words = cnt + ((size_t)(B + 3) << cshift);
    for (int i = threadIdx.x; i < (B + 3) * copies + kLutThreads; i += kLutThreads) cnt[i] = 0;
    RangeC r;
    float run_lo = 0.f, run_hi = 0.f, thr_min = 0.f, thr_max = 0.f;
    bool track_all = false;
    if (SPEC) {
        run_lo = a.state_minmax[0];
        run_hi = a.state_minmax[1];
        const float rg[4] = {run_lo, run_hi, round_io<IO>(run_lo), round_io<IO>(run_hi)};
        r = load_range(rg, 0);
        thr_min = a.state_edges[0];
        thr_max = a.state_edges[B];
        track_all = (run_lo == run_hi) | (thr_max < run_hi) | (thr_min > run_lo);
    } else {
        r = load_range(a.ranges, 0);
    }
    auto entry_of = [&](uint32_t pattern) -> uint32_t {
        IO io;
        io.bits = (uint16_t)pattern;
        const float v = load_f32(io);
        if ((v >= r.lo) & (v <= r.hi)) return (uint32_t)bin_exact(v, r, Bf, B);
        return v < r.thr_lo ? (uint32_t)B : (v > r.thr_hi ? (uint32_t)B + 1u : (uint32_t)B + 2u);
    };
    // The table.  The entry is a monotone function of the value on either side of zero, and a run of 64 neighbouring
    // patterns (one sign, rising magnitude) almost always lies inside one bin or outside the range altogether: only
    // the few binades the range's bins are as narrow as 16-bit values are dense in need their entries one by one.
    // So a thread first looks at the two ends of one run; where they agree the run is filled with that entry.  (The
    // entry "neither below nor above" sits on both sides of the range, so agreement on it proves nothing.)  The exact
    // arithmetic per pattern -- a division -- for all 65536 of them cost every workgroup 4 us of a 50 us kernel.
    {
        const uint32_t first = entry_of(threadIdx.x * 64u), last = entry_of(threadIdx.x * 64u + 63u);
        chunk_entry[threadIdx.x] = (uint16_t)((first == last && first != (uint32_t)B + 2u) ? first : 0xffffu);
    }
    __syncthreads();
    for (uint32_t q = threadIdx.x; q < kLutEntries / 2; q += kLutThreads) {
        const uint32_t same = chunk_entry[q >> 5];
        const uint32_t e0 = same != 0xffffu ? same : entry_of(2u * q);
        const uint32_t e1 = same != 0xffffu ? same : entry_of(2u * q + 1u);
        lds[q] = e0 | (e1 << 16);
    }
    __syncthreads();
    float ext_min = __builtin_inff(), ext_max = -__builtin_inff();
    auto track = [&](float v) {  // finite elements beyond the outermost edges (see hist_bin_kernel)
        const bool fin = __builtin_fabsf(v) < __builtin_inff();
        ext_min = fminf(ext_min, (fin & (v < thr_min)) ? v : __builtin_inff());
        ext_max = fmaxf(ext_max, (fin & (v > thr_max)) ? v : -__builtin_inff());
    };
    const uint32_t copy = threadIdx.x & (copies - 1);
    uint32_t* mine = cnt + copy;
    // Exact zeros (half of a rectified activation) would all meet in one LDS word; each thread adds them to a word
    // of its own instead and moves the sum to the bin of zero once, at the end.
    const uint32_t zero_at = (uint32_t)((B + 3) << cshift) + threadIdx.x;
    const IO* __restrict__ x = static_cast<const IO*>(a.x);
    int64_t done = 0;  // elements binned by the vector loop
    if (VEC > 1) {
        // Rounds of kLutU vectors per lane: all the round's table reads are issued before the first increment, so
        // the LDS unit always has independent work queued (an increment waits for its table read).
        const int64_t rounds = a.nvec / (kLutThreads * kLutU);
        for (int64_t t = blockIdx.x; t < rounds; t += gridDim.x) {
            Pack<IO, VEC> in[kLutU];
#pragma unroll
            for (int u = 0; u < kLutU; ++u) in[u] = load_pack_stream<IO, VEC>(x + ((t * kLutU + u) * kLutThreads + threadIdx.x) * VEC);
            uint32_t e[kLutU][VEC];
#pragma unroll
            for (int u = 0; u < kLutU; ++u)
#pragma unroll
                for (int k = 0; k < VEC; ++k) e[u][k] = lut[in[u].v[k].bits];
            bool outside = false;
#pragma unroll
            for (int u = 0; u < kLutU; ++u)
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    const bool zero = (in[u].v[k].bits & 0x7fffu) == 0;
                    atomicAdd(cnt + (zero ? zero_at : (e[u][k] << cshift) + copy), 1u);
                    if (SPEC) outside |= e[u][k] >= (uint32_t)B;
                }
            if (SPEC && (track_all || __builtin_amdgcn_ballot_w64(outside) != 0)) {
#pragma unroll
                for (int u = 0; u < kLutU; ++u)
                    for (int k = 0; k < VEC; ++k) track(load_f32(in[u].v[k]));
            }
        }
        done = rounds * kLutThreads * kLutU * VEC;
    }
    // what the rounds leave (less than one round; everything when the tensor is not 16-byte aligned), element by
    // element, spread over the workgroups
    for (int64_t i = done + (int64_t)blockIdx.x * kLutThreads + threadIdx.x; i < a.numel; i += (int64_t)gridDim.x * kLutThreads) {
        const uint32_t bits = x[i].bits;
        const uint32_t e = lut[bits];
        atomicAdd(cnt + ((bits & 0x7fffu) == 0 ? zero_at : (e << cshift) + copy), 1u);
        if (SPEC && (track_all || e >= (uint32_t)B)) track(load_f32(x[i]));
    }
    __syncthreads();
    {
        const uint32_t zeros = zero_words[threadIdx.x];
        if (zeros != 0) atomicAdd(mine + ((uint32_t)lut[0] << cshift), zeros);
    }
    if (SPEC) {
#pragma unroll
        for (int m = kWave / 2; m >= 1; m >>= 1) {
            ext_min = fminf(ext_min, __shfl_xor(ext_min, m, kWave));
            ext_max = fmaxf(ext_max, __shfl_xor(ext_max, m, kWave));
        }
        if ((threadIdx.x & (kWave - 1)) == 0) {
            ext_smem[threadIdx.x / kWave][0] = ext_min;
            ext_smem[threadIdx.x / kWave][1] = ext_max;
        }
    }
    __syncthreads();
    if (SPEC && threadIdx.x == 0) {
        float mn = ext_smem[0][0], mx = ext_smem[0][1];
        for (int wv = 1; wv < kLutThreads / kWave; ++wv) {
            mn = fminf(mn, ext_smem[wv][0]);
            mx = fmaxf(mx, ext_smem[wv][1]);
        }
        a.part_min[blockIdx.x] = mn;
        a.part_max[blockIdx.x] = mx;
    }
    // partial counts in the layout hist_bin_kernel leaves them in: entries 0..B-1 the bins, B below, B + 1 above
    const size_t np = gridDim.x;
    for (int e = threadIdx.x; e < B + 2; e += kLutThreads) {
        uint32_t c = 0;
        for (int cp = 0; cp < copies; ++cp) c += cnt[((size_t)e << cshift) + cp];
        a.partials[(((size_t)(e / kPartBins)) * np + blockIdx.x) * kPartBins + e % kPartBins] = c;
    }
}

// The table kernels need more dynamic LDS than a kernel gets by default: asked for once per device and dtype, for
// the most any launch uses; false when the runtime refuses (the callers then keep the arithmetic kernels).
static bool lut_lds_available(int dtype) {
    constexpr int kMost = (int)(kLdsMax - 4096);
    constexpr int kMaxDevices = 64;
    static std::atomic<int> state[kMaxDevices][2];  // 0 not asked yet, 1 granted, 2 refused
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return false;
    std::atomic<int>& st = state[dev][dtype == AHQ_F16 ? 0 : 1];
    int v = st.load(std::memory_order_acquire);
    if (v == 0) {
        auto allow = [](auto kernel) {
            return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kMost) == hipSuccess;
        };
        const bool ok = dtype == AHQ_F16
            ? allow(&hist_bin16_kernel<f16_t, 1, true>) && allow(&hist_bin16_kernel<f16_t, 1, false>) &&
              allow(&hist_bin16_kernel<f16_t, 8, true>) && allow(&hist_bin16_kernel<f16_t, 8, false>)
            : allow(&hist_bin16_kernel<bf16_t, 1, true>) && allow(&hist_bin16_kernel<bf16_t, 1, false>) &&
              allow(&hist_bin16_kernel<bf16_t, 8, true>) && allow(&hist_bin16_kernel<bf16_t, 8, false>);
        if (!ok) (void)hipGetLastError();  // the refusal is handled here, not reported by the next launch check
        v = ok ? 1 : 2;
        st.store(v, std::memory_order_release);
    }
    return v == 1;
}

// Several slots whose runs are long enough that a tile lies inside one run (per-channel weights, per-channel
// activations with large feature maps): one workgroup per tile bins into LDS sub-histograms of its slot and adds the
// non-empty bins to the slot's zero-initialised counters in global memory.
template <typename IO, int VEC, int NH>
__global__ __launch_bounds__(kBlock, 6) void hist_bin_rows_kernel(const BinArgs a, const Geom rows) {
    extern __shared__ uint32_t lds[];  // [NH][B][copies]
    __shared__ uint32_t cnt_smem[kBlock / kWave][NH][2];
    const int B = a.num_bins;
    const float Bf = (float)B;
    const int copies = a.copies;
    const Tile t = make_tile(rows, blockIdx.x);
    for (int i = threadIdx.x; i < copies * NH * B; i += kBlock) lds[i] = 0;
    RangeC r[NH];
#pragma unroll
    for (int h = 0; h < NH; ++h) r[h] = load_range(a.ranges + t.e0 * kRng, h);
    __syncthreads();
    const int cshift = a.copy_shift, bshift = cshift + 2;
    const uint32_t limit_bits = f32_to_bits(Bf) - 4u;
    uint32_t* mine[NH];
#pragma unroll
    for (int h = 0; h < NH; ++h) mine[h] = lds + (size_t)h * B * copies + (threadIdx.x & (copies - 1));
    const IO* __restrict__ x = static_cast<const IO*>(a.x) + t.v0 * VEC;
    uint32_t below[NH], above[NH];
#pragma unroll
    for (int h = 0; h < NH; ++h) below[h] = above[h] = 0;
    auto bin_slow = [&](float v, bool only_flagged) {
#pragma unroll
        for (int h = 0; h < NH; ++h) {
            const bool inr = (v >= r[h].lo) & (v <= r[h].hi);
            bool fast = false;
            if (only_flagged) (void)bin_estimate(v, r[h], Bf, limit_bits, fast);
            if (inr & !fast) atomicAdd(&mine[h][bin_exact(v, r[h], Bf, B) << cshift], 1u);
            if (!inr) {
                below[h] += v < r[h].thr_lo ? 1u : 0u;
                above[h] += v > r[h].thr_hi ? 1u : 0u;
            }
        }
    };
    if (t.nv == kTileVec) {
        Pack<IO, VEC> in[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) in[u] = load_pack_stream<IO, VEC>(x + (int64_t)(u * kBlock + threadIdx.x) * VEC);
        uint32_t binned = 0;
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                const float v = load_f32(in[u].v[k]);
#pragma unroll
                for (int h = 0; h < NH; ++h) {
                    bool fast;
                    const int b = bin_estimate(v, r[h], Bf, limit_bits, fast);
                    if (fast) {
                        atomicAdd(reinterpret_cast<uint32_t*>(reinterpret_cast<char*>(mine[h]) + ((uint32_t)b << bshift)), 1u);
                        ++binned;
                    }
                }
            }
        if (__builtin_amdgcn_ballot_w64(binned != (uint32_t)(kUnroll * VEC * NH)) != 0) {
            for (int u = 0; u < kUnroll; ++u)
                for (int k = 0; k < VEC; ++k) bin_slow(load_f32(in[u].v[k]), true);
        }
    } else {
        for (int u = 0; u < kUnroll; ++u) {
            const int lv = u * kBlock + threadIdx.x;
            if (lv < t.nv) {
                const Pack<IO, VEC> pk = load_pack_stream<IO, VEC>(x + (int64_t)lv * VEC);
                for (int k = 0; k < VEC; ++k) bin_slow(load_f32(pk.v[k]), false);
            }
        }
    }
    const int wave = threadIdx.x / kWave;
#pragma unroll
    for (int h = 0; h < NH; ++h) {
        uint32_t bl = below[h], ab = above[h];
#pragma unroll
        for (int m = kWave / 2; m >= 1; m >>= 1) {
            bl += __shfl_xor(bl, m, kWave);
            ab += __shfl_xor(ab, m, kWave);
        }
        if ((threadIdx.x & (kWave - 1)) == 0) {
            cnt_smem[wave][h][0] = bl;
            cnt_smem[wave][h][1] = ab;
        }
    }
    __syncthreads();
    uint32_t* out = a.counts + (size_t)t.e0 * NH * (B + 2);
    for (int i = threadIdx.x; i < NH * B; i += kBlock) {
        const int h = i / B, b = i - h * B;
        uint32_t c = 0;
        for (int cp = 0; cp < copies; ++cp) c += lds[(size_t)i * copies + cp];
        if (c) atomicAdd(&out[h * (B + 2) + b], c);
    }
    if (threadIdx.x < NH * 2) {
        const int h = threadIdx.x / 2, w = threadIdx.x & 1;
        uint32_t c = 0;
        for (int wv = 0; wv < kBlock / kWave; ++wv) c += cnt_smem[wv][h][w];
        if (c) atomicAdd(&out[h * (B + 2) + B + w], c);
    }
}

// Several slots (or histograms too large for LDS): every element adds to its slot's counters in global memory.
template <typename IO>
__global__ __launch_bounds__(kBlock) void hist_bin_generic_kernel(const BinArgs a) {
    const int B = a.num_bins;
    const float Bf = (float)B;
    const IO* __restrict__ x = static_cast<const IO*>(a.x);
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < a.numel; i += (int64_t)gridDim.x * kBlock) {
        int64_t e;
        if (a.nseg > 0) e = generic_enc_index(a, i);
        else e = a.J == 1 ? 0 : (i / a.K) % a.J;
        const float v = load_f32(x[i]);
        const float* rg = a.ranges + e * kRng;
        uint32_t* c = a.counts + (size_t)e * a.nhist * (B + 2);
        for (int h = 0; h < a.nhist; ++h) {
            const RangeC r = load_range(rg, h);
            if ((v >= r.lo) & (v <= r.hi)) atomicAdd(&c[h * (B + 2) + bin_exact(v, r, Bf, B)], 1u);
            if (v < r.thr_lo) atomicAdd(&c[h * (B + 2) + B], 1u);
            if (v > r.thr_hi) atomicAdd(&c[h * (B + 2) + B + 1], 1u);
        }
    }
}

__global__ void zero_u32_kernel(uint32_t* p, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0;
}

// ----------------------------------------------------------------------------------------------------- finish --
struct FinArgs {
    int32_t num_slots, num_bins, nhist, first;
    int32_t nparts;            // partial histograms per slot (1 when `counts` is used)
    const uint32_t* counts;    // several slots: [S][NH][B + 2] (nparts == 1); one slot: see hist_bin_kernel
    const float* carried;      // [S][B]
    const float* upd_edges;    // [S][B+1]
    float* hist;               // [S][B] running (out)
    float* edges;              // [S][B+1] running (out)
    float* new_hist;           // [S][B] (out)
    // single-slot fold-and-finish only:
    const int32_t* rebin;      // optional: leave at once when *rebin == 0 (the speculative pass already was the update)
    const float* ranges;       // optional, with `minmax`: the new running range (ranges[4], ranges[5]) is stored into
    float* minmax;             //   the state here, by the launch that ends the update
};

__global__ __launch_bounds__(kBlock) void hist_finish_kernel(const FinArgs a) {
    // grid: (ceil(B/64), S); thread = (bin within 64, group of partials)
    __shared__ unsigned long long sm[4][2][64];
    __shared__ unsigned long long edge_cnt[2][2];
    const int B = a.num_bins, NH = a.nhist;
    const int bl = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int b = blockIdx.x * 64 + bl;
    // the y dimension of a grid ends at 65535: slots beyond it are taken in further rounds
    for (int s = blockIdx.y; s < a.num_slots; s += gridDim.y) {
    if (s != (int)blockIdx.y) __syncthreads();  // the previous slot's sums in LDS are still being read
    const uint32_t* base = a.counts + (size_t)s * a.nparts * NH * (B + 2);
    unsigned long long c[2] = {0, 0};
    if (b < B) {
        for (int p = grp; p < a.nparts; p += 4)
            for (int h = 0; h < NH; ++h) c[h] += base[((size_t)p * NH + h) * (B + 2) + b];
    }
    sm[grp][0][bl] = c[0];
    sm[grp][1][bl] = c[1];
    // below/above totals (needed by the workgroups that own bin 0 and bin B-1; cheap enough to do everywhere)
    {
        // wave w (0..3) owns edge counter (h = w / 2, side = w % 2); its lanes stride over the partials
        const int w4 = threadIdx.x >> 6, lane = threadIdx.x & 63;
        const int h = w4 >> 1, side = w4 & 1;
        unsigned long long t = 0;
        if (h < NH)
            for (int p = lane; p < a.nparts; p += 64) t += base[((size_t)p * NH + h) * (B + 2) + B + side];
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) t += __shfl_xor(t, m, kWave);
        if (lane == 0) edge_cnt[h][side] = t;
    }
    __syncthreads();
    if (grp != 0 || b >= B) continue;
    unsigned long long tot[2];
    for (int h = 0; h < 2; ++h) tot[h] = sm[0][h][bl] + sm[1][h][bl] + sm[2][h][bl] + sm[3][h][bl];
    // the batch's own histogram: counts, then "+= below" on bin 0 and "+= above" on the last bin
    float nh = (float)tot[0];
    if (b == 0) nh += (float)edge_cnt[0][0];
    if (b == B - 1) nh += (float)edge_cnt[0][1];
    if (a.new_hist) a.new_hist[(size_t)s * B + b] = nh;
    float uh;
    if (a.first) {
        uh = nh;
    } else {
        const int h = NH - 1;
        uh = (float)tot[h] + a.carried[(size_t)s * B + b];
        if (b == 0) uh += (float)edge_cnt[h][0];
        if (b == B - 1) uh += (float)edge_cnt[h][1];
    }
    a.hist[(size_t)s * B + b] = uh;
    a.edges[(size_t)s * (B + 1) + b] = a.upd_edges[(size_t)s * (B + 1) + b];
    if (b == B - 1) a.edges[(size_t)s * (B + 1) + B] = a.upd_edges[(size_t)s * (B + 1) + B];
    }
}

// --------------------------------------------------------- single slot: fold of the partial counts and finish --
// One launch instead of a fold and a finish: a workgroup of 1024 threads owns one block of kPartBins bins, whose
// partial counts from all workgroups of the binning pass are one contiguous run of memory (see hist_bin_kernel), so
// the threads read it as whole cache lines, every thread always the same bin.  The integer sums are order-independent,
// the float operations per bin are those of hist_finish_kernel.  `carried` may be the running histogram itself (a
// bin is read and written by one thread); upd_edges == NULL leaves the running edges as they are.
constexpr int kFfThreads = 1024;

__device__ __forceinline__ const uint32_t* part_block(const FinArgs& a, int h, int blk) {
    const int nblk = (a.num_bins + 2 + kPartBins - 1) / kPartBins;
    return a.counts + ((size_t)h * nblk + blk) * (size_t)a.nparts * kPartBins;
}

// this thread's share of the sums of bin blockIdx.x * kPartBins + thread % kPartBins; all its loads in flight at once
__device__ __forceinline__ void fold_load(const FinArgs& a, unsigned long long (&c)[2]) {
    c[0] = c[1] = 0;
    const int n = a.nparts * kPartBins;
    constexpr int kFlight = 16;  // 16 * 1024 entries = 2048 workgroups per round: one round for any binning grid
    for (int h = 0; h < a.nhist; ++h) {
        const uint32_t* run = part_block(a, h, blockIdx.x);
        unsigned long long t = 0;
        for (int j = threadIdx.x; j < n; j += kFlight * kFfThreads) {
            uint32_t v[kFlight];
#pragma unroll
            for (int k = 0; k < kFlight; ++k) v[k] = j + k * kFfThreads < n ? run[j + k * kFfThreads] : 0u;
#pragma unroll
            for (int k = 0; k < kFlight; ++k) t += v[k];
        }
        c[h] = t;
    }
}

__device__ void fold_finish_bins(const FinArgs& a, unsigned long long (&c)[2]) {
    __shared__ unsigned long long sm[kFfThreads / kWave][2][kPartBins];
    __shared__ unsigned long long wave_edge[kFfThreads / kWave][4];
    const int B = a.num_bins, NH = a.nhist;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
    const int b = blockIdx.x * kPartBins + threadIdx.x;  // for the threads that finish a bin (the first kPartBins)
    const bool owner = threadIdx.x < kPartBins && b < B;
    const float carried_b = (owner && !a.first) ? a.carried[b] : 0.f;  // fetched ahead of the barrier
#pragma unroll
    for (int m = kWave / 2; m >= kPartBins; m >>= 1) {
        c[0] += __shfl_xor(c[0], m, kWave);
        c[1] += __shfl_xor(c[1], m, kWave);
    }
    if (lane < kPartBins) {
        sm[wave][0][lane] = c[0];
        sm[wave][1][lane] = c[1];
    }
    // below / above totals (entries B and B + 1 of every partial histogram), wanted by the owners of bin 0 and of
    // bin B - 1: thread = (histogram, side, workgroups of the binning pass)
    const bool owns_end = blockIdx.x == 0 || (int)blockIdx.x == (B - 1) / kPartBins;
    if (owns_end) {
        const int combo = threadIdx.x & 3, h = combo >> 1, side = combo & 1;
        unsigned long long t = 0;
        if (h < NH) {
            const int entry = B + side;
            const uint32_t* run = part_block(a, h, entry / kPartBins) + entry % kPartBins;
            constexpr int kFlight = 8, kStep = kFfThreads / 4;  // 8 * 256 workgroups per round
            for (int p = threadIdx.x >> 2; p < a.nparts; p += kFlight * kStep) {
                uint32_t v[kFlight];
#pragma unroll
                for (int k = 0; k < kFlight; ++k)
                    v[k] = p + k * kStep < a.nparts ? run[(size_t)(p + k * kStep) * kPartBins] : 0u;
#pragma unroll
                for (int k = 0; k < kFlight; ++k) t += v[k];
            }
        }
#pragma unroll
        for (int m = kWave / 2; m >= 4; m >>= 1) t += __shfl_xor(t, m, kWave);
        if (lane < 4) wave_edge[wave][lane] = t;
    }
    __syncthreads();
    if (!owner) return;
    unsigned long long tot[2] = {0, 0};
    for (int w = 0; w < kFfThreads / kWave; ++w) {
        tot[0] += sm[w][0][threadIdx.x];
        tot[1] += sm[w][1][threadIdx.x];
    }
    unsigned long long edge_cnt[2][2] = {{0, 0}, {0, 0}};
    if (b == 0 || b == B - 1)
        for (int w = 0; w < kFfThreads / kWave; ++w)
            for (int q = 0; q < 4; ++q) edge_cnt[q >> 1][q & 1] += wave_edge[w][q];
    // the batch's own histogram: counts, then "+= below" on bin 0 and "+= above" on the last bin
    float nh = (float)tot[0];
    if (b == 0) nh += (float)edge_cnt[0][0];
    if (b == B - 1) nh += (float)edge_cnt[0][1];
    if (a.new_hist) a.new_hist[b] = nh;
    float uh;
    if (a.first) {
        uh = nh;
    } else {
        const int h = NH - 1;
        uh = (float)tot[h] + carried_b;
        if (b == 0) uh += (float)edge_cnt[h][0];
        if (b == B - 1) uh += (float)edge_cnt[h][1];
    }
    a.hist[b] = uh;
    if (a.upd_edges) {
        a.edges[b] = a.upd_edges[b];
        if (b == B - 1) a.edges[B] = a.upd_edges[B];
    }
}

__global__ __launch_bounds__(kFfThreads) void hist_fold_finish_kernel(const FinArgs a) {
    if (a.rebin && *a.rebin == 0) return;
    if (a.minmax && blockIdx.x == 0 && threadIdx.x == 0) {
        a.minmax[0] = a.ranges[4];
        a.minmax[1] = a.ranges[5];
    }
    unsigned long long c[2];
    fold_load(a, c);
    fold_finish_bins(a, c);
}

// After a speculative binning pass (hist_bin_kernel<SPEC>), single slot.  Every workgroup folds the pass's partial
// extrema and decides, from the same unchanged state, whether the running range holds.  If it does, the pass's counts
// are the batch's contribution: the workgroups fold them into the running histogram (16 bins each) and the update is
// complete -- the launches that follow see *rebin == 0 and leave at once.  If it does not, workgroup 0 prepares the
// second pass (new range and edges, running counts carried over to the new bins), the others leave; the state's min /
// max are left alone in this launch because the other workgroups compare against them.
template <typename IO>
__global__ __launch_bounds__(kFfThreads) void hist_resolve_kernel(const PrepArgs pa, const FinArgs fa) {
    float mn, mx, umin, umax;
    unsigned long long c[2];
    const RunningRange running = load_running_range(pa, 0);
    fold_load(fa, c);  // ahead of the decision: reading the counts is harmless, and the latencies overlap
    fold_partial_extrema(pa, mn, mx);
    const bool same = updated_range(running, mn, mx, umin, umax);
    if (same) {
        if (blockIdx.x == 0 && threadIdx.x == 0) pa.rebin[0] = 0;
        fold_finish_bins(fa, c);
    } else if (blockIdx.x == 0) {
        prepare_slot<IO>(pa, 0, mn, mx, true);
    }
}

}  // namespace ahq

using namespace ahq;

namespace {

struct HistPlan {
    Plan plan;
    Plan rows_plan;  // tiling by runs (valid when `rows`)
    bool fast;       // single slot through LDS
    bool rows;       // several slots, every tile inside one run: per-tile LDS histograms
    int copies;
    int nblocks;
    int64_t ntiles;
    size_t off_mm_ws, off_bmin, off_bmax, off_ranges, off_carried, off_upd_edges, off_scratch, off_rebin, off_counts, total;
};

size_t align_up(size_t v) { return (v + 255) & ~(size_t)255; }

bool make_hist_plan(int dtype, const ahq_layout& layout, const void* x, int num_bins, HistPlan* hp) {
    if (!make_plan(dtype, layout, aligned16(x), false, &hp->plan)) return false;
    const CanonLayout& c = hp->plan.cl;
    const int64_t S = c.num_enc;
    hp->fast = false;
    hp->copies = 0;
    if (c.kind == kIJK && c.J == 1) {
        // at most 16 KB of LDS per workgroup of four waves, so that eight workgroups (32 waves) fit a compute unit
        const int fit = (int)(16384 / ((size_t)2 * num_bins * 4));
        int copies = 0;
        for (int c = 8; c >= 1; c >>= 1)
            if (c <= fit) {
                copies = c;
                break;
            }
        if (copies >= 1) {
            hp->fast = true;
            hp->copies = copies;
        }
    }
    hp->rows = false;
    if (c.kind == kIJK && c.J > 1) {
        const int fit = (int)(16384 / ((size_t)2 * num_bins * 4));
        int copies = 0;
        for (int c2 = 8; c2 >= 1; c2 >>= 1)
            if (c2 <= fit) {
                copies = c2;
                break;
            }
        if (copies >= 1 && make_plan(dtype, layout, aligned16(x), true, &hp->rows_plan) && hp->rows_plan.mode == kRows) {
            hp->rows = true;
            hp->copies = copies;
        }
    }
    hp->ntiles = (hp->plan.nvec + kBlock * kHistBinU - 1) / (kBlock * kHistBinU);
    int64_t nb = hp->fast ? hp->ntiles : (c.numel + kBlock - 1) / kBlock;
    if (nb > kHistBlocksMax) nb = kHistBlocksMax;
    if (nb < 1) nb = 1;
    hp->nblocks = (int)nb;
    const size_t B = (size_t)num_bins;
    size_t o = 0;
    // (the same region holds the speculative pass's partial extrema: two floats per workgroup)
    hp->off_mm_ws = o;     o = align_up(o + std::max(ahq_minmax_workspace_bytes(&layout), (size_t)kHistBlocksMax * 8));
    hp->off_bmin = o;      o = align_up(o + (size_t)S * 4);
    hp->off_bmax = o;      o = align_up(o + (size_t)S * 4);
    hp->off_ranges = o;    o = align_up(o + (size_t)S * kRng * 4);
    hp->off_carried = o;   o = align_up(o + (size_t)S * B * 4);
    hp->off_upd_edges = o; o = align_up(o + (size_t)S * (B + 1) * 4);
    hp->off_scratch = o;   o = align_up(o + (size_t)S * 2 * B * 4);
    hp->off_rebin = o;     o = align_up(o + (size_t)S * 4);
    hp->off_counts = o;
    const size_t nparts = hp->fast ? (size_t)hp->nblocks : 1;
    const size_t entries = ((B + 2 + kPartBins - 1) / kPartBins) * kPartBins;  // the single-slot layout is in whole blocks
    o = align_up(o + (size_t)S * nparts * 2 * entries * 4);
    hp->total = o;
    return true;
}

}  // namespace

extern "C" size_t ahq_hist_update_workspace_bytes(int32_t dtype, const ahq_layout* layout, int32_t num_bins) {
    if (!layout || num_bins <= 0) return 0;
    HistPlan hp;
    size_t need = 0;
    // the plan depends on pointer alignment only through the vector width; take the larger of the two
    if (make_hist_plan(dtype, *layout, nullptr, num_bins, &hp)) need = hp.total;
    if (make_hist_plan(dtype, *layout, reinterpret_cast<const void*>(4), num_bins, &hp) && hp.total > need) need = hp.total;
    return need;
}

extern "C" int64_t ahq_hist_table_min_numel(int64_t set) {
    return set >= 0 ? g_table_min_numel.exchange(set) : g_table_min_numel.load();
}

extern "C" int ahq_hist_update(int32_t dtype, const ahq_layout* layout, const void* x, const ahq_hist_state* st,
                               int first_batch, void* workspace, size_t workspace_bytes, void* stream) {
    if (dtype < AHQ_F32 || dtype > AHQ_BF16) return set_error("bad dtype"), AHQ_ERR_INVALID;
    if (!layout || !st || !x) return set_error("null argument"), AHQ_ERR_INVALID;
    if (st->num_bins <= 0) return set_error("num_bins must be positive"), AHQ_ERR_INVALID;
    if (!st->hist || !st->edges || !st->minmax || !st->limits)
        return set_error("histogram state has a null buffer"), AHQ_ERR_INVALID;
    if ((st->new_edges == nullptr) != (st->new_minmax == nullptr) || (st->new_hist && !st->new_edges))
        return set_error("new_edges and new_minmax go together, and new_hist needs them"), AHQ_ERR_INVALID;
    if (!(st->growth_limit >= 1.0f)) return set_error("growth limit must be at least 1"), AHQ_ERR_INVALID;
    HistPlan hp;
    if (!make_hist_plan(dtype, *layout, x, st->num_bins, &hp)) return AHQ_ERR_INVALID;
    const CanonLayout& c = hp.plan.cl;
    if (c.numel == 0) return set_error("cannot observe an empty tensor"), AHQ_ERR_INVALID;
    if (c.num_enc != st->num_slots) return set_error("layout does not have num_slots encodings"), AHQ_ERR_INVALID;
    if (!workspace || workspace_bytes < hp.total) return set_error("workspace too small"), AHQ_ERR_WORKSPACE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    char* w = static_cast<char*>(workspace);
    const int S = st->num_slots, B = st->num_bins;
    // Without new_hist only the running histogram is formed: one LDS update per element instead of two (a first batch
    // forms a single histogram either way, its own one being the running one).
    const bool merged_only = !first_batch && !st->new_hist;
    const int NH = (first_batch || merged_only) ? 1 : 2;

    // A batch after the first, one slot, only the running histogram wanted: bin on the running range while reading
    // the batch for its extrema, and bin again only if the range turns out to have changed.
    const bool speculative = merged_only && !st->new_edges && hp.fast && (size_t)hp.nblocks * 8 <= hp.off_bmin - hp.off_mm_ws;
    BinArgs ba{};
    fill_geom(hp.plan, &ba);
    ba.x = x;
    ba.num_bins = B;
    ba.nhist = NH;
    ba.copies = hp.copies;
    ba.copy_shift = 0;
    while ((1 << ba.copy_shift) < hp.copies) ++ba.copy_shift;
    ba.ntiles = hp.ntiles;
    uint32_t* counts = reinterpret_cast<uint32_t*>(w + hp.off_counts);
    int32_t* rebin = reinterpret_cast<int32_t*>(w + hp.off_rebin);

    // 16-bit tensors, one histogram: the binning kernel that looks the bin up in a table (hist_bin16_kernel)
    int lut_copies = 0;
    if (hp.fast && NH == 1 && dtype != AHQ_F32 && c.numel >= g_table_min_numel.load(std::memory_order_relaxed)) {
        // static arrays of the kernel (4 KB), one word per thread for its zeros, then the counters
        const size_t room = kLdsMax - kLutBytes - 4096 - (size_t)kLutThreads * 4;
        for (int c2 = 8; c2 >= 1 && lut_copies == 0; c2 >>= 1)
            if ((size_t)c2 * (B + 3) * 4 <= room) lut_copies = c2;
        if (lut_copies > 0 && !lut_lds_available(dtype)) lut_copies = 0;  // refused: the arithmetic kernels bin
    }
    const int lut_blocks = lut_copies > 0 ? (int)std::min<int64_t>(std::max<int64_t>(hp.plan.nvec / kLutThreads, 1), std::min(256, hp.nblocks)) : 0;
    auto launch_lut = [&](BinArgs args, bool spec) {
        args.copies = lut_copies;
        args.copy_shift = 0;
        while ((1 << args.copy_shift) < lut_copies) ++args.copy_shift;
        const size_t lds = kLutBytes + (size_t)lut_copies * (B + 3) * 4 + (size_t)kLutThreads * 4;
        const dim3 g(lut_blocks), b(kLutThreads);
#define AHQ_LAUNCH_LUT_K(K) hipLaunchKernelGGL(K, g, b, lds, s, args)
#define AHQ_LAUNCH_LUT(IO)                                                                                          \
    do {                                                                                                            \
        if (hp.plan.vec == 1) {                                                                                     \
            if (spec) AHQ_LAUNCH_LUT_K((hist_bin16_kernel<IO, 1, true>));                                           \
            else AHQ_LAUNCH_LUT_K((hist_bin16_kernel<IO, 1, false>));                                               \
        } else {                                                                                                    \
            if (spec) AHQ_LAUNCH_LUT_K((hist_bin16_kernel<IO, 8, true>));                                           \
            else AHQ_LAUNCH_LUT_K((hist_bin16_kernel<IO, 8, false>));                                               \
        }                                                                                                           \
    } while (0)
        if (dtype == AHQ_F16) AHQ_LAUNCH_LUT(f16_t);
        else AHQ_LAUNCH_LUT(bf16_t);
#undef AHQ_LAUNCH_LUT
#undef AHQ_LAUNCH_LUT_K
    };
    const int bin_blocks = lut_copies > 0 ? lut_blocks : hp.nblocks;  // partial histograms the binning pass leaves

    // 1. finite range of the batch, in the tensor's dtype
    const float *part_min = nullptr, *part_max = nullptr;
    int64_t nparts = 0;
    if (speculative) {
        ba.partials = counts;
        ba.state_minmax = st->minmax;
        ba.state_edges = st->edges;
        ba.part_min = reinterpret_cast<float*>(w + hp.off_mm_ws);
        ba.part_max = ba.part_min + bin_blocks;
        const size_t lds = (size_t)hp.copies * B * 4;
        const dim3 g(hp.nblocks), b(kBlock);
#define AHQ_LAUNCH_SPEC(IO)                                                                                         \
    do {                                                                                                            \
        if (hp.plan.vec == 1) hipLaunchKernelGGL((hist_bin_kernel<IO, 1, 1, true>), g, b, lds, s, ba);              \
        else hipLaunchKernelGGL((hist_bin_kernel<IO, IoTraits<IO>::kVec, 1, true>), g, b, lds, s, ba);              \
    } while (0)
        if (lut_copies > 0) {
            launch_lut(ba, true);
        } else {
            switch (dtype) {
                case AHQ_F32: AHQ_LAUNCH_SPEC(float); break;
                case AHQ_F16: AHQ_LAUNCH_SPEC(f16_t); break;
                default: AHQ_LAUNCH_SPEC(bf16_t); break;
            }
        }
#undef AHQ_LAUNCH_SPEC
        part_min = ba.part_min;
        part_max = ba.part_max;
        nparts = bin_blocks;
        ba.rebin = rebin;  // for the second pass
    } else {
        int rc = ahq_minmax_finite_partials(dtype, layout, x, w + hp.off_bmin, w + hp.off_bmax, w + hp.off_mm_ws,
                                            hp.off_bmin - hp.off_mm_ws, stream, &part_min, &part_max, &nparts);
        if (rc != AHQ_OK) return rc;
    }

    // 2. edges, updated range, re-binned running counts
    PrepArgs pa{};
    pa.num_slots = S;
    pa.num_bins = B;
    pa.first = first_batch ? 1 : 0;
    pa.growth = st->growth_limit;
    pa.bmin = w + hp.off_bmin;
    pa.bmax = w + hp.off_bmax;
    pa.part_min = part_min;
    pa.part_max = part_max;
    pa.nparts = S == 1 ? nparts : 0;
    pa.hist = st->hist;
    pa.edges = st->edges;
    pa.minmax = st->minmax;
    pa.limits = st->limits;
    pa.new_edges = st->new_edges;
    pa.new_minmax = st->new_minmax;
    pa.carried = reinterpret_cast<float*>(w + hp.off_carried);
    pa.upd_edges = reinterpret_cast<float*>(w + hp.off_upd_edges);
    pa.ranges = reinterpret_cast<float*>(w + hp.off_ranges);
    pa.scratch = reinterpret_cast<int32_t*>(w + hp.off_scratch);
    pa.rebin = speculative ? rebin : nullptr;
    FinArgs fa{};
    fa.num_slots = S;
    fa.num_bins = B;
    const dim3 ffgrid((B + kPartBins - 1) / kPartBins);
    if (speculative) {
        // the counts of the speculative pass, folded straight into the running histogram if the range holds
        fa.nhist = 1;
        fa.first = 0;
        fa.nparts = bin_blocks;
        fa.counts = counts;
        fa.carried = st->hist;
        fa.hist = st->hist;
        switch (dtype) {
            case AHQ_F32: hipLaunchKernelGGL((hist_resolve_kernel<float>), ffgrid, dim3(kFfThreads), 0, s, pa, fa); break;
            case AHQ_F16: hipLaunchKernelGGL((hist_resolve_kernel<f16_t>), ffgrid, dim3(kFfThreads), 0, s, pa, fa); break;
            default: hipLaunchKernelGGL((hist_resolve_kernel<bf16_t>), ffgrid, dim3(kFfThreads), 0, s, pa, fa); break;
        }
    } else {
        const int pthreads = nparts > 0 ? 1024 : (B >= 512 ? 512 : (B >= 64 ? ((B + 63) / 64) * 64 : 64));
        switch (dtype) {
            case AHQ_F32: hipLaunchKernelGGL((hist_prepare_kernel<float>), dim3(S), dim3(pthreads), 0, s, pa); break;
            case AHQ_F16: hipLaunchKernelGGL((hist_prepare_kernel<f16_t>), dim3(S), dim3(pthreads), 0, s, pa); break;
            default: hipLaunchKernelGGL((hist_prepare_kernel<bf16_t>), dim3(S), dim3(pthreads), 0, s, pa); break;
        }
    }

    // 3. binning pass (after a speculative pass: only if the range changed)
    ba.ranges = merged_only ? pa.ranges + 4 : pa.ranges;  // per slot: the batch's own range, then the running one
    if (hp.fast) {
        ba.partials = counts;
        const size_t lds = (size_t)hp.copies * NH * B * 4;
        const dim3 g(hp.nblocks), b(kBlock);
#define AHQ_LAUNCH_BIN(IO)                                                                                          \
    do {                                                                                                            \
        if (hp.plan.vec == 1) {                                                                                     \
            if (NH == 1) hipLaunchKernelGGL((hist_bin_kernel<IO, 1, 1>), g, b, lds, s, ba);                         \
            else hipLaunchKernelGGL((hist_bin_kernel<IO, 1, 2>), g, b, lds, s, ba);                                 \
        } else {                                                                                                    \
            if (NH == 1) hipLaunchKernelGGL((hist_bin_kernel<IO, IoTraits<IO>::kVec, 1>), g, b, lds, s, ba);        \
            else hipLaunchKernelGGL((hist_bin_kernel<IO, IoTraits<IO>::kVec, 2>), g, b, lds, s, ba);                \
        }                                                                                                           \
    } while (0)
        if (lut_copies > 0) {
            launch_lut(ba, false);
        } else {
            switch (dtype) {
                case AHQ_F32: AHQ_LAUNCH_BIN(float); break;
                case AHQ_F16: AHQ_LAUNCH_BIN(f16_t); break;
                default: AHQ_LAUNCH_BIN(bf16_t); break;
            }
        }
#undef AHQ_LAUNCH_BIN
    } else {
        ba.counts = counts;
        const int64_t n = (int64_t)S * NH * (B + 2);
        hipLaunchKernelGGL(zero_u32_kernel, dim3((unsigned)((n + 255) / 256 > 1024 ? 1024 : (n + 255) / 256)), dim3(256), 0, s, counts, n);
        if (hp.rows) {
            Geom rg{};
            fill_geom(hp.rows_plan, &rg);
            const size_t lds = (size_t)hp.copies * NH * B * 4;
            const dim3 g(hp.rows_plan.nblocks), b(kBlock);
#define AHQ_LAUNCH_ROWS(IO)                                                                                         \
    do {                                                                                                            \
        if (hp.rows_plan.vec == 1) {                                                                                \
            if (NH == 1) hipLaunchKernelGGL((hist_bin_rows_kernel<IO, 1, 1>), g, b, lds, s, ba, rg);                \
            else hipLaunchKernelGGL((hist_bin_rows_kernel<IO, 1, 2>), g, b, lds, s, ba, rg);                        \
        } else {                                                                                                    \
            if (NH == 1) hipLaunchKernelGGL((hist_bin_rows_kernel<IO, IoTraits<IO>::kVec, 1>), g, b, lds, s, ba, rg); \
            else hipLaunchKernelGGL((hist_bin_rows_kernel<IO, IoTraits<IO>::kVec, 2>), g, b, lds, s, ba, rg);       \
        }                                                                                                           \
    } while (0)
            switch (dtype) {
                case AHQ_F32: AHQ_LAUNCH_ROWS(float); break;
                case AHQ_F16: AHQ_LAUNCH_ROWS(f16_t); break;
                default: AHQ_LAUNCH_ROWS(bf16_t); break;
            }
#undef AHQ_LAUNCH_ROWS
        } else
        switch (dtype) {
            case AHQ_F32: hipLaunchKernelGGL((hist_bin_generic_kernel<float>), dim3(hp.nblocks), dim3(kBlock), 0, s, ba); break;
            case AHQ_F16: hipLaunchKernelGGL((hist_bin_generic_kernel<f16_t>), dim3(hp.nblocks), dim3(kBlock), 0, s, ba); break;
            default: hipLaunchKernelGGL((hist_bin_generic_kernel<bf16_t>), dim3(hp.nblocks), dim3(kBlock), 0, s, ba); break;
        }
    }

    // 4. counts -> fp32 statistics
    fa.nhist = NH;
    fa.first = first_batch ? 1 : 0;
    fa.nparts = hp.fast ? bin_blocks : 1;
    fa.counts = counts;
    fa.carried = pa.carried;
    fa.upd_edges = pa.upd_edges;
    fa.hist = st->hist;
    fa.edges = st->edges;
    fa.new_hist = st->new_hist;
    if (hp.fast) {
        if (speculative) {  // only if the range moved; ends the update by storing the new range into the state
            fa.rebin = rebin;
            fa.ranges = pa.ranges;
            fa.minmax = st->minmax;
        }
        hipLaunchKernelGGL(hist_fold_finish_kernel, ffgrid, dim3(kFfThreads), 0, s, fa);
    } else {
        hipLaunchKernelGGL(hist_finish_kernel, dim3((B + 63) / 64, S < 65535 ? S : 65535), dim3(kBlock), 0, s, fa);
    }
    return check_launch("ahq_hist_update");
}
