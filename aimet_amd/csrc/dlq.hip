// DlQuantization calibration on the device: min/max encodings, the TF-enhanced 1536-bucket PDF and the TF-enhanced
// (delta, offset) candidate search.  The reference runs all of this on the host with scalar float/double loops
// (ModelOptimizations/DlQuantization/src); every float / double operation below is the same operation in the same
// order, so results are bit-identical to that path.
//
//   ahq_dlq_minmax_encodings : getComputedEncodings over E blocks (quantization_utils.cpp:23-99,
//                              MinMaxEncodingAnalyzer.cpp:97-119)
//   ahq_dlq_pdf_update       : TfEnhancedEncodingAnalyzer::updateStats -> UpdatePdf (math_functions.cpp:190-285, 364-381)
//   ahq_dlq_tfe_encodings    : TfEnhancedEncodingAnalyzer::computeEncoding (TfEnhancedEncodingAnalyzer.cpp:52-377)

#include "ahq_device.h"
#include "ahq_host.h"
#include "layout.h"
#include "tiling.h"

namespace ahq {

constexpr int kPdf = AHQ_DLQ_PDF_SIZE;
constexpr float kFltMax = 3.402823466e+38f;
constexpr double kDblMax = 1.7976931348623157e+308;

// std::min / std::max / std::clamp as the reference's host code evaluates them (NaN never wins the comparison)
__device__ __forceinline__ float std_max(float a, float b) { return (a < b) ? b : a; }
__device__ __forceinline__ float std_min(float a, float b) { return (b < a) ? b : a; }
__device__ __forceinline__ double std_max(double a, double b) { return (a < b) ? b : a; }
__device__ __forceinline__ double std_min(double a, double b) { return (b < a) ? b : a; }
__device__ __forceinline__ double std_clamp(double v, double lo, double hi) { return (v < lo) ? lo : (hi < v) ? hi : v; }
// float/double -> int as x86-64 converts (out of range and NaN give INT_MIN)
__device__ __forceinline__ int to_int(float v) { return (v >= -2147483648.0f && v < 2147483648.0f) ? (int)v : (int)0x80000000; }
__device__ __forceinline__ int to_int(double v) { return (v > -2147483649.0 && v < 2147483648.0) ? (int)v : (int)0x80000000; }

// ----------------------------------------------------------------------------------------- min/max encodings ------
__device__ void computed_encodings(int bw, double mn, double mx, bool symmetric, bool strict, bool unsigned_sym, double zps,
                                   double* out) {
    double num_steps = (double)(1ull << bw) - 1;
    if (symmetric && strict) num_steps -= 1;
    const double f32_min = (double)(-kFltMax) * 0.99;
    const double f32_max = (double)kFltMax * 0.99;
    mn = std_clamp(mn, f32_min, 0.0);
    mx = std_clamp(mx, 0.0, f32_max);
    unsigned_sym = unsigned_sym && (mn >= 0.0);
    const double min_scale = std_min(0.01 / num_steps, (double)1.1920928955078125e-7f);
    double delta, offset;
    if (symmetric && !unsigned_sym) {
        double pos = floor(num_steps / 2) + zps;
        const double neg = num_steps - pos;
        if (num_steps == 3 && zps == 0.0) pos = neg;
        delta = std_max(std_max(mx / pos, -mn / neg), min_scale);
        offset = -neg;
    } else {
        delta = std_max((mx - mn) / num_steps, min_scale);
        offset = std_clamp(round(mn / delta), -num_steps, 0.0);
    }
    if (offset < 0) delta = std_min(delta, f32_min / offset);
    if (offset + num_steps > 0) delta = std_min(delta, f32_max / (offset + num_steps));
    out[0] = delta * offset;
    out[1] = delta * (offset + num_steps);
    out[2] = delta;
    out[3] = offset;
    out[4] = bw;
}

__global__ void dlq_minmax_encodings_kernel(const float* stat_min, const float* stat_max, int64_t E, int bw, int symmetric,
                                            int strict, int unsigned_sym, double zps, double* out) {
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= E) return;
    const double mn = std_min(0.0f, stat_min[e]);
    const double mx = std_max(0.0f, stat_max[e]);
    computed_encodings(bw, mn, mx, symmetric != 0, strict != 0, unsigned_sym != 0, zps, out + 5 * e);
}

// ------------------------------------------------------------------------------------------- PDF statistics ------
// meta[s] = {iterations, initialized, stats_updated, reserved}
struct PdfPrepArgs {
    int32_t num_slots;
    int32_t with_init;
    int32_t stat_dtype;  // ahq_dtype of bmin / bmax (the tensor's own dtype)
    const void* bmin;    // [S] batch minimum / maximum (only read when with_init)
    const void* bmax;
    double* xleft;
    double* pdf;
    int32_t* meta;
    float* params;  // [S][4]: inv_bucket, float(pdf_offset), active, iterations so far (int bits)
};

__device__ __forceinline__ float load_stat(const void* p, int dtype, int s) {
    if (dtype == AHQ_F32) return static_cast<const float*>(p)[s];
    if (dtype == AHQ_F16) return load_f32(static_cast<const f16_t*>(p)[s]);
    return load_f32(static_cast<const bf16_t*>(p)[s]);
}

__global__ __launch_bounds__(kBlock) void dlq_pdf_prepare_kernel(const PdfPrepArgs a) {
    const int s = blockIdx.x;
    __shared__ int sh_init;
    __shared__ double sh_bucket;
    __shared__ float sh_min;
    int32_t* meta = a.meta + 4 * s;
    double* xl = a.xleft + (size_t)s * kPdf;
    if (threadIdx.x == 0) {
        meta[2] = 1;
        int init = 0;
        if (meta[1] == 0 && a.with_init) {
            float mn = load_stat(a.bmin, a.stat_dtype, s), mx = load_stat(a.bmax, a.stat_dtype, s);
            if (!(mn == 0 && mx == 0)) {
                // InitializePdf<float>, signed values (math_functions.cpp:190-234)
                if (mn == mx) mx = std_max(mx, mn + (float)0.01);
                const float center = (mx + mn) / 2;
                mn = std_max((float).99 * -kFltMax, center - 3 * (center - mn));
                mx = std_min((float).99 * kFltMax, center + 3 * (mx - center));
                sh_bucket = ((double)mx - (double)mn) / kPdf;
                sh_min = mn;
                init = 1;
            }
        }
        sh_init = init;
    }
    __syncthreads();
    if (sh_init) {
        const double bucket = sh_bucket;
        const float mn = sh_min;
        for (int i = threadIdx.x; i < kPdf; i += kBlock) {
            xl[i] = floor(mn / bucket + i) * bucket;
            a.pdf[(size_t)s * kPdf + i] = 0.0;
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        if (sh_init) {
            meta[0] = 0;
            meta[1] = 1;
        }
        float* p = a.params + 4 * s;
        if (meta[1]) {
            // the first two left edges: just computed (same expression as above) or carried from earlier batches
            const double x0 = sh_init ? floor(sh_min / sh_bucket + 0) * sh_bucket : xl[0];
            const double x1 = sh_init ? floor(sh_min / sh_bucket + 1) * sh_bucket : xl[1];
            const double bucket = x1 - x0;
            p[0] = (float)(1 / bucket);
            p[1] = (float)to_int(round(x0 / bucket));
            p[2] = 1.f;
        } else {
            p[0] = 0.f;
            p[1] = 0.f;
            p[2] = 0.f;
        }
        p[3] = __int_as_float(meta[0]);  // iterations before this batch, for the running average
    }
}

struct PdfBinArgs : Geom {
    const void* x;
    float* params;        // [S][4]
    // single slot, range already fixed: the kernel derives the binning parameters from the statistics itself and
    // leaves them in `params` for the kernel that averages the counts in (no separate preparation launch)
    const double* xleft;
    const int32_t* meta;
    int32_t from_state;
    uint32_t* partials;   // single slot: [nblocks][kPdf]
    uint32_t* counts;     // several slots: [S][kPdf], zero-initialised
    int32_t copies, copy_shift;
};

// GetHistogram_cpu (math_functions.cpp:364-381): index = int(floor(x * float(1/bucket)) - pdf_offset), the subtraction
// evaluated in float.  Both terms are integer-valued floats, so testing the float against [0, kPdf) before the
// conversion accepts exactly the elements the reference accepts (NaN and out-of-range values fail the test).
__device__ __forceinline__ bool pdf_index(float v, float inv, float off, int& idx) {
    const float f = __builtin_floorf(v * inv) - off;
    idx = (int)f;
    return (f >= 0.f) & (f < (float)kPdf);
}

// THREADS lanes share one workgroup-wide histogram in LDS.  Bucket i of copy c sits at word i * copies + c and lane l
// adds to copy l % copies, so with many copies the lanes of a wave land in different banks whatever the data looks
// like: real activations put most elements into a few dozen buckets, and with few copies the wave's 64 atomic adds
// pile onto a handful of banks and are replayed bank conflict by bank conflict.
constexpr int kFfBins = 16;    // buckets per block of the single-slot partial counts
constexpr int kPdfUnroll = 1;  // 16-byte loads in flight per lane: the workgroups are persistent, so this sets the bytes in flight

template <typename IO, int VEC, int THREADS>
__global__ __launch_bounds__(THREADS) void dlq_pdf_bin_kernel(const PdfBinArgs a) {
    extern __shared__ uint32_t lds[];  // [kPdf][copies]
    float inv, off;
    if (a.from_state) {
        // what dlq_pdf_prepare_kernel computes for an initialised slot, evaluated by every lane (a few dozen
        // instructions once per workgroup); workgroup 0 also records it for the averaging kernel
        const bool active = a.meta[1] != 0;
        const double x0 = a.xleft[0], x1 = a.xleft[1];
        const double bucket = x1 - x0;
        inv = active ? (float)(1 / bucket) : 0.f;
        off = active ? (float)to_int(round(x0 / bucket)) : 0.f;
        if (blockIdx.x == 0 && threadIdx.x == 0) {
            a.params[0] = inv;
            a.params[1] = off;
            a.params[2] = active ? 1.f : 0.f;
            a.params[3] = __int_as_float(a.meta[0]);
        }
        if (!active) return;
    } else {
        if (a.params[2] == 0.f) return;  // histogram not initialised (only all-zero batches so far): nothing to count
        inv = a.params[0];
        off = a.params[1];
    }
    constexpr int kTile = THREADS * kPdfUnroll;  // vectors per workgroup and iteration
    const int copies = a.copies;
    for (int i = threadIdx.x; i < copies * kPdf; i += THREADS) lds[i] = 0;
    __syncthreads();
    const int bshift = a.copy_shift + 2;
    char* mine = reinterpret_cast<char*>(lds + (threadIdx.x & (copies - 1)));
    const IO* __restrict__ x = static_cast<const IO*>(a.x);
    auto add = [&](float v) {
        int idx;
        if (pdf_index(v, inv, off, idx)) atomicAdd(reinterpret_cast<uint32_t*>(mine + ((uint32_t)idx << bshift)), 1u);
    };
    const int64_t full_tiles = a.nvec / kTile;
    // two register buffers used alternately, a tile's load issued one round ahead of its binning, one vector per lane
    // and buffer: the shape and the reasons are those of the histogram's binning pass (hist_bin_kernel)
    Pack<IO, VEC> bufa[kPdfUnroll], bufb[kPdfUnroll];
    // `real` false: the prefetch past the end.  It reads the tensor's first tile with ordinary loads -- every
    // workgroup the same 64 KB, cache hits after the first -- where a streaming load of the current tile again was
    // 9 % more traffic from memory (nothing of a streamed tile stays in the cache).
    auto load_tile = [&](Pack<IO, VEC>* buf, int64_t t, bool real) {
        if (real) {
#pragma unroll
            for (int u = 0; u < kPdfUnroll; ++u) buf[u] = load_pack_stream<IO, VEC>(x + (t * kTile + u * THREADS + threadIdx.x) * VEC);
        } else {
#pragma unroll
            for (int u = 0; u < kPdfUnroll; ++u) buf[u] = load_pack<IO, VEC>(x + (u * THREADS + threadIdx.x) * VEC);
        }
    };
    auto bin_tile = [&](const Pack<IO, VEC>* buf) {
#pragma unroll
        for (int u = 0; u < kPdfUnroll; ++u)
#pragma unroll
            for (int k = 0; k < VEC; ++k) add(load_f32(buf[u].v[k]));
    };
    const int64_t step = gridDim.x;
    int64_t tile = blockIdx.x;
    if (tile < full_tiles) load_tile(bufa, tile, true);
    // the prefetch is unconditional (past the end it reads a tile that is dropped): a conditional load would leave
    // the number of loads in flight unknown and force a full wait before every use
    while (tile < full_tiles) {
        load_tile(bufb, tile + step, tile + step < full_tiles);
        bin_tile(bufa);
        tile += step;
        if (tile >= full_tiles) break;
        load_tile(bufa, tile + step, tile + step < full_tiles);
        bin_tile(bufb);
        tile += step;
    }
    if (blockIdx.x == 0) {  // ragged last tile and the elements past the last full vector
        for (int64_t v = full_tiles * kTile + threadIdx.x; v < a.nvec; v += THREADS) {
            const Pack<IO, VEC> pk = load_pack_stream<IO, VEC>(x + v * VEC);
            for (int k = 0; k < VEC; ++k) add(load_f32(pk.v[k]));
        }
        for (int64_t i = a.nvec * VEC + threadIdx.x; i < a.numel; i += THREADS) add(load_f32(x[i]));
    }
    __syncthreads();
    // partial counts in blocks of kFfBins buckets, [block][workgroup][kFfBins]: a workgroup stores 64-byte pieces, and
    // the launch that folds the partials reads all workgroups' counts of a block as one contiguous run
    for (int i = threadIdx.x; i < kPdf; i += THREADS) {
        uint32_t c = 0;
        for (int cp = 0; cp < copies; ++cp) c += lds[(size_t)i * copies + cp];
        a.partials[((size_t)(i / kFfBins) * gridDim.x + blockIdx.x) * kFfBins + i % kFfBins] = c;
    }
}

template <typename IO>
__global__ __launch_bounds__(kBlock) void dlq_pdf_bin_generic_kernel(const PdfBinArgs a) {
    const IO* __restrict__ x = static_cast<const IO*>(a.x);
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < a.numel; i += (int64_t)gridDim.x * kBlock) {
        int64_t e;
        if (a.nseg > 0) e = generic_enc_index(a, i);
        else e = a.J == 1 ? 0 : (i / a.K) % a.J;
        const float* p = a.params + 4 * e;
        if (p[2] == 0.f) continue;
        int idx;
        if (pdf_index(load_f32(x[i]), p[0], p[1], idx)) atomicAdd(&a.counts[(size_t)e * kPdf + idx], 1u);
    }
}

// Several slots, each one contiguous run of the tensor (per-channel statistics of a weight): a workgroup bins its
// slot's run into an LDS histogram and stores it as the slot's counts -- no global atomics, no zeroing pass.
template <typename IO, int VEC>
__global__ __launch_bounds__(kBlock) void dlq_pdf_bin_runs_kernel(const PdfBinArgs a) {
    __shared__ uint32_t hist[kPdf];
    const int64_t e = blockIdx.x;
    for (int i = threadIdx.x; i < kPdf; i += kBlock) hist[i] = 0;
    __syncthreads();
    const float* p = a.params + 4 * e;
    if (p[2] != 0.f) {
        const float inv = p[0], off = p[1];
        const IO* __restrict__ x = static_cast<const IO*>(a.x) + e * a.K;
        const int64_t nv = a.K / VEC;
        for (int64_t v = threadIdx.x; v < nv; v += kBlock) {
            const Pack<IO, VEC> pk = load_pack_stream<IO, VEC>(x + v * VEC);
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                int idx;
                if (pdf_index(load_f32(pk.v[k]), inv, off, idx)) atomicAdd(&hist[idx], 1u);
            }
        }
        for (int64_t i = nv * VEC + threadIdx.x; i < a.K; i += kBlock) {
            int idx;
            if (pdf_index(load_f32(x[i]), inv, off, idx)) atomicAdd(&hist[idx], 1u);
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < kPdf; i += kBlock) a.counts[(size_t)e * kPdf + i] = hist[i];
}

__global__ void dlq_zero_u32_kernel(uint32_t* p, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0;
}

constexpr int kPdfFoldGroups = 16;

struct PdfFinArgs {
    const uint32_t* counts;  // [S][nparts][kPdf]
    int32_t nparts;
    const float* params;
    double* pdf;
    int32_t* meta;
    unsigned long long cnt;  // elements per slot in this batch
    uint32_t* hist_out;      // optional [S][kPdf]: this batch's integer histogram
    int32_t num_slots;
};

// Average the batch into the running PDF (math_functions.cpp:274-284)
__global__ __launch_bounds__(kBlock) void dlq_pdf_finish_kernel(const PdfFinArgs a) {
    const int i = blockIdx.x * kBlock + threadIdx.x;
    // the y dimension of a grid ends at 65535: slots beyond it are taken in further rounds
    for (int s = blockIdx.y; s < a.num_slots; s += gridDim.y) {
    const bool active = a.params[4 * s + 2] != 0.f;
    uint32_t h = 0;
    if (active) {
        const uint32_t* c = a.counts + (size_t)s * a.nparts * kPdf;
        for (int p = 0; p < a.nparts; ++p) h += c[(size_t)p * kPdf + i];
        const int it = __float_as_int(a.params[4 * s + 3]);
        const double prob = (double)h / (double)a.cnt;
        double* pdf = a.pdf + (size_t)s * kPdf;
        pdf[i] = (pdf[i] * it + prob) / (it + 1);
    }
    if (a.hist_out) a.hist_out[(size_t)s * kPdf + i] = h;
    // pdf.iterations++ ; every thread above took the old count from `params`, so nothing else reads this word here
    if (active && i == 0) a.meta[4 * s] = __float_as_int(a.params[4 * s + 3]) + 1;
    }
}

// Single slot, many partial histograms: fold and average in one launch.  A workgroup owns one block of kFfBins
// neighbouring buckets, whose partial counts from all workgroups of the binning pass are one contiguous run (see
// dlq_pdf_bin_kernel): its threads read it as whole cache lines, every thread always the same bucket, all loads in
// flight at once; then one lane per bucket adds the group sums (integers: the order does not matter) and does what
// dlq_pdf_finish_kernel does.
constexpr int kFfGroups = kBlock / kFfBins;
__global__ __launch_bounds__(kBlock) void dlq_pdf_fold_finish_kernel(const PdfFinArgs a) {
    __shared__ uint32_t sm[kFfGroups][kFfBins];
    const int bl = threadIdx.x & (kFfBins - 1), grp = threadIdx.x / kFfBins;
    const int i = blockIdx.x * kFfBins + bl;
    const bool active = a.params[2] != 0.f;
    uint32_t acc = 0;
    if (active) {
        const uint32_t* run = a.counts + (size_t)blockIdx.x * a.nparts * kFfBins;
        const int n = a.nparts * kFfBins;
        constexpr int kFlight = 16;
        for (int j = threadIdx.x; j < n; j += kFlight * kBlock) {
            uint32_t v[kFlight];
#pragma unroll
            for (int k = 0; k < kFlight; ++k) v[k] = j + k * kBlock < n ? run[j + k * kBlock] : 0u;
#pragma unroll
            for (int k = 0; k < kFlight; ++k) acc += v[k];
        }
    }
    sm[grp][bl] = acc;
    __syncthreads();
    if (grp != 0) return;
    uint32_t h = 0;
#pragma unroll
    for (int g = 0; g < kFfGroups; ++g) h += sm[g][bl];
    if (active) {
        const int it = __float_as_int(a.params[3]);
        const double prob = (double)h / (double)a.cnt;
        a.pdf[i] = (a.pdf[i] * it + prob) / (it + 1);
        if (i == 0) a.meta[0] = it + 1;
    }
    if (a.hist_out) a.hist_out[i] = h;
    if (i == 0) a.meta[2] = 1;  // _statsUpdated
}

__global__ void dlq_pdf_mark_kernel(int32_t* meta, int S) {
    const int s = blockIdx.x * blockDim.x + threadIdx.x;
    if (s < S) meta[4 * s + 2] = 1;
}

// ------------------------------------------------------------------------------------------ TF-enhanced search ---
constexpr int kMaxCand = 512;

struct TfeArgs {
    int32_t num_slots, bw, symmetric, strict, unsigned_sym;
    const double* xleft;
    const double* pdf;
    const int32_t* meta;
    float* cand_delta;  // [S][kMaxCand]
    int32_t* cand_off;  // [S][kMaxCand]
    int32_t* cand_ok;   // [S][kMaxCand]
    float* centers;     // [S][kPdf]
    float* head;        // [S][4]: num_steps used for the final range, unused...
    double* cost;       // [S][kMaxCand]
    double* out;        // [S][5]
    int32_t* best;      // [S][2]: chosen candidate index, number of candidates (optional)
};

// _clampToObservedMinMax (TfEnhancedEncodingAnalyzer.cpp:129-155)
__device__ bool clamp_to_observed(float obs_min, float obs_max, float num_steps, float& delta, int& offset) {
    float tmin = std_max(delta * offset, -kFltMax);
    float tmax = std_min(delta * (offset + num_steps), kFltMax);
    if (tmin < obs_min && tmax > obs_max) return false;
    tmin = std_max(obs_min, tmin);
    tmax = std_min(obs_max, tmax);
    if (tmin == tmax) return false;
    delta = (float)(((double)tmax - tmin) / num_steps);
    offset = to_int(__builtin_roundf(tmin / delta));
    return true;
}

// One workgroup per slot: range of the aggregate statistics, bucket centres and the candidate list.
__global__ __launch_bounds__(kMaxCand) void dlq_tfe_candidates_kernel(const TfeArgs a) {
    const int s = blockIdx.x;
    const int t = threadIdx.x;
    if (a.meta[4 * s + 1] == 0) return;
    const double* xl = a.xleft + (size_t)s * kPdf;
    const double* pdf = a.pdf + (size_t)s * kPdf;
    __shared__ int sh_first, sh_last;
    __shared__ float sh_min, sh_max, sh_steps;
    if (t == 0) {
        sh_first = kPdf;
        sh_last = 0;
    }
    __syncthreads();
    // _findRangeOfAggregateStats (TfEnhancedEncodingAnalyzer.cpp:235-271): lowest bucket with probability > 0; highest
    // such bucket among indices 1 .. kPdf-1
    int first = kPdf, last = 0;
    for (int i = t; i < kPdf; i += kMaxCand)
        if (pdf[i] > 0) {
            first = first < i ? first : i;
            last = last > i ? last : i;
        }
    atomicMin(&sh_first, first);
    atomicMax(&sh_last, last);
    // bucket centres (_findBestCandidate, TfEnhancedEncodingAnalyzer.cpp:100-105): left edge narrowed to float first
    const double half = (xl[1] - xl[0]) / 2;
    for (int i = t; i < kPdf; i += kMaxCand) a.centers[(size_t)s * kPdf + i] = (float)((float)xl[i] + half);
    __syncthreads();
    if (t == 0) {
        float lo = (float)xl[0], hi = (float)xl[kPdf - 1];
        if (sh_first < kPdf) lo = (float)xl[sh_first];
        if (sh_last > 0) hi = (float)xl[sh_last];
        lo = std_min(lo, 0.0f);
        hi = std_max(hi, 0.0f);
        hi = std_max(hi, lo + (float)0.01);
        float num_steps = (float)((double)(1ull << a.bw) - 1);
        if (a.symmetric && a.strict) num_steps -= 1;
        sh_min = lo;
        sh_max = hi;
        sh_steps = num_steps;
        a.head[4 * s] = num_steps;
    }
    __syncthreads();
    const float num_steps = sh_steps;
    float delta = 0.f;
    int offset = 0;
    bool ok = false;
    if (a.symmetric) {
        // _pickTestCandidatesSymmetric (TfEnhancedEncodingAnalyzer.cpp:196-233)
        float delta_max;
        int test_offset;
        if (sh_min == 0.0 && a.unsigned_sym) {
            delta_max = sh_max / num_steps;
            test_offset = 0;
        } else {
            const float abs_max = std_max(__builtin_fabsf(sh_max), __builtin_fabsf(sh_min));
            delta_max = (float)(abs_max / (num_steps / 2.0));
            test_offset = to_int(__builtin_floorf(-num_steps / 2));
        }
        // f runs 0.01, 0.01 + 0.01, ... in float with each increment added in double; candidate t uses the (t+1)-th
        // value and exists while that value is <= 1.01
        float f = (float)(1.0 / 100);
        for (int k = 0; k < t; ++k) f = (float)(f + 1.0 / 100);
        ok = (double)f <= 1 + 1.0 / 100;
        delta = f * delta_max;
        offset = test_offset;
    } else {
        // _pickTestCandidatesAsymmetric (TfEnhancedEncodingAnalyzer.cpp:157-194): 17 deltas x 21 offsets in that
        // order, then the observed (delta, offset)
        float obs_min = sh_min, obs_max = sh_max;
        const float obs_delta = (float)(((double)obs_max - (double)obs_min) / num_steps);
        const int obs_offset = to_int(__builtin_roundf(obs_min / obs_delta));
        obs_min = std_max(obs_delta * obs_offset, -kFltMax);
        obs_max = std_min(obs_delta * (obs_offset + num_steps), kFltMax);
        if (t < 17 * 21) {
            const int fi = t / 21, i = t - fi * 21;
            const float f = (float)(fi + 1) * 0.0625f;  // k/16 is exact in float
            delta = f * obs_delta;
            offset = to_int(-num_steps + num_steps / 20.0 * i);
            ok = clamp_to_observed(obs_min, obs_max, num_steps, delta, offset);
        } else if (t == 17 * 21) {
            delta = obs_delta;
            offset = obs_offset;
            ok = true;
        }
    }
    a.cand_delta[(size_t)s * kMaxCand + t] = delta;
    a.cand_off[(size_t)s * kMaxCand + t] = offset;
    a.cand_ok[(size_t)s * kMaxCand + t] = ok ? 1 : 0;
}

// _quantAndSatCost (TfEnhancedEncodingAnalyzer.cpp:273-335), one candidate per lane.  The three sums run over the
// buckets in increasing order like the reference's three loops; pow(x, 2) is x*x.
// One workgroup per slot: its waves share one staged copy of the slot's statistics (18 KB of LDS, so eight
// workgroups = 64 waves fit a CU; with a workgroup per wave the LDS allowed two waves per SIMD and every wave staged
// the statistics for itself).  Waves without a valid candidate leave at once.
__global__ __launch_bounds__(kMaxCand) void dlq_tfe_cost_kernel(const TfeArgs a) {
    const int s = blockIdx.x;
    if (a.meta[4 * s + 1] == 0) return;
    __shared__ double sh_pdf[kPdf];
    __shared__ float sh_c[kPdf];
    for (int i = threadIdx.x; i < kPdf; i += kMaxCand) {
        sh_pdf[i] = a.pdf[(size_t)s * kPdf + i];
        sh_c[i] = a.centers[(size_t)s * kPdf + i];
    }
    __syncthreads();
    const int k = threadIdx.x;
    const bool ok = a.cand_ok[(size_t)s * kMaxCand + k] != 0;
    if (__builtin_amdgcn_ballot_w64(ok) == 0) {
        a.cost[(size_t)s * kMaxCand + k] = kDblMax;
        return;
    }
    const float delta = a.cand_delta[(size_t)s * kMaxCand + k];
    const int offset = a.cand_off[(size_t)s * kMaxCand + k];
    const double* xl = a.xleft + (size_t)s * kPdf;
    const float min_val = delta * offset;
    const float step_size = (float)((double)(1ull << a.bw) - 1);
    const float max_val = delta * (offset + step_size);
    const float pdf_start = (float)xl[0];
    const double pdf_step = xl[1] - xl[0];
    int min_ind = to_int(floor((min_val - pdf_start) / pdf_step));
    min_ind = min_ind < 0 ? 0 : (min_ind > kPdf - 1 ? kPdf - 1 : min_ind);
    int max_ind = to_int(floor((max_val - pdf_start) / pdf_step));
    max_ind = max_ind < 0 ? 0 : (max_ind > kPdf - 1 ? kPdf - 1 : max_ind);
    const float min_mid = sh_c[min_ind], max_mid = sh_c[max_ind];
    const float inv_delta = 1 / delta;
    double sat_bottom = 0, sat_top = 0, quant = 0;
    for (int i = 0; i < kPdf; ++i) {
        const float c = sh_c[i];
        const double p = sh_pdf[i];
        if (i < min_ind) {
            const double d = (double)c - min_mid;
            sat_bottom += p * (d * d);
        }
        if (i >= max_ind) {
            const double d = (double)c - max_mid;
            sat_top += p * (d * d);
        }
        if (i >= min_ind && i < max_ind) {
            const float deq = __builtin_floorf(c * inv_delta + 0.5f) * delta;
            const double d = (double)(c - deq);
            quant += p * (d * d);
        }
    }
    const double cost = 3.0 * (sat_bottom + sat_top) + quant;
    a.cost[(size_t)s * kMaxCand + k] = ok ? std_min(cost, kDblMax) : kDblMax;
}

// the value that lane j (a constant) holds, as a wave-uniform scalar
__device__ __forceinline__ double lane_value(double v, int j) {
    const long long b = __double_as_longlong(v);
    const unsigned int lo = __builtin_amdgcn_readlane((int)(unsigned int)b, j);
    const unsigned int hi = __builtin_amdgcn_readlane((int)(unsigned int)((unsigned long long)b >> 32), j);
    return __longlong_as_double((long long)(((unsigned long long)hi << 32) | lo));
}

// The same costs with one wave per candidate, for few slots (a per-tensor search has 358 candidates: six waves of
// the kernel above, each doing the arithmetic of all 1536 buckets for 64 candidates, leave the GPU idle).  The lanes
// work out the terms of 64 buckets at a time; the additions into the three sums then run over those 64 terms in
// bucket order on values read lane by lane, so every sum sees exactly the sequence of roundings of the serial loop
// (a term that does not belong to a sum is +0, which leaves a non-negative sum unchanged).
__global__ __launch_bounds__(kWave) void dlq_tfe_cost_wave_kernel(const TfeArgs a) {
    const int s = blockIdx.y;
    const int k = blockIdx.x;
    if (a.meta[4 * s + 1] == 0) return;
    const int lane = threadIdx.x;
    const bool ok = a.cand_ok[(size_t)s * kMaxCand + k] != 0;
    if (!ok) {
        if (lane == 0) a.cost[(size_t)s * kMaxCand + k] = kDblMax;
        return;
    }
    const float delta = a.cand_delta[(size_t)s * kMaxCand + k];
    const int offset = a.cand_off[(size_t)s * kMaxCand + k];
    const double* xl = a.xleft + (size_t)s * kPdf;
    const double* pdf = a.pdf + (size_t)s * kPdf;
    const float* centers = a.centers + (size_t)s * kPdf;
    const float min_val = delta * offset;
    const float step_size = (float)((double)(1ull << a.bw) - 1);
    const float max_val = delta * (offset + step_size);
    const float pdf_start = (float)xl[0];
    const double pdf_step = xl[1] - xl[0];
    int min_ind = to_int(floor((min_val - pdf_start) / pdf_step));
    min_ind = min_ind < 0 ? 0 : (min_ind > kPdf - 1 ? kPdf - 1 : min_ind);
    int max_ind = to_int(floor((max_val - pdf_start) / pdf_step));
    max_ind = max_ind < 0 ? 0 : (max_ind > kPdf - 1 ? kPdf - 1 : max_ind);
    const float min_mid = centers[min_ind], max_mid = centers[max_ind];
    const float inv_delta = 1 / delta;
    double sat_bottom = 0, sat_top = 0, quant = 0;
    // the next chunk's statistics are fetched before the additions of this one, whose chain hides the latency
    float c_next = centers[lane];
    double p_next = pdf[lane];
    for (int i0 = 0; i0 < kPdf; i0 += kWave) {
        const int i = i0 + lane;
        const float c = c_next;
        const double p = p_next;
        if (i0 + kWave < kPdf) {
            c_next = centers[i + kWave];
            p_next = pdf[i + kWave];
        }
        double tb = 0, tt = 0, tq = 0;
        if (i < min_ind) {
            const double d = (double)c - min_mid;
            tb = p * (d * d);
        }
        if (i >= max_ind) {
            const double d = (double)c - max_mid;
            tt = p * (d * d);
        }
        if (i >= min_ind && i < max_ind) {
            const float deq = __builtin_floorf(c * inv_delta + 0.5f) * delta;
            const double d = (double)(c - deq);
            tq = p * (d * d);
        }
        // The three sums take their buckets from three consecutive ranges, so a chunk of 64 buckets that lies within
        // one range is a single chain of additions; only the (at most two) chunks that straddle a boundary feed all
        // three sums.
        const int last = i0 + kWave - 1;
        const int phase = i0 < min_ind ? 0 : (i0 < max_ind ? 1 : 2);
        const int phase_last = last < min_ind ? 0 : (last < max_ind ? 1 : 2);
        if (phase == phase_last && min_ind <= max_ind) {
            const double t = phase == 0 ? tb : (phase == 1 ? tq : tt);
            double acc = phase == 0 ? sat_bottom : (phase == 1 ? quant : sat_top);
#pragma unroll
            for (int j = 0; j < kWave; ++j) acc += lane_value(t, j);
            if (phase == 0) sat_bottom = acc;
            else if (phase == 1) quant = acc;
            else sat_top = acc;
        } else {
#pragma unroll
            for (int j = 0; j < kWave; ++j) {
                sat_bottom += lane_value(tb, j);
                sat_top += lane_value(tt, j);
                quant += lane_value(tq, j);
            }
        }
    }
    const double cost = 3.0 * (sat_bottom + sat_top) + quant;
    if (lane == 0) a.cost[(size_t)s * kMaxCand + k] = std_min(cost, kDblMax);
}

// _findBestCandidate (first strictly smaller cost wins) and the final encoding (TfEnhancedEncodingAnalyzer.cpp:88-127,
// 337-377); also the two cases without a histogram (TfEnhancedEncodingAnalyzer.cpp:58-80)
__global__ __launch_bounds__(kWave) void dlq_tfe_select_kernel(const TfeArgs a) {
    const int s = blockIdx.x;
    const int lane = threadIdx.x;
    double* out = a.out + 5 * s;
    if (a.meta[4 * s + 1] == 0) {
        if (lane == 0) {
            if (a.best) a.best[2 * s] = -1, a.best[2 * s + 1] = 0;
            if (a.meta[4 * s + 2]) {
                const float num_steps = (float)((double)(1ull << a.bw) - 1);
                double mn = -1, mx = 1;
                const double delta = (mx - mn) / (int)num_steps;
                const double offset = floor(mn / delta);
                mn = offset * delta;
                mx = mn + (int)num_steps * delta;
                out[0] = mn; out[1] = mx; out[2] = delta; out[3] = offset; out[4] = a.bw;
            } else {
                out[0] = out[1] = out[2] = out[3] = out[4] = 0.0;
            }
        }
        return;
    }
    // each lane scans every 64th candidate in rising order (all loads are issued before the first comparison), then
    // the lanes are compared by (cost, index)
    constexpr int kPer = kMaxCand / kWave;
    double cs[kPer];
    int oks[kPer];
#pragma unroll
    for (int r = 0; r < kPer; ++r) {
        cs[r] = a.cost[(size_t)s * kMaxCand + r * kWave + lane];
        oks[r] = a.cand_ok[(size_t)s * kMaxCand + r * kWave + lane];
    }
    double bc = kDblMax;
    int bi = -1, n = 0;
#pragma unroll
    for (int r = 0; r < kPer; ++r) {
        n += oks[r];
        if (cs[r] < bc) {
            bc = cs[r];
            bi = r * kWave + lane;
        }
    }
#pragma unroll
    for (int m = 1; m < kWave; m <<= 1) {
        const double oc = __shfl_xor(bc, m, kWave);
        const int oi = __shfl_xor(bi, m, kWave);
        n += __shfl_xor(n, m, kWave);
        // the other lane's run precedes ours when its lane index is lower: ties go to the lower candidate index
        const bool take = (oi >= 0) && (bi < 0 || oc < bc || (oc == bc && oi < bi));
        if (take) {
            bc = oc;
            bi = oi;
        }
    }
    // index of the winner among the accepted candidates, as a host loop that skips rejected ones would count
    int rank = 0;
#pragma unroll
    for (int r = 0; r < kPer; ++r) rank += (r * kWave + lane < bi) ? oks[r] : 0;
#pragma unroll
    for (int m = 1; m < kWave; m <<= 1) rank += __shfl_xor(rank, m, kWave);
    if (lane == 0) {
        float best_delta = -1;
        int best_offset = -1;
        if (bi >= 0) {
            best_delta = a.cand_delta[(size_t)s * kMaxCand + bi];
            best_offset = a.cand_off[(size_t)s * kMaxCand + bi];
        }
        const float num_steps = a.head[4 * s];
        const float best_min = std_max(best_delta * best_offset, -kFltMax);
        const float best_max = std_min(best_delta * (best_offset + num_steps), kFltMax);
        out[0] = best_min;
        out[1] = best_max;
        out[2] = best_delta;
        out[3] = best_offset;
        out[4] = a.bw;
        if (a.best) {
            a.best[2 * s] = bi >= 0 ? rank : -1;
            a.best[2 * s + 1] = n;
        }
    }
}

// --------------------------------------------------------------------------------------------------- percentile ---
// PercentileEncodingAnalyzer::computeEncoding (PercentileEncodingAnalyzer.cpp:52-169).  One workgroup per slot; the
// cumulative distribution is a sequential sum in the reference, so one lane forms it (1536 additions).
__global__ __launch_bounds__(kWave) void dlq_percentile_kernel(const double* xleft, const double* pdfs, const int32_t* meta,
                                                               float percentile, int bw, int symmetric, int strict,
                                                               int unsigned_sym, double* outs) {
    const int s = blockIdx.x;
    const double* xl = xleft + (size_t)s * kPdf;
    const double* pdf = pdfs + (size_t)s * kPdf;
    double* out = outs + 5 * s;
    __shared__ double cdf[kPdf];
    if (threadIdx.x != 0) return;
    float num_steps = (float)((double)(1ull << bw) - 1);
    if (symmetric && strict) num_steps -= 1;
    if (meta[4 * s + 1] == 0) {
        if (meta[4 * s + 2]) {
            double mn = -1, mx = 1;
            const double delta = (mx - mn) / (int)num_steps;
            const double offset = floor(mn / delta);
            mn = offset * delta;
            mx = mn + (int)num_steps * delta;
            out[0] = mn; out[1] = mx; out[2] = delta; out[3] = offset; out[4] = bw;
        } else {
            out[0] = out[1] = out[2] = out[3] = out[4] = 0.0;
        }
        return;
    }
    // findOriginalRange (math_functions.cpp:401-435)
    float lo = (float)xl[0], hi = (float)xl[kPdf - 1];
    for (int i = 0; i < kPdf; ++i)
        if (pdf[i] > 0) { lo = (float)xl[i]; break; }
    for (int i = kPdf - 1; i > 0; --i)
        if (pdf[i] > 0) { hi = (float)xl[i]; break; }
    lo = std_min(lo, 0.0f);
    hi = std_max(hi, 0.0f);
    hi = std_max(hi, lo + (float)0.01);
    float a_min = lo, a_max = hi;
    if (percentile != 100.0f) {
        const float bin_width = (float)(xl[1] - xl[0]);
        float pmin = (float)xl[0];
        float pmax = (float)(xl[kPdf - 1] + bin_width);
        cdf[0] = pdf[0];
        for (int i = 1; i < kPdf; ++i) cdf[i] = pdf[i] + cdf[i - 1];
        const float left = 1 - percentile / 100;
        for (int i = 0; i < kPdf; ++i)
            if (cdf[i] >= left) { pmin = (float)xl[i]; break; }
        const float right = percentile / 100;
        for (int i = kPdf - 1; i >= 0; --i)
            if (cdf[i] < right && xl[i] < hi) { pmax = (float)(xl[i] + bin_width); break; }
        if (pmin == pmax) pmax += bin_width;
        a_min = pmin;
        a_max = pmax;
    }
    a_min = std_min(a_min, 0.f);
    a_max = std_max(a_max, 0.f);
    computed_encodings(bw, a_min, a_max, symmetric != 0, strict != 0, unsigned_sym != 0, 0.0, out);
}

// -------------------------------------------------------------------------------------------------- host side ---
namespace {

constexpr int kPdfThreads = 1024;  // two workgroups per compute unit: 8 copies x 1536 buckets x 4 B = 48 KB of LDS each
constexpr int kPdfCopies = 8;
constexpr int kPdfBlocksMax = 512;

size_t up256(size_t v) { return (v + 255) & ~(size_t)255; }

struct PdfPlan {
    Plan plan;
    bool fast;
    int copies, nblocks;
    size_t off_mm_ws, off_bmin, off_bmax, off_params, off_counts, total;
};

bool make_pdf_plan(int dtype, const ahq_layout& layout, const void* x, PdfPlan* pp) {
    if (!make_plan(dtype, layout, aligned16(x), false, &pp->plan)) return false;
    const CanonLayout& c = pp->plan.cl;
    const size_t S = (size_t)c.num_enc;
    pp->fast = c.kind == kIJK && c.J == 1;
    pp->copies = kPdfCopies;
    const int64_t ntiles = (pp->plan.nvec + kPdfThreads * kPdfUnroll - 1) / (kPdfThreads * kPdfUnroll);
    int64_t nb = pp->fast ? ntiles : (c.numel + kBlock - 1) / kBlock;
    if (nb > kPdfBlocksMax) nb = kPdfBlocksMax;
    if (nb < 1) nb = 1;
    pp->nblocks = (int)nb;
    size_t o = 0;
    pp->off_mm_ws = o;   o = up256(o + ahq_minmax_workspace_bytes(&layout));
    pp->off_bmin = o;    o = up256(o + S * 4);
    pp->off_bmax = o;    o = up256(o + S * 4);
    pp->off_params = o;  o = up256(o + S * 16);
    pp->off_counts = o;  o = up256(o + (pp->fast ? (size_t)pp->nblocks : S) * kPdf * 4);
    pp->total = o;
    return true;
}

bool check_pdf_state(const ahq_dlq_pdf_state* st) {
    if (!st) return set_error("pdf state is null"), false;
    if (st->num_slots <= 0) return set_error("num_slots must be positive"), false;
    if (!st->xleft || !st->pdf || !st->meta) return set_error("pdf state has a null buffer"), false;
    return true;
}

}  // namespace
}  // namespace ahq

using namespace ahq;

extern "C" int ahq_dlq_minmax_encodings(const float* stat_min, const float* stat_max, int64_t num_encodings, int32_t bw,
                                        int32_t symmetric, int32_t strict, int32_t unsigned_sym, double zero_point_shift,
                                        double* out, void* stream) {
    if (!stat_min || !stat_max || !out) return set_error("null argument"), AHQ_ERR_INVALID;
    if (num_encodings < 0) return set_error("negative encoding count"), AHQ_ERR_INVALID;
    if (bw < 1 || bw > 32) return set_error("bitwidth must be in 1..32"), AHQ_ERR_INVALID;
    if (zero_point_shift != 0.0) {
        // the reference throws std::runtime_error with these messages (quantization_utils.cpp:44-58); unsigned symmetric
        // only disqualifies when it would actually apply (min >= 0), which depends on the data: rejected up front here
        if (!symmetric) return set_error("zero_point_shift is only supported when useSymmetricEncodings is set to true"), AHQ_ERR_UNSUPPORTED;
        if (unsigned_sym) return set_error("zero_point_shift is only supported when useUnsignedSymmetric is set to false"), AHQ_ERR_UNSUPPORTED;
        if (strict) return set_error("zero_point_shift is only supported when useStrictSymmetric is set to false"), AHQ_ERR_UNSUPPORTED;
    }
    if (num_encodings == 0) return AHQ_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const unsigned blocks = (unsigned)((num_encodings + 255) / 256);
    hipLaunchKernelGGL(dlq_minmax_encodings_kernel, dim3(blocks), dim3(256), 0, s, stat_min, stat_max, num_encodings, bw,
                       symmetric, strict, unsigned_sym, zero_point_shift, out);
    return check_launch("dlq_minmax_encodings");
}

extern "C" size_t ahq_dlq_pdf_update_workspace_bytes(int32_t dtype, const ahq_layout* layout) {
    if (!layout) return 0;
    PdfPlan pp;
    size_t need = 0;
    if (make_pdf_plan(dtype, *layout, nullptr, &pp)) need = pp.total;
    if (make_pdf_plan(dtype, *layout, reinterpret_cast<const void*>(4), &pp) && pp.total > need) need = pp.total;
    return need;
}

extern "C" int ahq_dlq_pdf_update(int32_t dtype, const ahq_layout* layout, const void* x, const ahq_dlq_pdf_state* st,
                                  int32_t with_init, uint32_t* hist_out, void* workspace, size_t workspace_bytes,
                                  void* stream) {
    if (dtype < AHQ_F32 || dtype > AHQ_BF16) return set_error("bad dtype"), AHQ_ERR_INVALID;
    if (!layout) return set_error("layout is null"), AHQ_ERR_INVALID;
    if (!check_pdf_state(st)) return AHQ_ERR_INVALID;
    PdfPlan pp;
    if (!make_pdf_plan(dtype, *layout, x, &pp)) return AHQ_ERR_INVALID;
    const CanonLayout& c = pp.plan.cl;
    if (c.num_enc != st->num_slots) return set_error("layout does not have num_slots encodings"), AHQ_ERR_INVALID;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int S = st->num_slots;
    if (c.numel == 0) {
        // UpdatePdf returns at once for an empty tensor (math_functions.cpp:240-243); only _statsUpdated changes
        hipLaunchKernelGGL(dlq_pdf_mark_kernel, dim3((S + 255) / 256), dim3(256), 0, s, st->meta, S);
        if (hist_out) hipLaunchKernelGGL(dlq_zero_u32_kernel, dim3(8), dim3(256), 0, s, hist_out, (int64_t)S * kPdf);
        return check_launch("dlq_pdf_update");
    }
    if (!x) return set_error("x is null"), AHQ_ERR_INVALID;
    if (!workspace || workspace_bytes < pp.total) return set_error("workspace too small"), AHQ_ERR_WORKSPACE;
    char* w = static_cast<char*>(workspace);
    void* bmin = w + pp.off_bmin;
    void* bmax = w + pp.off_bmax;
    float* params = reinterpret_cast<float*>(w + pp.off_params);

    if (with_init) {
        // range of the batch, NaN skipped (GetMin / GetMax, math_functions.cpp:324-345).  16-bit inputs: the
        // reference converts the tensor to float first, and the extrema of the converted values are the converted
        // extrema, so min/max are taken in the tensor's dtype and widened in the prepare step.
        const int rc = ahq_minmax(dtype, layout, x, bmin, bmax, nullptr, nullptr, 2, w + pp.off_mm_ws,
                                  pp.off_bmin - pp.off_mm_ws, stream);
        if (rc != AHQ_OK) return rc;
    }
    PdfPrepArgs pa{};
    pa.num_slots = S;
    pa.with_init = with_init ? 1 : 0;
    pa.stat_dtype = dtype;
    pa.bmin = bmin;
    pa.bmax = bmax;
    pa.xleft = st->xleft;
    pa.pdf = st->pdf;
    pa.meta = st->meta;
    pa.params = params;
    // one slot whose range is already fixed: the binning kernel works the parameters out itself
    const bool from_state = !with_init && S == 1 && pp.fast && pp.nblocks > kPdfFoldGroups;
    if (!from_state) hipLaunchKernelGGL(dlq_pdf_prepare_kernel, dim3(S), dim3(kBlock), 0, s, pa);

    PdfBinArgs ba{};
    fill_geom(pp.plan, &ba);
    ba.x = x;
    ba.params = params;
    ba.xleft = st->xleft;
    ba.meta = st->meta;
    ba.from_state = from_state ? 1 : 0;
    ba.copies = pp.copies;
    ba.copy_shift = 0;
    while ((1 << ba.copy_shift) < pp.copies) ++ba.copy_shift;
    uint32_t* counts = reinterpret_cast<uint32_t*>(w + pp.off_counts);
    PdfFinArgs fa{};
    fa.params = params;
    fa.pdf = st->pdf;
    fa.meta = st->meta;
    fa.cnt = (unsigned long long)(c.numel / S);
    fa.hist_out = hist_out;
    fa.num_slots = S;
    if (pp.fast) {
        ba.partials = counts;
        const size_t lds = (size_t)pp.copies * kPdf * 4;
        const dim3 g(pp.nblocks), b(kPdfThreads);
        static_assert((size_t)kPdfCopies * kPdf * 4 <= 64 * 1024, "dynamic LDS beyond 64 KB needs hipFuncSetAttribute");
#define AHQ_LAUNCH_PDF_K(K) hipLaunchKernelGGL(K, g, b, lds, s, ba)
#define AHQ_LAUNCH_PDF(IO)                                                                                     \
    do {                                                                                                       \
        if (pp.plan.vec == 1) AHQ_LAUNCH_PDF_K((dlq_pdf_bin_kernel<IO, 1, kPdfThreads>));                      \
        else AHQ_LAUNCH_PDF_K((dlq_pdf_bin_kernel<IO, IoTraits<IO>::kVec, kPdfThreads>));                      \
    } while (0)
        switch (dtype) {
            case AHQ_F32: AHQ_LAUNCH_PDF(float); break;
            case AHQ_F16: AHQ_LAUNCH_PDF(f16_t); break;
            default: AHQ_LAUNCH_PDF(bf16_t); break;
        }
#undef AHQ_LAUNCH_PDF
#undef AHQ_LAUNCH_PDF_K
        // (one slot: the layout of the partial counts is the one dlq_pdf_fold_finish_kernel reads)
        fa.counts = counts;
        fa.nparts = pp.nblocks;
        hipLaunchKernelGGL(dlq_pdf_fold_finish_kernel, dim3(kPdf / kFfBins), dim3(kBlock), 0, s, fa);
        return check_launch("dlq_pdf_update");
    } else if (pp.plan.cl.kind == kIJK && pp.plan.cl.I == 1 && pp.plan.cl.J > 1 && pp.plan.cl.K >= kBlock &&
               pp.plan.cl.J <= 0x7fffffff) {
        // one run per slot
        ba.counts = counts;
        const bool vec = aligned16(x) && pp.plan.cl.K % io_vec(dtype) == 0;
        const dim3 g((unsigned)pp.plan.cl.J), b(kBlock);
#define AHQ_LAUNCH_RUNS(IO)                                                                                         \
    do {                                                                                                            \
        if (vec) hipLaunchKernelGGL((dlq_pdf_bin_runs_kernel<IO, IoTraits<IO>::kVec>), g, b, 0, s, ba);             \
        else hipLaunchKernelGGL((dlq_pdf_bin_runs_kernel<IO, 1>), g, b, 0, s, ba);                                  \
    } while (0)
        switch (dtype) {
            case AHQ_F32: AHQ_LAUNCH_RUNS(float); break;
            case AHQ_F16: AHQ_LAUNCH_RUNS(f16_t); break;
            default: AHQ_LAUNCH_RUNS(bf16_t); break;
        }
#undef AHQ_LAUNCH_RUNS
        fa.counts = counts;
        fa.nparts = 1;
    } else {
        ba.counts = counts;
        const int64_t n = (int64_t)S * kPdf;
        hipLaunchKernelGGL(dlq_zero_u32_kernel, dim3((unsigned)((n + 255) / 256 > 1024 ? 1024 : (n + 255) / 256)), dim3(256), 0,
                           s, counts, n);
        switch (dtype) {
            case AHQ_F32: hipLaunchKernelGGL((dlq_pdf_bin_generic_kernel<float>), dim3(pp.nblocks), dim3(kBlock), 0, s, ba); break;
            case AHQ_F16: hipLaunchKernelGGL((dlq_pdf_bin_generic_kernel<f16_t>), dim3(pp.nblocks), dim3(kBlock), 0, s, ba); break;
            default: hipLaunchKernelGGL((dlq_pdf_bin_generic_kernel<bf16_t>), dim3(pp.nblocks), dim3(kBlock), 0, s, ba); break;
        }
        fa.counts = counts;
        fa.nparts = 1;
    }
    hipLaunchKernelGGL(dlq_pdf_finish_kernel, dim3(kPdf / kBlock, S < 65535 ? S : 65535), dim3(kBlock), 0, s, fa);
    return check_launch("dlq_pdf_update");
}

// Running float min / max <- std::min / std::max with a batch's extrema given in the tensor's dtype (a 16-bit tensor is
// widened value by value before the fold, MinMaxEncodingAnalyzer.cpp:32-95 with tensor_utils.hpp's widening).
template <typename IO>
__global__ void dlq_minmax_fold_kernel(const IO* bmin, const IO* bmax, float* rmin, float* rmax, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float mn = load_f32(bmin[i]), mx = load_f32(bmax[i]);
    const float pmn = rmin[i], pmx = rmax[i];
    rmin[i] = mn < pmn ? mn : pmn;
    rmax[i] = pmx < mx ? mx : pmx;
}

extern "C" int ahq_dlq_minmax_fold(int32_t dtype, const void* batch_min, const void* batch_max, int64_t num_encodings,
                                   float* run_min, float* run_max, void* stream) {
    if (dtype < AHQ_F32 || dtype > AHQ_BF16) return set_error("bad dtype"), AHQ_ERR_INVALID;
    if (!batch_min || !batch_max || !run_min || !run_max) return set_error("null argument"), AHQ_ERR_INVALID;
    if (num_encodings < 0) return set_error("negative encoding count"), AHQ_ERR_INVALID;
    if (num_encodings == 0) return AHQ_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 g((unsigned)((num_encodings + 255) / 256)), b(256);
    switch (dtype) {
        case AHQ_F32: hipLaunchKernelGGL((dlq_minmax_fold_kernel<float>), g, b, 0, s, static_cast<const float*>(batch_min), static_cast<const float*>(batch_max), run_min, run_max, num_encodings); break;
        case AHQ_F16: hipLaunchKernelGGL((dlq_minmax_fold_kernel<f16_t>), g, b, 0, s, static_cast<const f16_t*>(batch_min), static_cast<const f16_t*>(batch_max), run_min, run_max, num_encodings); break;
        default: hipLaunchKernelGGL((dlq_minmax_fold_kernel<bf16_t>), g, b, 0, s, static_cast<const bf16_t*>(batch_min), static_cast<const bf16_t*>(batch_max), run_min, run_max, num_encodings); break;
    }
    return check_launch("dlq_minmax_fold");
}

extern "C" size_t ahq_dlq_tfe_encodings_workspace_bytes(int32_t num_slots) {
    if (num_slots <= 0) return 0;
    const size_t S = (size_t)num_slots;
    return up256(S * kMaxCand * 4) * 3 + up256(S * kPdf * 4) + up256(S * 16) + up256(S * kMaxCand * 8);
}

extern "C" int ahq_dlq_tfe_encodings(const ahq_dlq_pdf_state* st, int32_t bw, int32_t symmetric, int32_t strict,
                                     int32_t unsigned_sym, double* out, int32_t* best_index, void* workspace,
                                     size_t workspace_bytes, void* stream) {
    if (!check_pdf_state(st)) return AHQ_ERR_INVALID;
    if (!out) return set_error("out is null"), AHQ_ERR_INVALID;
    if (bw < 1 || bw > 31) return set_error("bitwidth must be in 1..31"), AHQ_ERR_INVALID;
    const size_t need = ahq_dlq_tfe_encodings_workspace_bytes(st->num_slots);
    if (!workspace || workspace_bytes < need) return set_error("workspace too small"), AHQ_ERR_WORKSPACE;
    const size_t S = (size_t)st->num_slots;
    char* w = static_cast<char*>(workspace);
    TfeArgs a{};
    a.num_slots = st->num_slots;
    a.bw = bw;
    a.symmetric = symmetric ? 1 : 0;
    a.strict = strict ? 1 : 0;
    a.unsigned_sym = unsigned_sym ? 1 : 0;
    a.xleft = st->xleft;
    a.pdf = st->pdf;
    a.meta = st->meta;
    size_t o = 0;
    a.cand_delta = reinterpret_cast<float*>(w + o);  o += up256(S * kMaxCand * 4);
    a.cand_off = reinterpret_cast<int32_t*>(w + o);  o += up256(S * kMaxCand * 4);
    a.cand_ok = reinterpret_cast<int32_t*>(w + o);   o += up256(S * kMaxCand * 4);
    a.centers = reinterpret_cast<float*>(w + o);     o += up256(S * kPdf * 4);
    a.head = reinterpret_cast<float*>(w + o);        o += up256(S * 16);
    a.cost = reinterpret_cast<double*>(w + o);       o += up256(S * kMaxCand * 8);
    a.out = out;
    a.best = best_index;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(dlq_tfe_candidates_kernel, dim3(st->num_slots), dim3(kMaxCand), 0, s, a);
    // Few slots: one wave per candidate (the candidates beyond the list are marked invalid and cost nothing).  That
    // form issues about eight times the instructions of the lane-per-candidate one, so it pays only while the latter
    // cannot fill the GPU.
    if (st->num_slots <= 16) hipLaunchKernelGGL(dlq_tfe_cost_wave_kernel, dim3(kMaxCand, st->num_slots), dim3(kWave), 0, s, a);
    else hipLaunchKernelGGL(dlq_tfe_cost_kernel, dim3(st->num_slots), dim3(kMaxCand), 0, s, a);
    hipLaunchKernelGGL(dlq_tfe_select_kernel, dim3(st->num_slots), dim3(kWave), 0, s, a);
    return check_launch("dlq_tfe_encodings");
}

extern "C" int ahq_dlq_percentile_encodings(const ahq_dlq_pdf_state* st, float percentile, int32_t bw, int32_t symmetric,
                                            int32_t strict, int32_t unsigned_sym, double* out, void* stream) {
    if (!check_pdf_state(st)) return AHQ_ERR_INVALID;
    if (!out) return set_error("out is null"), AHQ_ERR_INVALID;
    if (bw < 1 || bw > 31) return set_error("bitwidth must be in 1..31"), AHQ_ERR_INVALID;
    hipLaunchKernelGGL(dlq_percentile_kernel, dim3(st->num_slots), dim3(kWave), 0, static_cast<hipStream_t>(stream),
                       st->xleft, st->pdf, st->meta, percentile, bw, symmetric, strict, unsigned_sym, out);
    return check_launch("dlq_percentile_encodings");
}
