// SQNR / TF-enhanced encoding search over a histogram (aimet_torch/quantization/encoding_analyzer.py:695-899).
//
// The (histogram, delta, offset, bin) tensor of the reference is never materialised: one workgroup owns one
// (histogram, delta) row, its waves take the offset candidates in turn, lanes stride over the bins with the histogram
// and bin mid-points held in LDS, and the clipping/quantisation noise of a candidate is accumulated in fp64.  A second
// single-workgroup launch per histogram picks the first minimum and writes the encoding.  Searches over many histograms
// (per-channel analyzers) price one candidate per lane instead (sqnr_noise_lanes_kernel).
//
// Candidate generation repeats the reference's fp32 operations one by one (encoding_analyzer.py:728-820); the only
// host-made input is the rounded offset grid, because torch.arange computes it in double precision on the CPU.

#include "ahq_device.h"
#include "ahq_host.h"

namespace ahq {

struct SqnrArgs {
    int32_t num_slots, num_bins, num_deltas, num_offsets;  // num_offsets counts the observed offset (asymmetric)
    int32_t symmetric;
    int32_t stat_dtype;     // dtype the stored min/max live in (arithmetic on them happens in that dtype)
    int32_t pairs_per_block;  // (delta, offset) candidates one workgroup prices
    float num_steps;
    float min_scale;        // minimum_scale as float
    float min_range;        // float(minimum_scale * num_steps)
    float sym_offset;       // (-num_steps) // 2
    float gamma;
    float p;
    const float* hist;      // [S][B]
    const float* edges;     // [S][B+1]
    const float* minmax;    // [S][2]
    const float* offset_grid;  // [num_offsets - 1] rounded offsets (asymmetric)
    float* noise;           // [S][D][O]
    float* deltas;          // [S][D][O] clamped candidates
    float* offsets;         // [S][D][O]
    float* out;             // [S][4]: best delta, best offset, encoding min, encoding max
    long long* best_index;  // [S]
};

__device__ __forceinline__ float rnd_rt(float v, int dt) {
    if (dt == AHQ_BF16) return rnd<AHQ_BF16>(v);
    if (dt == AHQ_F16) return rnd<AHQ_F16>(v);
    return v;
}

struct Cand {
    float delta, offset;
};

// (delta, offset) of candidate (d, o) for histogram s, after clamping to the observed range.
__device__ __forceinline__ Cand candidate(const SqnrArgs& a, int s, int d, int o) {
    const int dt = a.stat_dtype;
    float lo = a.minmax[2 * s], hi = a.minmax[2 * s + 1];
    lo = fminf(lo, 0.f);
    hi = fmaxf(hi, 0.f);
    hi = fmaxf(hi, rnd_rt(lo + a.min_range, dt));
    Cand c;
    if (a.symmetric) {
        const float dmax = (2.f * fmaxf(hi, -lo)) / a.num_steps;
        c.delta = fmaxf((dmax * (float)(d + 1)) / (float)(a.num_deltas - 1), a.min_scale);
        c.offset = a.sym_offset;
        return c;
    }
    const float dmax = rnd_rt(hi - lo, dt) / a.num_steps;
    const float obs_off = __builtin_rintf(lo / dmax);
    const float obs_min = dmax * obs_off;
    const float obs_max = obs_min + dmax * a.num_steps;
    const float td = (dmax * (float)(d + 1)) / (float)(a.num_deltas - 1);
    const float to = o < a.num_offsets - 1 ? a.offset_grid[o] : obs_off;
    float tmin = td * to;
    float tmax = tmin + td * a.num_steps;
    tmin = fmaxf(obs_min, tmin);
    tmax = fminf(obs_max, tmax);
    c.delta = fmaxf((tmax - tmin) / a.num_steps, a.min_scale);
    c.offset = __builtin_rintf(tmin / c.delta);
    return c;
}

constexpr int kSqnrMaxBins = 4096;
constexpr int kMaxGridY = 65535;  // largest y dimension of a grid

// A workgroup stages one slot's histogram and bin centres and prices kPairsPerBlock (delta, offset) candidates, one
// wave per candidate at a time.  Candidates are numbered delta-major across the whole grid, so a symmetric search
// (one offset) fills its workgroups as well as an asymmetric one.
constexpr int kPairsPerBlock = 64;  // at most; fewer when that leaves the GPU short of workgroups

__global__ __launch_bounds__(kBlock) void sqnr_noise_kernel(const SqnrArgs a) {
    extern __shared__ float sqnr_lds[];  // [2][num_bins]
    const int B = a.num_bins, O = a.num_offsets;
    float* h_lds = sqnr_lds;
    float* m_lds = sqnr_lds + B;
    // the y dimension of a grid ends at 65535: slots beyond it are taken in further rounds
    for (int s = blockIdx.y; s < a.num_slots; s += gridDim.y) {
    if (s != (int)blockIdx.y) __syncthreads();  // the previous slot's staged histogram is still being read
    const float* e = a.edges + (size_t)s * (B + 1);
    const float w = e[1] - e[0];
    const float first_mid = e[0] + w / 2.f;
    for (int b = threadIdx.x; b < B; b += kBlock) {
        h_lds[b] = a.hist[(size_t)s * B + b];
        m_lds[b] = first_mid + w * (float)b;
    }
    __syncthreads();
    const int lane = threadIdx.x & (kWave - 1);
    const bool use_gamma = a.gamma != 1.0f;
    const int pairs = a.num_deltas * O;
    const int p0 = blockIdx.x * a.pairs_per_block;
    const int p1 = p0 + a.pairs_per_block < pairs ? p0 + a.pairs_per_block : pairs;
    for (int p = p0 + threadIdx.x / kWave; p < p1; p += kBlock / kWave) {
        const int d = p / O, o = p - d * O;
        const Cand c = candidate(a, s, d, o);
        double acc = 0.0;
        for (int b = lane; b < B; b += kWave) {
            const float mid = m_lds[b];
            float q = __builtin_rintf(mid / c.delta - c.offset);
            const bool clipped = (q < 0.f) | (q > a.num_steps);
            q = q < 0.f ? 0.f : (q > a.num_steps ? a.num_steps : q);
            const float y = (q + c.offset) * c.delta;
            const float ad = __builtin_fabsf(y - mid);
            float err = (a.p == 2.0f ? ad * ad : __builtin_powf(ad, a.p)) * h_lds[b];
            if (use_gamma && clipped) err = err * a.gamma;
            acc += (double)err;
        }
        acc = wave_reduce(acc, OpAddD());
        if (lane == 0) {
            const size_t i = ((size_t)s * a.num_deltas + d) * O + o;
            a.noise[i] = (float)acc;
            a.deltas[i] = c.delta;
            a.offsets[i] = c.offset;
        }
    }
    }
}

// The same sums with one lane per candidate, for searches with enough candidates to fill the GPU that way (per-channel
// and blockwise analyzers).  A lane walks every bin of its slot's staged histogram -- all lanes read the same LDS word,
// a broadcast -- so a candidate is derived once instead of once per lane of a wave, no cross-lane sum is needed, and
// the divisor of the bin loop is a per-lane constant: with its reciprocal at hand the quotient takes the
// division-free form (two residual corrections, correctly rounded like the IEEE sequence as long as nothing under- or
// overflows: bin centres up to 2^60 and a step in [2^-60, 2^60]; a wave with a lane outside that takes the plain
// division).  The bins are summed in fp64 in two interleaved chains.
constexpr float kSqnrFastDivMax = 1.152921504606846976e18f;   // 2^60
constexpr float kSqnrFastDivMin = 8.673617379884035472e-19f;  // 2^-60
constexpr int kLaneBlockMax = 512;

template <bool FAST, bool P2>
__device__ __forceinline__ double lane_noise(const SqnrArgs& a, const float2* hm, int B, Cand c, float rs) {
    double acc0 = 0.0, acc1 = 0.0;
    auto term = [&](float2 v) {
        const float mid = v.y;
        float t;
        if (FAST) {
            const float q0 = mid * rs;
            const float q1 = __builtin_fmaf(__builtin_fmaf(-q0, c.delta, mid), rs, q0);
            t = __builtin_fmaf(__builtin_fmaf(-q1, c.delta, mid), rs, q1);
        } else {
            t = mid / c.delta;
        }
        float q = __builtin_rintf(t - c.offset);
        const bool clipped = (q < 0.f) | (q > a.num_steps);
        q = q < 0.f ? 0.f : (q > a.num_steps ? a.num_steps : q);
        const float y = (q + c.offset) * c.delta;
        const float ad = __builtin_fabsf(y - mid);
        const float err = (P2 ? ad * ad : __builtin_powf(ad, a.p)) * v.x;
        // gamma == 1 leaves the term as it is, like the reference's skipped multiplication
        return (double)(clipped ? err * a.gamma : err);
    };
    int b = 0;
#pragma unroll 4
    for (; b + 1 < B; b += 2) {
        acc0 += term(hm[b]);
        acc1 += term(hm[b + 1]);
    }
    if (b < B) acc0 += term(hm[b]);
    return acc0 + acc1;
}

__global__ __launch_bounds__(kLaneBlockMax) void sqnr_noise_lanes_kernel(const SqnrArgs a) {
    extern __shared__ float2 sqnr_hm[];  // [num_bins] (count, bin centre)
    const int B = a.num_bins, O = a.num_offsets;
    for (int s = blockIdx.y; s < a.num_slots; s += gridDim.y) {  // slots beyond the y limit of a grid: further rounds
    if (s != (int)blockIdx.y) __syncthreads();
    const float* e = a.edges + (size_t)s * (B + 1);
    const float w = e[1] - e[0];
    const float first_mid = e[0] + w / 2.f;
    for (int b = threadIdx.x; b < B; b += blockDim.x)
        sqnr_hm[b] = make_float2(a.hist[(size_t)s * B + b], first_mid + w * (float)b);
    __syncthreads();
    const int pairs = a.num_deltas * O;
    const int p = blockIdx.x * blockDim.x + threadIdx.x;
    const bool live = p < pairs;
    const int d = live ? p / O : 0, o = live ? p - d * O : 0;
    const Cand c = candidate(a, s, d, o);
    const float last_mid = first_mid + w * (float)(B - 1);
    const float dm = __builtin_fabsf(c.delta);
    const bool fast = __builtin_fabsf(first_mid) <= kSqnrFastDivMax && __builtin_fabsf(last_mid) <= kSqnrFastDivMax &&
                      dm >= kSqnrFastDivMin && dm <= kSqnrFastDivMax;
    const bool all_fast = __builtin_amdgcn_ballot_w64(!fast) == 0;
    const float rs = all_fast ? 1.0f / c.delta : 0.f;
    double acc;
    if (a.p == 2.0f)
        acc = all_fast ? lane_noise<true, true>(a, sqnr_hm, B, c, rs) : lane_noise<false, true>(a, sqnr_hm, B, c, rs);
    else
        acc = all_fast ? lane_noise<true, false>(a, sqnr_hm, B, c, rs) : lane_noise<false, false>(a, sqnr_hm, B, c, rs);
    if (live) {
        const size_t i = (size_t)s * pairs + p;
        a.noise[i] = (float)acc;
        a.deltas[i] = c.delta;
        a.offsets[i] = c.offset;
    }
    }
}

// torch.min over the flattened candidates (encoding_analyzer.py:822-839): the first minimum, and a NaN counts as
// smaller than every number, so the first NaN wins when there is one.
__device__ __forceinline__ bool sqnr_better(float v, int i, float bv, int bi) {
    const bool vn = v != v, bn = bv != bv;
    if (vn | bn) return vn && (!bn || i < bi);
    return v < bv || (v == bv && i < bi);
}

__global__ __launch_bounds__(kBlock) void sqnr_select_kernel(const SqnrArgs a) {
    __shared__ float v_sm[kBlock / kWave];
    __shared__ int i_sm[kBlock / kWave];
    const int s = blockIdx.x;
    const int n = a.num_deltas * a.num_offsets;
    const float* noise = a.noise + (size_t)s * n;
    float best = __builtin_inff();
    int bi = n;
    constexpr int kLoads = 4;  // loads in flight per lane
    for (int i0 = threadIdx.x; i0 < n; i0 += kLoads * kBlock) {
        float v[kLoads];
#pragma unroll
        for (int u = 0; u < kLoads; ++u) v[u] = i0 + u * kBlock < n ? noise[i0 + u * kBlock] : __builtin_inff();
#pragma unroll
        for (int u = 0; u < kLoads; ++u) {
            const int i = i0 + u * kBlock < n ? i0 + u * kBlock : n;
            if (sqnr_better(v[u], i, best, bi)) {
                best = v[u];
                bi = i;
            }
        }
    }
#pragma unroll
    for (int m = kWave / 2; m >= 1; m >>= 1) {
        const float ov = __shfl_xor(best, m, kWave);
        const int oi = __shfl_xor(bi, m, kWave);
        if (sqnr_better(ov, oi, best, bi)) {
            best = ov;
            bi = oi;
        }
    }
    if ((threadIdx.x & (kWave - 1)) == 0) {
        v_sm[threadIdx.x / kWave] = best;
        i_sm[threadIdx.x / kWave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kBlock / kWave; ++w)
            if (sqnr_better(v_sm[w], i_sm[w], v_sm[0], i_sm[0])) {
                v_sm[0] = v_sm[w];
                i_sm[0] = i_sm[w];
            }
    }
    if (threadIdx.x == 0) {
        int idx = i_sm[0];
        if (idx >= n) idx = 0;
        const float delta = a.deltas[(size_t)s * n + idx];
        const float off = a.offsets[(size_t)s * n + idx];
        const float mn = off * delta;
        const float mx = mn + a.num_steps * delta;
        a.out[4 * s] = delta;
        a.out[4 * s + 1] = off;
        a.out[4 * s + 2] = mn;
        a.out[4 * s + 3] = mx;
        a.best_index[s] = idx;
    }
}

}  // namespace ahq

using namespace ahq;

extern "C" int ahq_sqnr_search(const ahq_sqnr_params* p, const float* hist, const float* edges, const float* minmax,
                               const float* offset_grid, float* noise, float* deltas, float* offsets, float* out,
                               long long* best_index, void* stream) {
    if (!p || !hist || !edges || !minmax || !noise || !deltas || !offsets || !out || !best_index)
        return set_error("null argument"), AHQ_ERR_INVALID;
    if (p->num_slots <= 0 || p->num_deltas <= 1 || p->num_offsets <= 0) return set_error("bad candidate grid"), AHQ_ERR_INVALID;
    if (p->num_bins <= 1 || p->num_bins > kSqnrMaxBins) return set_error("num_bins must be in [2, 4096]"), AHQ_ERR_UNSUPPORTED;
    if (p->num_steps <= 0) return set_error("num_steps must be positive"), AHQ_ERR_INVALID;
    if (!p->symmetric && (p->num_offsets < 2 || !offset_grid)) return set_error("asymmetric search needs an offset grid"), AHQ_ERR_INVALID;
    if (p->stat_dtype < AHQ_F32 || p->stat_dtype > AHQ_BF16) return set_error("bad stat_dtype"), AHQ_ERR_INVALID;
    SqnrArgs a{};
    a.num_slots = p->num_slots;
    a.num_bins = p->num_bins;
    a.num_deltas = p->num_deltas;
    a.num_offsets = p->symmetric ? 1 : p->num_offsets;
    a.symmetric = p->symmetric;
    a.stat_dtype = p->stat_dtype;
    a.num_steps = (float)p->num_steps;
    a.min_scale = (float)p->minimum_scale;
    a.min_range = (float)(p->minimum_scale * (double)p->num_steps);
    // Python floor division of -num_steps by 2
    a.sym_offset = (float)(-((p->num_steps + 1) / 2));
    a.gamma = (float)p->gamma;
    a.p = (float)p->p;
    a.hist = hist;
    a.edges = edges;
    a.minmax = minmax;
    a.offset_grid = offset_grid;
    a.noise = noise;
    a.deltas = deltas;
    a.offsets = offsets;
    a.out = out;
    a.best_index = best_index;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int pairs = a.num_deltas * a.num_offsets;
    // One lane per candidate costs about 19 instructions per bin for a whole wave of candidates; one wave per candidate
    // about 30 per 64 bins plus 150 for deriving the candidate and summing across lanes.  The first form also needs
    // enough waves of candidates to occupy the GPU, which a per-tensor search does not have.
    const int64_t cand_waves = (pairs + kWave - 1) / kWave;
    const unsigned grid_y = (unsigned)(a.num_slots < kMaxGridY ? a.num_slots : kMaxGridY);
    const int64_t cost_lanes = cand_waves * a.num_bins * 19;
    const int64_t cost_waves = (int64_t)pairs * ((int64_t)a.num_bins * 30 / kWave + 150);
    if (cand_waves * a.num_slots >= 512 && cost_lanes < cost_waves) {
        const int block = (int)(cand_waves * kWave < kLaneBlockMax ? cand_waves * kWave : kLaneBlockMax);
        hipLaunchKernelGGL(sqnr_noise_lanes_kernel, dim3((unsigned)((pairs + block - 1) / block), grid_y), dim3(block),
                           (size_t)a.num_bins * sizeof(float2), st, a);
    } else {
        // a per-tensor search has a few thousand candidates in all: one per wave, so that its latency is that of a
        // single candidate; with many slots a workgroup prices up to 64 per staged histogram
        int64_t ppb = ((int64_t)pairs * a.num_slots) / 2048;
        ppb = ppb < kBlock / kWave ? kBlock / kWave : (ppb > kPairsPerBlock ? kPairsPerBlock : ppb);
        a.pairs_per_block = (int)ppb;
        hipLaunchKernelGGL(sqnr_noise_kernel, dim3((unsigned)((pairs + ppb - 1) / ppb), grid_y), dim3(kBlock),
                           2 * (size_t)a.num_bins * sizeof(float), st, a);
    }
    hipLaunchKernelGGL(sqnr_select_kernel, dim3(a.num_slots), dim3(kBlock), 0, st, a);
    return check_launch("ahq_sqnr_search");
}
