// Min/max statistics -> encoding range, one thread per encoding.
//
// Replaces the dozen elementwise torch launches of MinMaxEncodingAnalyzer.compute_encodings_from_stats
// (aimet_torch/quantization/encoding_analyzer.py:425-481) and the range checks of _flag_extreme_min_max (:484-498)
// with one launch.  A whole-model calibration ends hundreds of quantizer contexts, each on a handful of values, so the
// launches -- not the arithmetic -- are the cost.  Every operation keeps the dtype torch's type promotion gives it:
// statistics arithmetic in the statistics dtype T (rounded after each operation), everything after the float32
// "widen" term in float32, the result rounded to T once.

#include <cstdio>

#include "ahq_device.h"
#include "ahq_host.h"
#include "layout.h"

namespace ahq {

struct EncArgs {
    const void* smin;
    const void* smax;
    void* out_min;
    void* out_max;
    int32_t* flags;  // optional [2]: any non-finite result, any result within 5 % of the dtype's largest value
    int64_t n;
    float num_steps;      // as float (exact up to 2^24)
    float tiny_t;         // minimum scale rounded to T (what the comparison sees)
    float tiny_f;         // minimum scale as float32 (what the product with the comparison result holds)
    float pos, neg, pos_extra;  // floor(n/2), ceil(n/2), floor(n/2) + (n == 3)
    float t_max;          // finfo(T).max
    float near_thr;       // T(1e-8 + 0.05 * finfo(T).max)
    int32_t symmetric;
};

template <typename T>
struct RoundTo;
template <>
struct RoundTo<float> { __device__ static float f(float v) { return v; } };
template <>
struct RoundTo<f16_t> { __device__ static float f(float v) { return rnd<AHQ_F16>(v); } };
template <>
struct RoundTo<bf16_t> { __device__ static float f(float v) { return rnd<AHQ_BF16>(v); } };

__device__ __forceinline__ float nan_max(float a, float b) { return (a != a || b != b) ? __builtin_nanf("") : fmaxf(a, b); }

// statistics (mn, mx) -> encoding range (lo, hi), both as T values widened to float; raises the flags
template <typename T>
__device__ __forceinline__ void encode_range(const EncArgs& a, float mn, float mx, T& lo_t, T& hi_t) {
    using R = RoundTo<T>;
    // clamp(min, max=0), clamp(max, min=0): NaN stays NaN
    float lo = (mn != mn) ? mn : fminf(mn, 0.f);
    float hi = (mx != mx) ? mx : fmaxf(mx, 0.f);
    const float step = R::f(R::f(hi - lo) / a.num_steps);       // (hi - lo) / num_steps in T
    const float widen = (step < a.tiny_t) ? a.tiny_f : 0.f;     // float32 from here on
    if (a.symmetric) {
        hi = hi + a.pos * widen;
        lo = lo - a.neg * widen;
        const float delta = nan_max(hi / a.pos_extra, (-lo) / a.neg);
        lo = (-1.f * a.neg) * delta;
        hi = a.pos * delta;
        lo = (lo != lo) ? lo : fmaxf(lo, -a.t_max);
    } else {
        hi = hi + a.num_steps * widen;
        // the lower end never left T; clamping it to finfo(T).min only turns -inf into the lowest finite value
        lo = (lo != lo) ? lo : fmaxf(lo, -a.t_max);
    }
    hi = (hi != hi) ? hi : fminf(hi, a.t_max);
    lo_t = store_cast<T>(lo);
    hi_t = store_cast<T>(hi);
    if (a.flags) {
        const float l = load_f32(lo_t), h = load_f32(hi_t);
        const bool nonfinite = !(__builtin_fabsf(l) < __builtin_inff()) || !(__builtin_fabsf(h) < __builtin_inff());
        const bool near = __builtin_fabsf(R::f(__builtin_fabsf(l) - a.t_max)) <= a.near_thr ||
                          __builtin_fabsf(R::f(__builtin_fabsf(h) - a.t_max)) <= a.near_thr;
        if (nonfinite) atomicOr(&a.flags[0], 1);
        if (near) atomicOr(&a.flags[1], 1);
    }
}

template <typename T>
__global__ void minmax_to_encodings_kernel(const EncArgs a) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= a.n) return;
    T lo_t, hi_t;
    encode_range<T>(a, load_f32(static_cast<const T*>(a.smin)[i]), load_f32(static_cast<const T*>(a.smax)[i]), lo_t, hi_t);
    static_cast<T*>(a.out_min)[i] = lo_t;
    static_cast<T*>(a.out_max)[i] = hi_t;
}

// ----------------------------------------------------------------------------------- range -> (scale, offset) --
// AffineQuantizerBase.get_scale / _get_offset for min/max quantizers with dtype = float32
// (aimet_torch/quantization/affine/quantizer.py:319-376):
//   scale  = clamp_min(|float(max) - float(min)| / num_steps, minimum_scale)
//   offset = clamp(round(min / scale) - qmin, -qmax, -qmin)          (asymmetric grids only)
// in float32 throughout (a 16-bit min is promoted by the division with the float32 scale), division by num_steps an
// IEEE division (what the CPU path does for tensor / number), round = half to even, NaN kept by both clamps.
struct ScaleOffArgs {
    const void* pmin;
    const void* pmax;
    float* scale;
    float* offset;  // null: symmetric grid, the offset is a constant the caller knows
    int64_t n;
    float num_steps, minimum_scale, qmin, lo, hi;  // lo = -qmax, hi = -qmin
};

template <typename T>
__global__ void range_to_scale_offset_kernel(const ScaleOffArgs a) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= a.n) return;
    const float mn = load_f32(static_cast<const T*>(a.pmin)[i]);
    const float mx = load_f32(static_cast<const T*>(a.pmax)[i]);
    float s = __builtin_fabsf((mx - mn) / a.num_steps);
    s = (s != s) ? s : fmaxf(s, a.minimum_scale);
    a.scale[i] = s;
    if (a.offset) {
        const float r = __builtin_rintf(mn / s) - a.qmin;
        a.offset[i] = (r != r) ? r : fminf(fmaxf(r, a.lo), a.hi);
    }
}

// ------------------------------------------------------ gradients of (scale, offset) -> gradients of (min, max) --
// What autograd derives for get_scale / _get_offset above when min / max are learned (the chain SubBackward,
// DivBackward, AbsBackward, ClampMinBackward and, for asymmetric grids, DivBackward, the straight-through round and
// ClampBackward: a dozen small launches per training step), operation by operation in float32:
//   gr     = goffset where -qmax <= round(min / s) - qmin <= -qmin, else 0            (clamp, straight-through round)
//   gmin1  = gr / s;   gs' = gscale + (-gr * ((min / s) / s))                          (min / s)
//   ga     = gs' where |d / n| >= minimum_scale, else 0;   g0 = ga * sgn(d / n)        (clamp_min, abs; d = max - min)
//   gd     = g0 / n;   gmax = gd;   gmin = gmin1 + (-gd)                               (division by num_steps, max - min)
// Symmetric grids have a constant offset: gr = 0.  Gradients that leave through a parameter of a narrower dtype P
// are rounded to P where autograd casts them (each of the two terms of gmin, then their sum).
struct RangeGradArgs {
    const void* pmin;
    const void* pmax;
    const float* gscale;
    const float* goffset;  // null: symmetric grid
    void* gmin;
    void* gmax;
    int64_t n;
    float num_steps, minimum_scale, qmin, lo, hi;  // lo = -qmax, hi = -qmin
};

template <typename P>
__global__ void range_grad_kernel(const RangeGradArgs a) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= a.n) return;
    using R = RoundTo<P>;
    const float mn = load_f32(static_cast<const P*>(a.pmin)[i]);
    const float mx = load_f32(static_cast<const P*>(a.pmax)[i]);
    const float s0 = (mx - mn) / a.num_steps;
    const float ab = __builtin_fabsf(s0);
    const float s = (ab != ab) ? ab : fmaxf(ab, a.minimum_scale);
    float gs = a.gscale[i];
    float gmin1 = 0.f;
    if (a.goffset) {
        const float r = mn / s;
        const float u = __builtin_rintf(r) - a.qmin;
        const float gr = (u >= a.lo && u <= a.hi) ? a.goffset[i] : 0.f;
        gmin1 = R::f(gr / s);
        gs = gs + (-gr) * (r / s);
    }
    const float ga = (ab >= a.minimum_scale) ? gs : 0.f;
    const float sg = (s0 > 0.f) ? 1.f : (s0 < 0.f) ? -1.f : 0.f;
    const float gd = (ga * sg) / a.num_steps;
    static_cast<P*>(a.gmax)[i] = store_cast<P>(gd);
    const float gmin2 = R::f(-gd);
    static_cast<P*>(a.gmin)[i] = store_cast<P>(a.goffset ? gmin1 + gmin2 : gmin2);
}

// ------------------------------------------------ statistics -> range, quantizer parameters, scale and offset --
// The end of a min/max calibration in one launch: the encoding range of the statistics (minmax_to_encodings_kernel),
// stored into the quantizer's min / max parameters in their own dtype P (what Tensor.copy_ does: round to nearest
// even), and scale / offset derived from the stored parameters (range_to_scale_offset_kernel).  A whole-model
// calibration ends a few hundred quantizer contexts; each is a handful of values.
struct FinalArgs {
    void* pmin;
    void* pmax;
    ScaleOffArgs so;  // pmin / pmax unused
};

template <typename T, typename P>
__device__ __forceinline__ void finalize_one(const EncArgs& a, const FinalArgs& f, int64_t i, float smin, float smax);

template <typename T, typename P>
__global__ void minmax_finalize_kernel(const EncArgs a, const FinalArgs f) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= a.n) return;
    finalize_one<T, P>(a, f, i, load_f32(static_cast<const T*>(a.smin)[i]), load_f32(static_cast<const T*>(a.smax)[i]));
}

// The same for a single encoding whose running extrema still lie in the slots of ahq_minmax_accumulate (min, max and
// a NaN flag per workgroup of that kernel): one workgroup folds the slots the way ahq_minmax_slots_read does -- a
// NaN seen anywhere makes both statistics NaN, as torch.amin / amax would -- and its first thread goes on.
constexpr int kSlotThreads = 256;

// Folds the slots; true in the one thread that holds the result (mn, mx as values of the tensor's dtype T: what the
// fold would have stored).
template <typename T>
__device__ __forceinline__ bool fold_slots(const float* slot_min, const float* slot_max, const int* slot_nan, float& mn,
                                           float& mx) {
    __shared__ float red[kSlotThreads / kWave][2];
    __shared__ int red_nan[kSlotThreads / kWave];
    mn = __builtin_inff();
    mx = -__builtin_inff();
    int nan = 0;
    for (int q = threadIdx.x; q < AHQ_MINMAX_SLOTS; q += kSlotThreads) {
        mn = fminf(mn, slot_min[q]);
        mx = fmaxf(mx, slot_max[q]);
        nan |= slot_nan[q];
    }
#pragma unroll
    for (int m = kWave / 2; m >= 1; m >>= 1) {
        mn = fminf(mn, __shfl_xor(mn, m, kWave));
        mx = fmaxf(mx, __shfl_xor(mx, m, kWave));
        nan |= __shfl_xor(nan, m, kWave);
    }
    if ((threadIdx.x & (kWave - 1)) == 0) {
        red[threadIdx.x / kWave][0] = mn;
        red[threadIdx.x / kWave][1] = mx;
        red_nan[threadIdx.x / kWave] = nan;
    }
    __syncthreads();
    if (threadIdx.x != 0) return false;
    for (int w = 1; w < kSlotThreads / kWave; ++w) {
        mn = fminf(mn, red[w][0]);
        mx = fmaxf(mx, red[w][1]);
        nan |= red_nan[w];
    }
    const float qnan = __builtin_nanf("");
    mn = load_f32(store_cast<T>(nan ? qnan : mn));
    mx = load_f32(store_cast<T>(nan ? qnan : mx));
    return true;
}

template <typename T, typename P>
__global__ __launch_bounds__(kSlotThreads) void minmax_slots_finalize_kernel(const float* slot_min, const float* slot_max,
                                                                             const int* slot_nan, const EncArgs a,
                                                                             const FinalArgs f) {
    float mn, mx;
    if (fold_slots<T>(slot_min, slot_max, slot_nan, mn, mx)) finalize_one<T, P>(a, f, 0, mn, mx);
}

// minmax_slots_finalize_kernel for up to kManySlots quantizers per launch, one workgroup each; every item carries
// its own dtypes, so the type dispatch happens in the kernel.
constexpr int kManySlots = 16;  // what fits the 4 KB a kernel takes as arguments
struct ManySlotItem {
    const float* slot_min;
    const float* slot_max;
    const int* slot_nan;
    EncArgs a;
    FinalArgs f;
    int32_t stat_dtype, param_dtype;
};
struct ManySlotArgs {
    ManySlotItem items[kManySlots];
};
static_assert(sizeof(ManySlotArgs) <= 4096, "kernel arguments are limited to 4 KB");

template <typename T>
__device__ __forceinline__ void many_slots_one(const ManySlotItem& it) {
    float mn, mx;
    if (!fold_slots<T>(it.slot_min, it.slot_max, it.slot_nan, mn, mx)) return;
    if (it.param_dtype == AHQ_F32) finalize_one<T, float>(it.a, it.f, 0, mn, mx);
    else if (it.param_dtype == AHQ_F16) finalize_one<T, f16_t>(it.a, it.f, 0, mn, mx);
    else finalize_one<T, bf16_t>(it.a, it.f, 0, mn, mx);
}

__global__ __launch_bounds__(kSlotThreads) void minmax_slots_finalize_many_kernel(const ManySlotArgs m) {
    const ManySlotItem& it = m.items[blockIdx.x];
    if (it.stat_dtype == AHQ_F32) many_slots_one<float>(it);
    else if (it.stat_dtype == AHQ_F16) many_slots_one<f16_t>(it);
    else many_slots_one<bf16_t>(it);
}

// minmax_to_encodings_kernel for one encoding whose statistics lie in such slots; stat_min / stat_max (optional)
// receive the folded statistics themselves.
template <typename T>
__global__ __launch_bounds__(kSlotThreads) void minmax_slots_to_encodings_kernel(const float* slot_min, const float* slot_max,
                                                                                 const int* slot_nan, const EncArgs a,
                                                                                 T* stat_min, T* stat_max) {
    float mn, mx;
    if (!fold_slots<T>(slot_min, slot_max, slot_nan, mn, mx)) return;
    T lo_t, hi_t;
    encode_range<T>(a, mn, mx, lo_t, hi_t);
    static_cast<T*>(a.out_min)[0] = lo_t;
    static_cast<T*>(a.out_max)[0] = hi_t;
    if (stat_min) stat_min[0] = store_cast<T>(mn);
    if (stat_max) stat_max[0] = store_cast<T>(mx);
}

template <typename T, typename P>
__device__ __forceinline__ void finalize_one(const EncArgs& a, const FinalArgs& f, const int64_t i, const float smin,
                                             const float smax) {
    T lo_t, hi_t;
    encode_range<T>(a, smin, smax, lo_t, hi_t);
    const P lo_p = store_cast<P>(load_f32(lo_t)), hi_p = store_cast<P>(load_f32(hi_t));
    static_cast<P*>(f.pmin)[i] = lo_p;
    static_cast<P*>(f.pmax)[i] = hi_p;
    const float mn = load_f32(lo_p), mx = load_f32(hi_p);
    float s = __builtin_fabsf((mx - mn) / f.so.num_steps);
    s = (s != s) ? s : fmaxf(s, f.so.minimum_scale);
    f.so.scale[i] = s;
    if (f.so.offset) {
        const float r = __builtin_rintf(mn / s) - f.so.qmin;
        f.so.offset[i] = (r != r) ? r : fminf(fmaxf(r, f.so.lo), f.so.hi);
    }
}

// ------------------------------------------------------------------------------- LPBQ: grouped block scales --
// GroupedBlockQuantizeDequantize._get_scale / _get_per_channel_scale (aimet_torch/quantization/affine/quantizer.py:
// 1363-1399) for a quantizer that holds min / max, dtype = float32:
//   raw         = clamp_min(|float(max) - float(min)| / num_steps, minimum_scale)            per block
//   per_channel = amax(raw over the group) / multipliers                                      per group
//   scale       = clamp(round(raw / per_channel), 1, multipliers) * per_channel               per block
// (the last line is quantize_dequantize(raw, per_channel, 0, 1, multipliers) in float32: true division, round half
// to even).  One wave per group of neighbouring blocks; the group is read twice (it is a few hundred bytes).
struct LpbqArgs {
    const void* pmin;
    const void* pmax;
    float* scale;
    float* per_channel;
    int64_t groups, group_size;
    float num_steps, minimum_scale, multipliers;
};

template <typename T>
__global__ __launch_bounds__(kBlock) void lpbq_scale_kernel(const LpbqArgs a) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t waves = (int64_t)gridDim.x * (kBlock / kWave);
    const T* __restrict__ pmin = static_cast<const T*>(a.pmin);
    const T* __restrict__ pmax = static_cast<const T*>(a.pmax);
    auto raw_at = [&](int64_t i) {
        const float s = __builtin_fabsf((load_f32(pmax[i]) - load_f32(pmin[i])) / a.num_steps);
        return (s != s) ? s : fmaxf(s, a.minimum_scale);
    };
    for (int64_t g = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave; g < a.groups; g += waves) {
        const int64_t base = g * a.group_size;
        float largest = -__builtin_inff();
        int nan = 0;
        for (int64_t k = lane; k < a.group_size; k += kWave) {
            const float s = raw_at(base + k);
            nan |= (s != s) ? 1 : 0;
            largest = fmaxf(largest, s);
        }
#pragma unroll
        for (int m = kWave / 2; m >= 1; m >>= 1) {
            largest = fmaxf(largest, __shfl_xor(largest, m, kWave));
            nan |= __shfl_xor(nan, m, kWave);
        }
        if (nan) largest = __builtin_nanf("");  // torch.amax propagates NaN
        const float pc = largest / a.multipliers;
        if (lane == 0) a.per_channel[g] = pc;
        for (int64_t k = lane; k < a.group_size; k += kWave) {
            const float s = raw_at(base + k);
            const float r = __builtin_rintf(s / pc);
            const float q = (r != r) ? r : fminf(fmaxf(r, 1.0f), a.multipliers);
            a.scale[base + k] = q * pc;
        }
    }
}

// LPBQ with learned ranges: the gradients of min / max given the gradient of the snapped block scales, i.e. the
// backward pass of everything lpbq_scale_kernel computes, as autograd derives it for the reference's composition
// (quantizer.py:1363-1399 on top of :319-342), in one launch.  Per group of blocks, with r_k the raw block scales,
// L their maximum, pc = L / M and t_k = r_k / pc:
//   quantize-dequantize of r by pc on the grid [1, M] (torch_builtins.py:727-831, float32 arithmetic, offset 0):
//       in_k   = 1 <= rint(t_k) <= M
//       gr1_k  = g_k where in_k, else 0
//       gpc    = sum_k g_k * (in_k ? rint(t_k) - t_k : clamp(rint(t_k), 1, M))      [+ the gradient of pc itself]
//   pc = L / M and L = amax(r):   gL = gpc / M;   gr2_k = (gL / #{k: r_k == L}) * [r_k == L]
//   r_k = clamp_min(|max_k - min_k| / n, eps):   the symmetric branch of range_grad_kernel on gr1_k + gr2_k.
// The sum runs in double precision in a fixed order (lanes stride over the group, then the fixed butterfly) and is
// rounded once; the reference's float32 sum differs from it in the last bits, as for every scale gradient.
struct LpbqGradArgs {
    const void* pmin;
    const void* pmax;
    const float* gscale;        // gradient of the snapped block scales
    const float* gper_channel;  // optional: gradient of the per-group scales themselves
    void* gmin;
    void* gmax;
    int64_t groups, group_size;
    float num_steps, minimum_scale, multipliers;
};

template <typename P>
__global__ __launch_bounds__(kBlock) void lpbq_scale_grad_kernel(const LpbqGradArgs a) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t waves = (int64_t)gridDim.x * (kBlock / kWave);
    const P* __restrict__ pmin = static_cast<const P*>(a.pmin);
    const P* __restrict__ pmax = static_cast<const P*>(a.pmax);
    P* __restrict__ gmin = static_cast<P*>(a.gmin);
    P* __restrict__ gmax = static_cast<P*>(a.gmax);
    for (int64_t g = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave; g < a.groups; g += waves) {
        const int64_t base = g * a.group_size;
        auto raw_at = [&](int64_t i, float& s0, float& ab) {
            s0 = (load_f32(pmax[i]) - load_f32(pmin[i])) / a.num_steps;
            ab = __builtin_fabsf(s0);
            return (ab != ab) ? ab : fmaxf(ab, a.minimum_scale);
        };
        // the group's maximum (NaN if any member is NaN, as torch.amax)
        float largest = -__builtin_inff();
        int nan = 0;
        for (int64_t k = lane; k < a.group_size; k += kWave) {
            float s0, ab;
            const float r = raw_at(base + k, s0, ab);
            nan |= (r != r) ? 1 : 0;
            largest = fmaxf(largest, r);
        }
#pragma unroll
        for (int m = kWave / 2; m >= 1; m >>= 1) {
            largest = fmaxf(largest, __shfl_xor(largest, m, kWave));
            nan |= __shfl_xor(nan, m, kWave);
        }
        if (nan) largest = __builtin_nanf("");
        const float pc = largest / a.multipliers;
        // gradient of pc and the number of members that attain the maximum
        double sum = 0.0;
        int ties = 0;
        for (int64_t k = lane; k < a.group_size; k += kWave) {
            float s0, ab;
            const float r = raw_at(base + k, s0, ab);
            const float t = r / pc;
            const float xr = __builtin_rintf(t);
            const bool in = (xr >= 1.f) & (xr <= a.multipliers);
            const float xc = xr < 1.f ? 1.f : (xr > a.multipliers ? a.multipliers : xr);
            sum += (double)(a.gscale[base + k] * (in ? xr - t : xc));
            ties += (r == largest) ? 1 : 0;
        }
        sum = wave_reduce(sum, OpAddD());
#pragma unroll
        for (int m = kWave / 2; m >= 1; m >>= 1) ties += __shfl_xor(ties, m, kWave);
        float gpc = (float)sum;
        if (a.gper_channel) gpc = gpc + a.gper_channel[g];
        const float share = (gpc / a.multipliers) / (float)ties;
        for (int64_t k = lane; k < a.group_size; k += kWave) {
            float s0, ab;
            const float r = raw_at(base + k, s0, ab);
            const float t = r / pc;
            const float xr = __builtin_rintf(t);
            const bool in = (xr >= 1.f) & (xr <= a.multipliers);
            const float gr = (in ? a.gscale[base + k] : 0.f) + share * ((r == largest) ? 1.f : 0.f);
            const float ga = (ab >= a.minimum_scale) ? gr : 0.f;
            const float sg = (s0 > 0.f) ? 1.f : (s0 < 0.f) ? -1.f : 0.f;
            const float gd = (ga * sg) / a.num_steps;
            gmax[base + k] = store_cast<P>(gd);
            gmin[base + k] = store_cast<P>(-gd);
        }
    }
}

// --------------------------------------------------------------------- "is this tensor already on a grid" test --
// The early exit of _decompose_prequantized_tensor (aimet_torch/utils.py:2098-2118), which runs on every weight at
// the start of a calibration: of the first 64 blocks take the first 2 * num_levels elements each, as float
// magnitudes; a block with more than num_levels distinct ones cannot lie on the grid.  The reference sorts each
// sample and counts the places where neighbours differ (NaN differs from everything).  One workgroup does the same
// with a bitonic sort in LDS over as many blocks at a time as fit, and writes the verdict: 1 = no sampled block rules
// the grid out.
constexpr int kProbeThreads = 1024;
constexpr int kProbeKeys = 8192;   // sort keys held in LDS (32 KB)
constexpr int kProbeBlocks = 64;   // blocks the reference samples

struct ProbeArgs {
    const void* x;
    uint8_t* verdict;
    int64_t I, J, K;     // flat = (i * J + j) * K + k, block index j
    int32_t nblocks;     // min(J, 64)
    int32_t n;           // sampled elements per block
    int32_t padded;      // n rounded up to a power of two
    int32_t num_levels;
};

template <typename T>
__global__ __launch_bounds__(kProbeThreads) void grid_probe_kernel(const ProbeArgs a) {
    __shared__ unsigned int keys[kProbeKeys];
    __shared__ int exceeded;
    if (threadIdx.x == 0) exceeded = 0;
    const int P = a.padded, per_round = kProbeKeys / P;
    const T* __restrict__ x = static_cast<const T*>(a.x);
    for (int b0 = 0; b0 < a.nblocks; b0 += per_round) {
        const int nb = a.nblocks - b0 < per_round ? a.nblocks - b0 : per_round;
        const int total = nb * P;
        __syncthreads();
        // magnitudes as unsigned keys (their order is the order of the magnitudes; NaN above infinity); the padding
        // sorts behind every element
        for (int t = threadIdx.x; t < total; t += kProbeThreads) {
            const int seg = t / P, m = t - seg * P;
            unsigned int key = 0xffffffffu;
            if (m < a.n) {
                const int64_t i = m / a.K, k = m - i * a.K;
                key = f32_to_bits(load_f32(x[(i * a.J + (b0 + seg)) * a.K + k])) & 0x7fffffffu;
            }
            keys[t] = key;
        }
        __syncthreads();
        for (int k = 2; k <= P; k <<= 1) {
            for (int j = k >> 1; j >= 1; j >>= 1) {
                for (int t = threadIdx.x; t < total; t += kProbeThreads) {
                    const int u = t ^ j;
                    if (u > t) {
                        const bool up = ((t & (P - 1)) & k) == 0;  // every segment ends ascending
                        const unsigned int kt = keys[t], ku = keys[u];
                        if ((kt > ku) == up) {
                            keys[t] = ku;
                            keys[u] = kt;
                        }
                    }
                }
                __syncthreads();
            }
        }
        // distinct values of a segment = 1 + places where float neighbours differ; one wave per segment at a time
        const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
        for (int seg = wave; seg < nb; seg += kProbeThreads / kWave) {
            int differ = 0;
            for (int m = 1 + lane; m < a.n; m += kWave) {
                const float v0 = bits_to_f32(keys[seg * P + m - 1]), v1 = bits_to_f32(keys[seg * P + m]);
                differ += (v1 != v0) ? 1 : 0;
            }
#pragma unroll
            for (int s = kWave / 2; s >= 1; s >>= 1) differ += __shfl_xor(differ, s, kWave);
            if (lane == 0 && differ + 1 > a.num_levels) atomicOr(&exceeded, 1);
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) *a.verdict = exceeded ? 0 : 1;
}

}  // namespace ahq

using namespace ahq;

extern "C" int ahq_grid_probe(int32_t dtype, const ahq_layout* layout, const void* x, int64_t num_levels,
                              uint8_t* verdict, void* stream) {
    if (dtype < AHQ_F32 || dtype > AHQ_BF16) return set_error("bad dtype"), AHQ_ERR_INVALID;
    if (!layout || !x || !verdict) return set_error("null argument"), AHQ_ERR_INVALID;
    if (num_levels < 1) return set_error("num_levels must be positive"), AHQ_ERR_INVALID;
    CanonLayout c;
    const char* err = nullptr;
    if (!canonicalize(*layout, &c, &err)) return set_error(err), AHQ_ERR_INVALID;
    if (c.kind != kIJK) return set_error("blocks along several dimensions are not supported by the grid test"), AHQ_ERR_UNSUPPORTED;
    if (c.numel == 0) return set_error("empty tensor"), AHQ_ERR_INVALID;
    const int64_t block_elems = c.I * c.K;
    if (block_elems <= num_levels) return set_error("blocks no larger than the grid need no test"), AHQ_ERR_INVALID;
    const int64_t n = block_elems < 2 * num_levels ? block_elems : 2 * num_levels;
    int64_t padded = 1;
    while (padded < n) padded <<= 1;
    if (padded > kProbeKeys) return set_error("grid too wide for the on-device grid test"), AHQ_ERR_UNSUPPORTED;
    ProbeArgs a{};
    a.x = x;
    a.verdict = verdict;
    a.I = c.I;
    a.J = c.J;
    a.K = c.K;
    a.nblocks = (int32_t)(c.J < kProbeBlocks ? c.J : kProbeBlocks);
    a.n = (int32_t)n;
    a.padded = (int32_t)(padded < 2 ? 2 : padded);
    a.num_levels = (int32_t)(num_levels > 0x7fffffff ? 0x7fffffff : num_levels);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case AHQ_F32: hipLaunchKernelGGL((grid_probe_kernel<float>), dim3(1), dim3(kProbeThreads), 0, s, a); break;
        case AHQ_F16: hipLaunchKernelGGL((grid_probe_kernel<f16_t>), dim3(1), dim3(kProbeThreads), 0, s, a); break;
        default: hipLaunchKernelGGL((grid_probe_kernel<bf16_t>), dim3(1), dim3(kProbeThreads), 0, s, a); break;
    }
    return check_launch("grid_probe");
}

extern "C" int ahq_range_to_scale_offset(int32_t dtype, const void* range_min, const void* range_max,
                                         int64_t num_encodings, int64_t qmin, int64_t qmax, double minimum_scale,
                                         float* scale, float* offset, void* stream) {
    if (dtype < AHQ_F32 || dtype > AHQ_BF16) return set_error("bad dtype"), AHQ_ERR_INVALID;
    if (!range_min || !range_max || !scale) return set_error("null argument"), AHQ_ERR_INVALID;
    if (num_encodings < 0) return set_error("negative encoding count"), AHQ_ERR_INVALID;
    if (qmin >= qmax) return set_error("qmax must be larger than qmin"), AHQ_ERR_INVALID;
    if (num_encodings == 0) return AHQ_OK;
    ScaleOffArgs a{};
    a.pmin = range_min;
    a.pmax = range_max;
    a.scale = scale;
    a.offset = offset;
    a.n = num_encodings;
    // Python numbers reach torch's float32 kernels rounded once from double
    a.num_steps = (float)(double)(qmax - qmin);
    a.minimum_scale = (float)minimum_scale;
    a.qmin = (float)(double)qmin;
    a.lo = (float)(double)(-qmax);
    a.hi = (float)(double)(-qmin);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 g((unsigned)((num_encodings + 255) / 256)), b(256);
    switch (dtype) {
        case AHQ_F32: hipLaunchKernelGGL((range_to_scale_offset_kernel<float>), g, b, 0, s, a); break;
        case AHQ_F16: hipLaunchKernelGGL((range_to_scale_offset_kernel<f16_t>), g, b, 0, s, a); break;
        default: hipLaunchKernelGGL((range_to_scale_offset_kernel<bf16_t>), g, b, 0, s, a); break;
    }
    return check_launch("range_to_scale_offset");
}

extern "C" int ahq_lpbq_scale(int32_t dtype, const ahq_layout* grouping, const void* range_min, const void* range_max,
                              int64_t qmin, int64_t qmax, double minimum_scale, int32_t num_multipliers, float* scale,
                              float* per_channel_scale, void* stream) {
    if (dtype < AHQ_F32 || dtype > AHQ_BF16) return set_error("bad dtype"), AHQ_ERR_INVALID;
    if (!grouping || !range_min || !range_max || !scale || !per_channel_scale) return set_error("null argument"), AHQ_ERR_INVALID;
    if (qmin >= qmax) return set_error("qmax must be larger than qmin"), AHQ_ERR_INVALID;
    if (num_multipliers < 1 || num_multipliers > (1 << 24)) return set_error("num_multipliers must be in 1..2^24"), AHQ_ERR_INVALID;
    CanonLayout c;
    const char* err = nullptr;
    if (!canonicalize(*grouping, &c, &err)) return set_error(err), AHQ_ERR_INVALID;
    if (c.numel == 0) return AHQ_OK;
    if (c.kind != kIJK || c.I != 1)
        return set_error("groups whose blocks are not neighbours in memory are not supported by the fused LPBQ scale"), AHQ_ERR_UNSUPPORTED;
    LpbqArgs a{};
    a.pmin = range_min;
    a.pmax = range_max;
    a.scale = scale;
    a.per_channel = per_channel_scale;
    a.groups = c.J;
    a.group_size = c.K;
    a.num_steps = (float)(double)(qmax - qmin);
    a.minimum_scale = (float)minimum_scale;
    a.multipliers = (float)num_multipliers;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t per_block = kBlock / kWave;
    int64_t nb = (c.J + per_block - 1) / per_block;
    if (nb > 65536) nb = 65536;
    const dim3 g((unsigned)nb), b(kBlock);
    switch (dtype) {
        case AHQ_F32: hipLaunchKernelGGL((lpbq_scale_kernel<float>), g, b, 0, s, a); break;
        case AHQ_F16: hipLaunchKernelGGL((lpbq_scale_kernel<f16_t>), g, b, 0, s, a); break;
        default: hipLaunchKernelGGL((lpbq_scale_kernel<bf16_t>), g, b, 0, s, a); break;
    }
    return check_launch("lpbq_scale");
}

extern "C" int ahq_lpbq_scale_backward(int32_t dtype, const ahq_layout* grouping, const void* range_min,
                                       const void* range_max, int64_t qmin, int64_t qmax, double minimum_scale,
                                       int32_t num_multipliers, const float* grad_scale,
                                       const float* grad_per_channel_scale, void* grad_min, void* grad_max,
                                       void* stream) {
    if (dtype < AHQ_F32 || dtype > AHQ_BF16) return set_error("bad dtype"), AHQ_ERR_INVALID;
    if (!grouping || !range_min || !range_max || !grad_scale || !grad_min || !grad_max) return set_error("null argument"), AHQ_ERR_INVALID;
    if (qmin >= qmax) return set_error("qmax must be larger than qmin"), AHQ_ERR_INVALID;
    if (num_multipliers < 1 || num_multipliers > (1 << 24)) return set_error("num_multipliers must be in 1..2^24"), AHQ_ERR_INVALID;
    CanonLayout c;
    const char* err = nullptr;
    if (!canonicalize(*grouping, &c, &err)) return set_error(err), AHQ_ERR_INVALID;
    if (c.numel == 0) return AHQ_OK;
    if (c.kind != kIJK || c.I != 1)
        return set_error("groups whose blocks are not neighbours in memory are not supported by the fused LPBQ scale"), AHQ_ERR_UNSUPPORTED;
    LpbqGradArgs a{};
    a.pmin = range_min;
    a.pmax = range_max;
    a.gscale = grad_scale;
    a.gper_channel = grad_per_channel_scale;
    a.gmin = grad_min;
    a.gmax = grad_max;
    a.groups = c.J;
    a.group_size = c.K;
    a.num_steps = (float)(double)(qmax - qmin);
    a.minimum_scale = (float)minimum_scale;
    a.multipliers = (float)num_multipliers;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t per_block = kBlock / kWave;
    int64_t nb = (c.J + per_block - 1) / per_block;
    if (nb > 65536) nb = 65536;
    const dim3 g((unsigned)nb), b(kBlock);
    switch (dtype) {
        case AHQ_F32: hipLaunchKernelGGL((lpbq_scale_grad_kernel<float>), g, b, 0, s, a); break;
        case AHQ_F16: hipLaunchKernelGGL((lpbq_scale_grad_kernel<f16_t>), g, b, 0, s, a); break;
        default: hipLaunchKernelGGL((lpbq_scale_grad_kernel<bf16_t>), g, b, 0, s, a); break;
    }
    return check_launch("lpbq_scale_backward");
}

extern "C" int ahq_range_backward(int32_t dtype, const void* range_min, const void* range_max, int64_t num_encodings,
                                  int64_t qmin, int64_t qmax, double minimum_scale, const float* grad_scale,
                                  const float* grad_offset, void* grad_min, void* grad_max, void* stream) {
    if (dtype < AHQ_F32 || dtype > AHQ_BF16) return set_error("bad dtype"), AHQ_ERR_INVALID;
    if (!range_min || !range_max || !grad_scale || !grad_min || !grad_max) return set_error("null argument"), AHQ_ERR_INVALID;
    if (num_encodings < 0) return set_error("negative encoding count"), AHQ_ERR_INVALID;
    if (qmin >= qmax) return set_error("qmax must be larger than qmin"), AHQ_ERR_INVALID;
    if (num_encodings == 0) return AHQ_OK;
    RangeGradArgs a{};
    a.pmin = range_min;
    a.pmax = range_max;
    a.gscale = grad_scale;
    a.goffset = grad_offset;
    a.gmin = grad_min;
    a.gmax = grad_max;
    a.n = num_encodings;
    a.num_steps = (float)(double)(qmax - qmin);
    a.minimum_scale = (float)minimum_scale;
    a.qmin = (float)(double)qmin;
    a.lo = (float)(double)(-qmax);
    a.hi = (float)(double)(-qmin);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 g((unsigned)((num_encodings + 255) / 256)), b(256);
    switch (dtype) {
        case AHQ_F32: hipLaunchKernelGGL((range_grad_kernel<float>), g, b, 0, s, a); break;
        case AHQ_F16: hipLaunchKernelGGL((range_grad_kernel<f16_t>), g, b, 0, s, a); break;
        default: hipLaunchKernelGGL((range_grad_kernel<bf16_t>), g, b, 0, s, a); break;
    }
    return check_launch("range_backward");
}

static int fill_enc_args(EncArgs* a, int32_t dtype, const void* stat_min, const void* stat_max, int64_t num_encodings,
                         int64_t num_steps, int32_t symmetric, float minimum_scale_in_dtype, float minimum_scale,
                         float dtype_max, float near_max_threshold, int32_t* flags) {
    if (dtype < AHQ_F32 || dtype > AHQ_BF16) return set_error("bad dtype"), AHQ_ERR_INVALID;
    if (!stat_min || !stat_max) return set_error("null argument"), AHQ_ERR_INVALID;
    if (num_encodings < 0) return set_error("negative encoding count"), AHQ_ERR_INVALID;
    if (num_steps <= 0 || num_steps > (1ll << 24)) return set_error("num_steps must be in 1..2^24"), AHQ_ERR_INVALID;
    a->smin = stat_min;
    a->smax = stat_max;
    a->flags = flags;
    a->n = num_encodings;
    a->num_steps = (float)num_steps;
    a->tiny_t = minimum_scale_in_dtype;
    a->tiny_f = minimum_scale;
    a->pos = (float)(num_steps / 2);
    a->neg = (float)(num_steps - num_steps / 2);
    a->pos_extra = a->pos + (num_steps == 3 ? 1.f : 0.f);
    a->t_max = dtype_max;
    a->near_thr = near_max_threshold;
    a->symmetric = symmetric ? 1 : 0;
    return AHQ_OK;
}

extern "C" int ahq_minmax_to_encodings(int32_t dtype, const void* stat_min, const void* stat_max, int64_t num_encodings,
                                       int64_t num_steps, int32_t symmetric, float minimum_scale_in_dtype,
                                       float minimum_scale, float dtype_max, float near_max_threshold, void* out_min,
                                       void* out_max, int32_t* flags, void* stream) {
    EncArgs a{};
    const int rc = fill_enc_args(&a, dtype, stat_min, stat_max, num_encodings, num_steps, symmetric,
                                 minimum_scale_in_dtype, minimum_scale, dtype_max, near_max_threshold, flags);
    if (rc != AHQ_OK) return rc;
    if (!out_min || !out_max) return set_error("null argument"), AHQ_ERR_INVALID;
    if (num_encodings == 0) return AHQ_OK;
    a.out_min = out_min;
    a.out_max = out_max;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 g((unsigned)((num_encodings + 255) / 256)), b(256);
    switch (dtype) {
        case AHQ_F32: hipLaunchKernelGGL((minmax_to_encodings_kernel<float>), g, b, 0, s, a); break;
        case AHQ_F16: hipLaunchKernelGGL((minmax_to_encodings_kernel<f16_t>), g, b, 0, s, a); break;
        default: hipLaunchKernelGGL((minmax_to_encodings_kernel<bf16_t>), g, b, 0, s, a); break;
    }
    return check_launch("minmax_to_encodings");
}

template <typename T>
static void launch_finalize(int32_t param_dtype, const dim3& g, const dim3& b, hipStream_t s, const EncArgs& a,
                            const FinalArgs& f) {
    switch (param_dtype) {
        case AHQ_F32: hipLaunchKernelGGL((minmax_finalize_kernel<T, float>), g, b, 0, s, a, f); break;
        case AHQ_F16: hipLaunchKernelGGL((minmax_finalize_kernel<T, f16_t>), g, b, 0, s, a, f); break;
        default: hipLaunchKernelGGL((minmax_finalize_kernel<T, bf16_t>), g, b, 0, s, a, f); break;
    }
}

extern "C" int ahq_minmax_finalize(int32_t stat_dtype, const void* stat_min, const void* stat_max, int64_t num_encodings,
                                   int64_t num_steps, int32_t symmetric, float minimum_scale_in_dtype,
                                   float minimum_scale, float dtype_max, float near_max_threshold, int32_t* flags,
                                   int32_t param_dtype, void* param_min, void* param_max, int64_t qmin, int64_t qmax,
                                   double grid_minimum_scale, float* scale, float* offset, void* stream) {
    EncArgs a{};
    const int rc = fill_enc_args(&a, stat_dtype, stat_min, stat_max, num_encodings, num_steps, symmetric,
                                 minimum_scale_in_dtype, minimum_scale, dtype_max, near_max_threshold, flags);
    if (rc != AHQ_OK) return rc;
    if (param_dtype < AHQ_F32 || param_dtype > AHQ_BF16) return set_error("bad parameter dtype"), AHQ_ERR_INVALID;
    if (!param_min || !param_max || !scale) return set_error("null argument"), AHQ_ERR_INVALID;
    if (qmin >= qmax) return set_error("qmax must be larger than qmin"), AHQ_ERR_INVALID;
    if (num_encodings == 0) return AHQ_OK;
    FinalArgs f{};
    f.pmin = param_min;
    f.pmax = param_max;
    f.so.scale = scale;
    f.so.offset = offset;
    f.so.n = num_encodings;
    f.so.num_steps = (float)(double)(qmax - qmin);
    f.so.minimum_scale = (float)grid_minimum_scale;
    f.so.qmin = (float)(double)qmin;
    f.so.lo = (float)(double)(-qmax);
    f.so.hi = (float)(double)(-qmin);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 g((unsigned)((num_encodings + 255) / 256)), b(256);
    switch (stat_dtype) {
        case AHQ_F32: launch_finalize<float>(param_dtype, g, b, s, a, f); break;
        case AHQ_F16: launch_finalize<f16_t>(param_dtype, g, b, s, a, f); break;
        default: launch_finalize<bf16_t>(param_dtype, g, b, s, a, f); break;
    }
    return check_launch("minmax_finalize");
}

template <typename T>
static void launch_slots_finalize(int32_t param_dtype, hipStream_t s, const float* mn, const float* mx, const int* nan,
                                  const EncArgs& a, const FinalArgs& f) {
    const dim3 g(1), b(kSlotThreads);
    switch (param_dtype) {
        case AHQ_F32: hipLaunchKernelGGL((minmax_slots_finalize_kernel<T, float>), g, b, 0, s, mn, mx, nan, a, f); break;
        case AHQ_F16: hipLaunchKernelGGL((minmax_slots_finalize_kernel<T, f16_t>), g, b, 0, s, mn, mx, nan, a, f); break;
        default: hipLaunchKernelGGL((minmax_slots_finalize_kernel<T, bf16_t>), g, b, 0, s, mn, mx, nan, a, f); break;
    }
}

extern "C" int ahq_minmax_slots_finalize(int32_t stat_dtype, const void* slots, int64_t num_steps, int32_t symmetric,
                                         float minimum_scale_in_dtype, float minimum_scale, float dtype_max,
                                         float near_max_threshold, int32_t* flags, int32_t param_dtype, void* param_min,
                                         void* param_max, int64_t qmin, int64_t qmax, double grid_minimum_scale,
                                         float* scale, float* offset, void* stream) {
    if (!slots || (reinterpret_cast<uintptr_t>(slots) & 3u)) return set_error("slots is null or misaligned"), AHQ_ERR_INVALID;
    EncArgs a{};
    const int rc = fill_enc_args(&a, stat_dtype, slots, slots, 1, num_steps, symmetric, minimum_scale_in_dtype,
                                 minimum_scale, dtype_max, near_max_threshold, flags);
    if (rc != AHQ_OK) return rc;
    if (param_dtype < AHQ_F32 || param_dtype > AHQ_BF16) return set_error("bad parameter dtype"), AHQ_ERR_INVALID;
    if (!param_min || !param_max || !scale) return set_error("null argument"), AHQ_ERR_INVALID;
    if (qmin >= qmax) return set_error("qmax must be larger than qmin"), AHQ_ERR_INVALID;
    a.smin = a.smax = nullptr;  // the statistics come from the slots
    FinalArgs f{};
    f.pmin = param_min;
    f.pmax = param_max;
    f.so.scale = scale;
    f.so.offset = offset;
    f.so.n = 1;
    f.so.num_steps = (float)(double)(qmax - qmin);
    f.so.minimum_scale = (float)grid_minimum_scale;
    f.so.qmin = (float)(double)qmin;
    f.so.lo = (float)(double)(-qmax);
    f.so.hi = (float)(double)(-qmin);
    const char* w = static_cast<const char*>(slots);
    const float* mn = reinterpret_cast<const float*>(w);
    const float* mx = reinterpret_cast<const float*>(w + 4 * AHQ_MINMAX_SLOTS);
    const int* nan = reinterpret_cast<const int*>(w + 8 * AHQ_MINMAX_SLOTS);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (stat_dtype) {
        case AHQ_F32: launch_slots_finalize<float>(param_dtype, s, mn, mx, nan, a, f); break;
        case AHQ_F16: launch_slots_finalize<f16_t>(param_dtype, s, mn, mx, nan, a, f); break;
        default: launch_slots_finalize<bf16_t>(param_dtype, s, mn, mx, nan, a, f); break;
    }
    return check_launch("minmax_slots_finalize");
}

extern "C" int ahq_minmax_slots_to_encodings(int32_t dtype, const void* slots, int64_t num_steps, int32_t symmetric,
                                             float minimum_scale_in_dtype, float minimum_scale, float dtype_max,
                                             float near_max_threshold, void* out_min, void* out_max, void* stat_min,
                                             void* stat_max, int32_t* flags, void* stream) {
    if (!slots || (reinterpret_cast<uintptr_t>(slots) & 3u)) return set_error("slots is null or misaligned"), AHQ_ERR_INVALID;
    EncArgs a{};
    const int rc = fill_enc_args(&a, dtype, slots, slots, 1, num_steps, symmetric, minimum_scale_in_dtype, minimum_scale,
                                 dtype_max, near_max_threshold, flags);
    if (rc != AHQ_OK) return rc;
    if (!out_min || !out_max) return set_error("null argument"), AHQ_ERR_INVALID;
    a.smin = a.smax = nullptr;  // the statistics come from the slots
    a.out_min = out_min;
    a.out_max = out_max;
    const char* w = static_cast<const char*>(slots);
    const float* mn = reinterpret_cast<const float*>(w);
    const float* mx = reinterpret_cast<const float*>(w + 4 * AHQ_MINMAX_SLOTS);
    const int* nan = reinterpret_cast<const int*>(w + 8 * AHQ_MINMAX_SLOTS);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 g(1), b(kSlotThreads);
    switch (dtype) {
        case AHQ_F32: hipLaunchKernelGGL((minmax_slots_to_encodings_kernel<float>), g, b, 0, s, mn, mx, nan, a, static_cast<float*>(stat_min), static_cast<float*>(stat_max)); break;
        case AHQ_F16: hipLaunchKernelGGL((minmax_slots_to_encodings_kernel<f16_t>), g, b, 0, s, mn, mx, nan, a, static_cast<f16_t*>(stat_min), static_cast<f16_t*>(stat_max)); break;
        default: hipLaunchKernelGGL((minmax_slots_to_encodings_kernel<bf16_t>), g, b, 0, s, mn, mx, nan, a, static_cast<bf16_t*>(stat_min), static_cast<bf16_t*>(stat_max)); break;
    }
    return check_launch("minmax_slots_to_encodings");
}

extern "C" int ahq_minmax_slots_finalize_many(const ahq_slots_finalize_item* items, int64_t count, int32_t* flags,
                                              void* stream) {
    if (count < 0 || (count > 0 && !items)) return set_error("null argument"), AHQ_ERR_INVALID;
    if (count == 0) return AHQ_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    for (int64_t base = 0; base < count; base += kManySlots) {
        const int n = (int)(count - base < kManySlots ? count - base : kManySlots);
        ManySlotArgs m{};
        for (int k = 0; k < n; ++k) {
            const ahq_slots_finalize_item& it = items[base + k];
            ManySlotItem& d = m.items[k];
            auto fail = [&](const char* what) {
                std::snprintf(error_buffer(), 512, "item %lld: %s", (long long)(base + k), what);
                return AHQ_ERR_INVALID;
            };
            if (!it.slots || (reinterpret_cast<uintptr_t>(it.slots) & 3u)) return fail("slots is null or misaligned");
            const int rc = fill_enc_args(&d.a, it.stat_dtype, it.slots, it.slots, 1, it.num_steps, it.symmetric,
                                         it.minimum_scale_in_dtype, it.minimum_scale, it.dtype_max,
                                         it.near_max_threshold, flags);
            if (rc != AHQ_OK) return fail(error_buffer());
            if (it.param_dtype < AHQ_F32 || it.param_dtype > AHQ_BF16) return fail("bad parameter dtype");
            if (!it.param_min || !it.param_max || !it.scale) return fail("null argument");
            if (it.qmin >= it.qmax) return fail("qmax must be larger than qmin");
            d.a.smin = d.a.smax = nullptr;
            d.f.pmin = it.param_min;
            d.f.pmax = it.param_max;
            d.f.so.scale = it.scale;
            d.f.so.offset = it.offset;
            d.f.so.n = 1;
            d.f.so.num_steps = (float)(double)(it.qmax - it.qmin);
            d.f.so.minimum_scale = (float)it.grid_minimum_scale;
            d.f.so.qmin = (float)(double)it.qmin;
            d.f.so.lo = (float)(double)(-it.qmax);
            d.f.so.hi = (float)(double)(-it.qmin);
            const char* w = static_cast<const char*>(it.slots);
            d.slot_min = reinterpret_cast<const float*>(w);
            d.slot_max = reinterpret_cast<const float*>(w + 4 * AHQ_MINMAX_SLOTS);
            d.slot_nan = reinterpret_cast<const int*>(w + 8 * AHQ_MINMAX_SLOTS);
            d.stat_dtype = it.stat_dtype;
            d.param_dtype = it.param_dtype;
        }
        hipLaunchKernelGGL(minmax_slots_finalize_many_kernel, dim3((unsigned)n), dim3(kSlotThreads), 0, s, m);
    }
    return check_launch("minmax_slots_finalize_many");
}
