// Min/max statistics -> encoding range, one thread per encoding.
//
// Replaces the dozen elementwise torch launches of MinMaxEncodingAnalyzer.compute_encodings_from_stats
// (aimet_torch/quantization/encoding_analyzer.py:425-481) and the range checks of _flag_extreme_min_max (:484-498)
// with one launch.  A whole-model calibration ends hundreds of quantizer contexts, each on a handful of values, so the
// launches -- not the arithmetic -- are the cost.  Every operation keeps the dtype torch's type promotion gives it:
// statistics arithmetic in the statistics dtype T (rounded after each operation), everything after the float32
// "widen" term in float32, the result rounded to T once.

#include "ahq_device.h"
#include "ahq_host.h"

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

template <typename T>
__global__ void minmax_to_encodings_kernel(const EncArgs a) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= a.n) return;
    using R = RoundTo<T>;
    const float mn = load_f32(static_cast<const T*>(a.smin)[i]);
    const float mx = load_f32(static_cast<const T*>(a.smax)[i]);
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
    const T lo_t = store_cast<T>(lo), hi_t = store_cast<T>(hi);
    static_cast<T*>(a.out_min)[i] = lo_t;
    static_cast<T*>(a.out_max)[i] = hi_t;
    if (a.flags) {
        const float l = load_f32(lo_t), h = load_f32(hi_t);
        const bool nonfinite = !(__builtin_fabsf(l) < __builtin_inff()) || !(__builtin_fabsf(h) < __builtin_inff());
        const bool near = __builtin_fabsf(R::f(__builtin_fabsf(l) - a.t_max)) <= a.near_thr ||
                          __builtin_fabsf(R::f(__builtin_fabsf(h) - a.t_max)) <= a.near_thr;
        if (nonfinite) atomicOr(&a.flags[0], 1);
        if (near) atomicOr(&a.flags[1], 1);
    }
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

}  // namespace ahq

using namespace ahq;

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

extern "C" int ahq_minmax_to_encodings(int32_t dtype, const void* stat_min, const void* stat_max, int64_t num_encodings,
                                       int64_t num_steps, int32_t symmetric, float minimum_scale_in_dtype,
                                       float minimum_scale, float dtype_max, float near_max_threshold, void* out_min,
                                       void* out_max, int32_t* flags, void* stream) {
    if (dtype < AHQ_F32 || dtype > AHQ_BF16) return set_error("bad dtype"), AHQ_ERR_INVALID;
    if (!stat_min || !stat_max || !out_min || !out_max) return set_error("null argument"), AHQ_ERR_INVALID;
    if (num_encodings < 0) return set_error("negative encoding count"), AHQ_ERR_INVALID;
    if (num_steps <= 0 || num_steps > (1ll << 24)) return set_error("num_steps must be in 1..2^24"), AHQ_ERR_INVALID;
    if (num_encodings == 0) return AHQ_OK;
    EncArgs a{};
    a.smin = stat_min;
    a.smax = stat_max;
    a.out_min = out_min;
    a.out_max = out_max;
    a.flags = flags;
    a.n = num_encodings;
    a.num_steps = (float)num_steps;
    a.tiny_t = minimum_scale_in_dtype;
    a.tiny_f = minimum_scale;
    a.pos = (float)(num_steps / 2);
    a.neg = (float)(num_steps - num_steps / 2);
    a.pos_extra = a.pos + (num_steps == 3 ? 1.f : 0.f);
    a.t_max = dtype_max;
    a.near_thr = near_max_threshold;
    a.symmetric = symmetric ? 1 : 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 g((unsigned)((num_encodings + 255) / 256)), b(256);
    switch (dtype) {
        case AHQ_F32: hipLaunchKernelGGL((minmax_to_encodings_kernel<float>), g, b, 0, s, a); break;
        case AHQ_F16: hipLaunchKernelGGL((minmax_to_encodings_kernel<f16_t>), g, b, 0, s, a); break;
        default: hipLaunchKernelGGL((minmax_to_encodings_kernel<bf16_t>), g, b, 0, s, a); break;
    }
    return check_launch("minmax_to_encodings");
}
