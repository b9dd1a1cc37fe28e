// Fake-quantization kernels: quantize-dequantize / quantize / dequantize forward and straight-through backward.
//
// One streaming pass per tensor: every element is read once and written once (forward: x -> y [+ 1-byte mask];
// backward: g, x -> gx [+ per-encoding scale/offset gradients]).  Threads move 16-byte vectors; a workgroup owns a
// tile of kTileVec vectors and first stages the encodings its tile touches in LDS, so per-channel and blockwise scales
// are fetched from memory once per tile with one coalesced load.
//
// Arithmetic reproduced (see include/aimet_amd.h for the reference locations):
//   AHQ_ARITH_ATEN      reciprocal multiply, round-half-even, clamp on the code          (fp32 math)
//   AHQ_ARITH_AUTOGRAD  true division, round-half-even, every intermediate rounded to the compute dtype
//   AHQ_ARITH_DLQ       clamp on the value, true division, round-half-away-from-zero     (fp32 math)
// Built with -ffp-contract=off: fusing a multiply into an add would change the rounding of any of them.

#include <cstdio>

#include "ahq_device.h"
#include "ahq_host.h"
#include "layout.h"
#include "tiling.h"

namespace ahq {

constexpr int kStage = kTileVec + 2;  // most encodings a tile can touch
// Vectors per thread and tile in the forward kernels.  One input stream runs fastest with two 16-byte loads per lane
// in flight (four cost about 5 %); the backward kernels, with two input streams, keep kUnroll = 4.
constexpr int kFwdUnroll = 2;

struct GridC {
    float qmin, qmax, zps;
    int flags;  // float fake-cast only: kCastOverflowNaN | kCastUnsignedZero
};
constexpr int kCastOverflowNaN = 1;    // a value that rounds past the largest one becomes NaN (else infinity)
constexpr int kCastUnsignedZero = 2;   // the format has no negative zero
constexpr int kCastLogForm = 4;        // 16-bit tensors: the reference's logarithm formula, rounded step by step
constexpr int kCastKeepScaled = 8;     // stop before the multiplication by the scale (quantize only)
constexpr int kCastRescaleOnly = 16;   // only the multiplication by the scale (dequantize)

struct EncP {
    float p0, p1, p2, p3;
    float rs;  // 1 / scale correctly rounded, or 0 when the division-free path must not be used for this encoding
};

// x / s, correctly rounded.  FAST: two residual corrections of x * (1/s) with fused multiply-adds.  With rs = RN(1/s)
// the first correction leaves a quotient that is off by at most a few 2^-47 relative, and the second is then the
// correctly rounded one (Markstein's division theorem); the residuals are exact as long as nothing under- or
// overflows, which the callers guarantee by taking this path only for |x| <= 2^60 and 2^-60 <= |s| <= 2^60 (a
// quotient below 2^-120 cannot arise there, and one too small to matter rounds to code 0 either way).  Five
// instructions instead of the thirteen of the general IEEE sequence, whose divisor scaling, reciprocal refinement and
// fix-up are work per element that does not depend on the element.
//
// CD = the dtype the caller rounds the quotient to next.  For the 16-bit dtypes one correction is enough: x and s then
// have p <= 11 significant bits, so an exact quotient that is not itself a rounding tie of that dtype lies at least
// 2^-(2p+1) >= 2^-23 (relative) away from every tie, while the once-corrected quotient is exact whenever the true
// quotient is a float (every tie is) and within 2^-24 otherwise: both round to the same 16-bit value.
template <bool FAST, int CD>
__device__ __forceinline__ float divide(float x, float s, float rs) {
    if (!FAST) return x / s;
    const float q0 = x * rs;
    const float r0 = __builtin_fmaf(-q0, s, x);
    const float q1 = __builtin_fmaf(r0, rs, q0);
    if (CD != AHQ_F32) return q1;
    const float r1 = __builtin_fmaf(-q1, s, x);
    return __builtin_fmaf(r1, rs, q1);
}

constexpr float kFastDivMax = 1.152921504606846976e18f;     // 2^60
constexpr float kFastDivMin = 8.673617379884035472e-19f;    // 2^-60

__device__ __forceinline__ float safe_reciprocal(float s) {
    const float m = __builtin_fabsf(s);
    return (m >= kFastDivMin && m <= kFastDivMax) ? 1.0f / s : 0.f;
}

// --------------------------------------------------------------------------------------------------- arithmetic --
// Each Math type: kNP staged floats per encoding; prep() turns (scale, offset, min, max) into them; fwd() returns the
// output value (already rounded to the compute dtype) and whether the code was in range; bwd() returns the three
// per-element gradient terms.

// Largest integer magnitude n such that every integer up to n + 1 is a value of the compute dtype.
template <int CD> struct ExactInt { static constexpr float kMax = 16777215.f; };
template <> struct ExactInt<AHQ_F16> { static constexpr float kMax = 2047.f; };
template <> struct ExactInt<AHQ_BF16> { static constexpr float kMax = 255.f; };

// The FAST form (no zero-point shift) needs more than a divisible scale: an integer offset, and grid bounds, offset
// and shifted bounds lo = offset + qmin, hi = offset + qmax small enough that every integer the reference's
// intermediate steps can produce near the grid is exact in the compute dtype.  Then
//   r = rnd(rint(t) - offset) is in [qmin, qmax]  <=>  lo <= rint(t) <= hi        (integers, roundings monotone and
//                                                                                   exact up to one past the bounds)
//   rnd(clamp(r) + offset) = clamp(rint(t), lo, hi)
// so the subtraction, the addition and two of the roundings drop out, and the clamp is one median-of-three.  The
// median does not propagate NaN: tiles holding a NaN take the general form (lane_can_divide_fast).  Encodings that do
// not qualify get rs = 0, which sends their tile to the general form too.
template <int CD, bool ZPS>
struct MathAutogradQdq {
    static constexpr int kNP = 2;
    static constexpr int kCD = CD;
    static constexpr bool kDiv = true;
    static constexpr bool kHasBwd = true;
    __device__ static EncP prep(float s, float off, float, float, const GridC& g) {
        const float sr = rnd<CD>(s), offr = rnd<CD>(off);
        float rs = safe_reciprocal(sr);
        if (!ZPS) {
            constexpr float K = ExactInt<CD>::kMax;
            const float lo = offr + g.qmin, hi = offr + g.qmax;
            const bool small = (offr == __builtin_rintf(offr)) & (__builtin_fabsf(offr) <= K) &
                               (__builtin_fabsf(g.qmin) <= K) & (__builtin_fabsf(g.qmax) <= K) &
                               (__builtin_fabsf(lo) <= K) & (__builtin_fabsf(hi) <= K);
            if (!small) rs = 0.f;
        }
        return {sr, offr, 0.f, 0.f, rs};
    }
    // Returns the output before its last rounding to the compute dtype (the caller rounds while storing).
    template <bool FAST>
    __device__ static float fwd(float x, const EncP& e, const GridC& g, bool& inr) {
        float t = rnd<CD>(divide<FAST, CD>(x, e.p0, e.rs));
        if (FAST && !ZPS) {
            const float xr = __builtin_rintf(t);
            const float m = __builtin_amdgcn_fmed3f(xr, e.p1 + g.qmin, e.p1 + g.qmax);
            inr = (m == xr);
            // the reference's (q + offset) is never a negative zero: adding +0 to the exact product turns -0 * scale
            // into +0 and changes nothing else
            return __builtin_fmaf(m, e.p0, 0.f);
        }
        if (ZPS) t = rnd<CD>(t - g.zps);
        const float r = rnd<CD>(__builtin_rintf(t) - e.p1);
        inr = (r >= g.qmin) & (r <= g.qmax);
        const float q = r < g.qmin ? g.qmin : (r > g.qmax ? g.qmax : r);
        const float offp = ZPS ? rnd<CD>(e.p1 + g.zps) : e.p1;
        return rnd<CD>(q + offp) * e.p0;
    }
    // The FAST backward in two steps, so that a caller can look at a whole vector's in-range flags before it spends
    // work on the out-of-range terms (calibrated data is almost always inside the grid): pre() gives the rounded
    // quotient t, rint(t) and its clamp; an element is in range when the clamp left rint(t) alone.
    static constexpr bool kSplitBwd = !ZPS;
    __device__ static void bwd_pre(float x, const EncP& e, float lo, float hi, float& t, float& xr, float& m) {
        t = rnd<CD>(divide<true, CD>(x, e.p0, e.rs));
        xr = __builtin_rintf(t);
        m = __builtin_amdgcn_fmed3f(xr, lo, hi);
    }
    __device__ static float bwd_gs_in(float gr, float t, float xr) { return rnd<CD>(gr * (xr - t)); }
    __device__ static float bwd_gs_out(float gr, float m) { return rnd<CD>(gr * m); }
    __device__ static float bwd_goff_out(float gr, const EncP& e) { return rnd<CD>(gr * e.p0); }

    template <bool FAST>
    __device__ static void bwd(float gr, float x, const EncP& e, const GridC& g, float& gx, float& gs, float& goff) {
        float t = rnd<CD>(divide<FAST, CD>(x, e.p0, e.rs));
        if (FAST && !ZPS) {
            const float xr = __builtin_rintf(t);
            const float m = __builtin_amdgcn_fmed3f(xr, e.p1 + g.qmin, e.p1 + g.qmax);
            const bool in = (m == xr);
            // rint(t) - t is a multiple of ulp(t) no larger than 1/2: exact in the compute dtype, no rounding needed
            gx = in ? gr : 0.f;
            gs = rnd<CD>(gr * (in ? xr - t : m));
            goff = in ? 0.f : rnd<CD>(gr * e.p0);
            return;
        }
        if (ZPS) t = rnd<CD>(t - g.zps);
        const float xr = __builtin_rintf(t);
        const float err = rnd<CD>(xr - t);
        const float r = rnd<CD>(xr - e.p1);
        const bool inr = (r >= g.qmin) & (r <= g.qmax);
        const float lo = rnd<CD>(e.p1 + g.qmin), hi = rnd<CD>(e.p1 + g.qmax);
        float xc = xr < lo ? lo : (xr > hi ? hi : xr);
        if (ZPS) xc = rnd<CD>(xc + g.zps);
        gx = inr ? gr : 0.f;
        gs = rnd<CD>(gr * (inr ? err : xc));
        goff = inr ? 0.f : rnd<CD>(gr * e.p0);
    }
};

template <int CD>
struct MathAutogradQuantize {
    static constexpr bool kSplitBwd = false;
    static constexpr int kNP = 2;
    static constexpr int kCD = AHQ_F32;  // its outputs are already values of CD
    static constexpr bool kDiv = true;
    static constexpr bool kHasBwd = true;
    __device__ static EncP prep(float s, float off, float, float, const GridC&) {
        const float sr = rnd<CD>(s);
        return {sr, rnd<CD>(off), 0.f, 0.f, safe_reciprocal(sr)};
    }
    template <bool FAST>
    __device__ static float fwd(float x, const EncP& e, const GridC& g, bool& inr) {
        float t = divide<FAST, CD>(x, e.p0, e.rs);
        // the division-free quotient of a zero comes out as +0; with a zero offset the code of -0 is -0 in the reference
        if (FAST && t == 0.f) t = bits_to_f32((f32_to_bits(x) ^ f32_to_bits(e.p0)) & 0x80000000u);
        const float r = rnd<CD>(__builtin_rintf(rnd<CD>(t)) - e.p1);
        inr = (r >= g.qmin) & (r <= g.qmax);
        return r < g.qmin ? g.qmin : (r > g.qmax ? g.qmax : r);
    }
    template <bool FAST>
    __device__ static void bwd(float gr, float x, const EncP& e, const GridC& g, float& gx, float& gs, float& goff) {
        const float xs = rnd<CD>(divide<FAST, CD>(x, e.p0, e.rs));
        const float r = rnd<CD>(__builtin_rintf(xs) - e.p1);
        const bool inr = (r >= g.qmin) & (r <= g.qmax);
        const float mg = rnd<CD>(gr * (inr ? 1.f : 0.f));
        gx = rnd<CD>(mg / e.p0);  // the gradient's magnitude is not bounded like x: general division
        gs = rnd<CD>((-gx) * xs);
        goff = -mg;
    }
};

template <int CD>
struct MathAutogradDequantize {
    static constexpr bool kSplitBwd = false;
    static constexpr int kNP = 2;
    static constexpr int kCD = CD;
    static constexpr bool kDiv = false;
    static constexpr bool kHasBwd = true;
    __device__ static EncP prep(float s, float off, float, float, const GridC&) { return {rnd<CD>(s), rnd<CD>(off), 0.f, 0.f, 0.f}; }
    template <bool FAST>
    __device__ static float fwd(float x, const EncP& e, const GridC&, bool& inr) {
        inr = true;
        return rnd<CD>(x + e.p1) * e.p0;  // last rounding by the caller
    }
    template <bool FAST>
    __device__ static void bwd(float gr, float x, const EncP& e, const GridC&, float& gx, float& gs, float& goff) {
        gx = rnd<CD>(gr * e.p0);
        gs = rnd<CD>(gr * rnd<CD>(x + e.p1));
        goff = gx;
    }
};

struct MathAten {
    static constexpr bool kSplitBwd = false;
    static constexpr int kCD = AHQ_F32;
    static constexpr int kNP = 3;
    static constexpr bool kDiv = false;
    static constexpr bool kHasBwd = true;
    // p0 = scale, p1 = zero point as float, p2 = 1.0f/scale
    __device__ static EncP prep(float s, float off, float, float, const GridC&) { return {s, (float)(-(int)off), 1.0f / s, 0.f, 0.f}; }
    template <bool FAST>
    __device__ static float fwd(float x, const EncP& e, const GridC& g, bool& inr) {
        const float q = __builtin_rintf(x * e.p2) + e.p1;
        inr = (q >= g.qmin) & (q <= g.qmax);
        const float qc = fminf(fmaxf(q, g.qmin), g.qmax);
        return (qc - e.p1) * e.p0;
    }
    template <bool FAST>
    __device__ static void bwd(float gr, float x, const EncP& e, const GridC& g, float& gx, float& gs, float& goff) {
        const float q = __builtin_rintf(x * e.p2) + e.p1;
        const bool inr = (q >= g.qmin) & (q <= g.qmax);
        gx = gr * (inr ? 1.f : 0.f);
        gs = 0.f;
        goff = 0.f;
    }
};

struct MathDlq {
    static constexpr bool kSplitBwd = false;
    static constexpr int kCD = AHQ_F32;
    static constexpr int kNP = 4;
    static constexpr bool kDiv = true;
    static constexpr bool kHasBwd = false;
    // p0 = delta, p1 = offset, p2 = min, p3 = max.  The value is clamped to [min, max] before it is divided, so the
    // division-free path only needs the encoding itself to be in range.
    __device__ static EncP prep(float s, float off, float mn, float mx, const GridC&) {
        const bool bounded = __builtin_fabsf(mn) <= kFastDivMax && __builtin_fabsf(mx) <= kFastDivMax;
        return {s, off, mn, mx, bounded ? safe_reciprocal(s) : 0.f};
    }
    template <bool FAST>
    __device__ static float fwd(float x, const EncP& e, const GridC&, bool& inr) {
        inr = true;
        float v = (x != x) ? e.p2 : x;
        v = fmaxf(fminf(v, e.p3), e.p2);
        v = divide<FAST, AHQ_F32>(v, e.p0, e.rs) - e.p1;
        v = roundf(v);
        return e.p0 * (v + e.p1);
    }
    template <bool FAST>
    __device__ static void bwd(float, float, const EncP&, const GridC&, float& gx, float& gs, float& goff) { gx = gs = goff = 0.f; }
};

// DlQuantization FP8 fake-cast (fakeCastToFp8 / quantizeDequantizeFp8Cpu, DLQ/src/trim_functions.cpp:49-67, 243-258):
// v = clamp(x / scale, -max, max); e = max(frexp exponent of v - 1, exponent_min); step = 2^(e - mantissa bits);
// y = rint(v / step) * step * scale.  The grid constants travel in GridC: qmin = exponent_min, qmax = max value,
// zps = mantissa bits.  Dividing by a power of two is exact, so it is done by scaling the exponent.
struct MathDlqFp8 {
    static constexpr bool kSplitBwd = false;
    static constexpr int kCD = AHQ_F32;
    static constexpr int kNP = 2;
    static constexpr bool kDiv = true;
    static constexpr bool kHasBwd = false;
    __device__ static EncP prep(float s, float, float, float, const GridC&) { return {s, 0.f, 0.f, 0.f, safe_reciprocal(s)}; }
    template <bool FAST>
    __device__ static float fwd(float x, const EncP& e, const GridC& g, bool& inr) {
        inr = true;
        float v = divide<FAST, AHQ_F32>(x, e.p0, e.rs);
        v = (v < -g.qmax) ? -g.qmax : (g.qmax < v) ? g.qmax : v;  // std::clamp: NaN passes through
        int ex = __builtin_amdgcn_frexp_expf(v);                   // v = m * 2^ex, |m| in [0.5, 1); 0 for v == 0
        ex = ex - 1 < (int)g.qmin ? (int)g.qmin : ex - 1;
        const int sh = ex - (int)g.zps;
        const float y = __builtin_ldexpf(__builtin_rintf(__builtin_ldexpf(v, -sh)), sh) * e.p0;
        // a zero result carries the sign of x in the reference (quotient, rounding and product all keep it); the
        // corrected quotient of divide<true> does not keep the sign of a zero
        return y == 0.f ? __builtin_copysignf(0.f, x) : y;
    }
    template <bool FAST>
    __device__ static void bwd(float, float, const EncP&, const GridC&, float& gx, float& gs, float& goff) { gx = gs = goff = 0.f; }
};

// aimet_torch's float fake-cast (quantization/float/quantizer.py:634-716): in the arithmetic dtype CD of the call,
//   t = x / scale;  t = clamp(t, -max, max);  v = t rounded to the simulated format and brought back to CD;
//   y = v * scale.
// The simulated format is given by its mantissa bits, the exponent of its smallest normal binade and its largest
// value (GridC: zps, qmin, qmax); rounding is to nearest even on that grid, exactly what a conversion to a storage
// type of that layout does and what the reference's logarithm-based formula evaluates to
// (fp_quantization.py:148-214).  The clamp bound is the largest value as CD holds it, like the Python scalar the
// reference hands to torch.clamp; where that rounds upward (65504 in bfloat16) a clamped value can round past the
// format's largest value and overflows like the conversion would.
template <int CD>
struct MathFloatCast {
    static constexpr bool kSplitBwd = false;
    static constexpr int kCD = CD;
    static constexpr int kNP = 2;
    static constexpr bool kDiv = true;
    static constexpr bool kHasBwd = false;
    // The scale stays a float whatever CD is: a float32 scale with one element per tensor is an operand torch keeps
    // at full precision next to a 16-bit tensor (and any larger float32 scale widens the whole computation), so the
    // quotient is the correctly rounded float one, rounded once more to CD.
    __device__ static EncP prep(float s, float, float, float, const GridC&) { return {s, 0.f, 0.f, 0.f, safe_reciprocal(s)}; }
    template <bool FAST>
    __device__ static float fwd(float x, const EncP& e, const GridC& g, bool& inr) {
        inr = true;
        if (g.flags & kCastRescaleOnly) return x * e.p0;  // last rounding by the caller
        const float back = (g.flags & kCastKeepScaled) ? 1.f : e.p0;
        float t = rnd<CD>(divide<FAST, AHQ_F32>(x, e.p0, e.rs));
        // the corrected quotient of divide<true> does not keep the sign of a zero
        if (FAST && t == 0.f) t = bits_to_f32((f32_to_bits(x) ^ f32_to_bits(e.p0)) & 0x80000000u);
        const float mx = rnd<CD>(g.qmax);
        t = (t < -mx) ? -mx : (mx < t) ? mx : t;
        if constexpr (CD != AHQ_F32) {
            if (g.flags & kCastLogForm) {
                // fake_cast_to_ieee_float (aimet_torch/fp_quantization.py:177-201) on a 16-bit tensor, every torch
                // operation with its own rounding to that dtype:
                //   log_scales = clamp(floor(log2|x| + bias), 1);  scales = 2 ** (log_scales - mantissa_bits - bias)
                //   out = round(x / scales) * scales
                // Near the top of a binade the rounded logarithm reaches the next integer, so such values land on the
                // next binade's coarser grid, and a clamp bound that rounds upward in the tensor's dtype is returned
                // as it is: this is what the reference computes, and it is reproduced rather than corrected.
                const float bias = rnd<CD>(1.f - g.qmin);
                float ls = __builtin_floorf(rnd<CD>(rnd<CD>(__builtin_log2f(__builtin_fabsf(t))) + bias));
                ls = (ls != ls) ? ls : fmaxf(ls, 1.f);
                const float ex2 = rnd<CD>(rnd<CD>(ls - g.zps) - bias);
                const float sc = rnd<CD>(__builtin_exp2f(ex2));
                const float q = rnd<CD>(t / sc);
                return rnd<CD>(__builtin_rintf(q) * sc) * back;  // last rounding by the caller
            }
        }
        int ex = __builtin_amdgcn_frexp_expf(t) - 1;
        ex = ex < (int)g.qmin ? (int)g.qmin : ex;
        const int sh = ex - (int)g.zps;
        float v = __builtin_ldexpf(__builtin_rintf(__builtin_ldexpf(t, -sh)), sh);
        if (__builtin_fabsf(v) > g.qmax)
            v = (g.flags & kCastOverflowNaN) ? __builtin_nanf("") : __builtin_copysignf(__builtin_inff(), v);
        if ((g.flags & kCastUnsignedZero) && v == 0.f) v = 0.f;
        return rnd<CD>(v) * back;  // last rounding by the caller
    }
    template <bool FAST>
    __device__ static void bwd(float, float, const EncP&, const GridC&, float& gx, float& gs, float& goff) {
        gx = gs = goff = 0.f;
    }
};

// ------------------------------------------------------------------------------------------------ kernel arguments --
struct QdqArgs : Geom {
    const void* x;
    void* y;
    uint8_t* mask;
    const void* g;
    void* gx;
    const float* scale;
    const float* offset;
    const float* emin;
    const float* emax;
    float* gscale;
    float* goffset;
    double* partials;  // kRedTile: [nblocks][2]; kRedAtomic: [num_enc][2]
    GridC gc;
    int32_t red;
    int32_t out_cd;  // compute dtype the reduced gradients are rounded through
    // one encoding handed over by value (scale, offset, min, max) instead of through the four pointers: what the
    // per-tensor entry points use, so that their callers need no device copy of the encoding
    int32_t by_value;
    float value_enc[4];
};

template <typename M>
__device__ __forceinline__ void stage_encodings(const QdqArgs& a, const Tile& t, float (*sp)[kStage]) {
    for (int i = threadIdx.x; i < t.nstage; i += kBlock) {
        int64_t e = t.e0 + i;
        if (e >= a.J) e %= a.J;
        const float s = a.by_value ? a.value_enc[0] : a.scale[e];
        const float off = a.by_value ? a.value_enc[1] : (a.offset ? a.offset[e] : 0.f);
        const float mn = a.by_value ? a.value_enc[2] : (a.emin ? a.emin[e] : 0.f);
        const float mx = a.by_value ? a.value_enc[3] : (a.emax ? a.emax[e] : 0.f);
        const EncP p = M::prep(s, off, mn, mx, a.gc);
        sp[0][i] = p.p0;
        sp[1][i] = p.p1;
        if (M::kNP > 2) sp[2][i] = p.p2;
        if (M::kNP > 3) sp[3][i] = p.p3;
        if (M::kDiv) sp[M::kNP][i] = p.rs;
    }
}

// LPBQ forward with the grouped block scales derived by the kernel itself (GroupedBlockQuantizeDequantize._get_scale,
// aimet_torch/quantization/affine/quantizer.py:1363-1399, which the reference runs before every forward): a tile's
// workgroup evaluates, for the groups its blocks belong to, the largest raw block scale (a group is a run of
// neighbouring blocks, a few hundred bytes of min / max), then snaps the raw scales of its own blocks to integer
// multiples of the group's per-channel scale, writes them out for the backward pass and stages them.  The float
// operations are those of lpbq_scale_kernel, in the same order.
struct LpbqFuse {
    const void* pmin;        // per block, `dtype`
    const void* pmax;
    float* scale_out;        // per block
    float* per_channel_out;  // per group, optional
    int64_t group;           // neighbouring blocks per group
    int32_t group_shift;     // log2(group) when it is a power of two, else -1
    int32_t dtype;
    float num_steps, minimum_scale, multipliers;
};

__device__ __forceinline__ void lpbq_load_range(const LpbqFuse& f, int64_t i, float& mn, float& mx) {
    if (f.dtype == AHQ_F32) {
        mn = static_cast<const float*>(f.pmin)[i];
        mx = static_cast<const float*>(f.pmax)[i];
    } else if (f.dtype == AHQ_F16) {
        mn = load_f32(static_cast<const f16_t*>(f.pmin)[i]);
        mx = load_f32(static_cast<const f16_t*>(f.pmax)[i]);
    } else {
        mn = load_f32(static_cast<const bf16_t*>(f.pmin)[i]);
        mx = load_f32(static_cast<const bf16_t*>(f.pmax)[i]);
    }
}

__device__ __forceinline__ float lpbq_raw_from(const LpbqFuse& f, float mn, float mx) {
    const float s = __builtin_fabsf((mx - mn) / f.num_steps);
    return (s != s) ? s : fmaxf(s, f.minimum_scale);
}

__device__ __forceinline__ float lpbq_raw_scale(const LpbqFuse& f, int64_t i) {
    float mn, mx;
    lpbq_load_range(f, i, mn, mx);
    return lpbq_raw_from(f, mn, mx);
}

// min / max of the block this thread stages first, requested ahead of the tile's elements: loads return in the order
// they were issued, so the scale derivation can then run while the elements are still in flight
__device__ __forceinline__ void lpbq_preload(const LpbqFuse& f, const Tile& t, float& mn, float& mx) {
    mn = mx = 0.f;
    if ((int)threadIdx.x < t.nstage) lpbq_load_range(f, t.e0 + threadIdx.x, mn, mx);
}

template <typename M>
__device__ __forceinline__ void stage_lpbq(const QdqArgs& a, const LpbqFuse& f, const Tile& t, float (*sp)[kStage],
                                           const float pre_mn, const float pre_mx) {
    __shared__ float per_channel[kStage];  // of the groups this tile touches
    const int64_t G = f.group;
    const int lane = threadIdx.x & (kWave - 1);
    auto stage_one = [&](int i, int64_t e, int64_t g, float raw, float pc) {
        const float r = __builtin_rintf(raw / pc);
        const float q = (r != r) ? r : fminf(fmaxf(r, 1.0f), f.multipliers);
        const float s = q * pc;
        f.scale_out[e] = s;  // a block lies in one tile, or in two neighbouring ones that store the same value
        if (f.per_channel_out && e == g * G) f.per_channel_out[g] = pc;
        const EncP p = M::prep(s, a.offset ? a.offset[e] : 0.f, 0.f, 0.f, a.gc);
        sp[0][i] = p.p0;
        sp[1][i] = p.p1;
        if (M::kNP > 2) sp[2][i] = p.p2;
        if (M::kNP > 3) sp[3][i] = p.p3;
        if (M::kDiv) sp[M::kNP][i] = p.rs;
    };
    if (f.group_shift >= 0 && G <= kWave && (t.e0 & (G - 1)) == 0 && (t.nstage & (G - 1)) == 0) {
        // whole groups, each inside a power-of-two run of lanes: one read of min / max per block, the group's largest
        // raw scale by shuffles (a maximum does not depend on the order), no second barrier
        const int padded = (t.nstage + kWave - 1) & ~(kWave - 1);
        for (int i = threadIdx.x; i < padded; i += kBlock) {
            const bool live = i < t.nstage;
            const int64_t e = t.e0 + i;
            const float raw = !live ? -__builtin_inff()
                              : i == (int)threadIdx.x ? lpbq_raw_from(f, pre_mn, pre_mx) : lpbq_raw_scale(f, e);
            float largest = raw;
            int nan = (raw != raw) ? 1 : 0;
            for (int m = 1; m < (int)G; m <<= 1) {
                largest = fmaxf(largest, __shfl_xor(largest, m, kWave));
                nan |= __shfl_xor(nan, m, kWave);
            }
            if (nan) largest = __builtin_nanf("");  // torch.amax propagates NaN
            if (live) stage_one(i, e, e >> f.group_shift, raw, largest / f.multipliers);
        }
        return;
    }
    const int64_t g0 = t.e0 / G;
    const int ng = t.nstage > 0 ? (int)((t.e0 + t.nstage - 1) / G - g0) + 1 : 0;
    for (int gi = threadIdx.x / kWave; gi < ng; gi += kBlock / kWave) {
        const int64_t base = (g0 + gi) * G;
        float largest = -__builtin_inff();
        int nan = 0;
        for (int64_t k = lane; k < G; k += kWave) {
            const float s = lpbq_raw_scale(f, base + k);
            nan |= (s != s) ? 1 : 0;
            largest = fmaxf(largest, s);
        }
#pragma unroll
        for (int m = kWave / 2; m >= 1; m >>= 1) {
            largest = fmaxf(largest, __shfl_xor(largest, m, kWave));
            nan |= __shfl_xor(nan, m, kWave);
        }
        if (nan) largest = __builtin_nanf("");  // torch.amax propagates NaN
        if (lane == 0) per_channel[gi] = largest / f.multipliers;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < t.nstage; i += kBlock) {
        const int64_t e = t.e0 + i;
        const int64_t g = e / G;
        stage_one(i, e, g, lpbq_raw_scale(f, e), per_channel[g - g0]);
    }
}

template <typename M>
__device__ __forceinline__ EncP staged(float (*sp)[kStage], int i) {
    EncP e;
    e.p0 = sp[0][i];
    e.p1 = sp[1][i];
    e.p2 = M::kNP > 2 ? sp[2][i] : 0.f;
    e.p3 = M::kNP > 3 ? sp[3][i] : 0.f;
    e.rs = M::kDiv ? sp[M::kNP][i] : 0.f;
    return e;
}

template <typename M>
__device__ __forceinline__ EncP load_enc(const QdqArgs& a, int64_t e) {
    if (a.by_value) return M::prep(a.value_enc[0], a.value_enc[1], a.value_enc[2], a.value_enc[3], a.gc);
    return M::prep(a.scale[e], a.offset ? a.offset[e] : 0.f, a.emin ? a.emin[e] : 0.f, a.emax ? a.emax[e] : 0.f, a.gc);
}

// -------------------------------------------------------------------------------------------------------- forward --
// FULL: every lane of the tile has work, so loads and stores carry no per-lane bounds checks (all tiles but the last).
// True when every element and encoding this lane handles allows the division-free path (see divide()).
template <typename IO, int VEC, typename M, bool FULL, int U>
__device__ __forceinline__ bool lane_can_divide_fast(const QdqArgs& a, const Tile& t, float (*sp)[kStage],
                                                     const Pack<IO, VEC>* in) {
    if (!M::kDiv) return true;
    // One addition per element instead of a comparison each: the sum of the magnitudes is at least every magnitude
    // (rounded sums of non-negative terms never fall below a term), a NaN or an infinity makes it fail the comparison,
    // and 32 elements below the bound cannot overflow it.
    bool ok = true;
    float sum = 0.f;
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int lv = u * kBlock + threadIdx.x;
        if (FULL || lv < t.nv) {
            ok &= sp[M::kNP][stage_index(a, t, lv)] != 0.f;
#pragma unroll
            for (int k = 0; k < VEC; ++k) sum += __builtin_fabsf(load_f32(in[u].v[k]));
        }
    }
    return ok & (sum <= kFastDivMax);
}

template <typename IO, int VEC, typename M, bool FULL, bool FAST, int U>
__device__ __forceinline__ void fwd_math(const QdqArgs& a, const Tile& t, float (*sp)[kStage], const Pack<IO, VEC>* in,
                                         IO* __restrict__ y, uint8_t* __restrict__ mask) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int lv = u * kBlock + threadIdx.x;
        if (FULL || lv < t.nv) {
            const EncP e = staged<M>(sp, stage_index(a, t, lv));
            Pack<IO, VEC> out;
            Pack<uint8_t, VEC> mk;
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                bool inr;
                const float r = M::template fwd<FAST>(load_f32(in[u].v[k]), e, a.gc, inr);
                out.v[k] = store_rounded<IO, M::kCD>(r);
                mk.v[k] = inr ? 1 : 0;
            }
            store_pack_stream<IO, VEC>(y + (int64_t)lv * VEC, out);
            if (mask) store_pack_stream<uint8_t, VEC>(mask + (int64_t)lv * VEC, mk);
        }
    }
}

// FULL: every lane of the tile has work, so loads and stores carry no per-lane bounds checks (all tiles but the last).
// The tile's elements are requested first; the encodings are fetched, prepared and staged while those loads are in
// flight, and the workgroup meets at the barrier once before the arithmetic.
template <typename IO, int VEC, typename M, bool FULL, int U, bool LPBQ = false>
__device__ __forceinline__ void fwd_tile(const QdqArgs& a, const Tile& t, float (*sp)[kStage],
                                         const LpbqFuse* lpbq = nullptr) {
    const IO* __restrict__ x = static_cast<const IO*>(a.x) + t.v0 * VEC;
    IO* __restrict__ y = static_cast<IO*>(a.y) + t.v0 * VEC;
    uint8_t* __restrict__ mask = a.mask ? a.mask + t.v0 * VEC : nullptr;
    Pack<IO, VEC> in[U];
    float pre_mn = 0.f, pre_mx = 0.f;
    if constexpr (LPBQ) lpbq_preload(*lpbq, t, pre_mn, pre_mx);
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int lv = u * kBlock + threadIdx.x;
        if (FULL || lv < t.nv) in[u] = load_pack<IO, VEC>(x + (int64_t)lv * VEC);
    }
    if constexpr (LPBQ) stage_lpbq<M>(a, *lpbq, t, sp, pre_mn, pre_mx);
    else stage_encodings<M>(a, t, sp);
    __syncthreads();
    // one wave-uniform choice per tile: huge or infinite inputs and out-of-range scales take the general division
    if (!M::kDiv || __builtin_amdgcn_ballot_w64(!lane_can_divide_fast<IO, VEC, M, FULL, U>(a, t, sp, in)) == 0)
        fwd_math<IO, VEC, M, FULL, true, U>(a, t, sp, in, y, mask);
    else
        fwd_math<IO, VEC, M, FULL, false, U>(a, t, sp, in, y, mask);
}

template <typename IO, int VEC, typename M>
__global__ __launch_bounds__(kBlock) void qdq_fwd_kernel(const QdqArgs a) {
    __shared__ float sp[M::kNP + (M::kDiv ? 1 : 0)][kStage];
    const Tile t = make_tile(a, blockIdx.x);
    if (t.nv == kBlock * kFwdUnroll) fwd_tile<IO, VEC, M, true, kFwdUnroll>(a, t, sp);
    else fwd_tile<IO, VEC, M, false, kFwdUnroll>(a, t, sp);
    // elements past the last full vector (only possible with a single encoding)
    if (VEC > 1 && blockIdx.x == 0) {
        const int64_t i = a.nvec * VEC + threadIdx.x;
        if (i < a.numel) {
            const IO* x = static_cast<const IO*>(a.x);
            IO* y = static_cast<IO*>(a.y);
            const EncP e = staged<M>(sp, 0);
            bool inr;
            const float r = M::template fwd<false>(load_f32(x[i]), e, a.gc, inr);
            y[i] = store_rounded<IO, M::kCD>(r);
            if (a.mask) a.mask[i] = inr ? 1 : 0;
        }
    }
}

// The tiled forward kernel with the LPBQ block scales derived in place of read (no elements past the last full vector:
// the host side sends such tensors to the two-launch form).
template <typename IO, int VEC, typename M>
__global__ __launch_bounds__(kBlock) void qdq_fwd_lpbq_kernel(const QdqArgs a, const LpbqFuse f) {
    __shared__ float sp[M::kNP + (M::kDiv ? 1 : 0)][kStage];
    const Tile t = make_tile(a, blockIdx.x);
    if (t.nv == kBlock * kFwdUnroll) fwd_tile<IO, VEC, M, true, kFwdUnroll, true>(a, t, sp, &f);
    else fwd_tile<IO, VEC, M, false, kFwdUnroll, true>(a, t, sp, &f);
}

// Encodings that change with every element (run length 1: per-channel along the fastest axis).  The tiled kernel
// would prepare one encoding per element; here a lane owns VEC neighbouring encodings, prepares them once and walks
// down the rows, so loads and stores stay coalesced 16-byte vectors.  A workgroup is 64 lanes across x a few waves
// down; each wave takes kColUnroll rows per step.  kColWaves is the unit the grids are sized in (workgroups of sixteen
// waves, the first shape); the kernels run with fewer waves per workgroup and correspondingly more workgroups, which
// measured faster (forward 8192 x 4096 fp32: 43.6 us with sixteen waves, 40.8 us with four) and leaves a lane more
// registers.
constexpr int kColWaves = 16;
constexpr int kFwdColWaves = 4;
constexpr int kColUnroll = 2;

// the division-free form is allowed for this lane's VEC elements of one row
template <typename IO, int VEC>
__device__ __forceinline__ bool row_can_divide_fast(const Pack<IO, VEC>& p) {
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < VEC; ++k) sum += __builtin_fabsf(load_f32(p.v[k]));
    return sum <= kFastDivMax;  // fails for NaN and infinity
}

template <typename IO, int VEC, typename M, int WAVES>
__global__ __launch_bounds__(WAVES * kWave) void qdq_fwd_cols_kernel(const QdqArgs a) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int64_t c0 = ((int64_t)blockIdx.x * kWave + lane) * VEC;
    if (c0 >= a.J) return;
    const IO* __restrict__ x = static_cast<const IO*>(a.x);
    IO* __restrict__ y = static_cast<IO*>(a.y);
    EncP e[VEC];
    bool enc_fast = true;
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
        e[k] = load_enc<M>(a, c0 + k);
        enc_fast &= !M::kDiv || e[k].rs != 0.f;
    }
    const int64_t step = (int64_t)gridDim.y * WAVES * kColUnroll;
    for (int64_t r0 = ((int64_t)blockIdx.y * WAVES + wave) * kColUnroll; r0 < a.I; r0 += step) {
        Pack<IO, VEC> in[kColUnroll];
        bool ok = enc_fast;
#pragma unroll
        for (int u = 0; u < kColUnroll; ++u)
            if (r0 + u < a.I) in[u] = load_pack<IO, VEC>(x + (r0 + u) * a.J + c0);
#pragma unroll
        for (int u = 0; u < kColUnroll; ++u)
            if (M::kDiv && r0 + u < a.I) ok &= row_can_divide_fast<IO, VEC>(in[u]);
        const bool fast = !M::kDiv || __builtin_amdgcn_ballot_w64(!ok) == 0;  // wave-uniform, like the tiled kernel
#pragma unroll
        for (int u = 0; u < kColUnroll; ++u) {
            if (r0 + u >= a.I) continue;
            Pack<IO, VEC> out;
            Pack<uint8_t, VEC> mk;
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                bool inr;
                const float v = load_f32(in[u].v[k]);
                const float r = fast ? M::template fwd<true>(v, e[k], a.gc, inr) : M::template fwd<false>(v, e[k], a.gc, inr);
                out.v[k] = store_rounded<IO, M::kCD>(r);
                mk.v[k] = inr ? 1 : 0;
            }
            store_pack_stream<IO, VEC>(y + (r0 + u) * a.J + c0, out);
            if (a.mask) store_pack_stream<uint8_t, VEC>(a.mask + (r0 + u) * a.J + c0, mk);
        }
    }
}

template <typename IO, typename M>
__global__ __launch_bounds__(kBlock) void qdq_fwd_generic_kernel(const QdqArgs a) {
    const IO* __restrict__ x = static_cast<const IO*>(a.x);
    IO* __restrict__ y = static_cast<IO*>(a.y);
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < a.numel; i += (int64_t)gridDim.x * kBlock) {
        const EncP e = load_enc<M>(a, generic_enc_index(a, i));
        bool inr;
        const float r = M::template fwd<false>(load_f32(x[i]), e, a.gc, inr);
        y[i] = store_rounded<IO, M::kCD>(r);
        if (a.mask) a.mask[i] = inr ? 1 : 0;
    }
}

// ------------------------------------------------------------------------------------------------------- backward --
__device__ __forceinline__ float finish_sum_rt(double s, int cd) {
    if (cd == AHQ_BF16) return rnd<AHQ_BF16>((float)s);
    if (cd == AHQ_F16) return rnd<AHQ_F16>((float)s);
    return (float)s;
}

template <typename IO, int VEC, typename M, int RED, bool FULL, bool FAST>
__device__ __forceinline__ void bwd_math(const QdqArgs& a, const Tile& t, float (*sp)[kStage], const Pack<IO, VEC>* xin,
                                         const Pack<IO, VEC>* gin, IO* __restrict__ gxp, double& acc_s, double& acc_o,
                                         double* stage_sums, float* vec_sums) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const int lv = u * kBlock + threadIdx.x;
        float vs = 0.f, vo = 0.f;
        int si = 0;
        bool wave_all_in = false;  // only the split form below sets it
        if constexpr (FAST && M::kSplitBwd) {
            const bool work = FULL || lv < t.nv;
            EncP e{};
            float tq[VEC], xr[VEC], m[VEC];
            bool all_in = true;
            if (work) {
                si = stage_index(a, t, lv);
                e = staged<M>(sp, si);
                const float lo = e.p1 + a.gc.qmin, hi = e.p1 + a.gc.qmax;
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    M::bwd_pre(load_f32(xin[u].v[k]), e, lo, hi, tq[k], xr[k], m[k]);
                    all_in &= (m[k] == xr[k]);
                }
            }
            wave_all_in = __builtin_amdgcn_ballot_w64(!all_in) == 0;
            if (wave_all_in) {
                // every element of this vector, in every lane, is inside the grid: the input gradient is the output
                // gradient, the offset gradient gets no term
                if (work) {
#pragma unroll
                    for (int k = 0; k < VEC; ++k) vs += M::bwd_gs_in(load_f32(gin[u].v[k]), tq[k], xr[k]);
                    if (gxp) store_pack_stream<IO, VEC>(gxp + (int64_t)lv * VEC, gin[u]);
                }
            } else if (work) {
                Pack<IO, VEC> out;
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    const float gr = load_f32(gin[u].v[k]);
                    const bool in = (m[k] == xr[k]);
                    out.v[k] = store_cast<IO>(in ? gr : 0.f);
                    vs += in ? M::bwd_gs_in(gr, tq[k], xr[k]) : M::bwd_gs_out(gr, m[k]);
                    vo += in ? 0.f : M::bwd_goff_out(gr, e);
                }
                if (gxp) store_pack_stream<IO, VEC>(gxp + (int64_t)lv * VEC, out);
            }
        } else if (FULL || lv < t.nv) {
            si = stage_index(a, t, lv);
            const EncP e = staged<M>(sp, si);
            Pack<IO, VEC> out;
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                float gx, gs, go;
                M::template bwd<FAST>(load_f32(gin[u].v[k]), load_f32(xin[u].v[k]), e, a.gc, gx, gs, go);
                out.v[k] = store_cast<IO>(gx);
                vs += gs;
                vo += go;
            }
            if (gxp) store_pack_stream<IO, VEC>(gxp + (int64_t)lv * VEC, out);
        }
        if (RED == kRedTile) {
            acc_s += (double)vs;
            acc_o += (double)vo;
        } else if (RED == kRedSeg) {
            // runs of Kv (power of two <= 64) neighbouring lanes share an encoding; runs never straddle a wave.  At most
            // 64 x VEC terms per encoding, so single precision (what the reference's own sum accumulates in) is enough
            const int kv = (int)a.Kv;
            const float fs = segment_reduce(vs, kv, OpAddF());
            const float fo = wave_all_in ? 0.f : segment_reduce(vo, kv, OpAddF());
            if ((FULL || lv < t.nv) && (threadIdx.x & (kv - 1)) == 0) {
                const int64_t e = t.e0 + si;
                a.gscale[e] = finish_sum_rt((double)fs, a.out_cd);
                a.goffset[e] = finish_sum_rt((double)fo, a.out_cd);
            }
        } else if (RED == kRedAtomic) {
            // into the tile's own table in LDS first (one entry per run the tile touches); the table is added to the
            // global sums once per run and tile instead of once per vector
            if (FULL || lv < t.nv) {
                atomicAdd(&stage_sums[2 * si], (double)vs);
                atomicAdd(&stage_sums[2 * si + 1], (double)vo);
            }
        } else if (RED == kRedRuns) {
            // one pair per vector; the runs are added up in a fixed order once the tile is through
            if (FULL || lv < t.nv) {
                vec_sums[lv] = vs;
                vec_sums[kTileVec + lv] = vo;
            }
        }
    }
}

template <typename IO, int VEC, typename M, int RED, bool FULL>
__device__ __forceinline__ void bwd_tile(const QdqArgs& a, const Tile& t, float (*sp)[kStage], double& acc_s, double& acc_o,
                                         double* stage_sums, float* vec_sums) {
    const IO* __restrict__ x = static_cast<const IO*>(a.x) + t.v0 * VEC;
    const IO* __restrict__ g = static_cast<const IO*>(a.g) + t.v0 * VEC;
    IO* __restrict__ gxp = a.gx ? static_cast<IO*>(a.gx) + t.v0 * VEC : nullptr;
    Pack<IO, VEC> xin[kUnroll], gin[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const int lv = u * kBlock + threadIdx.x;
        if (FULL || lv < t.nv) {
            xin[u] = load_pack<IO, VEC>(x + (int64_t)lv * VEC);
            gin[u] = load_pack<IO, VEC>(g + (int64_t)lv * VEC);
        }
    }
    // the encodings are staged while the loads above are in flight
    stage_encodings<M>(a, t, sp);
    if (RED == kRedAtomic)
        for (int i = threadIdx.x; i < 2 * t.nstage; i += kBlock) stage_sums[i] = 0.0;
    __syncthreads();
    if (!M::kDiv || __builtin_amdgcn_ballot_w64(!lane_can_divide_fast<IO, VEC, M, FULL, kUnroll>(a, t, sp, xin)) == 0)
        bwd_math<IO, VEC, M, RED, FULL, true>(a, t, sp, xin, gin, gxp, acc_s, acc_o, stage_sums, vec_sums);
    else
        bwd_math<IO, VEC, M, RED, FULL, false>(a, t, sp, xin, gin, gxp, acc_s, acc_o, stage_sums, vec_sums);
}

template <typename IO, int VEC, typename M, int RED>
__global__ __launch_bounds__(kBlock) void qdq_bwd_kernel(const QdqArgs a) {
    __shared__ float sp[M::kNP + (M::kDiv ? 1 : 0)][kStage];
    __shared__ double red_smem[kBlock / kWave];
    __shared__ double stage_sums[RED == kRedAtomic ? 2 * kStage : 1];  // kRedAtomic: (scale, offset) sums per run
    __shared__ float vec_sums[RED == kRedRuns ? 2 * kTileVec : 1];     // kRedRuns: (scale, offset) terms per vector
    const Tile t = make_tile(a, blockIdx.x);
    double acc_s = 0.0, acc_o = 0.0;  // kRedTile: per-thread totals
    if (t.nv == kTileVec) bwd_tile<IO, VEC, M, RED, true>(a, t, sp, acc_s, acc_o, stage_sums, vec_sums);
    else bwd_tile<IO, VEC, M, RED, false>(a, t, sp, acc_s, acc_o, stage_sums, vec_sums);
    if (RED == kRedRuns) {
        // The tile holds t.nstage whole runs of Kv vectors.  Short runs: one thread adds a run front to back.  Longer
        // ones: one wave per run, every lane adds its strided share front to back, then the lanes are combined in
        // the fixed pattern of wave_reduce.  Either way the order of additions depends on the layout alone.
        __syncthreads();
        const int kv = (int)a.Kv;
        const int64_t run0 = (int64_t)blockIdx.x * a.tpr;
        auto emit = [&](int run, double s, double o) {
            if (a.I == 1) {
                a.gscale[run0 + run] = finish_sum_rt(s, a.out_cd);
                a.goffset[run0 + run] = finish_sum_rt(o, a.out_cd);
            } else {
                a.partials[2 * (run0 + run)] = s;
                a.partials[2 * (run0 + run) + 1] = o;
            }
        };
        if (kv <= 16) {
            for (int run = threadIdx.x; run < t.nstage; run += kBlock) {
                double s = 0.0, o = 0.0;
                for (int k = 0; k < kv; ++k) {
                    s += (double)vec_sums[run * kv + k];
                    o += (double)vec_sums[kTileVec + run * kv + k];
                }
                emit(run, s, o);
            }
        } else {
            const int lane = threadIdx.x & (kWave - 1);
            for (int run = threadIdx.x / kWave; run < t.nstage; run += kBlock / kWave) {
                double s = 0.0, o = 0.0;
                for (int k = lane; k < kv; k += kWave) {
                    s += (double)vec_sums[run * kv + k];
                    o += (double)vec_sums[kTileVec + run * kv + k];
                }
                s = wave_reduce(s, OpAddD());
                o = wave_reduce(o, OpAddD());
                if (lane == 0) emit(run, s, o);
            }
        }
        return;
    }
    if (RED == kRedAtomic) {
        __syncthreads();
        for (int i = threadIdx.x; i < t.nstage; i += kBlock) {
            int64_t e = t.e0 + i;
            if (e >= a.J) e %= a.J;
            atomicAdd(&a.partials[2 * e], stage_sums[2 * i]);
            atomicAdd(&a.partials[2 * e + 1], stage_sums[2 * i + 1]);
        }
    }
    if (VEC > 1 && blockIdx.x == 0) {  // tail elements, single encoding only
        const int64_t i = a.nvec * VEC + threadIdx.x;
        if (i < a.numel) {
            const IO* x = static_cast<const IO*>(a.x);
            const IO* g = static_cast<const IO*>(a.g);
            IO* gxp = static_cast<IO*>(a.gx);
            const EncP e = staged<M>(sp, 0);
            float gx, gs, go;
            M::template bwd<false>(load_f32(g[i]), load_f32(x[i]), e, a.gc, gx, gs, go);
            if (gxp) gxp[i] = store_cast<IO>(gx);
            if (RED == kRedTile) {
                acc_s += (double)gs;
                acc_o += (double)go;
            } else if (RED == kRedAtomic) {
                atomicAdd(&a.partials[0], (double)gs);
                atomicAdd(&a.partials[1], (double)go);
            }
        }
    }
    if (RED == kRedTile) {
        const double bs = block_reduce(acc_s, OpAddD(), red_smem);
        const double bo = block_reduce(acc_o, OpAddD(), red_smem);
        // number of tiles that feed one encoding
        const int64_t per_enc = a.mode == kRows ? a.I * (int64_t)a.tpr : (int64_t)a.nblocks;
        if (per_enc == 1) {
            if (threadIdx.x == 0) {
                a.gscale[t.e0] = finish_sum_rt(bs, a.out_cd);
                a.goffset[t.e0] = finish_sum_rt(bo, a.out_cd);
            }
            return;
        }
        if (threadIdx.x == 0) {
            a.partials[2 * (int64_t)blockIdx.x] = bs;
            a.partials[2 * (int64_t)blockIdx.x + 1] = bo;
        }
    }
}

// Adds the per-tile partial sums of every encoding in a fixed order (second launch: a kernel boundary makes the
// partials visible without any in-kernel fence, which on a multi-die GPU would flush the L2 once per workgroup).
constexpr int kFinishThreads = 1024;
__global__ __launch_bounds__(kFinishThreads) void qdq_bwd_finish_kernel(const QdqArgs a) {
    __shared__ double red_smem[2][kFinishThreads / kWave];
    const int64_t per_enc = a.mode == kRows ? a.I * (int64_t)a.tpr : (int64_t)a.nblocks;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    if (a.mode != kRows) {
        // single encoding: independent loads per thread, then one tree
        double s = 0.0, o = 0.0;
#pragma unroll 4
        for (int64_t q = threadIdx.x; q < per_enc; q += kFinishThreads) {
            s += a.partials[2 * q];
            o += a.partials[2 * q + 1];
        }
        s = wave_reduce(s, OpAddD());
        o = wave_reduce(o, OpAddD());
        if (lane == 0) {
            red_smem[0][wave] = s;
            red_smem[1][wave] = o;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            double ts = 0.0, to = 0.0;
            for (int w = 0; w < kFinishThreads / kWave; ++w) {
                ts += red_smem[0][w];
                to += red_smem[1][w];
            }
            a.gscale[0] = finish_sum_rt(ts, a.out_cd);
            a.goffset[0] = finish_sum_rt(to, a.out_cd);
        }
        return;
    }
    // one wave per encoding, lanes stride over that encoding's tiles
    const int64_t wave0 = (int64_t)blockIdx.x * (kFinishThreads / kWave) + wave;
    for (int64_t j = wave0; j < a.J; j += (int64_t)gridDim.x * (kFinishThreads / kWave)) {
        double s = 0.0, o = 0.0;
        for (int64_t q = lane; q < per_enc; q += kWave) {
            const int64_t i = q / a.tpr, tt = q - i * a.tpr;
            const int64_t blk = (i * a.J + j) * a.tpr + tt;
            s += a.partials[2 * blk];
            o += a.partials[2 * blk + 1];
        }
        s = wave_reduce(s, OpAddD());
        o = wave_reduce(o, OpAddD());
        if (lane == 0) {
            a.gscale[j] = finish_sum_rt(s, a.out_cd);
            a.goffset[j] = finish_sum_rt(o, a.out_cd);
        }
    }
}

// Adds, for every encoding, `count` partial pairs that lie `stride` pairs apart (the first one at the encoding's own
// index), in a fixed order: one wave per encoding, every lane its strided share front to back, then wave_reduce.
// kRedRuns with I > 1: count = I runs per encoding, stride = J.  Column kernel: count = row groups, stride = J.
__global__ __launch_bounds__(kBlock) void qdq_bwd_strided_finish_kernel(const double* __restrict__ partials, int64_t count,
                                                                        int64_t stride, int64_t num_enc, float* gscale,
                                                                        float* goffset, int cd) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t waves = (int64_t)gridDim.x * (kBlock / kWave);
    for (int64_t e = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave; e < num_enc; e += waves) {
        double s = 0.0, o = 0.0;
        for (int64_t q = lane; q < count; q += kWave) {
            s += partials[2 * (q * stride + e)];
            o += partials[2 * (q * stride + e) + 1];
        }
        s = wave_reduce(s, OpAddD());
        o = wave_reduce(o, OpAddD());
        if (lane == 0) {
            gscale[e] = finish_sum_rt(s, cd);
            goffset[e] = finish_sum_rt(o, cd);
        }
    }
}

template <typename IO, typename M>
__global__ __launch_bounds__(kBlock) void qdq_bwd_generic_kernel(const QdqArgs a) {
    const IO* __restrict__ x = static_cast<const IO*>(a.x);
    const IO* __restrict__ g = static_cast<const IO*>(a.g);
    IO* __restrict__ gxp = static_cast<IO*>(a.gx);
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    const int64_t first = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    // whole waves iterate together (lanes past the end carry zeros), so the exchanges below are wave-wide
    for (int64_t base = first - lane; base < a.numel; base += stride) {
        const int64_t i = base + lane;
        const bool active = i < a.numel;
        int64_t ei = -1;
        float gx = 0.f, gs = 0.f, go = 0.f;
        if (active) {
            ei = generic_enc_index(a, i);
            const EncP e = load_enc<M>(a, ei);
            M::template bwd<false>(load_f32(g[i]), load_f32(x[i]), e, a.gc, gx, gs, go);
            if (gxp) gxp[i] = store_cast<IO>(gx);
        }
        if (a.partials) {
            // neighbouring elements mostly share an encoding: the lanes of each distinct encoding are summed first
            // and one lane issues the two atomics
            uint64_t todo = __builtin_amdgcn_ballot_w64(active);
            while (todo != 0) {
                const int lead = __builtin_ctzll(todo);
                const int64_t el = __shfl(ei, lead, kWave);
                const bool mine = active && ei == el;
                double ss = mine ? (double)gs : 0.0, so = mine ? (double)go : 0.0;
#pragma unroll
                for (int k = kWave / 2; k >= 1; k >>= 1) {
                    ss += __shfl_xor(ss, k, kWave);
                    so += __shfl_xor(so, k, kWave);
                }
                if (lane == lead) {
                    atomicAdd(&a.partials[2 * el], ss);
                    atomicAdd(&a.partials[2 * el + 1], so);
                }
                todo &= ~__builtin_amdgcn_ballot_w64(mine);
            }
        }
    }
}

// Backward for run length 1 (see qdq_fwd_cols_kernel): every lane keeps the sums of its VEC encodings over the rows
// it walks, the waves of a workgroup add theirs up in LDS one after the other, and the workgroup's sums go to its own
// row of the partials ([row group][encoding]), which qdq_bwd_strided_finish_kernel adds up in order.
template <typename IO, int VEC, typename M, int WAVES>
__global__ __launch_bounds__(WAVES * kWave) void qdq_bwd_cols_kernel(const QdqArgs a) {
    __shared__ double sums[2 * VEC * kWave];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int64_t c0 = ((int64_t)blockIdx.x * kWave + lane) * VEC;
    const bool live = c0 < a.J;
    const bool want_pg = a.partials != nullptr;
    if (want_pg) {
        for (int i = threadIdx.x; i < 2 * VEC * kWave; i += WAVES * kWave) sums[i] = 0.0;
        __syncthreads();
    }
    double acc_s[VEC], acc_o[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) acc_s[k] = acc_o[k] = 0.0;
    if (live) {
        const IO* __restrict__ x = static_cast<const IO*>(a.x);
        const IO* __restrict__ g = static_cast<const IO*>(a.g);
        IO* __restrict__ gxp = static_cast<IO*>(a.gx);
        EncP e[VEC];
        bool enc_fast = true;
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            e[k] = load_enc<M>(a, c0 + k);
            enc_fast &= !M::kDiv || e[k].rs != 0.f;
        }
        const int64_t step = (int64_t)gridDim.y * WAVES * kColUnroll;
        for (int64_t r0 = ((int64_t)blockIdx.y * WAVES + wave) * kColUnroll; r0 < a.I; r0 += step) {
            Pack<IO, VEC> xin[kColUnroll], gin[kColUnroll];
            bool ok = enc_fast;
#pragma unroll
            for (int u = 0; u < kColUnroll; ++u)
                if (r0 + u < a.I) {
                    xin[u] = load_pack<IO, VEC>(x + (r0 + u) * a.J + c0);
                    gin[u] = load_pack<IO, VEC>(g + (r0 + u) * a.J + c0);
                }
#pragma unroll
            for (int u = 0; u < kColUnroll; ++u)
                if (M::kDiv && r0 + u < a.I) ok &= row_can_divide_fast<IO, VEC>(xin[u]);
            const bool fast = !M::kDiv || __builtin_amdgcn_ballot_w64(!ok) == 0;
#pragma unroll
            for (int u = 0; u < kColUnroll; ++u) {
                if (r0 + u >= a.I) continue;
                Pack<IO, VEC> out;
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    float gx, gs, go;
                    const float gr = load_f32(gin[u].v[k]), v = load_f32(xin[u].v[k]);
                    if (fast) M::template bwd<true>(gr, v, e[k], a.gc, gx, gs, go);
                    else M::template bwd<false>(gr, v, e[k], a.gc, gx, gs, go);
                    out.v[k] = store_cast<IO>(gx);
                    acc_s[k] += (double)gs;
                    acc_o[k] += (double)go;
                }
                if (gxp) store_pack_stream<IO, VEC>(gxp + (r0 + u) * a.J + c0, out);
            }
        }
    }
    if (!want_pg) return;
    // the waves take turns, so the sums do not depend on which wave finishes first
    for (int w = 0; w < WAVES; ++w) {
        if (wave == w && live) {
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                sums[(2 * k) * kWave + lane] += acc_s[k];
                sums[(2 * k + 1) * kWave + lane] += acc_o[k];
            }
        }
        __syncthreads();
    }
    if (wave == 0 && live) {
        double* row = a.partials + 2 * (int64_t)blockIdx.y * a.J;
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            row[2 * (c0 + k)] = sums[(2 * k) * kWave + lane];
            row[2 * (c0 + k) + 1] = sums[(2 * k + 1) * kWave + lane];
        }
    }
}

__global__ void zero_f64_kernel(double* p, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0.0;
}

__global__ void finish_atomic_kernel(const double* acc, float* gscale, float* goffset, int64_t nenc, int cd) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nenc; i += (int64_t)gridDim.x * blockDim.x) {
        gscale[i] = finish_sum_rt(acc[2 * i], cd);
        goffset[i] = finish_sum_rt(acc[2 * i + 1], cd);
    }
}

// ------------------------------------------------------------------------------------------------ host dispatch --
static void fill_args(const ahq_grid& grid, const Plan& p, QdqArgs* a) {
    fill_geom(p, a);
    a->gc.qmin = (float)grid.qmin;
    a->gc.qmax = (float)grid.qmax;
    a->gc.zps = (float)grid.zero_point_shift;
    a->gc.flags = 0;
    a->red = p.red;
    a->out_cd = grid.compute_dtype;
}

static bool validate_grid(const ahq_grid* g, bool backward) {
    if (!g) return set_error("grid is null"), false;
    if (g->io_dtype < AHQ_F32 || g->io_dtype > AHQ_BF16) return set_error("bad io_dtype"), false;
    if (g->compute_dtype != g->io_dtype && g->compute_dtype != AHQ_F32) return set_error("compute_dtype must equal io_dtype or be fp32"), false;
    if (g->arith < AHQ_ARITH_ATEN || g->arith > AHQ_ARITH_DLQ) return set_error("bad arith"), false;
    if (g->op < AHQ_OP_QDQ || g->op > AHQ_OP_DEQUANTIZE) return set_error("bad op"), false;
    if (g->arith != AHQ_ARITH_AUTOGRAD && g->op != AHQ_OP_QDQ) return set_error("only quantize-dequantize exists for this arithmetic"), false;
    if (g->op != AHQ_OP_DEQUANTIZE && g->qmin > g->qmax) return set_error("qmin must not exceed qmax"), false;
    if (g->op == AHQ_OP_DEQUANTIZE && g->compute_dtype != g->io_dtype) return set_error("dequantize computes in the io dtype"), false;
    if (g->zero_point_shift != 0.0 && g->zero_point_shift != 0.5) return set_error("zero_point_shift must be 0.0 or 0.5"), false;
    if (g->zero_point_shift != 0.0 && (g->arith != AHQ_ARITH_AUTOGRAD || g->op != AHQ_OP_QDQ)) return set_error("zero_point_shift needs the autograd quantize-dequantize arithmetic"), false;
    if (g->qmax - g->qmin >= (1ll << 24) || g->qmin < -(1ll << 24) || g->qmax > (1ll << 24)) return set_error("grid wider than fp32 can represent exactly"), false;
    if (backward && g->arith == AHQ_ARITH_DLQ) return set_error("no backward exists for the DlQuantization arithmetic"), false;
    return true;
}

// Expands to a call of F<IO, ...> for the io dtype at run time.
#define AHQ_IO_SWITCH(dtype, CALL)                                      \
    switch (dtype) {                                                    \
        case AHQ_F32: { using IO = float; CALL; } break;                \
        case AHQ_F16: { using IO = f16_t; CALL; } break;                \
        default: { using IO = bf16_t; CALL; } break;                    \
    }

// Run length 1 over several rows, whole 16-byte vectors per row: the column-walking kernels apply.
template <typename IO>
static bool cols_layout(const Plan& p, bool aligned) {
    constexpr int V = IoTraits<IO>::kVec;
    // at least half a wave of lanes must own columns, or the tiled kernel's full waves win
    return aligned && p.cl.kind == kIJK && p.cl.K == 1 && p.cl.I > 1 && p.cl.J % V == 0 && p.cl.J / V >= kWave / 2;
}

// grid of the column-walking kernels: x over groups of 64 lanes x VEC encodings, y over row groups; about `target`
// workgroups, every wave with at least one step of rows
template <typename IO>
static dim3 cols_grid(const Plan& p, int64_t target, int waves = kColWaves) {
    constexpr int V = IoTraits<IO>::kVec;
    const int64_t gx = (p.cl.J / V + kWave - 1) / kWave;
    const int64_t row_groups = (p.cl.I + (int64_t)waves * kColUnroll - 1) / ((int64_t)waves * kColUnroll);
    int64_t gy = (target + gx - 1) / gx;
    gy = gy < 1 ? 1 : (gy > row_groups ? row_groups : gy);
    if (gy > 65535) gy = 65535;
    return dim3((unsigned)gx, (unsigned)gy);
}

template <typename IO, typename M>
static void launch_fwd(const Plan& p, const QdqArgs& a, hipStream_t st, bool aligned) {
    if (cols_layout<IO>(p, aligned) && (p.cl.J / IoTraits<IO>::kVec + kWave - 1) / kWave <= 0x7fffffff) {
        // a lane prepares kVec encodings before its first row: the more of them, the more rows it should walk
        constexpr int W = kFwdColWaves;
        hipLaunchKernelGGL((qdq_fwd_cols_kernel<IO, IoTraits<IO>::kVec, M, W>),
                           cols_grid<IO>(p, (IoTraits<IO>::kVec > 4 ? 768 : 2048) * (kColWaves / W), W), dim3(W * kWave), 0, st, a);
        return;
    }
    if (p.cl.kind == kGeneric) {
        hipLaunchKernelGGL((qdq_fwd_generic_kernel<IO, M>), dim3(p.nblocks), dim3(kBlock), 0, st, a);
    } else if (p.vec == 1) {
        hipLaunchKernelGGL((qdq_fwd_kernel<IO, 1, M>), dim3(p.nblocks), dim3(kBlock), 0, st, a);
    } else {
        hipLaunchKernelGGL((qdq_fwd_kernel<IO, IoTraits<IO>::kVec, M>), dim3(p.nblocks), dim3(kBlock), 0, st, a);
    }
}

// the column-walking backward kernel takes run length 1 whatever reduction the plan would otherwise use for it
template <typename IO>
static bool bwd_cols_layout(const Plan& p, bool aligned) {
    return cols_layout<IO>(p, aligned) && (p.red == kRedAtomic || p.red == kRedRuns || p.red == kRedNone);
}

static bool bwd_cols_layout(int io_dtype, const Plan& p, bool aligned) {
    return io_dtype == AHQ_F32 ? bwd_cols_layout<float>(p, aligned) : bwd_cols_layout<f16_t>(p, aligned);
}

// The backward kernel keeps eight encodings, sixteen double sums and two rows of two tensors per lane on a 16-bit
// tensor: more than the 128 registers a workgroup of sixteen waves leaves a lane (36 of them were spilled: 92 us on
// 8192 x 4096 bf16 with learned encodings; 73 us with eight waves, 62 us with four, 71 us with two).  float32:
// 73.6 us with sixteen waves, 69.5 us with eight, 72 us with four.
template <typename IO>
constexpr int bwd_cols_waves() { return IoTraits<IO>::kVec > 4 ? kColWaves / 4 : kColWaves / 2; }

template <typename IO>
static dim3 bwd_cols_grid(const Plan& p) {
    return cols_grid<IO>(p, 512 * (kColWaves / bwd_cols_waves<IO>()), bwd_cols_waves<IO>());
}

static unsigned bwd_cols_row_groups(int io_dtype, const Plan& p) {
    return io_dtype == AHQ_F32 ? bwd_cols_grid<float>(p).y : bwd_cols_grid<f16_t>(p).y;
}

// pairs of doubles the backward pass needs as scratch for its parameter gradients
static size_t bwd_scratch_pairs(int io_dtype, const Plan& p, bool aligned, bool want_pg) {
    if (!want_pg) return 0;
    if (bwd_cols_layout(io_dtype, p, aligned)) return (size_t)bwd_cols_row_groups(io_dtype, p) * (size_t)p.cl.J;
    return p.ws_elems;
}

template <typename IO, typename M, int RED>
static void launch_bwd_red(const Plan& p, const QdqArgs& a, hipStream_t st) {
    if (p.vec == 1) {
        hipLaunchKernelGGL((qdq_bwd_kernel<IO, 1, M, RED>), dim3(p.nblocks), dim3(kBlock), 0, st, a);
    } else {
        hipLaunchKernelGGL((qdq_bwd_kernel<IO, IoTraits<IO>::kVec, M, RED>), dim3(p.nblocks), dim3(kBlock), 0, st, a);
    }
}

template <typename IO, typename M>
static void launch_bwd(const Plan& p, const QdqArgs& a, hipStream_t st, bool aligned) {
    if (bwd_cols_layout<IO>(p, aligned)) {
        // few row groups: every workgroup ends with one row of partial sums
        constexpr int W = bwd_cols_waves<IO>();
        hipLaunchKernelGGL((qdq_bwd_cols_kernel<IO, IoTraits<IO>::kVec, M, W>), bwd_cols_grid<IO>(p), dim3(W * kWave), 0, st, a);
        return;
    }
    if (p.cl.kind == kGeneric) {
        hipLaunchKernelGGL((qdq_bwd_generic_kernel<IO, M>), dim3(p.nblocks), dim3(kBlock), 0, st, a);
        return;
    }
    switch (p.red) {
        case kRedNone: launch_bwd_red<IO, M, kRedNone>(p, a, st); break;
        case kRedTile: launch_bwd_red<IO, M, kRedTile>(p, a, st); break;
        case kRedSeg: launch_bwd_red<IO, M, kRedSeg>(p, a, st); break;
        case kRedRuns: launch_bwd_red<IO, M, kRedRuns>(p, a, st); break;
        default: launch_bwd_red<IO, M, kRedAtomic>(p, a, st); break;
    }
}

// Calls F with the Math type selected by (arith, op, compute dtype).
#define AHQ_MATH_SWITCH(grid, CALL)                                                                  \
    do {                                                                                             \
        if ((grid).arith == AHQ_ARITH_ATEN) { using M = MathAten; CALL; }                            \
        else if ((grid).arith == AHQ_ARITH_DLQ) { using M = MathDlq; CALL; }                         \
        else if ((grid).op == AHQ_OP_QDQ) {                                                          \
            if ((grid).zero_point_shift != 0.0) {                                                    \
                if ((grid).compute_dtype == AHQ_F32) { using M = MathAutogradQdq<AHQ_F32, true>; CALL; }       \
                else if ((grid).compute_dtype == AHQ_F16) { using M = MathAutogradQdq<AHQ_F16, true>; CALL; }  \
                else { using M = MathAutogradQdq<AHQ_BF16, true>; CALL; }                            \
            } else if ((grid).compute_dtype == AHQ_F32) { using M = MathAutogradQdq<AHQ_F32, false>; CALL; }   \
            else if ((grid).compute_dtype == AHQ_F16) { using M = MathAutogradQdq<AHQ_F16, false>; CALL; }     \
            else { using M = MathAutogradQdq<AHQ_BF16, false>; CALL; }                               \
        } else if ((grid).op == AHQ_OP_QUANTIZE) {                                                   \
            if ((grid).compute_dtype == AHQ_F32) { using M = MathAutogradQuantize<AHQ_F32>; CALL; }  \
            else if ((grid).compute_dtype == AHQ_F16) { using M = MathAutogradQuantize<AHQ_F16>; CALL; } \
            else { using M = MathAutogradQuantize<AHQ_BF16>; CALL; }                                 \
        } else {                                                                                     \
            if ((grid).compute_dtype == AHQ_F32) { using M = MathAutogradDequantize<AHQ_F32>; CALL; } \
            else if ((grid).compute_dtype == AHQ_F16) { using M = MathAutogradDequantize<AHQ_F16>; CALL; } \
            else { using M = MathAutogradDequantize<AHQ_BF16>; CALL; }                               \
        }                                                                                            \
    } while (0)

}  // namespace ahq

using namespace ahq;

extern "C" int ahq_qdq_forward(const ahq_grid* grid, const ahq_layout* layout, const void* x, void* y, uint8_t* mask_out,
                               const float* scale, const float* offset, const float* enc_min, const float* enc_max,
                               void* stream) {
    if (!validate_grid(grid, false)) return AHQ_ERR_INVALID;
    if (!layout) return set_error("layout is null"), AHQ_ERR_INVALID;
    if (!scale) return set_error("scale is null"), AHQ_ERR_INVALID;
    if (grid->arith == AHQ_ARITH_DLQ && (!enc_min || !enc_max || !offset)) return set_error("DlQuantization arithmetic needs offset, enc_min and enc_max"), AHQ_ERR_INVALID;
    if (grid->arith != AHQ_ARITH_DLQ && (enc_min || enc_max)) return set_error("enc_min/enc_max only apply to the DlQuantization arithmetic"), AHQ_ERR_INVALID;
    Plan p;
    const bool al = aligned16(x) && aligned16(y) && (!mask_out || (reinterpret_cast<uintptr_t>(mask_out) & 7u) == 0);
    if (!make_plan(grid->io_dtype, *layout, al, false, &p, kFwdUnroll)) return AHQ_ERR_INVALID;
    if (p.cl.numel == 0) return AHQ_OK;
    if (!x || !y) return set_error("x or y is null"), AHQ_ERR_INVALID;
    QdqArgs a{};
    a.x = x;
    a.y = y;
    a.mask = mask_out;
    a.scale = scale;
    a.offset = offset;
    a.emin = enc_min;
    a.emax = enc_max;
    fill_args(*grid, p, &a);
    hipStream_t st = static_cast<hipStream_t>(stream);
    AHQ_IO_SWITCH(grid->io_dtype, AHQ_MATH_SWITCH(*grid, (launch_fwd<IO, M>(p, a, st, al))));
    return check_launch("ahq_qdq_forward");
}

template <typename IO, typename M>
static void launch_fwd_lpbq(const Plan& p, const QdqArgs& a, const LpbqFuse& f, hipStream_t st) {
    if (p.vec == 1) hipLaunchKernelGGL((qdq_fwd_lpbq_kernel<IO, 1, M>), dim3(p.nblocks), dim3(kBlock), 0, st, a, f);
    else hipLaunchKernelGGL((qdq_fwd_lpbq_kernel<IO, IoTraits<IO>::kVec, M>), dim3(p.nblocks), dim3(kBlock), 0, st, a, f);
}

extern "C" int ahq_lpbq_qdq_forward(const ahq_grid* grid, const ahq_layout* layout, const void* x, void* y,
                                    uint8_t* mask_out, int32_t range_dtype, const void* range_min,
                                    const void* range_max, int64_t blocks_per_group, double minimum_scale,
                                    int32_t num_multipliers, const float* offset, float* scale,
                                    float* per_channel_scale, void* stream) {
    if (!validate_grid(grid, false)) return AHQ_ERR_INVALID;
    if (!layout || !range_min || !range_max || !scale) return set_error("null argument"), AHQ_ERR_INVALID;
    if (range_dtype < AHQ_F32 || range_dtype > AHQ_BF16) return set_error("bad range dtype"), AHQ_ERR_INVALID;
    if (blocks_per_group < 1) return set_error("blocks_per_group must be positive"), AHQ_ERR_INVALID;
    if (grid->qmin >= grid->qmax) return set_error("qmax must be larger than qmin"), AHQ_ERR_INVALID;
    if (num_multipliers < 1 || num_multipliers > (1 << 24)) return set_error("num_multipliers must be in 1..2^24"), AHQ_ERR_INVALID;
    if (grid->arith != AHQ_ARITH_AUTOGRAD || grid->op != AHQ_OP_QDQ || grid->zero_point_shift != 0.0 ||
        grid->compute_dtype != grid->io_dtype)
        return set_error("the fused LPBQ forward covers the autograd quantize-dequantize arithmetic computed in the tensor's dtype"), AHQ_ERR_UNSUPPORTED;
    Plan p;
    const bool al = aligned16(x) && aligned16(y) && (!mask_out || (reinterpret_cast<uintptr_t>(mask_out) & 7u) == 0);
    if (!make_plan(grid->io_dtype, *layout, al, false, &p, kFwdUnroll)) return AHQ_ERR_INVALID;
    if (p.cl.numel == 0) return AHQ_OK;
    if (!x || !y) return set_error("x or y is null"), AHQ_ERR_INVALID;
    if (p.cl.kind != kIJK || p.cl.I != 1 || p.cl.J % blocks_per_group != 0 || p.nvec * p.vec != p.cl.numel)
        return set_error("the fused LPBQ forward needs blocks that follow each other in memory, in whole groups"), AHQ_ERR_UNSUPPORTED;
    QdqArgs a{};
    a.x = x;
    a.y = y;
    a.mask = mask_out;
    a.offset = offset;
    fill_args(*grid, p, &a);
    LpbqFuse f{};
    f.pmin = range_min;
    f.pmax = range_max;
    f.scale_out = scale;
    f.per_channel_out = per_channel_scale;
    f.group = blocks_per_group;
    f.group_shift = -1;
    if (is_pow2(blocks_per_group))
        for (int b = 0; b < 62; ++b)
            if (((int64_t)1 << b) == blocks_per_group) f.group_shift = b;
    f.dtype = range_dtype;
    f.num_steps = (float)(double)(grid->qmax - grid->qmin);
    f.minimum_scale = (float)minimum_scale;
    f.multipliers = (float)num_multipliers;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (grid->io_dtype) {
        case AHQ_F32: launch_fwd_lpbq<float, MathAutogradQdq<AHQ_F32, false>>(p, a, f, st); break;
        case AHQ_F16: launch_fwd_lpbq<f16_t, MathAutogradQdq<AHQ_F16, false>>(p, a, f, st); break;
        default: launch_fwd_lpbq<bf16_t, MathAutogradQdq<AHQ_BF16, false>>(p, a, f, st); break;
    }
    return check_launch("ahq_lpbq_qdq_forward");
}

extern "C" int ahq_dlq_fp8_qdq(int32_t dtype, const ahq_layout* layout, const void* x, void* y, const float* scale,
                               int32_t mantissa_bits, int32_t exponent_min, float max_value, void* stream) {
    if (dtype != AHQ_F32) return set_error("FP8 quantize-dequantize supports float tensors only"), AHQ_ERR_UNSUPPORTED;
    if (!layout) return set_error("layout is null"), AHQ_ERR_INVALID;
    if (!scale) return set_error("scale is null"), AHQ_ERR_INVALID;
    if (mantissa_bits < 0 || mantissa_bits > 23 || exponent_min < -126 || exponent_min > 127 || !(max_value > 0.f))
        return set_error("bad FP8 format description"), AHQ_ERR_INVALID;
    Plan p;
    if (!make_plan(dtype, *layout, aligned16(x) && aligned16(y), false, &p, kFwdUnroll)) return AHQ_ERR_INVALID;
    if (p.cl.numel == 0) return AHQ_OK;
    if (!x || !y) return set_error("x or y is null"), AHQ_ERR_INVALID;
    QdqArgs a{};
    a.x = x;
    a.y = y;
    a.scale = scale;
    ahq_grid grid{};
    grid.compute_dtype = AHQ_F32;
    fill_args(grid, p, &a);
    a.gc.qmin = (float)exponent_min;
    a.gc.qmax = max_value;
    a.gc.zps = (float)mantissa_bits;
    hipStream_t st = static_cast<hipStream_t>(stream);
    launch_fwd<float, MathDlqFp8>(p, a, st, aligned16(x) && aligned16(y));
    return check_launch("ahq_dlq_fp8_qdq");
}

// One encoding by value over a flat tensor of `count` elements.
static bool flat_plan(int32_t dtype, uint64_t count, const void* x, const void* y, Plan* p, bool* aligned) {
    if (count > (uint64_t)1 << 62) return set_error("count too large"), false;
    ahq_layout layout{};
    layout.ndim = 1;
    layout.dims[0] = (int64_t)count;
    layout.block[0] = count ? (int64_t)count : 1;
    layout.enc_stride[0] = 0;
    *aligned = aligned16(x) && aligned16(y);
    return make_plan(dtype, layout, *aligned, false, p, kFwdUnroll);
}

extern "C" int ahq_dlq_qdq_per_tensor(int32_t dtype, const void* x, void* y, uint64_t count, double enc_min,
                                      double enc_max, double delta, double offset, void* stream) {
    if (dtype < AHQ_F32 || dtype > AHQ_BF16) return set_error("bad dtype"), AHQ_ERR_INVALID;
    Plan p;
    bool al;
    if (!flat_plan(dtype, count, x, y, &p, &al)) return AHQ_ERR_INVALID;
    if (p.cl.numel == 0) return AHQ_OK;
    if (!x || !y) return set_error("x or y is null"), AHQ_ERR_INVALID;
    ahq_grid grid{};
    grid.arith = AHQ_ARITH_DLQ;
    grid.op = AHQ_OP_QDQ;
    grid.io_dtype = dtype;
    grid.compute_dtype = AHQ_F32;
    QdqArgs a{};
    a.x = x;
    a.y = y;
    a.by_value = 1;
    // the encoding's doubles narrowed to float, as quantizeDequantizeCpu / Gpu do (trim_functions.cpp:211-226)
    a.value_enc[0] = (float)delta;
    a.value_enc[1] = (float)offset;
    a.value_enc[2] = (float)enc_min;
    a.value_enc[3] = (float)enc_max;
    fill_args(grid, p, &a);
    hipStream_t st = static_cast<hipStream_t>(stream);
    AHQ_IO_SWITCH(dtype, (launch_fwd<IO, MathDlq>(p, a, st, al)));
    return check_launch("ahq_dlq_qdq_per_tensor");
}

extern "C" int ahq_dlq_fp8_qdq_per_tensor(int32_t dtype, const void* x, void* y, uint64_t count, double delta,
                                          int32_t mantissa_bits, int32_t exponent_min, float max_value, void* stream) {
    if (dtype != AHQ_F32) return set_error("FP8 quantize-dequantize supports float tensors only"), AHQ_ERR_UNSUPPORTED;
    if (mantissa_bits < 0 || mantissa_bits > 23 || exponent_min < -126 || exponent_min > 127 || !(max_value > 0.f))
        return set_error("bad FP8 format description"), AHQ_ERR_INVALID;
    Plan p;
    bool al;
    if (!flat_plan(dtype, count, x, y, &p, &al)) return AHQ_ERR_INVALID;
    if (p.cl.numel == 0) return AHQ_OK;
    if (!x || !y) return set_error("x or y is null"), AHQ_ERR_INVALID;
    QdqArgs a{};
    a.x = x;
    a.y = y;
    a.by_value = 1;
    a.value_enc[0] = (float)delta;
    ahq_grid grid{};
    grid.compute_dtype = AHQ_F32;
    fill_args(grid, p, &a);
    a.gc.qmin = (float)exponent_min;
    a.gc.qmax = max_value;
    a.gc.zps = (float)mantissa_bits;
    launch_fwd<float, MathDlqFp8>(p, a, static_cast<hipStream_t>(stream), al);
    return check_launch("ahq_dlq_fp8_qdq_per_tensor");
}

static int float_cast_impl(const char* what, int stage_flags, int32_t dtype, const ahq_layout* layout, const void* x,
                           void* y, const float* scale, int32_t mantissa_bits, int32_t exponent_min, float max_value,
                           int32_t overflow_to_nan, int32_t unsigned_zero, int32_t logarithm_form, void* stream) {
    if (dtype < AHQ_F32 || dtype > AHQ_BF16) return set_error("bad dtype"), AHQ_ERR_INVALID;
    if (!layout) return set_error("layout is null"), AHQ_ERR_INVALID;
    if (!scale) return set_error("scale is null"), AHQ_ERR_INVALID;
    if (!(stage_flags & kCastRescaleOnly) &&
        (mantissa_bits < 0 || mantissa_bits > 23 || exponent_min < -126 || exponent_min > 127 || !(max_value > 0.f)))
        return set_error("bad float format description"), AHQ_ERR_INVALID;
    Plan p;
    if (!make_plan(dtype, *layout, aligned16(x) && aligned16(y), false, &p, kFwdUnroll)) return AHQ_ERR_INVALID;
    if (p.cl.numel == 0) return AHQ_OK;
    if (!x || !y) return set_error("x or y is null"), AHQ_ERR_INVALID;
    QdqArgs a{};
    a.x = x;
    a.y = y;
    a.scale = scale;
    ahq_grid grid{};
    grid.compute_dtype = dtype;
    fill_args(grid, p, &a);
    a.gc.qmin = (float)exponent_min;
    a.gc.qmax = max_value;
    a.gc.zps = (float)mantissa_bits;
    a.gc.flags = (overflow_to_nan ? kCastOverflowNaN : 0) | (unsigned_zero ? kCastUnsignedZero : 0) |
                 (logarithm_form ? kCastLogForm : 0) | stage_flags;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == AHQ_F32) launch_fwd<float, MathFloatCast<AHQ_F32>>(p, a, st, aligned16(x) && aligned16(y));
    else if (dtype == AHQ_F16) launch_fwd<f16_t, MathFloatCast<AHQ_F16>>(p, a, st, aligned16(x) && aligned16(y));
    else launch_fwd<bf16_t, MathFloatCast<AHQ_BF16>>(p, a, st, aligned16(x) && aligned16(y));
    return check_launch(what);
}

extern "C" int ahq_float_qdq(int32_t dtype, const ahq_layout* layout, const void* x, void* y, const float* scale,
                             int32_t mantissa_bits, int32_t exponent_min, float max_value, int32_t overflow_to_nan,
                             int32_t unsigned_zero, int32_t logarithm_form, void* stream) {
    return float_cast_impl("ahq_float_qdq", 0, dtype, layout, x, y, scale, mantissa_bits, exponent_min, max_value,
                           overflow_to_nan, unsigned_zero, logarithm_form, stream);
}

extern "C" int ahq_float_quantize(int32_t dtype, const ahq_layout* layout, const void* x, void* y, const float* scale,
                                  int32_t mantissa_bits, int32_t exponent_min, float max_value,
                                  int32_t overflow_to_nan, int32_t unsigned_zero, int32_t logarithm_form,
                                  void* stream) {
    return float_cast_impl("ahq_float_quantize", kCastKeepScaled, dtype, layout, x, y, scale, mantissa_bits,
                           exponent_min, max_value, overflow_to_nan, unsigned_zero, logarithm_form, stream);
}

extern "C" int ahq_float_dequantize(int32_t dtype, const ahq_layout* layout, const void* x, void* y,
                                    const float* scale, void* stream) {
    return float_cast_impl("ahq_float_dequantize", kCastRescaleOnly, dtype, layout, x, y, scale, 0, 0, 1.f, 0, 0, 0,
                           stream);
}

extern "C" size_t ahq_qdq_backward_workspace_bytes(const ahq_grid* grid, const ahq_layout* layout, int want_param_grads) {
    if (!grid || !layout) return 0;
    const bool pg = want_param_grads != 0;
    Plan p;
    if (!make_plan(grid->io_dtype, *layout, true, pg, &p, kUnroll, true)) return 0;
    size_t a = bwd_scratch_pairs(grid->io_dtype, p, true, pg) * 2 * sizeof(double);
    // an unaligned tensor falls back to the scalar path whose strategy may need a different amount
    Plan q;
    if (make_plan(grid->io_dtype, *layout, false, pg, &q, kUnroll, true)) {
        const size_t b = bwd_scratch_pairs(grid->io_dtype, q, false, pg) * 2 * sizeof(double);
        if (b > a) a = b;
    }
    return a;
}

extern "C" int ahq_qdq_backward(const ahq_grid* grid, const ahq_layout* layout, const void* g, const void* x, void* gx,
                                float* gscale, float* goffset, const float* scale, const float* offset, void* workspace,
                                size_t workspace_bytes, void* stream) {
    if (!validate_grid(grid, true)) return AHQ_ERR_INVALID;
    if (!layout) return set_error("layout is null"), AHQ_ERR_INVALID;
    if (!scale) return set_error("scale is null"), AHQ_ERR_INVALID;
    if ((gscale == nullptr) != (goffset == nullptr)) return set_error("gscale and goffset must be given together"), AHQ_ERR_INVALID;
    const bool want_pg = gscale != nullptr;
    if (want_pg && grid->arith == AHQ_ARITH_ATEN) return set_error("the ATen arithmetic has no scale/offset gradient"), AHQ_ERR_INVALID;
    Plan p;
    const bool al = aligned16(x) && aligned16(g) && (!gx || aligned16(gx));
    if (!make_plan(grid->io_dtype, *layout, al, want_pg, &p, kUnroll, true)) return AHQ_ERR_INVALID;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (p.cl.numel == 0) return AHQ_OK;  // nothing to read: outputs are left untouched
    if (!x || !g) return set_error("x or g is null"), AHQ_ERR_INVALID;
    if (!gx && !want_pg) return AHQ_OK;
    const bool cols = bwd_cols_layout(grid->io_dtype, p, al);
    const size_t ws_need = bwd_scratch_pairs(grid->io_dtype, p, al, want_pg) * 2 * sizeof(double);
    if (ws_need > 0 && (!workspace || workspace_bytes < ws_need)) return set_error("workspace too small"), AHQ_ERR_WORKSPACE;
    QdqArgs a{};
    a.x = x;
    a.g = g;
    a.gx = gx;
    a.scale = scale;
    a.offset = offset;
    a.gscale = gscale;
    a.goffset = goffset;
    a.partials = ws_need ? static_cast<double*>(workspace) : nullptr;
    fill_args(*grid, p, &a);
    const bool atomic = p.red == kRedAtomic && !cols;
    if (atomic) {
        const int64_t n = p.cl.num_enc * 2;
        hipLaunchKernelGGL(zero_f64_kernel, dim3((unsigned)((n + 255) / 256 > 1024 ? 1024 : (n + 255) / 256)), dim3(256), 0, st, a.partials, n);
    }
    AHQ_IO_SWITCH(grid->io_dtype, AHQ_MATH_SWITCH(*grid, (launch_bwd<IO, M>(p, a, st, al))));
    if (p.red == kRedTile) {
        const int64_t per_enc = p.mode == kRows ? p.cl.I * (int64_t)p.tpr : (int64_t)p.nblocks;
        if (per_enc > 1) {
            const int64_t waves = kFinishThreads / kWave;
            const int64_t nb = p.mode == kRows ? (p.cl.J + waves - 1) / waves : 1;
            hipLaunchKernelGGL(qdq_bwd_finish_kernel, dim3((unsigned)(nb > 4096 ? 4096 : nb)), dim3(kFinishThreads), 0, st, a);
        }
    }
    if (atomic) {
        const int64_t n = p.cl.num_enc;
        hipLaunchKernelGGL(finish_atomic_kernel, dim3((unsigned)((n + 255) / 256 > 1024 ? 1024 : (n + 255) / 256)), dim3(256), 0, st,
                           (const double*)a.partials, gscale, goffset, n, (int)grid->compute_dtype);
    }
    if (want_pg && (cols || (p.red == kRedRuns && p.cl.I > 1))) {
        // one slot per (row group, encoding) or per run: added up per encoding in a fixed order
        const int64_t count = cols ? (int64_t)bwd_cols_row_groups(grid->io_dtype, p) : p.cl.I;
        const int64_t nb = (p.cl.J + kBlock / kWave - 1) / (kBlock / kWave);
        hipLaunchKernelGGL(qdq_bwd_strided_finish_kernel, dim3((unsigned)(nb > 4096 ? 4096 : nb)), dim3(kBlock), 0, st,
                           (const double*)a.partials, count, p.cl.J, p.cl.J, gscale, goffset, (int)grid->compute_dtype);
    }
    return check_launch("ahq_qdq_backward");
}
