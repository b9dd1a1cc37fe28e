// Shared by the fake-quantization translation units (qdq.hip: forward kernels; qdq_bwd.hip: backward kernels):
// the three arithmetics, the kernel arguments, the staging of a tile's encodings in LDS and the host-side dispatch
// helpers.
//
// One streaming pass per tensor: every element is read once and written once (forward: x -> y [+ 1-byte mask];
// backward: g, x -> gx [+ per-encoding scale/offset gradients]).  Threads move 16-byte vectors; a workgroup owns a
// tile of vectors (kBlock x kFwdUnroll forward, kBwdTileVec backward) and first stages the encodings its tile touches
// in LDS, so per-channel and blockwise scales are fetched from memory once per tile with one coalesced load.
//
// Arithmetic reproduced (see include/aimet_amd.h for the reference locations):
//   AHQ_ARITH_ATEN      reciprocal multiply, round-half-even, clamp on the code          (fp32 math)
//   AHQ_ARITH_AUTOGRAD  true division, round-half-even, every intermediate rounded to the compute dtype
//   AHQ_ARITH_DLQ       clamp on the value, true division, round-half-away-from-zero     (fp32 math)
// Built with -ffp-contract=off: fusing a multiply into an add would change the rounding of any of them.
#pragma once

#include <cstdio>

#include "ahq_device.h"
#include "ahq_host.h"
#include "layout.h"
#include "tiling.h"

namespace ahq {

// Vectors per thread and tile.  Measured on tensors that come from HBM (buffers taken in rotation, nothing cached),
// bare kernels of the same shapes, one tile per workgroup of 256 threads: one read + one write runs at 0.735 of the
// 8 TB/s peak with two 16-byte loads per lane in flight and 0.80 with one; two reads + one write at 0.70 with four per
// stream, 0.76 with two, 0.80 with one -- always with non-temporal loads, which are worth 4 to 8 % there.  On this
// memory system a wave with fewer bytes in flight is answered sooner, and the workgroups are plentiful.
constexpr int kFwdUnroll = 2;
// A backward tile is one round of kBwdUnroll vectors per lane and stream, or -- when that makes a whole row of a
// per-channel tensor one tile, so that its sums need no second launch (4096 float32 values per row: 35.9 against
// 37.5 us) -- kBwdRounds such rounds one after the other: the loads of a round are issued when the round before has
// been worked off, so a lane never has more than kBwdUnroll loads per stream in flight.  Two rounds everywhere cost
// 5 % where no launch is saved.
constexpr int kBwdUnroll = 2;
constexpr int kBwdRounds = 2;
constexpr int kBwdTileUnroll = kBwdUnroll * kBwdRounds;
constexpr int kBwdTileVec = kBlock * kBwdTileUnroll;
constexpr int kStage = kBwdTileVec + 2;  // most encodings a tile can touch

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
    static constexpr bool kHasBwd = true;  // the input gradient of the exact form (formats with a storage type)
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
        return rnd<CD>(to_format(t, g)) * back;  // last rounding by the caller
    }
    // the conversion to the simulated storage type and back: round to nearest even on its grid, overflow as it does
    __device__ static float to_format(float t, const GridC& g) {
        int ex = __builtin_amdgcn_frexp_expf(t) - 1;
        ex = ex < (int)g.qmin ? (int)g.qmin : ex;
        const int sh = ex - (int)g.zps;
        float v = __builtin_ldexpf(__builtin_rintf(__builtin_ldexpf(t, -sh)), sh);
        if (__builtin_fabsf(v) > g.qmax)
            v = (g.flags & kCastOverflowNaN) ? __builtin_nanf("") : __builtin_copysignf(__builtin_inff(), v);
        if ((g.flags & kCastUnsignedZero) && v == 0.f) v = 0.f;
        return v;
    }
    // What autograd derives for the reference's composition with a storage type (float/quantizer.py:687-710:
    // div, clamp, .to(storage type), .to(dtype), mul), operation by operation and each rounded to CD:
    //   g * scale  ->  through the two casts backwards, i.e. converted to the storage type and back (the gradient
    //   is rounded onto the simulated format's grid, and overflows like any other value)  ->  times the clamp's mask
    //   (bounds included; a NaN quotient is outside)  ->  / scale.
    template <bool FAST>
    __device__ static void bwd(float gr, float x, const EncP& e, const GridC& g, float& gx, float& gs, float& goff) {
        const float t = rnd<CD>(divide<FAST, AHQ_F32>(x, e.p0, e.rs));
        const float mx = rnd<CD>(g.qmax);
        const float c = rnd<CD>(to_format(rnd<CD>(gr * e.p0), g));
        const float masked = ((t >= -mx) & (t <= mx)) ? c : 0.f;  // clamp's backward selects: +0 outside, whatever c is
        gx = rnd<CD>(masked / e.p0);  // the gradient's magnitude is not bounded like x: general division
        gs = goff = 0.f;
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
    int32_t stream_loads;  // read the tensors with non-temporal loads (see kStreamLoadBytes)
};

// a tile's load of one vector: non-temporal for large tensors (wave-uniform choice)
template <typename IO, int VEC>
__device__ __forceinline__ Pack<IO, VEC> load_pack_hinted(const IO* p, bool stream) {
    return stream ? load_pack_stream<IO, VEC>(p) : load_pack<IO, VEC>(p);
}

// The values of one encoding as the caller passed them.
struct EncRaw {
    float s, off, mn, mx;
};

__device__ __forceinline__ EncRaw load_raw_encoding(const QdqArgs& a, const Tile& t, int i) {
    int64_t e = t.e0 + i;
    if (e >= a.J) e %= a.J;
    EncRaw r;
    r.s = a.by_value ? a.value_enc[0] : a.scale[e];
    r.off = a.by_value ? a.value_enc[1] : (a.offset ? a.offset[e] : 0.f);
    r.mn = a.by_value ? a.value_enc[2] : (a.emin ? a.emin[e] : 0.f);
    r.mx = a.by_value ? a.value_enc[3] : (a.emax ? a.emax[e] : 0.f);
    return r;
}

// The encoding this thread stages first, requested ahead of the tile's elements: loads return in the order they were
// issued, so the preparation of the encodings (a division among other things) and the barrier behind it can then
// run while the elements are still in flight instead of after the last of them has arrived.
__device__ __forceinline__ EncRaw preload_encoding(const QdqArgs& a, const Tile& t) {
    EncRaw r{1.f, 0.f, 0.f, 0.f};
    if ((int)threadIdx.x < t.nstage) r = load_raw_encoding(a, t, threadIdx.x);
    return r;
}

template <typename M>
__device__ __forceinline__ void stage_encodings(const QdqArgs& a, const Tile& t, float (*sp)[kStage], const EncRaw& pre) {
    for (int i = threadIdx.x; i < t.nstage; i += kBlock) {
        const EncRaw r = i == (int)threadIdx.x ? pre : load_raw_encoding(a, t, i);
        const EncP p = M::prep(r.s, r.off, r.mn, r.mx, a.gc);
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
            // (one ballot says which lanes hold NaN; a lane looks at the bits of its own group)
            float largest = segment_max_any(raw, (int)G);
            const uint64_t group_lanes = G >= kWave ? ~0ull : (((1ull << G) - 1) << (lane & ~((int)G - 1)));
            if (__builtin_amdgcn_ballot_w64(raw != raw) & group_lanes) largest = __builtin_nanf("");  // torch.amax propagates NaN
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
                                                     const Pack<IO, VEC>* in, int base = 0) {
    if (!M::kDiv) return true;
    // One addition per element instead of a comparison each: the sum of the magnitudes is at least every magnitude
    // (rounded sums of non-negative terms never fall below a term), a NaN or an infinity makes it fail the comparison,
    // and 32 elements below the bound cannot overflow it.
    bool ok = true;
    float sum = 0.f;
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int lv = base + u * kBlock + threadIdx.x;
        if (FULL || lv < t.nv) {
            ok &= sp[M::kNP][stage_index(a, t, lv)] != 0.f;
#pragma unroll
            for (int k = 0; k < VEC; ++k) sum += __builtin_fabsf(load_f32(in[u].v[k]));
        }
    }
    return ok & (sum <= kFastDivMax);
}

// Encodings that change with every element (run length 1: per-channel along the fastest axis).  The tiled kernel
// would prepare one encoding per element; here a lane owns VEC neighbouring encodings, prepares them once and walks
// down the rows, so loads and stores stay coalesced vectors.  A workgroup is 64 lanes across x a few waves down; each
// wave takes kColUnroll rows per step.  Few waves per workgroup measured faster than many (forward 8192 x 4096 fp32:
// 43.6 us with sixteen waves, 40.8 us with four) and leave a lane more registers.
constexpr int kFwdColWaves = 4;
constexpr int kColUnroll = 2;

// The VEC neighbouring encodings of a lane, starting at column c0 (a multiple of VEC; VEC is 4 or 8).  Read as 16-byte
// vectors when the arrays allow it: read one float at a time, a wave's load touches sixteen cache lines for 256 useful
// bytes, and the 2 * VEC such loads of the set-up move as many lines through the vector cache as sixteen steps of rows.
template <typename M, int VEC>
__device__ __forceinline__ void load_col_encodings(const QdqArgs& a, int64_t c0, EncP* e) {
    if (a.by_value) {
        const EncP p = M::prep(a.value_enc[0], a.value_enc[1], a.value_enc[2], a.value_enc[3], a.gc);
#pragma unroll
        for (int k = 0; k < VEC; ++k) e[k] = p;
        return;
    }
    float s[VEC], off[VEC], mn[VEC], mx[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) off[k] = mn[k] = mx[k] = 0.f;
    const bool wide = ((reinterpret_cast<uintptr_t>(a.scale) | reinterpret_cast<uintptr_t>(a.offset) |
                        reinterpret_cast<uintptr_t>(a.emin) | reinterpret_cast<uintptr_t>(a.emax)) & 15) == 0;
    if (VEC % 4 == 0 && wide) {
#pragma unroll
        for (int k = 0; k < VEC; k += 4) {
            const Pack<float, 4> ps = load_pack<float, 4>(a.scale + c0 + k);
            Pack<float, 4> po = ps, pn = ps, px = ps;
            if (a.offset) po = load_pack<float, 4>(a.offset + c0 + k);
            if (M::kNP > 3 && a.emin) pn = load_pack<float, 4>(a.emin + c0 + k);
            if (M::kNP > 3 && a.emax) px = load_pack<float, 4>(a.emax + c0 + k);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                s[k + j] = ps.v[j];
                if (a.offset) off[k + j] = po.v[j];
                if (M::kNP > 3 && a.emin) mn[k + j] = pn.v[j];
                if (M::kNP > 3 && a.emax) mx[k + j] = px.v[j];
            }
        }
    } else {
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            s[k] = a.scale[c0 + k];
            if (a.offset) off[k] = a.offset[c0 + k];
            if (M::kNP > 3 && a.emin) mn[k] = a.emin[c0 + k];
            if (M::kNP > 3 && a.emax) mx[k] = a.emax[c0 + k];
        }
    }
#pragma unroll
    for (int k = 0; k < VEC; ++k) e[k] = M::prep(s[k], off[k], mn[k], mx[k], a.gc);
}

// the division-free form is allowed for this lane's VEC elements of one row
template <typename IO, int VEC>
__device__ __forceinline__ bool row_can_divide_fast(const Pack<IO, VEC>& p) {
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < VEC; ++k) sum += __builtin_fabsf(load_f32(p.v[k]));
    return sum <= kFastDivMax;  // fails for NaN and infinity
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
    a->stream_loads = p.cl.numel * (int64_t)io_size(grid.io_dtype) >= kStreamLoadBytes ? 1 : 0;
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

// grid of the column-walking kernels: x over groups of 64 lanes x VEC encodings, y over row groups, z over stacked
// problems; about `target` workgroups, every wave with at least one step of rows
template <int V>
static dim3 cols_grid(const Plan& p, int64_t target, int waves) {
    const int64_t gx = ((p.cl.J + V - 1) / V + kWave - 1) / kWave;
    const int64_t row_groups = (p.cl.I + (int64_t)waves * kColUnroll - 1) / ((int64_t)waves * kColUnroll);
    int64_t gy = (target + gx * p.cl.A - 1) / (gx * p.cl.A);
    gy = gy < 1 ? 1 : (gy > row_groups ? row_groups : gy);
    if (gy > 65535) gy = 65535;
    return dim3((unsigned)gx, (unsigned)gy, (unsigned)p.cl.A);
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
