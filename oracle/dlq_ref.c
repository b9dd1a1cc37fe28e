/*
 * dlq_ref.c -- TEST INFRASTRUCTURE ONLY.  A plain-C restatement of the DlQuantization CPU path (scalar loops, same
 * operation order and the same float/double types at every step).  Only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may load it; nothing under aimet_amd/ does.
 *
 * Each function names the reference lines it follows (paths relative to ModelOptimizations/DlQuantization/src).
 *
 * Pinned by (tests/test_oracle_dlq.py): the expected outputs of the reference's own tests -- broadcast QDQ vectors
 * (test/TestQuantizationFunctions.cpp:62-255), per-channel encodings and outputs (test/TestTensorQuantizer.cpp:197-300,
 * 568-728), block min/max encodings (test/TestMinMaxEncodingAnalyzer.cpp:17-130), the all-zero TF-enhanced encoding
 * (test/TestTfEnhancedEncodingAnalyzer.cpp:133-153) -- plus closed forms (uniform grids, brute-force histogram).
 * dlq_pdf_update and dlq_tfe_compute_encoding, whose results the reference's tests only bound
 * (test/TestTfEnhancedEncodingAnalyzer.cpp:57-286; those bounds are checked too), are pinned exactly: the statistics
 * on inputs at binary fractions strictly inside their buckets against a brute-force count with no slack and a
 * hand-computed running average of three unequal batches; the search against tests/tfe_enumeration.py, an
 * independent array-arithmetic statement of the algorithm (identical delta, offset, candidate index and candidate
 * count on hand-built tables, for every mode and 2/4/8/16 bits), against two searches solved by hand (first of equal
 * costs wins; the float running sum yields 101 symmetric multipliers) and on tables where the factor 3 on the
 * saturation cost decides the winner.
 *
 * Conversions of out-of-range or NaN floats to int are undefined in C; the reference relies on what x86-64 does
 * (cvttss2si yields INT_MIN).  to_int() states that behaviour explicitly.
 */
#include <float.h>
#include <limits.h>
#include <math.h>
#include <stdint.h>
#include <string.h>

#define DLQ_PDF_SIZE 1536 /* math_functions.hpp:49 */

static int to_int_f(float v) { return (v >= -2147483648.0f && v < 2147483648.0f) ? (int)v : INT_MIN; }
static int to_int_d(double v) { return (v > -2147483649.0 && v < 2147483648.0) ? (int)v : INT_MIN; }
static float fmax_std(float a, float b) { return (a < b) ? b : a; } /* std::max */
static float fmin_std(float a, float b) { return (b < a) ? b : a; } /* std::min */
static double dmax_std(double a, double b) { return (a < b) ? b : a; }
static double dmin_std(double a, double b) { return (b < a) ? b : a; }
static double dclamp(double v, double lo, double hi) { return (v < lo) ? lo : (hi < v) ? hi : v; } /* std::clamp */

/* ------------------------------------------------------------------ quantize-dequantize ---------------------------
 * quantizeValueCpu / dequantizeValueCpu with EncType = float, ROUND_NEAREST (trim_functions.cpp:177-209) */
static float qdq_value(float x, float emin, float emax, float delta, float offset) {
    float v = isnan(x) ? emin : x;
    v = fmaxf(fminf(v, emax), emin);
    v = v / delta - offset;
    v = roundf(v);
    return delta * (v + offset);
}

/* quantizeDequantizeCpu (trim_functions.cpp:211-241); encoding fields are doubles narrowed to float */
void dlq_qdq(const float* in, uint64_t cnt, double emin, double emax, double delta, double offset, float* out) {
    for (uint64_t i = 0; i < cnt; ++i) out[i] = qdq_value(in[i], (float)emin, (float)emax, (float)delta, (float)offset);
}

/* quantizeDequantizeBroadcast (trim_functions.cpp:909-948 -> 724-789) with getBroadcastableShapes
 * (tensor_utils.cpp:28-58): the encoding shape is right-aligned against the tensor shape; a tensor dim d that is a
 * multiple of the encoding dim e splits into (e, d/e).  enc is [E][4] = min, max, delta, offset.
 * Returns 0, or 1 when the shapes do not broadcast. */
int dlq_qdq_broadcast(const float* in, float* out, const int64_t* tshape, int tnd, const int64_t* eshape, int end_,
                      const double* enc) {
    int64_t bt[16], be[16];
    int nd = 0;
    if (end_ > tnd || tnd > 8) return 1;
    for (int i = 0; i < tnd; ++i) {
        const int64_t d1 = tshape[i];
        const int64_t d2 = (i < tnd - end_) ? 1 : eshape[i - (tnd - end_)];
        if (d1 == d2 || (d1 == 1 && d2 == 1)) {
            bt[nd] = d1; be[nd] = d2; ++nd;
        } else {
            if (d1 < d2 || d1 % d2 != 0) return 1;
            bt[nd] = d2; be[nd] = d2; ++nd;
            bt[nd] = d1 / d2; be[nd] = 1; ++nd;
        }
    }
    int64_t estride[16], s = 1, numel = 1;
    for (int i = nd - 1; i >= 0; --i) { estride[i] = (be[i] == 1) ? 0 : s; s *= be[i]; numel *= bt[i]; }
    int64_t coords[16];
    memset(coords, 0, sizeof coords);
    int64_t ei = 0;
    for (int64_t i = 0; i < numel; ++i) {
        const double* e = enc + 4 * ei;
        out[i] = qdq_value(in[i], (float)e[0], (float)e[1], (float)e[2], (float)e[3]);
        for (int d = nd - 1; d >= 0; --d) {
            if (++coords[d] < bt[d]) { ei += estride[d]; break; }
            coords[d] = 0;
            ei -= estride[d] * (bt[d] - 1);
        }
    }
    return 0;
}

/* ------------------------------------------------------------------ FP8 fake-cast ---------------------------------
 * fakeCastToFp8<float> (trim_functions.cpp:49-67) under round-to-nearest-even, and quantizeDequantizeFp8Cpu
 * (trim_functions.cpp:243-258): out = fakeCast(in / scale) * scale, scale = float(encoding.delta). */
static float fake_cast_fp8(float value, int mantissa_bits, int exponent_min, float max_value) {
    value = (value < -max_value) ? -max_value : (max_value < value) ? max_value : value; /* std::clamp */
    int exponent;
    frexpf(value, &exponent);
    exponent = (exponent - 1 < exponent_min) ? exponent_min : exponent - 1;
    const float step = ldexpf(1.0f, exponent - mantissa_bits);
    return nearbyintf(value / step) * step;
}

void dlq_fp8_qdq(const float* in, uint64_t cnt, double delta, int mantissa_bits, int exponent_min, double max_value,
                 float* out) {
    const float scale = (float)delta;
    for (uint64_t i = 0; i < cnt; ++i)
        out[i] = fake_cast_fp8(in[i] / scale, mantissa_bits, exponent_min, (float)max_value) * scale;
}

/* ------------------------------------------------------------------ min/max statistics ----------------------------
 * GetMin_cpu / GetMax_cpu (math_functions.cpp:324-345): std::min / std::max folds, so NaN never replaces the running
 * value and the minimum starts from FLT_MAX */
void dlq_minmax(const float* data, uint64_t cnt, float* mn, float* mx) {
    float lo = FLT_MAX, hi = -FLT_MAX;
    for (uint64_t i = 0; i < cnt; ++i) {
        lo = fmin_std(lo, data[i]);
        hi = fmax_std(hi, data[i]);
    }
    *mn = lo;
    *mx = hi;
}

/* getComputedEncodings (quantization_utils.cpp:23-99).  out = min, max, delta, offset, bw.
 * Returns 0, or 1 where the reference throws (zero-point shift with an unsupported mode). */
int dlq_computed_encodings(int bw, double min, double max, int symmetric, int strict, int unsigned_sym, double zps,
                           double* out) {
    double num_steps = pow(2, bw) - 1;
    if (symmetric && strict) num_steps -= 1;
    const double F32_MIN = (double)(-FLT_MAX) * 0.99;
    const double F32_MAX = (double)FLT_MAX * 0.99;
    min = dclamp(min, F32_MIN, 0.0);
    max = dclamp(max, 0.0, F32_MAX);
    unsigned_sym = unsigned_sym && (min >= 0.0);
    if (zps != 0.0 && (!symmetric || unsigned_sym || strict)) return 1;
    const double min_scale = dmin_std(0.01 / num_steps, (double)FLT_EPSILON);
    double delta, offset;
    if (symmetric && !unsigned_sym) {
        double pos = floor(num_steps / 2) + zps;
        const double neg = num_steps - pos;
        if (num_steps == 3 && zps == 0.0) pos = neg;
        delta = dmax_std(dmax_std(max / pos, -min / neg), min_scale); /* std::max({a, b, c}) */
        offset = -neg;
    } else {
        delta = dmax_std((max - min) / num_steps, min_scale);
        offset = dclamp(round(min / delta), -num_steps, 0.0);
    }
    if (offset < 0) delta = dmin_std(delta, F32_MIN / offset);
    if (offset + num_steps > 0) delta = dmin_std(delta, F32_MAX / (offset + num_steps));
    out[0] = delta * offset;
    out[1] = delta * (offset + num_steps);
    out[2] = delta;
    out[3] = offset;
    out[4] = bw;
    return 0;
}

/* MinMaxEncodingAnalyzer::computeEncoding for one block (MinMaxEncodingAnalyzer.cpp:97-119): float statistics, zero
 * forced into the range, then getComputedEncodings in double */
int dlq_minmax_encoding(float stat_min, float stat_max, int bw, int symmetric, int strict, int unsigned_sym, double zps,
                        double* out) {
    const double new_min = fmin_std(0.0f, stat_min);
    const double new_max = fmax_std(0.0f, stat_max);
    return dlq_computed_encodings(bw, new_min, new_max, symmetric, strict, unsigned_sym, zps, out);
}

/* ------------------------------------------------------------------ TF-enhanced statistics ------------------------ */
typedef struct {
    double xleft[DLQ_PDF_SIZE];
    double pdf[DLQ_PDF_SIZE];
    int32_t iterations;
    int32_t initialized;   /* xLeft.size() != 0 */
    int32_t stats_updated; /* _statsUpdated */
    int32_t pad;
} dlq_pdf;

void dlq_pdf_init(dlq_pdf* p) { memset(p, 0, sizeof *p); } /* a freshly constructed analyzer */

/* resetStats (TfEnhancedEncodingAnalyzer.cpp:44-50): the histogram goes, _statsUpdated stays as it was */
void dlq_pdf_reset(dlq_pdf* p) {
    const int32_t updated = p->stats_updated;
    memset(p, 0, sizeof *p);
    p->stats_updated = updated;
}

/* InitializePdf<float>, signed values (math_functions.cpp:190-234) */
static void pdf_initialize(dlq_pdf* p, float min_val, float max_val) {
    if (min_val == max_val) max_val = fmax_std(max_val, min_val + (float)0.01);
    const float center = (max_val + min_val) / 2;
    min_val = fmax_std((float).99 * -FLT_MAX, center - 3 * (center - min_val));
    max_val = fmin_std((float).99 * FLT_MAX, center + 3 * (max_val - center));
    const double bucket = ((double)max_val - (double)min_val) / DLQ_PDF_SIZE;
    for (int i = 0; i < DLQ_PDF_SIZE; ++i) {
        p->xleft[i] = floor(min_val / bucket + i) * bucket;
        p->pdf[i] = 0.0;
    }
    p->iterations = 0;
    p->initialized = 1;
}

/* TfEnhancedEncodingAnalyzer::updateStats -> UpdatePdf<float> (TfEnhancedEncodingAnalyzer.cpp:34-42,
 * math_functions.cpp:236-285) with GetHistogram_cpu (math_functions.cpp:364-381).  hist_out (optional) receives this
 * batch's integer histogram. */
void dlq_pdf_update(dlq_pdf* p, const float* data, uint64_t cnt, uint32_t* hist_out) {
    p->stats_updated = 1;
    if (hist_out) memset(hist_out, 0, sizeof(uint32_t) * DLQ_PDF_SIZE);
    if (cnt == 0) return;
    if (!p->initialized) {
        float mn, mx;
        dlq_minmax(data, cnt, &mn, &mx);
        if (mn == 0 && mx == 0) return;
        pdf_initialize(p, mn, mx);
    }
    const double bucket = p->xleft[1] - p->xleft[0];
    const double min_val = p->xleft[0];
    const int pdf_offset = to_int_d(round(min_val / bucket));
    uint32_t hist[DLQ_PDF_SIZE];
    memset(hist, 0, sizeof hist);
    const float inv_bucket = (float)(1 / bucket);
    for (uint64_t i = 0; i < cnt; ++i) {
        /* floor() of a float stays a float; float - int is evaluated in float, then truncated to int */
        const int index = to_int_f(floorf(data[i] * inv_bucket) - (float)pdf_offset);
        if (index >= 0 && index < DLQ_PDF_SIZE) hist[index] += 1;
    }
    for (int i = 0; i < DLQ_PDF_SIZE; ++i) {
        const double prob = (double)hist[i] / (double)cnt;
        p->pdf[i] = (p->pdf[i] * p->iterations + prob) / (p->iterations + 1);
    }
    p->iterations++;
    if (hist_out) memcpy(hist_out, hist, sizeof hist);
}

/* ------------------------------------------------------------------ TF-enhanced search ---------------------------- */
#define DLQ_MAX_CAND 512
typedef struct { float delta; int offset; } cand_t;

/* _clampToObservedMinMax (TfEnhancedEncodingAnalyzer.cpp:129-155) */
static int clamp_to_observed(float obs_min, float obs_max, float num_steps, float* delta, int* offset) {
    float tmin = fmax_std(*delta * *offset, -FLT_MAX);
    float tmax = fmin_std(*delta * (*offset + num_steps), FLT_MAX);
    if (tmin < obs_min && tmax > obs_max) return 0;
    tmin = fmax_std(obs_min, tmin);
    tmax = fmin_std(obs_max, tmax);
    if (tmin == tmax) return 0;
    *delta = (float)(((double)tmax - tmin) / num_steps);
    *offset = to_int_f(roundf(tmin / *delta));
    return 1;
}

/* _pickTestCandidatesAsymmetric (TfEnhancedEncodingAnalyzer.cpp:157-194) */
static int pick_asymmetric(float obs_min, float obs_max, float num_steps, cand_t* c) {
    int n = 0;
    const float obs_delta = (float)(((double)obs_max - (double)obs_min) / num_steps);
    const int obs_offset = to_int_f(roundf(obs_min / obs_delta));
    obs_min = fmax_std(obs_delta * obs_offset, -FLT_MAX);
    obs_max = fmin_std(obs_delta * (obs_offset + num_steps), FLT_MAX);
    const float delta_max = obs_delta;
    for (float f = 1.0 / 16; f <= 1 + 1.0 / 16; f += 1.0 / 16) {
        for (int i = 0; i <= 20; ++i) {
            float test_delta = f * delta_max;
            int test_offset = to_int_d(-num_steps + num_steps / 20.0 * i);
            if (!clamp_to_observed(obs_min, obs_max, num_steps, &test_delta, &test_offset)) continue;
            c[n].delta = test_delta;
            c[n].offset = test_offset;
            ++n;
        }
    }
    c[n].delta = obs_delta;
    c[n].offset = obs_offset;
    return n + 1;
}

/* _pickTestCandidatesSymmetric (TfEnhancedEncodingAnalyzer.cpp:196-233) */
static int pick_symmetric(float min_val, float max_val, float num_steps, int unsigned_sym, cand_t* c) {
    float delta_max;
    int test_offset;
    if (min_val == 0.0 && unsigned_sym) {
        delta_max = max_val / num_steps;
        test_offset = 0;
    } else {
        const float abs_max = fmax_std(fabsf(max_val), fabsf(min_val));
        delta_max = (float)(abs_max / (num_steps / 2.0));
        test_offset = to_int_f(floorf(-num_steps / 2));
    }
    int n = 0;
    for (float f = 1.0 / 100; f <= 1 + 1.0 / 100 && n < DLQ_MAX_CAND; f += 1.0 / 100) {
        c[n].delta = f * delta_max;
        c[n].offset = test_offset;
        ++n;
    }
    return n;
}

/* _findRangeOfAggregateStats (TfEnhancedEncodingAnalyzer.cpp:235-271) */
static void find_range(const dlq_pdf* p, float* mn, float* mx) {
    float lo = (float)p->xleft[0], hi = (float)p->xleft[DLQ_PDF_SIZE - 1];
    for (int i = 0; i < DLQ_PDF_SIZE; ++i)
        if (p->pdf[i] > 0) { lo = (float)p->xleft[i]; break; }
    for (int i = DLQ_PDF_SIZE - 1; i > 0; --i)
        if (p->pdf[i] > 0) { hi = (float)p->xleft[i]; break; }
    lo = fmin_std(lo, 0.0f);
    hi = fmax_std(hi, 0.0f);
    hi = fmax_std(hi, lo + (float)0.01);
    *mn = lo;
    *mx = hi;
}

/* _quantAndSatCost (TfEnhancedEncodingAnalyzer.cpp:273-335); pow(x, 2) is x*x */
static double quant_and_sat_cost(const dlq_pdf* p, const float* centers, int bw, float delta, int offset) {
    const float min_val = delta * offset;
    const float step_size = (float)(pow(2, bw) - 1);
    const float max_val = delta * (offset + step_size);
    const float pdf_start = (float)p->xleft[0];
    const double pdf_step = p->xleft[1] - p->xleft[0];
    int min_ind = to_int_d(floor((min_val - pdf_start) / pdf_step));
    min_ind = min_ind < 0 ? 0 : min_ind > DLQ_PDF_SIZE - 1 ? DLQ_PDF_SIZE - 1 : min_ind;
    int max_ind = to_int_d(floor((max_val - pdf_start) / pdf_step));
    max_ind = max_ind < 0 ? 0 : max_ind > DLQ_PDF_SIZE - 1 ? DLQ_PDF_SIZE - 1 : max_ind;
    double sat_bottom = 0;
    const float min_mid = centers[min_ind];
    for (int i = 0; i < min_ind; ++i) {
        const double mid = centers[i];
        const double d = mid - min_mid;
        sat_bottom += p->pdf[i] * (d * d);
    }
    double sat_top = 0;
    const float max_mid = centers[max_ind];
    for (int i = max_ind; i < DLQ_PDF_SIZE; ++i) {
        const double mid = centers[i];
        const double d = mid - max_mid;
        sat_top += p->pdf[i] * (d * d);
    }
    double quant = 0;
    const float inv_delta = 1 / delta;
    for (int i = min_ind; i < max_ind; ++i) {
        const float v = centers[i];
        const float deq = floorf(v * inv_delta + 0.5f) * delta;
        const double d = (double)(v - deq);
        quant += p->pdf[i] * (d * d);
    }
    const double cost = 3.0f * (sat_bottom + sat_top) + quant;
    return dmin_std(cost, DBL_MAX);
}

/* TfEnhancedEncodingAnalyzer::computeEncoding + getComputedEncodings + _findBestCandidate
 * (TfEnhancedEncodingAnalyzer.cpp:52-127, 337-377).  out = min, max, delta, offset, bw; cand_out (optional) receives
 * the number of candidates and best_out the index of the chosen one. */
void dlq_tfe_compute_encoding(const dlq_pdf* p, int bw, int symmetric, int strict, int unsigned_sym, double* out,
                              int* cand_out, int* best_out) {
    float num_steps = (float)(pow(2, bw) - 1);
    memset(out, 0, 5 * sizeof(double));
    if (cand_out) *cand_out = 0;
    if (best_out) *best_out = -1;
    if (!p->initialized) {
        if (p->stats_updated) {
            double mn = -1, mx = 1;
            const double delta = (mx - mn) / (int)num_steps;
            const double offset = floor(mn / delta);
            mn = offset * delta;
            mx = mn + (int)num_steps * delta;
            out[0] = mn; out[1] = mx; out[2] = delta; out[3] = offset; out[4] = bw;
        }
        return;
    }
    float min_val, max_val;
    find_range(p, &min_val, &max_val);
    cand_t cands[DLQ_MAX_CAND];
    int n;
    if (symmetric) {
        if (strict) num_steps -= 1;
        n = pick_symmetric(min_val, max_val, num_steps, unsigned_sym, cands);
    } else {
        n = pick_asymmetric(min_val, max_val, num_steps, cands);
    }
    const double half = (p->xleft[1] - p->xleft[0]) / 2;
    float centers[DLQ_PDF_SIZE];
    for (int i = 0; i < DLQ_PDF_SIZE; ++i) centers[i] = (float)((float)p->xleft[i] + half);
    float best_delta = -1;
    int best_offset = -1, best = -1;
    double best_cost = DBL_MAX;
    for (int k = 0; k < n; ++k) {
        const double cost = quant_and_sat_cost(p, centers, bw, cands[k].delta, cands[k].offset);
        if (cost < best_cost) { best_cost = cost; best_delta = cands[k].delta; best_offset = cands[k].offset; best = k; }
    }
    const float best_min = fmax_std(best_delta * best_offset, -FLT_MAX);
    const float best_max = fmin_std(best_delta * (best_offset + num_steps), FLT_MAX);
    out[0] = best_min; out[1] = best_max; out[2] = best_delta; out[3] = best_offset; out[4] = bw;
    if (cand_out) *cand_out = n;
    if (best_out) *best_out = best;
}

/* ------------------------------------------------------------------ percentile --------------------------------------
 * PercentileEncodingAnalyzer::computeEncoding / _computePercentileRange (PercentileEncodingAnalyzer.cpp:52-169) with
 * findOriginalRange (math_functions.cpp:401-435).  The statistics are the same PDF as the TF-enhanced analyzer's. */
void dlq_percentile_compute_encoding(const dlq_pdf* p, float percentile, int bw, int symmetric, int strict,
                                     int unsigned_sym, double* out) {
    float num_steps = (float)(pow(2, bw) - 1);
    if (symmetric && strict) num_steps -= 1;
    memset(out, 0, 5 * sizeof(double));
    if (!p->initialized) {
        if (p->stats_updated) {
            double mn = -1, mx = 1;
            const double delta = (mx - mn) / (int)num_steps;
            const double offset = floor(mn / delta);
            mn = offset * delta;
            mx = mn + (int)num_steps * delta;
            out[0] = mn; out[1] = mx; out[2] = delta; out[3] = offset; out[4] = bw;
        }
        return;
    }
    float min_val, max_val;
    find_range(p, &min_val, &max_val); /* findOriginalRange is the same search as _findRangeOfAggregateStats */
    float a_min = min_val, a_max = max_val;
    if (percentile != 100.0f) {
        const float bin_width = (float)(p->xleft[1] - p->xleft[0]);
        const float hist_min = (float)p->xleft[0];
        const float hist_max = (float)(p->xleft[DLQ_PDF_SIZE - 1] + bin_width);
        float pmin = hist_min, pmax = hist_max;
        double cdf[DLQ_PDF_SIZE];
        cdf[0] = p->pdf[0];
        for (int i = 1; i < DLQ_PDF_SIZE; ++i) cdf[i] = p->pdf[i] + cdf[i - 1];
        const float left = 1 - percentile / 100;
        for (int i = 0; i < DLQ_PDF_SIZE; ++i)
            if (cdf[i] >= left) { pmin = (float)p->xleft[i]; break; }
        const float right = percentile / 100;
        for (int i = DLQ_PDF_SIZE - 1; i >= 0; --i)
            if (cdf[i] < right && p->xleft[i] < max_val) { pmax = (float)(p->xleft[i] + bin_width); break; }
        if (pmin == pmax) pmax += bin_width;
        a_min = pmin;
        a_max = pmax;
    }
    a_min = fmin_std(a_min, 0.f);
    a_max = fmax_std(a_max, 0.f);
    dlq_computed_encodings(bw, a_min, a_max, symmetric, strict, unsigned_sym, 0.0, out);
}

/* size of dlq_pdf, for callers that allocate it from another language */
uint64_t dlq_pdf_sizeof(void) { return sizeof(dlq_pdf); }
