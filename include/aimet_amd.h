/*
 * aimet_amd.h -- C ABI of libaimet_amd.so: MI355X (gfx950) kernels for AIMET's quantization-simulation hot path.
 *
 * Conventions
 *   - every tensor pointer is a DEVICE pointer; tensors are dense and contiguous in the dimension order given
 *   - every function enqueues work on `stream` (a hipStream_t passed as void*) and returns without synchronising
 *   - return value: AHQ_OK or an ahq_status error code; ahq_last_error() returns a thread-local message
 *   - the library never allocates device memory: scratch is a caller-provided `workspace` whose required size is
 *     returned by the matching *_workspace_bytes() query (the buffer does not need to be cleared by the caller)
 *
 * Reference interfaces each entry point stands in for (paths relative to the AIMET checkout):
 *   AT  = TrainingExtensions/torch/src/python/aimet_torch
 *   DLQ = ModelOptimizations/DlQuantization
 */
#ifndef AIMET_AMD_H
#define AIMET_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AHQ_MAX_DIMS 8

typedef enum {
    AHQ_OK              = 0,
    AHQ_ERR_INVALID     = 1, /* malformed argument (null pointer, negative size, bad enum, ...) */
    AHQ_ERR_UNSUPPORTED = 2, /* well-formed request this library has no kernel for */
    AHQ_ERR_LAUNCH      = 3, /* HIP runtime reported an error */
    AHQ_ERR_WORKSPACE   = 4  /* workspace missing or too small */
} ahq_status;

typedef enum { AHQ_F32 = 0, AHQ_F16 = 1, AHQ_BF16 = 2 } ahq_dtype;

/* Which of the reference's three quantize-dequantize arithmetics to reproduce. */
typedef enum {
    /* ATen fake_quantize_per_{tensor,channel}_affine as called from AT/quantization/affine/backends/torch_builtins.py:485-491,526-533:
       inv = 1.0f/scale; q = rint(float(x)*inv) + zp; y = T((clamp(q,qmin,qmax) - zp) * scale); zp = -int32(offset) */
    AHQ_ARITH_ATEN = 1,
    /* QuantDequantFunc / QuantizeFunc / DequantizeFunc, torch_builtins.py:588-831: every intermediate rounded to the
       compute dtype; t = x/scale [- zps]; r = rint(t) - offset; y = (clamp(r,qmin,qmax) + offset [+ zps]) * scale */
    AHQ_ARITH_AUTOGRAD = 2,
    /* DlQuantization quantizeValueCpu/dequantizeValueCpu, DLQ/src/trim_functions.cpp:177-209:
       v = isnan(x) ? min : x; v = fmax(fmin(v,max),min); v = round(v/delta - offset); y = delta*(v + offset) */
    AHQ_ARITH_DLQ = 3
} ahq_arith;

typedef enum {
    AHQ_OP_QDQ = 0,       /* quantize-dequantize */
    AHQ_OP_QUANTIZE = 1,  /* integer codes stored as floating point */
    AHQ_OP_DEQUANTIZE = 2 /* (x + offset) * scale */
} ahq_op;

/*
 * How encodings map onto a dense tensor.  The tensor has `ndim` dimensions `dims[]` (row-major, dims[ndim-1]
 * fastest).  Along dimension d, `block[d]` consecutive coordinates share an encoding, and moving to the next block
 * advances the encoding index by `enc_stride[d]` (0 = the encoding is broadcast along d).  The encoding index of an
 * element with coordinates c[] is  sum_d (c[d] / block[d]) * enc_stride[d].
 *   per-tensor:               ndim=1, dims={N}, block={N}, enc_stride={0}
 *   per-channel axis 0 of RxC: dims={R,C}, block={1,C}, enc_stride={1,0}
 *   blockwise (1,B) on RxC:    dims={R,C}, block={1,B}, enc_stride={C/B,1}
 * This is the flattened form of the interleaved reshape in torch_builtins.py:285-289 and of
 * getBroadcastableShapes/shapeToStrides in DLQ/src/tensor_utils.cpp:28-77.
 */
typedef struct {
    int32_t ndim;
    int64_t dims[AHQ_MAX_DIMS];
    int64_t block[AHQ_MAX_DIMS];
    int64_t enc_stride[AHQ_MAX_DIMS];
} ahq_layout;

/* Parameters of one quantization grid. */
typedef struct {
    int32_t arith;           /* ahq_arith */
    int32_t op;              /* ahq_op */
    int32_t io_dtype;        /* ahq_dtype of x / y / g / gx */
    int32_t compute_dtype;   /* ahq_dtype every intermediate is rounded to (torch_builtins.py:268-277); == io_dtype or AHQ_F32 */
    int64_t qmin;
    int64_t qmax;
    double  zero_point_shift; /* 0.0 or 0.5 (AT/quantization/affine/quantizer.py:170-174) */
} ahq_grid;

const char* ahq_last_error(void);
int         ahq_version(void);

/* ---------------------------------------------------------------- QDQ forward / backward --------------------------
 * Replaces: torch_builtins.quantize / quantize_dequantize / dequantize (torch_builtins.py:166-302, 537-571), the ATen
 * fast path (torch_builtins.py:335-431), and for AHQ_ARITH_DLQ DlQuantization::quantizeDequantize /
 * quantizeDequantizeBroadcast (DLQ/src/trim_functions.cpp:108-128, 909-948).
 *
 * scale/offset: fp32 arrays with one entry per encoding (AHQ_ARITH_ATEN/AUTOGRAD).  For AHQ_ARITH_DLQ pass
 * enc_min/enc_max as well (the float-narrowed TfEncoding fields, DLQ/src/trim_functions.cpp:211-226); otherwise
 * they must be NULL.
 * mask_out: optional (may be NULL) one byte per element, 1 where the code was inside [qmin,qmax]
 * (torch_builtins.py:743-746).
 */
int ahq_qdq_forward(const ahq_grid* grid, const ahq_layout* layout, const void* x, void* y, uint8_t* mask_out,
                    const float* scale, const float* offset, const float* enc_min, const float* enc_max,
                    void* stream);

/* Replaces DlQuantization::quantizeDequantize<T>(in, cnt, encoding, out, COMP_MODE_GPU, ROUND_NEAREST, stream)
 * (DLQ/src/trim_functions.hpp:35-37, trim_functions.cpp:108-128), the per-tensor form BlockTensorQuantizer uses when
 * its shape has one element (DLQ/src/TensorQuantizer.cpp:106-111): the encoding travels by value, so the caller needs
 * no device copy of it.  x / y: `count` elements of `dtype`; the four doubles are the TfEncoding fields, narrowed to
 * float inside as the reference does.
 */
int ahq_dlq_qdq_per_tensor(int32_t dtype, const void* x, void* y, uint64_t count, double enc_min, double enc_max,
                           double delta, double offset, void* stream);

/* Backward of the above with the straight-through estimator (torch_builtins.py:637-655, 691-701, 779-831).  The mask
 * is recomputed from x.  gx may be NULL; gscale/goffset may be NULL (both or neither); when given they receive the
 * gradient already reduced to one fp32 value per encoding (what autograd's sum-to-size produces in the reference).
 * workspace: ahq_qdq_backward_workspace_bytes() bytes of device memory, 16-byte aligned (NULL if that is 0).
 */
size_t ahq_qdq_backward_workspace_bytes(const ahq_grid* grid, const ahq_layout* layout, int want_param_grads);
int    ahq_qdq_backward(const ahq_grid* grid, const ahq_layout* layout, const void* g, const void* x, void* gx,
                        float* gscale, float* goffset, const float* scale, const float* offset, void* workspace,
                        size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------- min / max statistics ----------------------------
 * Replaces: _MinMaxObserver.collect_stats = utils.reduce(amin/amax) (AT/quantization/encoding_analyzer.py:80-94,
 * AT/utils.py:1115-1148), _HistogramObserver._get_min_max (encoding_analyzer.py:213-219, finite_only=1) and
 * DlQuantization GetMinMax (DLQ/src/math_functions.cpp:72-117).
 * out_min/out_max: one value per encoding in the tensor's own dtype.  finite_only selects the NaN / infinity rule:
 *   0  NaN propagates like torch.amin/amax
 *   1  non-finite values are ignored (an all-non-finite slice yields +inf / -inf)
 *   2  DlQuantization's std::min / std::max folds: NaN is skipped, the minimum starts from FLT_MAX and the maximum
 *      from -FLT_MAX (math_functions.cpp:324-345); run_min/run_max are folded the same way
 * run_min/run_max (optional, both or neither): running statistics of the same shape and dtype that the batch result is
 * folded into with torch.minimum / torch.maximum semantics (_MinMaxObserver.merge_stats, encoding_analyzer.py:96-112).
 */
size_t ahq_minmax_workspace_bytes(const ahq_layout* layout);
int    ahq_minmax(int32_t dtype, const ahq_layout* layout, const void* x, void* out_min, void* out_max,
                  void* run_min, void* run_max, int finite_only, void* workspace, size_t workspace_bytes, void* stream);

/* ahq_minmax that also writes y = x (same dtype and layout, y not aliasing x).  Replaces the observe-then-clone of an
 * input / output quantizer in pass-through calibration: AffineQuantizerBase._compute_encodings(passthrough=True)
 * observes the tensor and returns torch.Tensor.clone(input) (AT/quantization/affine/quantizer.py:601-640).  With one
 * encoding the pass that reads the tensor writes the copy; other layouts reduce and copy separately.
 */
int    ahq_minmax_copy(int32_t dtype, const ahq_layout* layout, const void* x, void* y, void* out_min, void* out_max,
                       void* run_min, void* run_max, int finite_only, void* workspace, size_t workspace_bytes,
                       void* stream);

/* ahq_minmax for callers that cannot allocate device memory and have no workspace to pass: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  Same arguments and
 * results as ahq_minmax without the workspace pair: the partial extrema / per-encoding keys go to a file-scope
 * device array of AHQ_MINMAX_STATIC_SCRATCH_BYTES that every device the library runs on holds until the process ends.
 * The call allocates nothing (no hipMalloc / hipFree, no allocating library routine); the first call on a device
 * looks the array's address up (hipGetSymbolAddress), so make that call outside a capture.
 * A reduction that needs more scratch than the array holds returns AHQ_ERR_WORKSPACE and launches nothing (a
 * per-tensor reduction needs 6 KB whatever its size; others 12 bytes per encoding or per tile; per-channel along the
 * fastest axis needs 12 bytes per encoding and uses more when it is there, which is what
 * ahq_minmax_workspace_bytes() reports for that layout).
 * All calls on one device share the array: calls that overlap on one device (different streams) race; calls on one
 * stream are ordered and each clears what it needs.
 */
#define AHQ_MINMAX_STATIC_SCRATCH_BYTES (1u << 20)
int    ahq_minmax_static(int32_t dtype, const ahq_layout* layout, const void* x, void* out_min, void* out_max,
                         void* run_min, void* run_max, int finite_only, void* stream);

/* Running per-tensor extrema without a second launch per batch.  Replaces the same reference code as ahq_minmax
 * (_MinMaxObserver.collect_stats + merge_stats, AT/quantization/encoding_analyzer.py:69-118) for a single encoding when
 * the caller does not need the statistics between batches: `slots` (AHQ_MINMAX_SLOTS_BYTES bytes, 4-byte aligned,
 * owned by the caller) holds one (min, max, saw-NaN) triple per workgroup of the streaming kernel; each call folds the
 * batch into them in place (minimum and maximum are exact in any order and grouping), `first` != 0 starts them
 * afresh.  copy_to (optional) receives a copy of the `count` elements of x from the same pass.  batch_slots
 * (optional, a second array of the same size that must not alias `slots`) receives the batch's OWN partial extrema,
 * written, not merged: what update_stats() returns (the statistics of this tensor alone, :369-374) without a launch
 * that folds them.  ahq_minmax_slots_read folds either array into one (min, max) of `dtype`, with torch.amin / amax
 * semantics (NaN if any element was NaN); ahq_minmax_slots_to_encodings and ahq_minmax_slots_finalize fold them inside
 * the launch that consumes them.
 */
#define AHQ_MINMAX_SLOTS 512
#define AHQ_MINMAX_SLOTS_BYTES (12 * AHQ_MINMAX_SLOTS)
int ahq_minmax_accumulate(int32_t dtype, const void* x, int64_t count, void* copy_to, void* slots, void* batch_slots,
                          int32_t first, void* stream);
int ahq_minmax_slots_read(int32_t dtype, const void* slots, void* out_min, void* out_max, void* stream);

/* Replaces MinMaxEncodingAnalyzer.compute_encodings_from_stats (AT/quantization/encoding_analyzer.py:425-481) and the
 * checks of _flag_extreme_min_max (:484-498): zero forced into the range, ranges narrower than the minimum scale
 * widened, symmetric grids re-centred, the result clamped to the statistics dtype.  stat_min / stat_max / out_min /
 * out_max hold num_encodings values of `dtype`.  The three thresholds are passed the way torch's scalar handling
 * produces them: minimum_scale_in_dtype = the minimum scale rounded to `dtype` (the comparison), minimum_scale = the
 * same as float32 (the widening term), near_max_threshold = dtype(1e-8 + 0.05 * dtype_max).
 * flags (optional, int32[2], accumulated with OR, cleared by the caller): [0] a result is NaN or infinite, [1] a
 * result lies within 5 % of dtype_max.
 */
int ahq_minmax_to_encodings(int32_t dtype, const void* stat_min, const void* stat_max, int64_t num_encodings,
                            int64_t num_steps, int32_t symmetric, float minimum_scale_in_dtype, float minimum_scale,
                            float dtype_max, float near_max_threshold, void* out_min, void* out_max, int32_t* flags,
                            void* stream);

/* ahq_minmax_to_encodings for one encoding whose statistics lie in the slots of ahq_minmax_accumulate (the running
 * ones or a batch's own): the launch folds the slots as ahq_minmax_slots_read would and goes on from there, so a
 * per-tensor analyzer's update_stats() + compute_encodings() are two launches, not four.  stat_min / stat_max
 * (optional, one value of `dtype` each) receive the folded statistics.  The slots are only read.
 */
int ahq_minmax_slots_to_encodings(int32_t dtype, const void* slots, int64_t num_steps, int32_t symmetric,
                                  float minimum_scale_in_dtype, float minimum_scale, float dtype_max,
                                  float near_max_threshold, void* out_min, void* out_max, void* stat_min,
                                  void* stat_max, int32_t* flags, void* stream);

/* Replaces AffineQuantizerBase.get_scale / _get_offset with dtype = float32 for a quantizer that holds min / max
 * (AT/quantization/affine/quantizer.py:319-376), the half-dozen elementwise launches a quantizer spends on its first
 * forward after its range was written:
 *   scale  = clamp_min(|float(max) - float(min)| / (qmax - qmin), minimum_scale)
 *   offset = clamp(round(min / scale) - qmin, -qmax, -qmin)
 * range_min / range_max: num_encodings values of `dtype`; scale / offset: float32 outputs.  offset may be NULL (a
 * symmetric grid, whose offset is the constant -round((qmin + qmax) / 2)).  minimum_scale = _get_minimum_scale(qmax -
 * qmin) as the Python float.
 */
int ahq_range_to_scale_offset(int32_t dtype, const void* range_min, const void* range_max, int64_t num_encodings,
                              int64_t qmin, int64_t qmax, double minimum_scale, float* scale, float* offset,
                              void* stream);

/* The end of a min/max calibration in one launch: replaces, for a quantizer that holds min / max, the sequence
 * MinMaxEncodingAnalyzer.compute_encodings_from_stats (AT/quantization/encoding_analyzer.py:425-481) with the checks of
 * _flag_extreme_min_max (:484-498), set_range (AT/quantization/affine/quantizer.py:378-438: min.copy_(lo),
 * max.copy_(hi)) and the get_scale / _get_offset the next forward would run (:319-376).  The first ten arguments and
 * `flags` are those of ahq_minmax_to_encodings; the range is stored into param_min / param_max (num_encodings values
 * of `param_dtype`, rounded to nearest even from `stat_dtype` as Tensor.copy_ does), and scale / offset (float32,
 * offset may be NULL for a symmetric grid) are derived from the stored values exactly as ahq_range_to_scale_offset
 * derives them; qmin, qmax and grid_minimum_scale are that function's arguments.
 */
int ahq_minmax_finalize(int32_t stat_dtype, const void* stat_min, const void* stat_max, int64_t num_encodings,
                        int64_t num_steps, int32_t symmetric, float minimum_scale_in_dtype, float minimum_scale,
                        float dtype_max, float near_max_threshold, int32_t* flags, int32_t param_dtype,
                        void* param_min, void* param_max, int64_t qmin, int64_t qmax, double grid_minimum_scale,
                        float* scale, float* offset, void* stream);

/* ahq_minmax_finalize for a single encoding whose running extrema still lie in the slots of ahq_minmax_accumulate:
 * the launch folds the slots (as ahq_minmax_slots_read would: a NaN seen in any batch makes both statistics NaN) and
 * goes on from there, so that leaving a whole-model calibration costs one launch per activation quantizer instead of
 * two.  The slots are only read.  Remaining arguments as in ahq_minmax_finalize with num_encodings = 1.
 */
int ahq_minmax_slots_finalize(int32_t stat_dtype, const void* slots, int64_t num_steps, int32_t symmetric,
                              float minimum_scale_in_dtype, float minimum_scale, float dtype_max,
                              float near_max_threshold, int32_t* flags, int32_t param_dtype, void* param_min,
                              void* param_max, int64_t qmin, int64_t qmax, double grid_minimum_scale, float* scale,
                              float* offset, void* stream);

/* The calibration of a parameter followed by its first quantize-dequantize, as one call: what
 * BaseQuantizationMixin._compute_param_encodings (AT/nn/base.py:331-386: the parameter quantizer observes the
 * parameter inside its compute_encodings() context and sets its range on leaving it) and the quantizer's next forward
 * pass do for a min/max-calibrated affine quantizer.  The launches and the results are those of ahq_minmax on x,
 * ahq_minmax_finalize on the extrema and ahq_qdq_forward with the scale / offset just derived; a whole-model
 * calibration makes this call once per weight, and the host time of three calls with their arguments was the larger
 * part of entering it.  grid: AHQ_OP_QDQ, AHQ_ARITH_ATEN or AHQ_ARITH_AUTOGRAD, as the forward pass would choose;
 * num_steps .. grid_minimum_scale as in ahq_minmax_finalize (qmin / qmax are the grid's); scale: float32 output;
 * offset: float32, written for an asymmetric grid, READ for a symmetric one (the caller's constant offsets), one
 * value per encoding either way.  workspace: ahq_minmax_calibrate_qdq_workspace_bytes(grid->io_dtype, layout) bytes.
 */
size_t ahq_minmax_calibrate_qdq_workspace_bytes(int32_t dtype, const ahq_layout* layout);
int    ahq_minmax_calibrate_qdq(const ahq_grid* grid, const ahq_layout* layout, const void* x, void* y,
                                int64_t num_steps, int32_t symmetric, float minimum_scale_in_dtype,
                                float minimum_scale, float dtype_max, float near_max_threshold, int32_t* flags,
                                int32_t param_dtype, void* param_min, void* param_max, double grid_minimum_scale,
                                float* scale, float* offset, void* workspace, size_t workspace_bytes, void* stream);

/* Whole-model calibration, where a model's quantized modules enter and leave their compute_encodings() contexts
 * together (AT/nn/base.py:392-427 for every module of a QuantizationSimModel, AT/quantsim/quantsim.py:514-560): the
 * calls above for ALL quantizers behind one call each, in the order given, so that the host spends one call on
 * entering (every parameter: the grid test of _decompose_prequantized_tensor, then calibration + first
 * quantize-dequantize) and one on leaving (every per-tensor activation quantizer) instead of one per quantizer.
 * Each item holds the arguments of the single call of the same name; `flags` is shared by all items.  The items are
 * read on the host during the call.  Returns the first failing item's status (its index is in ahq_last_error());
 * items before it have been launched.
 * ahq_grid_probe_many: item i writes verdicts[i]; an item the single call would answer with AHQ_ERR_UNSUPPORTED gets
 * unsupported[i] = 1 (host array, optional) and no launch, and the call goes on.
 * ahq_minmax_slots_finalize_many launches one workgroup per item, 16 items per launch.
 */
typedef struct {
    int32_t dtype;
    ahq_layout layout;
    const void* x;
    int64_t num_levels;
} ahq_grid_probe_item;
int ahq_grid_probe_many(const ahq_grid_probe_item* items, int64_t count, uint8_t* verdicts, uint8_t* unsupported,
                        void* stream);

typedef struct {
    ahq_grid grid;
    ahq_layout layout;
    const void* x;
    void* y;
    int64_t num_steps;
    int32_t symmetric;
    float minimum_scale_in_dtype, minimum_scale, dtype_max, near_max_threshold;
    int32_t param_dtype;
    void* param_min;
    void* param_max;
    double grid_minimum_scale;
    float* scale;
    float* offset;
    void* workspace;
    size_t workspace_bytes;
} ahq_calibrate_qdq_item;
int ahq_minmax_calibrate_qdq_many(const ahq_calibrate_qdq_item* items, int64_t count, int32_t* flags, void* stream);

typedef struct {
    int32_t stat_dtype;
    int32_t symmetric;
    const void* slots;
    int64_t num_steps;
    float minimum_scale_in_dtype, minimum_scale, dtype_max, near_max_threshold;
    int32_t param_dtype;
    int32_t reserved;
    void* param_min;
    void* param_max;
    int64_t qmin, qmax;
    double grid_minimum_scale;
    float* scale;
    float* offset;   /* NULL for a symmetric grid */
} ahq_slots_finalize_item;
int ahq_minmax_slots_finalize_many(const ahq_slots_finalize_item* items, int64_t count, int32_t* flags, void* stream);

/* The backward pass of ahq_lpbq_scale: replaces the autograd chain of GroupedBlockQuantizeDequantize._get_scale
 * (AT/quantization/affine/quantizer.py:1363-1399 on top of :319-342) when min / max are learned -- the backward of
 * the quantize-dequantize of the block scales (AT/quantization/affine/backends/torch_builtins.py:727-831), of the
 * division by the number of multipliers, of torch.amax over each group and of get_scale -- with one launch.
 * grad_scale: float32 gradient with respect to `scale`; grad_per_channel_scale: optional float32 gradient with respect
 * to `per_channel_scale`; grad_min / grad_max: outputs in `dtype`.  Same grouping restriction as ahq_lpbq_scale.
 */
int ahq_lpbq_scale_backward(int32_t dtype, const ahq_layout* grouping, const void* range_min, const void* range_max,
                            int64_t qmin, int64_t qmax, double minimum_scale, int32_t num_multipliers,
                            const float* grad_scale, const float* grad_per_channel_scale, void* grad_min,
                            void* grad_max, void* stream);

/* The backward pass of ahq_range_to_scale_offset: replaces the autograd chain of get_scale / _get_offset
 * (AT/quantization/affine/quantizer.py:319-376) when min / max are learned -- SubBackward, DivBackward, AbsBackward,
 * ClampMinBackward and, for asymmetric grids, DivBackward, the straight-through round (AT/utils.py:1250-1257) and
 * ClampBackward -- with one launch that evaluates the same float32 operations.  grad_scale / grad_offset: float32
 * gradients with respect to scale and offset (grad_offset NULL: symmetric grid); grad_min / grad_max: outputs in
 * `dtype`, the dtype of range_min / range_max.
 */
int ahq_range_backward(int32_t dtype, const void* range_min, const void* range_max, int64_t num_encodings,
                       int64_t qmin, int64_t qmax, double minimum_scale, const float* grad_scale,
                       const float* grad_offset, void* grad_min, void* grad_max, void* stream);

/* Replaces GroupedBlockQuantizeDequantize._get_scale / _get_per_channel_scale with dtype = float32 (LPBQ,
 * AT/quantization/affine/quantizer.py:1363-1399), which the reference runs on every forward through get_encodings():
 *   raw               = clamp_min(|float(max) - float(min)| / (qmax - qmin), minimum_scale)     (quantizer.py:319-339)
 *   per_channel_scale = amax(raw over each group of blocks) / num_multipliers
 *   scale             = quantize_dequantize(raw, per_channel_scale, offset 0, qmin 1, qmax num_multipliers)
 * range_min / range_max: one value of `dtype` per block.  grouping: the layout of the GROUPS over the array of blocks
 * (dims = the quantizer shape, block = blocks per group along each dimension, enc_stride = strides of the
 * per-channel-scale array); scale: float32 per block, per_channel_scale: float32 per group.  num_multipliers =
 * 2^(decompressed_bw - bitwidth).  AHQ_ERR_UNSUPPORTED: groups whose blocks are not neighbours in memory (the caller
 * then composes ahq_range_to_scale_offset, ahq_minmax and ahq_qdq_forward, or the reference's torch form).
 */
int ahq_lpbq_scale(int32_t dtype, const ahq_layout* grouping, const void* range_min, const void* range_max,
                   int64_t qmin, int64_t qmax, double minimum_scale, int32_t num_multipliers, float* scale,
                   float* per_channel_scale, void* stream);

/* ahq_lpbq_scale and ahq_qdq_forward in one launch: the forward pass of GroupedBlockQuantizeDequantize
 * (AT/quantization/affine/quantizer.py:1363-1399 for the scale, which the reference derives before every forward, then
 * AT/quantization/affine/backends/torch_builtins.py:705-725).  Every workgroup derives the grouped scales of the blocks
 * its tile touches from range_min / range_max (one value of `range_dtype` per block, in the order of the encodings of
 * `layout`), stores them into `scale` (float32 per block, bit for bit what ahq_lpbq_scale stores; the backward pass
 * reads them) and `per_channel_scale` (float32 per group, may be NULL), and quantize-dequantizes x with them.  A group
 * is blocks_per_group encodings that follow each other in that order.  offset: float32 per block or NULL (zero).
 * minimum_scale / num_multipliers as for ahq_lpbq_scale.
 * AHQ_ERR_UNSUPPORTED (the caller then makes the two calls): another arithmetic than the autograd quantize-dequantize
 * computed in the tensor's dtype without zero-point shift, blocks that do not follow each other in memory (encodings
 * that repeat over a leading dimension, strided layouts), a number of blocks that is no multiple of blocks_per_group.
 */
int ahq_lpbq_qdq_forward(const ahq_grid* grid, const ahq_layout* layout, const void* x, void* y, uint8_t* mask_out,
                         int32_t range_dtype, const void* range_min, const void* range_max, int64_t blocks_per_group,
                         double minimum_scale, int32_t num_multipliers, const float* offset, float* scale,
                         float* per_channel_scale, void* stream);

/* Replaces the early exit of _decompose_prequantized_tensor (AT/utils.py:2098-2118), the test every weight goes
 * through when a calibration starts: of the first 64 blocks of the layout, the first 2 * num_levels elements each are
 * taken as float magnitudes; *verdict = 0 if one of those samples holds more than num_levels distinct values (the
 * tensor is not an already-quantized one), else 1.  verdict: one byte of device memory (a torch.bool element).
 * The caller handles blocks of at most num_levels elements itself (the reference skips the test for them).
 * AHQ_ERR_UNSUPPORTED: blocks along several dimensions, or num_levels above 4096.
 */
int ahq_grid_probe(int32_t dtype, const ahq_layout* layout, const void* x, int64_t num_levels, uint8_t* verdict,
                   void* stream);

/* ---------------------------------------------------------------- histogram statistics ----------------------------
 * Replaces: _HistogramObserver.collect_stats + merge_stats (AT/quantization/encoding_analyzer.py:189-332), i.e. what
 * PercentileEncodingAnalyzer / SqnrEncodingAnalyzer / TfEnhancedEncodingAnalyzer.update_stats do per batch.
 * One call: finite min/max of the batch, the batch's own num_bins-bin histogram over its own range (returned as
 * new_*), the running range widened to cover the batch (clamped to growth_limit x the first batch's range), the
 * running counts re-binned onto that range, and the batch binned onto it and added.  Bin index formula and
 * out-of-range handling are torch.histc's on CPU; counts are fp32 like the reference's.
 * All buffers are fp32 device arrays owned by the caller; hist/edges/minmax/limits persist between calls.
 * new_hist may be NULL: the batch's own histogram is then not formed, which leaves one histogram update per element
 * instead of two for every batch after the first.  new_edges and new_minmax may be NULL as well (both, and then
 * new_hist too): only the running statistics are kept up, and a batch after the first that stays inside the running
 * range is read once instead of twice (it is binned on the running range while its out-of-range elements are looked
 * for; only a batch that moves the range is binned again).  A caller that turns out to need a batch's own statistics
 * gets the same values from a first_batch call on a scratch state (collect_stats alone).
 */
typedef struct {
    int32_t num_slots;     /* number of histograms = number of encodings of the layout */
    int32_t num_bins;
    float   growth_limit;  /* >= 1; +inf for no limit (encoding_analyzer.py:138-145) */
    float*  hist;          /* [num_slots][num_bins]     running histogram */
    float*  edges;         /* [num_slots][num_bins+1]   running bin edges */
    float*  minmax;        /* [num_slots][2]            running stats.min / stats.max */
    float*  limits;        /* [num_slots][2]            range limits fixed by the first batch */
    float*  new_hist;      /* [num_slots][num_bins]     out: this batch's own histogram (optional) */
    float*  new_edges;     /* [num_slots][num_bins+1]   out (optional, with new_minmax) */
    float*  new_minmax;    /* [num_slots][2]            out: this batch's finite min / max (optional) */
} ahq_hist_state;

size_t ahq_hist_update_workspace_bytes(int32_t dtype, const ahq_layout* layout, int32_t num_bins);
int    ahq_hist_update(int32_t dtype, const ahq_layout* layout, const void* x, const ahq_hist_state* state,
                       int first_batch, void* workspace, size_t workspace_bytes, void* stream);

/* No counterpart in the reference: a tuning knob of ahq_hist_update.  A single-slot update of a 16-bit tensor that
 * forms one histogram is binned through a 64K-entry table in LDS once the tensor has at least this many elements
 * (default 48 Mi; below it filling the table costs more than it saves), and arithmetically below.  Both ways give the
 * same counts.  set >= 0 replaces the threshold (0: always the table), set < 0 only reads it; returns the value that
 * was in force before the call.  Process-wide.
 */
int64_t ahq_hist_table_min_numel(int64_t set);

/* ---------------------------------------------------------------- SQNR / TF-enhanced search ------------------------
 * Replaces: _LpNormEncodingAnalyzer._pick_test_candidates / _clamp_delta_offset_values /
 * _estimate_clip_and_quant_noise / _select_best_candidates (encoding_analyzer.py:728-899).
 * offset_grid: the rounded offsets `round(arange(-num_steps, step, step))` (encoding_analyzer.py:763-770), made by the
 * caller; num_offsets = len(offset_grid) + 1 (the observed offset is appended).  Ignored when symmetric.
 * noise/deltas/offsets: [num_slots][num_deltas][num_offsets] fp32 outputs (every candidate, for inspection).
 * out: [num_slots][4] = best delta, best offset, encoding min, encoding max; best_index: flat argmin (first minimum).
 */
typedef struct {
    int32_t num_slots, num_bins, num_deltas, num_offsets;
    int32_t symmetric;
    int32_t stat_dtype;      /* ahq_dtype the running min/max are stored in (their arithmetic happens in it) */
    int64_t num_steps;
    double  minimum_scale;   /* _get_minimum_scale(num_steps) */
    double  gamma;
    double  p;
} ahq_sqnr_params;

int ahq_sqnr_search(const ahq_sqnr_params* params, const float* hist, const float* edges, const float* minmax,
                    const float* offset_grid, float* noise, float* deltas, float* offsets, float* out,
                    long long* best_index, void* stream);

/* ---------------------------------------------------------------- DlQuantization calibration ----------------------
 * Encodings are rows of five doubles: min, max, delta, offset, bw (DLQ TfEncoding, QuantizationType.hpp).
 *
 * ahq_dlq_minmax_encodings replaces MinMaxEncodingAnalyzer::computeEncoding -> getComputedEncodings
 * (DLQ/src/MinMaxEncodingAnalyzer.cpp:97-119, DLQ/src/quantization_utils.cpp:23-99): stat_min/stat_max are the running
 * per-block float statistics (ahq_minmax with finite_only = 2); out is [num_encodings][5].  A non-zero
 * zero_point_shift with a mode the reference rejects returns AHQ_ERR_UNSUPPORTED with the reference's message.
 */
int ahq_dlq_minmax_encodings(const float* stat_min, const float* stat_max, int64_t num_encodings, int32_t bw,
                             int32_t symmetric, int32_t strict, int32_t unsigned_sym, double zero_point_shift,
                             double* out, void* stream);

/* Folds a batch's per-block extrema (values of `dtype`, e.g. the out_min / out_max of ahq_minmax with finite_only = 2
 * on a 16-bit tensor) into the running float statistics with std::min / std::max: what MinMaxEncodingAnalyzer::
 * updateStats does after widening a half / bfloat16 tensor (DLQ/src/MinMaxEncodingAnalyzer.cpp:32-95).
 */
int ahq_dlq_minmax_fold(int32_t dtype, const void* batch_min, const void* batch_max, int64_t num_encodings,
                        float* run_min, float* run_max, void* stream);

/* TF-enhanced statistics: one 1536-bucket PDF per encoding block (DLQ/src/math_functions.hpp:28-49).
 * xleft/pdf: [num_slots][AHQ_DLQ_PDF_SIZE] doubles; meta: [num_slots][4] int32 = iterations, initialized (xLeft not
 * empty), stats_updated, reserved.  All zero = a freshly constructed analyzer; resetStats zeroes everything but
 * stats_updated (DLQ/src/TfEnhancedEncodingAnalyzer.cpp:44-50).
 */
#define AHQ_DLQ_PDF_SIZE 1536
typedef struct {
    int32_t  num_slots;
    double*  xleft;
    double*  pdf;
    int32_t* meta;
} ahq_dlq_pdf_state;

/* Replaces TfEnhancedEncodingAnalyzer::updateStats -> UpdatePdf / InitializePdf / GetHistogram
 * (DLQ/src/TfEnhancedEncodingAnalyzer.cpp:26-42, DLQ/src/math_functions.cpp:190-285, 364-381) for every block of the
 * layout (EncodingAnalyzerWrapper::updateStats, DLQ/src/EncodingAnalyzerWrapper.cpp:27-46).
 * with_init: non-zero adds the pass that finds the batch's range, needed while any slot is still uninitialised (a
 * slot stays uninitialised while it has only seen all-zero batches); callers pass 1 until meta says every slot is
 * initialised, 0 afterwards (one read of the tensor instead of two).  With 0, an uninitialised slot ignores the batch.
 * hist_out (optional): [num_slots][AHQ_DLQ_PDF_SIZE] counts of this batch alone.
 */
size_t ahq_dlq_pdf_update_workspace_bytes(int32_t dtype, const ahq_layout* layout);
int    ahq_dlq_pdf_update(int32_t dtype, const ahq_layout* layout, const void* x, const ahq_dlq_pdf_state* state,
                          int32_t with_init, uint32_t* hist_out, void* workspace, size_t workspace_bytes, void* stream);

/* Replaces TfEnhancedEncodingAnalyzer::computeEncoding (DLQ/src/TfEnhancedEncodingAnalyzer.cpp:52-377): range of the
 * aggregate statistics, the 17 x 21 + 1 asymmetric or 101 symmetric (delta, offset) candidates, the quantization +
 * 3 x saturation cost of each over the PDF, first minimum.  out: [num_slots][5]; best_index (optional):
 * [num_slots][2] = position of the chosen candidate in the reference's candidate list, length of that list.
 */
size_t ahq_dlq_tfe_encodings_workspace_bytes(int32_t num_slots);
int    ahq_dlq_tfe_encodings(const ahq_dlq_pdf_state* state, int32_t bw, int32_t symmetric, int32_t strict,
                             int32_t unsigned_sym, double* out, int32_t* best_index, void* workspace,
                             size_t workspace_bytes, void* stream);

/* Replaces quantizeDequantizeFp8 / quantizeDequantizeFp8Broadcast (DLQ/include/DlQuantization/Quantization.hpp,
 * DLQ/src/trim_functions.cpp:49-67, 243-258, 791-900): y = fakeCastToFp8(x / scale) * scale under round-to-nearest-
 * even, for the FP8 format given by its mantissa bits, minimum normal exponent and largest value
 * (FloatQuantizationSpec, DLQ/include/DlQuantization/QuantizationType.hpp:24-33; E4M3FN = 3, -6, 448; E5M2 = 2, -14,
 * 57344).  scale: one float per encoding of the layout (float(encoding.delta)).  Float tensors only, as in the
 * reference.
 */
int ahq_dlq_fp8_qdq(int32_t dtype, const ahq_layout* layout, const void* x, void* y, const float* scale,
                    int32_t mantissa_bits, int32_t exponent_min, float max_value, void* stream);

/* The per-tensor form of ahq_dlq_fp8_qdq with the scale (TfEncoding.delta) by value: quantizeDequantizeFp8
 * (DLQ/src/trim_functions.hpp:39-41, trim_functions.cpp:243-258).
 */
int ahq_dlq_fp8_qdq_per_tensor(int32_t dtype, const void* x, void* y, uint64_t count, double delta,
                               int32_t mantissa_bits, int32_t exponent_min, float max_value, void* stream);

/* Replaces _float_quantize_dequantize of aimet_torch (aimet_torch/quantization/float/quantizer.py:634-716, with
 * _cast_decast :709-710 and fake_cast_to_ieee_float, aimet_torch/fp_quantization.py:148-214): in the arithmetic of
 * `dtype` (x, y and every intermediate), y = cast(clamp(x / scale, -max_value, max_value)) * scale, where cast rounds
 * to nearest even onto the floating-point grid with `mantissa_bits` explicit mantissa bits whose smallest normal
 * binade starts at 2^exponent_min, and max_value is the largest value of the simulated format.  overflow_to_nan: what
 * a value that still rounds past max_value becomes (1: NaN, as the "fn" / "fnuz" storage types do; 0: infinity).
 * unsigned_zero: the format has no negative zero.  scale: one float per encoding of the layout, used at float
 * precision (quotient and product are formed in float and rounded once to `dtype`), which is how torch treats a
 * one-element float32 operand next to a 16-bit tensor.
 * logarithm_form (16-bit `dtype` only, ignored for float32): cast the way fake_cast_to_ieee_float does for a format
 * without a torch storage type, scales = 2 ** (clamp(floor(log2|x| + bias), 1) - mantissa_bits - bias), out =
 * round(x / scales) * scales with bias = 1 - exponent_min and every operation rounded to `dtype`: values within one
 * unit of `dtype` below a power of two land on the next binade's grid and a clamp bound that `dtype` rounds upward is
 * returned as it is, as in the reference; overflow_to_nan and unsigned_zero do not apply.
 * workspace (optional): ahq_float_cast_workspace_bytes() bytes of 16-byte aligned device memory, or null.  With it,
 * a 16-bit tensor with a single encoding and at least 2^22 elements is cast through a table of the function's value
 * for each of the 65536 bit patterns (filled by the same arithmetic, so the results are the same bits) instead of
 * once per element; without it, and for every other tensor, the arithmetic runs per element.  The query returns 0
 * where the table does not apply.
 */
size_t ahq_float_cast_workspace_bytes(int32_t dtype, const ahq_layout* layout);
int ahq_float_qdq(int32_t dtype, const ahq_layout* layout, const void* x, void* y, const float* scale,
                  int32_t mantissa_bits, int32_t exponent_min, float max_value, int32_t overflow_to_nan,
                  int32_t unsigned_zero, int32_t logarithm_form, void* workspace, size_t workspace_bytes, void* stream);

/* The input gradient autograd derives for _float_quantize_dequantize with a format that has a torch storage type
 * (aimet_torch/quantization/float/quantizer.py:634-710: div, clamp, _cast_decast = .to(storage type).to(dtype), mul),
 * in one pass: gx = (cast(g * scale) * [ -max_value <= x / scale <= max_value ]) / scale, every operation rounded to
 * `dtype` as torch's would be.  The backward of the two conversions converts the gradient to the storage type and
 * back, so the reference's gradient is rounded onto the simulated format's grid (and overflows like any other
 * value); this is reproduced.  Format arguments as for ahq_float_qdq.  (Formats without a storage type go through the
 * reference's logarithm formula, whose gradient is zero everywhere: no kernel needed.)
 */
int ahq_float_qdq_backward(int32_t dtype, const ahq_layout* layout, const void* g, const void* x, void* gx,
                           const float* scale, int32_t mantissa_bits, int32_t exponent_min, float max_value,
                           int32_t overflow_to_nan, int32_t unsigned_zero, void* stream);

/* Replaces _float_quantize of aimet_torch (aimet_torch/quantization/float/quantizer.py:687-706), which
 * FloatEncoding.quantize calls (aimet_torch/quantization/float/encoding.py:140-152): ahq_float_qdq without its last
 * multiplication, y = cast(clamp(x / scale, -max_value, max_value)); same arguments, same arithmetic.
 */
int ahq_float_quantize(int32_t dtype, const ahq_layout* layout, const void* x, void* y, const float* scale,
                       int32_t mantissa_bits, int32_t exponent_min, float max_value, int32_t overflow_to_nan,
                       int32_t unsigned_zero, int32_t logarithm_form, void* workspace, size_t workspace_bytes,
                       void* stream);

/* Replaces FloatEncoding.dequantize of aimet_torch (aimet_torch/quantization/float/encoding.py:154-165, a blockwise
 * torch.mul): y = x * scale, the product formed in float and rounded once to `dtype`; scale: one float per encoding
 * of the layout.
 */
int ahq_float_dequantize(int32_t dtype, const ahq_layout* layout, const void* x, void* y, const float* scale,
                         void* stream);

/* Replaces PercentileEncodingAnalyzer::computeEncoding (DLQ/src/PercentileEncodingAnalyzer.cpp:52-169) on the same PDF
 * statistics: the range that keeps `percentile` percent of the probability mass on each side, widened to contain
 * zero, then getComputedEncodings.  out: [num_slots][5].
 */
int ahq_dlq_percentile_encodings(const ahq_dlq_pdf_state* state, float percentile, int32_t bw, int32_t symmetric,
                                 int32_t strict, int32_t unsigned_sym, double* out, void* stream);

/* Diagnostics, outside the drop-in boundary: measurement aids for the benchmark with no counterpart in the reference;
 * nothing that replaces a reference call uses them and a binding of the reference need not declare them.
 * ahq_diag_read streams `bytes` bytes through
 * 16-byte loads (non-temporal ones if `nontemporal`) and folds them into one word per workgroup (out: `workgroups`
 * words); ahq_diag_copy copies them.  Both are persistent grid-stride kernels of `workgroups` x 256 threads.  x, y:
 * 16-byte aligned, bytes a multiple of 16.  What they reach on buffers that are not already in the last-level cache is
 * the ceiling the memory system offers the library's streaming kernels on this device.
 */
int ahq_diag_read(const void* x, size_t bytes, int32_t workgroups, int32_t nontemporal, uint32_t* out, void* stream);
int ahq_diag_copy(const void* x, void* y, size_t bytes, int32_t workgroups, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* AIMET_AMD_H */
