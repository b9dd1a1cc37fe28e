// Fake-quantization forward kernels: quantize-dequantize / quantize / dequantize, the LPBQ forward that derives its
// block scales in the launch, the DlQuantization and float fake-casts (arithmetic and arguments: qdq_common.h).

#include <atomic>

#include "qdq_common.h"

namespace ahq {

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
// The encodings a thread stages are requested first, then the tile's elements; the encodings are prepared and staged
// while the elements are in flight, and the workgroup meets at the barrier once before the arithmetic.
template <typename IO, int VEC, typename M, bool FULL, int U, bool LPBQ = false>
__device__ __forceinline__ void fwd_tile(const QdqArgs& a, const Tile& t, float (*sp)[kStage],
                                         const LpbqFuse* lpbq = nullptr) {
    const IO* __restrict__ x = static_cast<const IO*>(a.x) + t.v0 * VEC;
    IO* __restrict__ y = static_cast<IO*>(a.y) + t.v0 * VEC;
    uint8_t* __restrict__ mask = a.mask ? a.mask + t.v0 * VEC : nullptr;
    Pack<IO, VEC> in[U];
    float pre_mn = 0.f, pre_mx = 0.f;
    EncRaw pre{};
    if constexpr (LPBQ) lpbq_preload(*lpbq, t, pre_mn, pre_mx);
    else pre = preload_encoding(a, t);
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int lv = u * kBlock + threadIdx.x;
        if (FULL || lv < t.nv) in[u] = load_pack_hinted<IO, VEC>(x + (int64_t)lv * VEC, a.stream_loads != 0);
    }
    if constexpr (LPBQ) stage_lpbq<M>(a, *lpbq, t, sp, pre_mn, pre_mx);
    else stage_encodings<M>(a, t, sp, pre);
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

template <typename IO, int VEC, typename M, bool FAST>
__device__ __forceinline__ void fwd_cols_rows(const QdqArgs& a, const Pack<IO, VEC>* in, const EncP* e, IO* __restrict__ y,
                                              uint8_t* __restrict__ mask, int64_t r0, int64_t c0) {
#pragma unroll
    for (int u = 0; u < kColUnroll; ++u) {
        if (r0 + u >= a.I) continue;
        Pack<IO, VEC> out;
        Pack<uint8_t, VEC> mk;
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            bool inr;
            const float r = M::template fwd<FAST>(load_f32(in[u].v[k]), e[k], a.gc, inr);
            out.v[k] = store_rounded<IO, M::kCD>(r);
            mk.v[k] = inr ? 1 : 0;
        }
        store_pack_stream<IO, VEC>(y + (r0 + u) * a.J + c0, out);
        if (mask) store_pack_stream<uint8_t, VEC>(mask + (r0 + u) * a.J + c0, mk);
    }
}

template <typename IO, int VEC, typename M, int WAVES>
__global__ __launch_bounds__(WAVES * kWave) void qdq_fwd_cols_kernel(const QdqArgs a) {
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int64_t c0 = ((int64_t)blockIdx.x * kWave + lane) * VEC;
    if (c0 >= a.J) return;
    const int64_t z = blockIdx.z;  // stacked columns: problem z has its own I x J elements and J encodings
    const IO* __restrict__ x = static_cast<const IO*>(a.x) + z * a.I * a.J;
    IO* __restrict__ y = static_cast<IO*>(a.y) + z * a.I * a.J;
    uint8_t* __restrict__ mask = a.mask ? a.mask + z * a.I * a.J : nullptr;
    EncP e[VEC];
    bool enc_fast = true;
    load_col_encodings<M, VEC>(a, z * a.J + c0, e);
#pragma unroll
    for (int k = 0; k < VEC; ++k) enc_fast &= !M::kDiv || e[k].rs != 0.f;
    const int64_t step = (int64_t)gridDim.y * WAVES * kColUnroll;
    for (int64_t r0 = ((int64_t)blockIdx.y * WAVES + wave) * kColUnroll; r0 < a.I; r0 += step) {
        Pack<IO, VEC> in[kColUnroll];
        bool ok = enc_fast;
#pragma unroll
        for (int u = 0; u < kColUnroll; ++u)
            if (r0 + u < a.I) in[u] = load_pack_hinted<IO, VEC>(x + (r0 + u) * a.J + c0, a.stream_loads != 0);
#pragma unroll
        for (int u = 0; u < kColUnroll; ++u)
            if (M::kDiv && r0 + u < a.I) ok &= row_can_divide_fast<IO, VEC>(in[u]);
        // wave-uniform, like the tiled kernel: one branch per step, and each side a straight run of arithmetic over
        // all its elements (a choice per element costs a branch per element and keeps the compiler from interleaving
        // the elements' instruction chains)
        if (!M::kDiv || __builtin_amdgcn_ballot_w64(!ok) == 0) fwd_cols_rows<IO, VEC, M, true>(a, in, e, y, mask, r0, c0);
        else fwd_cols_rows<IO, VEC, M, false>(a, in, e, y, mask, r0, c0);
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

template <typename IO, typename M>
static void launch_fwd(const Plan& p, const QdqArgs& a, hipStream_t st, bool aligned) {
    const int lane_elems = cols_lane_elems(IoTraits<IO>::kDtype, p, aligned);
    if (lane_elems > 0) {
        // About as many workgroups as the chip holds at once (256 CUs; the 16-bit kernels run four waves per SIMD,
        // the float32 ones eight): every wave prepares its encodings before its first row, and a second round of
        // waves pays that set-up while the memory pipes drain (8192 x 4096 bf16: 25.5 us with 1024 workgroups,
        // 28.7 us with 3072, 32.3 us with 384; float32: 44.3 us with 8192, 45.6 us with 4096 or 16384).
        constexpr int V = IoTraits<IO>::kVec;
        if (lane_elems == V)
            hipLaunchKernelGGL((qdq_fwd_cols_kernel<IO, V, M, kFwdColWaves>), (cols_grid<V>(p, V > 4 ? 1024 : 8192, kFwdColWaves)),
                               dim3(kFwdColWaves * kWave), 0, st, a);
        else
            hipLaunchKernelGGL((qdq_fwd_cols_kernel<IO, 1, M, kFwdColWaves>), (cols_grid<1>(p, 8192, kFwdColWaves)),
                               dim3(kFwdColWaves * kWave), 0, st, a);
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

// ----------------------------------------------------------------------- float fake-cast of 16-bit tensors by table --
// With one encoding the result is a function of the element's 16 bits alone, and the cast is arithmetic-bound on
// 16-bit tensors (eight elements per 16 bytes, a logarithm, an exponential and a dozen roundings each: 71 to 117 us
// for 134 MB where the memory system needs 43).  So the function is tabulated first -- one launch evaluates
// MathFloatCast::fwd, the very code of the elementwise kernel, on all 65536 bit patterns and leaves the 128 KB table in
// the caller's workspace -- and the tensor is then streamed through a copy of the table in LDS: a 16-byte load, eight
// two-byte LDS reads, a 16-byte store.
namespace ahq {
constexpr int kCastTableEntries = 65536;
constexpr size_t kCastTableBytes = (size_t)kCastTableEntries * 2;
constexpr int64_t kCastTableMinNumel = (int64_t)1 << 22;  // below that the two extra launches cost more than they save
constexpr int kCastTableThreads = 1024;
constexpr int kCastTableUnroll = 1;  // 16-byte loads in flight per lane: 46.3 us with one, 49.3 with two, 50.4 with four (134 MB)

template <typename IO, int CD>
__global__ __launch_bounds__(256) void float_cast_table_kernel(const QdqArgs a, uint16_t* __restrict__ table) {
    using M = MathFloatCast<CD>;
    const int p = blockIdx.x * 256 + threadIdx.x;
    if (p >= kCastTableEntries) return;
    const EncP e = M::prep(a.scale[0], 0.f, 0.f, 0.f, a.gc);
    IO in;
    in.bits = (uint16_t)p;
    bool inr;
    const IO out = store_rounded<IO, CD>(M::template fwd<false>(load_f32(in), e, a.gc, inr));
    table[p] = out.bits;
}

template <typename IO>
__global__ __launch_bounds__(kCastTableThreads) void float_cast_lookup_kernel(const IO* __restrict__ x, IO* __restrict__ y,
                                                                              int64_t numel, const uint16_t* __restrict__ table) {
    extern __shared__ uint16_t lut[];
    {
        // 128 KB / 1024 threads: eight 16-byte vectors each, neighbouring threads neighbouring vectors
        const Pack<uint16_t, 8>* src = reinterpret_cast<const Pack<uint16_t, 8>*>(table);
        Pack<uint16_t, 8>* dst = reinterpret_cast<Pack<uint16_t, 8>*>(lut);
#pragma unroll
        for (int i = 0; i < kCastTableEntries / 8 / kCastTableThreads; ++i) dst[i * kCastTableThreads + threadIdx.x] = src[i * kCastTableThreads + threadIdx.x];
    }
    __syncthreads();
    const int64_t nvec = numel / 8;
    const int64_t stride = (int64_t)gridDim.x * kCastTableThreads * kCastTableUnroll;
    for (int64_t v0 = (int64_t)blockIdx.x * kCastTableThreads * kCastTableUnroll + threadIdx.x; v0 < nvec; v0 += stride) {
        Pack<IO, 8> in[kCastTableUnroll];
#pragma unroll
        for (int u = 0; u < kCastTableUnroll; ++u)
            if (v0 + u * kCastTableThreads < nvec) in[u] = load_pack_stream<IO, 8>(x + (v0 + u * kCastTableThreads) * 8);
#pragma unroll
        for (int u = 0; u < kCastTableUnroll; ++u) {
            if (v0 + u * kCastTableThreads >= nvec) continue;
            Pack<IO, 8> out;
#pragma unroll
            for (int k = 0; k < 8; ++k) out.v[k].bits = lut[in[u].v[k].bits];
            store_pack_stream<IO, 8>(y + (v0 + u * kCastTableThreads) * 8, out);
        }
    }
    // the elements behind the last whole vector, straight from the table in memory
    if (blockIdx.x == 0 && threadIdx.x < (int)(numel - nvec * 8)) {
        const int64_t i = nvec * 8 + threadIdx.x;
        IO out;
        out.bits = table[x[i].bits];
        y[i] = out;
    }
}

// The lookup kernel's 128 KB of dynamic LDS are more than a kernel gets by default: asked for once per device and
// dtype; false when the runtime refuses (the elementwise kernel then does the work).
static bool cast_table_lds_available(int dtype) {
    constexpr int kMaxDevices = 64;
    static std::atomic<int> state[kMaxDevices][2];  // 0 not asked yet, 1 granted, 2 refused
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return false;
    std::atomic<int>& st = state[dev][dtype == AHQ_F16 ? 0 : 1];
    int v = st.load(std::memory_order_acquire);
    if (v == 0) {
        const void* k = dtype == AHQ_F16 ? reinterpret_cast<const void*>(&float_cast_lookup_kernel<f16_t>)
                                         : reinterpret_cast<const void*>(&float_cast_lookup_kernel<bf16_t>);
        const bool ok = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kCastTableBytes) == hipSuccess;
        if (!ok) (void)hipGetLastError();  // the refusal is handled here, not reported by the next launch check
        v = ok ? 1 : 2;
        st.store(v, std::memory_order_release);
    }
    return v == 1;
}

// the table applies: a 16-bit tensor, dense and 16-byte aligned, one encoding, enough elements
static bool cast_table_applies(int dtype, const Plan& p) {
    return dtype != AHQ_F32 && p.cl.kind == kIJK && p.cl.J == 1 && p.cl.numel >= kCastTableMinNumel;
}
}  // namespace ahq

extern "C" size_t ahq_float_cast_workspace_bytes(int32_t dtype, const ahq_layout* layout) {
    if (dtype < AHQ_F32 || dtype > AHQ_BF16 || !layout) return 0;
    Plan p;
    if (!make_plan(dtype, *layout, true, false, &p, kFwdUnroll)) return 0;
    return cast_table_applies(dtype, p) ? kCastTableBytes : 0;
}

static int float_cast_impl(const char* what, int stage_flags, int32_t dtype, const ahq_layout* layout, const void* x,
                           void* y, const float* scale, int32_t mantissa_bits, int32_t exponent_min, float max_value,
                           int32_t overflow_to_nan, int32_t unsigned_zero, int32_t logarithm_form, void* workspace,
                           size_t workspace_bytes, void* stream) {
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
    grid.io_dtype = dtype;
    grid.compute_dtype = dtype;
    fill_args(grid, p, &a);
    a.gc.qmin = (float)exponent_min;
    a.gc.qmax = max_value;
    a.gc.zps = (float)mantissa_bits;
    a.gc.flags = (overflow_to_nan ? kCastOverflowNaN : 0) | (unsigned_zero ? kCastUnsignedZero : 0) |
                 (logarithm_form ? kCastLogForm : 0) | stage_flags;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (workspace && workspace_bytes >= kCastTableBytes && aligned16(workspace) && aligned16(x) && aligned16(y) &&
        cast_table_applies(dtype, p) && cast_table_lds_available(dtype)) {
        uint16_t* table = static_cast<uint16_t*>(workspace);
        const dim3 tg(kCastTableEntries / 256), tb(256);
        // one workgroup per compute unit and 128 KB of LDS each; fewer for tensors that would leave them idle
        const int64_t nvec = p.cl.numel / 8;
        int64_t nb = (nvec + (int64_t)kCastTableThreads * kCastTableUnroll - 1) / ((int64_t)kCastTableThreads * kCastTableUnroll);
        nb = nb < 1 ? 1 : (nb > 256 ? 256 : nb);
        if (dtype == AHQ_F16) {
            hipLaunchKernelGGL((float_cast_table_kernel<f16_t, AHQ_F16>), tg, tb, 0, st, a, table);
            hipLaunchKernelGGL((float_cast_lookup_kernel<f16_t>), dim3((unsigned)nb), dim3(kCastTableThreads), kCastTableBytes, st,
                               static_cast<const f16_t*>(x), static_cast<f16_t*>(y), p.cl.numel, (const uint16_t*)table);
        } else {
            hipLaunchKernelGGL((float_cast_table_kernel<bf16_t, AHQ_BF16>), tg, tb, 0, st, a, table);
            hipLaunchKernelGGL((float_cast_lookup_kernel<bf16_t>), dim3((unsigned)nb), dim3(kCastTableThreads), kCastTableBytes, st,
                               static_cast<const bf16_t*>(x), static_cast<bf16_t*>(y), p.cl.numel, (const uint16_t*)table);
        }
        return check_launch(what);
    }
    if (dtype == AHQ_F32) launch_fwd<float, MathFloatCast<AHQ_F32>>(p, a, st, aligned16(x) && aligned16(y));
    else if (dtype == AHQ_F16) launch_fwd<f16_t, MathFloatCast<AHQ_F16>>(p, a, st, aligned16(x) && aligned16(y));
    else launch_fwd<bf16_t, MathFloatCast<AHQ_BF16>>(p, a, st, aligned16(x) && aligned16(y));
    return check_launch(what);
}

extern "C" int ahq_float_qdq(int32_t dtype, const ahq_layout* layout, const void* x, void* y, const float* scale,
                             int32_t mantissa_bits, int32_t exponent_min, float max_value, int32_t overflow_to_nan,
                             int32_t unsigned_zero, int32_t logarithm_form, void* workspace, size_t workspace_bytes,
                             void* stream) {
    return float_cast_impl("ahq_float_qdq", 0, dtype, layout, x, y, scale, mantissa_bits, exponent_min, max_value,
                           overflow_to_nan, unsigned_zero, logarithm_form, workspace, workspace_bytes, stream);
}

extern "C" int ahq_float_quantize(int32_t dtype, const ahq_layout* layout, const void* x, void* y, const float* scale,
                                  int32_t mantissa_bits, int32_t exponent_min, float max_value,
                                  int32_t overflow_to_nan, int32_t unsigned_zero, int32_t logarithm_form,
                                  void* workspace, size_t workspace_bytes, void* stream) {
    return float_cast_impl("ahq_float_quantize", kCastKeepScaled, dtype, layout, x, y, scale, mantissa_bits,
                           exponent_min, max_value, overflow_to_nan, unsigned_zero, logarithm_form, workspace,
                           workspace_bytes, stream);
}

extern "C" int ahq_float_dequantize(int32_t dtype, const ahq_layout* layout, const void* x, void* y,
                                    const float* scale, void* stream) {
    return float_cast_impl("ahq_float_dequantize", kCastRescaleOnly, dtype, layout, x, y, scale, 0, 0, 1.f, 0, 0, 0,
                           nullptr, 0, stream);
}
