// Device-side helpers shared by all kernels (gfx950, wave64).
#pragma once

#include <type_traits>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/aimet_amd.h"

namespace ahq {

constexpr int kBlock = 256;          // threads per workgroup = 4 waves of 64
constexpr int kWave = 64;
constexpr int kUnroll = 4;           // 16-byte vectors per thread per tile
constexpr int kTileVec = kBlock * kUnroll;  // vectors per tile
// Tensors of at least this many bytes are read with non-temporal loads by the kernels that take the hint: they do not
// fit the caches anyway, and a streamed line that is not kept leaves room for what the rest of the step reads again.
// Smaller tensors are often still resident from the kernel that produced them and keep the ordinary loads.
constexpr long long kStreamLoadBytes = 32ll << 20;

// ------------------------------------------------------------------------------------------------ storage types --
struct f16_t { uint16_t bits; };
struct bf16_t { uint16_t bits; };

template <typename T> struct IoTraits;
template <> struct IoTraits<float> { static constexpr int kVec = 4; static constexpr int kDtype = AHQ_F32; };
template <> struct IoTraits<f16_t> { static constexpr int kVec = 8; static constexpr int kDtype = AHQ_F16; };
template <> struct IoTraits<bf16_t> { static constexpr int kVec = 8; static constexpr int kDtype = AHQ_BF16; };

__device__ __forceinline__ float bits_to_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f32_to_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

__device__ __forceinline__ float load_f32(float v) { return v; }
__device__ __forceinline__ float load_f32(f16_t v) { return (float)__builtin_bit_cast(_Float16, v.bits); }
__device__ __forceinline__ float load_f32(bf16_t v) { return bits_to_f32((uint32_t)v.bits << 16); }

// Round-to-nearest-even narrowing (one v_cvt_pk_bf16_f32 / v_cvt_f16_f32 each on gfx950).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }
// The value passes through an empty asm statement first: without it the compiler merges a preceding multiplication
// into v_fma_mixlo_f16 with a +0 addend, which turns a product of -0 into +0.
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
    asm("" : "+v"(f));
    return __builtin_bit_cast(uint16_t, (_Float16)f);
}

template <typename T> __device__ __forceinline__ T store_cast(float v);
template <> __device__ __forceinline__ float store_cast<float>(float v) { return v; }
template <> __device__ __forceinline__ f16_t store_cast<f16_t>(float v) { return f16_t{f32_to_f16_bits(v)}; }
template <> __device__ __forceinline__ bf16_t store_cast<bf16_t>(float v) { return bf16_t{f32_to_bf16_bits(v)}; }

// Round a float to the compute dtype and widen it again ("every intermediate is rounded to D").
template <int CD> __device__ __forceinline__ float rnd(float v);
template <> __device__ __forceinline__ float rnd<AHQ_F32>(float v) { return v; }
template <> __device__ __forceinline__ float rnd<AHQ_F16>(float v) { return (float)__builtin_bit_cast(_Float16, f32_to_f16_bits(v)); }
template <> __device__ __forceinline__ float rnd<AHQ_BF16>(float v) { return bits_to_f32((uint32_t)f32_to_bf16_bits(v) << 16); }

// Round to the compute dtype CD, then narrow to the storage type: one conversion when the two formats coincide.
template <typename IO, int CD>
__device__ __forceinline__ IO store_rounded(float v) {
    if constexpr (CD == AHQ_F32 || (CD == AHQ_BF16 && std::is_same<IO, bf16_t>::value) ||
                  (CD == AHQ_F16 && std::is_same<IO, f16_t>::value))
        return store_cast<IO>(v);
    else
        return store_cast<IO>(rnd<CD>(v));
}

// ------------------------------------------------------------------------------------------- 16-byte vector I/O --
template <typename T, int N> struct alignas(sizeof(T) * N) Pack { T v[N]; };

template <typename T, int N>
__device__ __forceinline__ Pack<T, N> load_pack(const T* p) {
    return *reinterpret_cast<const Pack<T, N>*>(p);
}
// Non-temporal load, for kernels that only read.  Which kernels gain is an empirical matter on this part (same box,
// back-to-back runs): a bare reduction over 1 GiB goes from 6.3 to 7.0 TB/s and the per-row min/max of a 67 MB tensor
// from 11.4 to 10.0 us, the histogram stream gains 8 % and the PDF stream 2.6 % (batches taken in turn, none
// found in the last-level cache); the quantize-dequantize kernels, which write as much as they
// read, lose 10 % and the 8-lane block min/max loses 9 %, so those keep load_pack.
template <typename T, int N>
__device__ __forceinline__ Pack<T, N> load_pack_stream(const T* p) {
    constexpr int kBytes = (int)sizeof(T) * N;
    if constexpr (kBytes == 16) {
        typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
        return __builtin_bit_cast(Pack<T, N>, __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)));
    } else if constexpr (kBytes == 8) {
        typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(Pack<T, N>, __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p)));
    } else if constexpr (kBytes == 4) {
        return __builtin_bit_cast(Pack<T, N>, __builtin_nontemporal_load(reinterpret_cast<const unsigned int*>(p)));
    } else if constexpr (kBytes == 2) {
        return __builtin_bit_cast(Pack<T, N>, __builtin_nontemporal_load(reinterpret_cast<const unsigned short*>(p)));
    } else {
        return load_pack<T, N>(p);
    }
}
template <typename T, int N>
__device__ __forceinline__ void store_pack(T* p, const Pack<T, N>& v) {
    *reinterpret_cast<Pack<T, N>*>(p) = v;
}
// Store of an output that this kernel never reads back: marked non-temporal, so the written lines do not displace the
// inputs from the caches (a backward pass re-reads the tensor its forward pass has just read).
template <typename T, int N>
__device__ __forceinline__ void store_pack_stream(T* p, const Pack<T, N>& v) {
    constexpr int kBytes = (int)sizeof(T) * N;
    if constexpr (kBytes == 16) {
        typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
        __builtin_nontemporal_store(__builtin_bit_cast(u32x4, v), reinterpret_cast<u32x4*>(p));
    } else if constexpr (kBytes == 8) {
        typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
        __builtin_nontemporal_store(__builtin_bit_cast(u32x2, v), reinterpret_cast<u32x2*>(p));
    } else if constexpr (kBytes == 4) {
        __builtin_nontemporal_store(__builtin_bit_cast(unsigned int, v), reinterpret_cast<unsigned int*>(p));
    } else {
        store_pack<T, N>(p, v);
    }
}

// ------------------------------------------------------------------------------------------- wave / block reduce --
// ------------------------------------------------------------------------------------------ segment exchange --
// Value of the lane whose index differs by XOR-ing `m` inside runs of `kv` lanes (kv a power of two, m < kv).
// Inside a row of 16 lanes the exchange is a data-parallel-primitive move in the vector ALU (quad permutes for m = 1
// and 2; for m = 4 and 8 the mirrored lane, which after the earlier steps holds the other half's partial result, so
// these are only valid as steps of a full butterfly over operands that are symmetric within the halves already
// combined); wider exchanges go through the LDS permute network.
template <int CTRL>
__device__ __forceinline__ int dpp_int(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, false);
}
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) { return __builtin_bit_cast(float, dpp_int<CTRL>(__builtin_bit_cast(int, v))); }
template <int CTRL>
__device__ __forceinline__ int dpp_move(int v) { return dpp_int<CTRL>(v); }
template <int CTRL>
__device__ __forceinline__ double dpp_move(double v) {
    const long long b = __builtin_bit_cast(long long, v);
    const int lo = dpp_int<CTRL>((int)(b & 0xffffffffll)), hi = dpp_int<CTRL>((int)(b >> 32));
    return __builtin_bit_cast(double, ((long long)hi << 32) | (unsigned int)lo);
}

// All-lanes butterfly reduction over runs of kv lanes (kv a power of two <= 64, uniform across the wave), written as
// straight-line steps so that each exchange is a compile-time DPP pattern.
template <typename T, typename Op>
__device__ __forceinline__ T segment_reduce(T v, int kv, Op op) {
    if (kv > 1) v = op(v, dpp_move<0xB1>(v));   // quad_perm [1,0,3,2]
    if (kv > 2) v = op(v, dpp_move<0x4E>(v));   // quad_perm [2,3,0,1]
    if (kv > 4) v = op(v, dpp_move<0x141>(v));  // row_half_mirror: lane i <-> 7 - i of each 8
    if (kv > 8) v = op(v, dpp_move<0x140>(v));  // row_mirror: lane i <-> 15 - i of each 16
    if (kv > 16) v = op(v, __shfl_xor(v, 16, kWave));
    if (kv > 32) v = op(v, __shfl_xor(v, 32, kWave));
    return v;
}

// Minimum / maximum of a float over runs of KV lanes (KV a power of two <= 16, known at compile time), every lane
// receiving the result: one vector instruction per step, the exchange being the instruction's own data-parallel
// operand (quad permutes, then the mirrored lane of each 8 and each 16; see segment_reduce for why those are valid as
// later steps of a butterfly).  The compiler's own form of such a step is four instructions: a move through the
// data-parallel network and two operand canonicalisations in front of the minimum.  v_min_f32 / v_max_f32 return the
// other operand when one is NaN, so NaN never wins; the callers track NaN separately.  The two wait states a
// data-parallel operand needs after the vector instruction that wrote it are spelled out, since the assembler does
// not add them inside an asm statement.
#define AHQ_DPP_STEP(OPC, CTRL) \
    asm volatile("s_nop 1\n\t" OPC " %0, %1, %1 " CTRL " row_mask:0xf bank_mask:0xf" : "=v"(v) : "v"(v))
template <int KV>
__device__ __forceinline__ float segment_min_f32(float v) {
    static_assert(KV >= 1 && KV <= 16 && (KV & (KV - 1)) == 0, "runs of 1, 2, 4, 8 or 16 lanes");
    if constexpr (KV > 1) AHQ_DPP_STEP("v_min_f32_dpp", "quad_perm:[1,0,3,2]");
    if constexpr (KV > 2) AHQ_DPP_STEP("v_min_f32_dpp", "quad_perm:[2,3,0,1]");
    if constexpr (KV > 4) AHQ_DPP_STEP("v_min_f32_dpp", "row_half_mirror");
    if constexpr (KV > 8) AHQ_DPP_STEP("v_min_f32_dpp", "row_mirror");
    return v;
}
template <int KV>
__device__ __forceinline__ float segment_max_f32(float v) {
    static_assert(KV >= 1 && KV <= 16 && (KV & (KV - 1)) == 0, "runs of 1, 2, 4, 8 or 16 lanes");
    if constexpr (KV > 1) AHQ_DPP_STEP("v_max_f32_dpp", "quad_perm:[1,0,3,2]");
    if constexpr (KV > 2) AHQ_DPP_STEP("v_max_f32_dpp", "quad_perm:[2,3,0,1]");
    if constexpr (KV > 4) AHQ_DPP_STEP("v_max_f32_dpp", "row_half_mirror");
    if constexpr (KV > 8) AHQ_DPP_STEP("v_max_f32_dpp", "row_mirror");
    return v;
}
#undef AHQ_DPP_STEP

// Maximum of a float over runs of `kv` lanes (a power of two up to 64, uniform across the wave), in every lane: the
// steps inside a row of 16 lanes are one instruction each, the two across rows go through the LDS permute network.
// NaN never wins (see segment_max_f32).
__device__ __forceinline__ float segment_max_any(float v, int kv) {
    switch (kv) {
        case 1: return v;
        case 2: return segment_max_f32<2>(v);
        case 4: return segment_max_f32<4>(v);
        case 8: return segment_max_f32<8>(v);
        default: break;
    }
    v = segment_max_f32<16>(v);
    if (kv > 16) v = fmaxf(v, __shfl_xor(v, 16, kWave));
    if (kv > 32) v = fmaxf(v, __shfl_xor(v, 32, kWave));
    return v;
}

template <typename T, typename Op>
__device__ __forceinline__ T wave_reduce(T v, Op op) {
#pragma unroll
    for (int m = kWave / 2; m >= 1; m >>= 1) v = op(v, __shfl_xor(v, m, kWave));
    return v;
}

// All threads get the result.  `smem` must hold kBlock/kWave elements of T and is reusable after the call returns.
template <typename T, typename Op>
__device__ __forceinline__ T block_reduce(T v, Op op, T* smem) {
    v = wave_reduce(v, op);
    const int wave = threadIdx.x / kWave;
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) smem[wave] = v;
    __syncthreads();
    T r = smem[0];
#pragma unroll
    for (int w = 1; w < kBlock / kWave; ++w) r = op(r, smem[w]);
    return r;
}

struct OpAddF { __device__ __forceinline__ float operator()(float a, float b) const { return a + b; } };
struct OpAddD { __device__ __forceinline__ double operator()(double a, double b) const { return a + b; } };
struct OpMinF { __device__ __forceinline__ float operator()(float a, float b) const { return fminf(a, b); } };
struct OpMaxF { __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); } };
struct OpOrI { __device__ __forceinline__ int operator()(int a, int b) const { return a | b; } };

}  // namespace ahq
