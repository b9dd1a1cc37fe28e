// Device-side helpers shared by all kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/aimet_amd.h"

namespace ahq {

constexpr int kBlock = 256;          // threads per workgroup = 4 waves of 64
constexpr int kWave = 64;
constexpr int kUnroll = 4;           // 16-byte vectors per thread per tile
constexpr int kTileVec = kBlock * kUnroll;  // vectors per tile

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
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); }

template <typename T> __device__ __forceinline__ T store_cast(float v);
template <> __device__ __forceinline__ float store_cast<float>(float v) { return v; }
template <> __device__ __forceinline__ f16_t store_cast<f16_t>(float v) { return f16_t{f32_to_f16_bits(v)}; }
template <> __device__ __forceinline__ bf16_t store_cast<bf16_t>(float v) { return bf16_t{f32_to_bf16_bits(v)}; }

// Round a float to the compute dtype and widen it again ("every intermediate is rounded to D").
template <int CD> __device__ __forceinline__ float rnd(float v);
template <> __device__ __forceinline__ float rnd<AHQ_F32>(float v) { return v; }
template <> __device__ __forceinline__ float rnd<AHQ_F16>(float v) { return (float)(_Float16)v; }
template <> __device__ __forceinline__ float rnd<AHQ_BF16>(float v) { return bits_to_f32((uint32_t)f32_to_bf16_bits(v) << 16); }

// ------------------------------------------------------------------------------------------- 16-byte vector I/O --
template <typename T, int N> struct alignas(sizeof(T) * N) Pack { T v[N]; };

template <typename T, int N>
__device__ __forceinline__ Pack<T, N> load_pack(const T* p) {
    return *reinterpret_cast<const Pack<T, N>*>(p);
}
template <typename T, int N>
__device__ __forceinline__ void store_pack(T* p, const Pack<T, N>& v) {
    *reinterpret_cast<Pack<T, N>*>(p) = v;
}

// ------------------------------------------------------------------------------------------- wave / block reduce --
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

struct OpAddD { __device__ __forceinline__ double operator()(double a, double b) const { return a + b; } };
struct OpMinF { __device__ __forceinline__ float operator()(float a, float b) const { return fminf(a, b); } };
struct OpMaxF { __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); } };
struct OpOrI { __device__ __forceinline__ int operator()(int a, int b) const { return a | b; } };

}  // namespace ahq
