// Minimum / maximum statistics in one pass over the tensor (both extrema from the same read).
//
// Per-lane running min/max over 16-byte vectors -> wave64 shuffle tree -> LDS across the four waves of a workgroup ->
// per-tile partials that a second, one-workgroup launch folds together.
// NaN handling follows torch.amin/amax (any NaN in a slice makes that slice's result NaN) unless `finite_only`, which
// reproduces the histogram observer's range (non-finite values ignored).

#include <mutex>

#include "ahq_device.h"
#include "ahq_host.h"
#include "layout.h"
#include "tiling.h"

// Scratch of ahq_minmax_static: partial extrema or per-encoding keys of one reduction.  Every device the library
// runs on holds its own copy of this array until the process ends.  In host code the name is only a handle for
// hipGetSymbolAddress; the address the kernels receive is looked up once per device (static_scratch below).
constexpr size_t kStaticScratchBytes = AHQ_MINMAX_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace ahq {

// Where results go (shared by every kernel family of this file).
struct MmOut {
    void* out_min;
    void* out_max;
    void* run_min;          // optional running statistics folded with torch.minimum / torch.maximum semantics
    void* run_max;
    int32_t finite_only;
};

struct MmArgs : Geom, MmOut {
    const void* x;
    float* part_min;      // kRedTile: [nblocks]
    float* part_max;
    int* part_nan;
    unsigned int* key_min;  // kRedAtomic: [num_enc] order-preserving keys
    unsigned int* key_max;
    int32_t red;
    void* copy;             // optional: the tensor is also copied there by the pass that reads it (single encoding)
};

// Arguments of the single-encoding kernels.
struct MmFlatArgs : MmOut {
    const void* x;
    void* copy;        // optional: the tensor is also copied there by the pass that reads it
    int64_t numel;
    int64_t nvec;
    float* part_min;   // [gridDim.x] partial extrema, folded by minmax_fold_kernel
    float* part_max;
    int* part_nan;
    // accumulate: the partials are running statistics, one slot per workgroup ([kFlatMaxBlocks] each): a workgroup
    // merges its result into its slot and nothing is folded; first: the slots hold nothing yet
    int32_t accumulate;
    int32_t first;
    // the workgroup that takes the vectors past the last full tile: (nvec / kFlatTileVec) % gridDim.x, formed on the
    // host (a 64-bit remainder is a hundred instructions that every workgroup would run as its last act)
    uint32_t tail_block;
    // accumulate, optional: slots of the same shape that receive this batch's own partials (nothing merged into them)
    float* batch_min;
    float* batch_max;
    int* batch_nan;
};

// Arguments of the two lean kernels below (runs of whole vectors on the leading axis): a few words instead of the
// whole tile geometry, because their workgroups live for about a microsecond and every scalar load and division at
// their start shows.
struct MmRunArgs : MmOut {
    const void* x;
    int64_t nvec;      // vectors in the tensor
    int64_t runs;      // number of encodings
    int32_t kv;        // vectors per run
    int32_t kv_shift;  // log2(kv) (segment kernel: kv is a power of two)
    int32_t stream_loads;  // segment kernel: non-temporal loads (tensors too large to be resident in the caches)
};

struct MinMax {
    float mn, mx;
    int nan;
};

__device__ __forceinline__ MinMax mm_identity() { return {__builtin_inff(), -__builtin_inff(), 0}; }

__device__ __forceinline__ void mm_add(MinMax& m, float v, bool finite_only) {
    if (finite_only) {
        const bool fin = __builtin_fabsf(v) < __builtin_inff();
        m.mn = fminf(m.mn, fin ? v : __builtin_inff());
        m.mx = fmaxf(m.mx, fin ? v : -__builtin_inff());
    } else {
        m.nan |= (v != v) ? 1 : 0;
        m.mn = fminf(m.mn, v);
        m.mx = fmaxf(m.mx, v);
    }
}

// Both extrema of one 16-byte vector.  The kernels are close enough to the memory system's limit that the vector
// instructions per element show in their run time, so: two elements per three-operand minimum / maximum, and NaN is
// looked for with one unordered comparison per PAIR of elements whose lane mask is OR-ed on the scalar unit
// (`unordered`: lanes that have seen a NaN), instead of a compare, a select and an OR per element.
// MODE 0: NaN is tracked (torch.amin / amax propagate it); 1: non-finite values are ignored; 2: NaN is simply never
// chosen (fminf / fmaxf), which is what DlQuantization's std::min / std::max folds do.
template <typename IO, int VEC, int MODE>
__device__ __forceinline__ void mm_pack(const Pack<IO, VEC>& p, float& mn, float& mx, uint64_t& unordered) {
    float f[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) f[k] = load_f32(p.v[k]);
    if (MODE == 1) {
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            const bool fin = __builtin_fabsf(f[k]) < __builtin_inff();
            mn = fminf(mn, fin ? f[k] : __builtin_inff());
            mx = fmaxf(mx, fin ? f[k] : -__builtin_inff());
        }
        return;
    }
#pragma unroll
    for (int k = 0; k + 1 < VEC; k += 2) {
        mn = fminf(fminf(mn, f[k]), f[k + 1]);
        mx = fmaxf(fmaxf(mx, f[k]), f[k + 1]);
        if (MODE == 0) unordered |= __builtin_amdgcn_ballot_w64(__builtin_isunordered(f[k], f[k + 1]));
    }
    if (VEC & 1) {
        mn = fminf(mn, f[VEC - 1]);
        mx = fmaxf(mx, f[VEC - 1]);
        if (MODE == 0) unordered |= __builtin_amdgcn_ballot_w64(f[VEC - 1] != f[VEC - 1]);
    }
}

constexpr int mm_mode(bool finite) { return finite ? 1 : 0; }

__device__ __forceinline__ MinMax mm_merge(const MinMax& a, const MinMax& b) {
    return {fminf(a.mn, b.mn), fmaxf(a.mx, b.mx), a.nan | b.nan};
}

__device__ __forceinline__ MinMax mm_shfl_xor(const MinMax& a, int m) {
    return {__shfl_xor(a.mn, m, kWave), __shfl_xor(a.mx, m, kWave), __shfl_xor(a.nan, m, kWave)};
}

// Extrema over the 64 lanes of a wave, every lane receiving them: the four steps inside a row of 16 lanes are one
// instruction each (segment_min_f32), two exchanges across rows follow; the NaN flags are one ballot.  (Eighteen
// dependent trips through the LDS permute network before: the tail of every workgroup of kernels that last a
// microsecond or two.)
__device__ __forceinline__ MinMax mm_wave_reduce(MinMax v) {
    v.mn = segment_min_f32<16>(v.mn);
    v.mx = segment_max_f32<16>(v.mx);
#pragma unroll
    for (int m = 16; m <= 32; m <<= 1) {
        v.mn = fminf(v.mn, __shfl_xor(v.mn, m, kWave));
        v.mx = fmaxf(v.mx, __shfl_xor(v.mx, m, kWave));
    }
    v.nan = __builtin_amdgcn_ballot_w64(v.nan != 0) != 0 ? 1 : 0;
    return v;
}

template <int BLOCK = kBlock>
__device__ __forceinline__ MinMax mm_block_reduce(MinMax v, MinMax* smem) {
    v = mm_wave_reduce(v);
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) smem[threadIdx.x / kWave] = v;
    __syncthreads();
    MinMax r = smem[0];
#pragma unroll
    for (int w = 1; w < BLOCK / kWave; ++w) r = mm_merge(r, smem[w]);
    return r;
}

template <typename IO>
__device__ __forceinline__ void mm_write(const MmOut& a, int64_t e, MinMax m) {
    IO* omn = static_cast<IO*>(a.out_min);
    IO* omx = static_cast<IO*>(a.out_max);
    const float qnan = __builtin_nanf("");
    float mn = m.nan ? qnan : m.mn;
    float mx = m.nan ? qnan : m.mx;
    if (a.finite_only == 2) {
        // std::min / std::max folds that start from the largest / lowest finite float: NaN never wins a comparison
        // and the minimum cannot exceed FLT_MAX (DlQuantization GetMin_cpu / GetMax_cpu)
        const float big = 3.402823466e+38f;
        mn = fminf(m.mn, big);
        mx = fmaxf(m.mx, -big);
    }
    omn[e] = store_cast<IO>(mn);
    omx[e] = store_cast<IO>(mx);
    if (a.run_min) {
        // torch.minimum / torch.maximum: NaN in either operand wins
        IO* rmn = static_cast<IO*>(a.run_min);
        IO* rmx = static_cast<IO*>(a.run_max);
        const float pmn = load_f32(rmn[e]), pmx = load_f32(rmx[e]);
        if (a.finite_only == 2) {
            rmn[e] = store_cast<IO>(mn < pmn ? mn : pmn);
            rmx[e] = store_cast<IO>(pmx < mx ? mx : pmx);
        } else {
            rmn[e] = store_cast<IO>((pmn != pmn || mn != mn) ? qnan : fminf(pmn, mn));
            rmx[e] = store_cast<IO>((pmx != pmx || mx != mx) ? qnan : fmaxf(pmx, mx));
        }
    }
}

__device__ __forceinline__ unsigned int f32_key(float f) {
    const unsigned int b = f32_to_bits(f);
    return b ^ ((b >> 31) ? 0xffffffffu : 0x80000000u);
}
__device__ __forceinline__ float key_f32(unsigned int k) {
    return bits_to_f32(k ^ ((k >> 31) ? 0x80000000u : 0xffffffffu));
}

// FULL: every lane of the tile has work (all tiles but the last).  FINITE: ignore non-finite values.
constexpr int kMmStage = kTileVec + 2;  // most runs a tile can touch

template <typename IO, int VEC, int RED, bool FINITE, bool FULL>
__device__ __forceinline__ void mm_tile(const MmArgs& a, const Tile& t, MinMax& acc, unsigned int* stage_keys) {
    const IO* __restrict__ x = static_cast<const IO*>(a.x) + t.v0 * VEC;
    Pack<IO, VEC> in[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const int lv = u * kBlock + threadIdx.x;
        if (FULL || lv < t.nv) in[u] = load_pack<IO, VEC>(x + (int64_t)lv * VEC);
    }
    // lanes of this lane's run, as a mask over the wave (kRedSeg): a NaN seen by any of them belongs to the run
    uint64_t run_lanes = ~0ull;
    if (RED == kRedSeg && a.Kv < kWave) run_lanes = ((1ull << a.Kv) - 1) << (threadIdx.x & (kWave - 1) & ~((int)a.Kv - 1));
    const uint64_t my_lane = 1ull << (threadIdx.x & (kWave - 1));
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const int lv = u * kBlock + threadIdx.x;
        MinMax v = mm_identity();
        int si = 0;
        uint64_t unordered = 0;  // lanes of the wave whose vector holds a NaN
        const bool live = FULL || lv < t.nv;
        if (RED != kRedTile && live) si = stage_index(a, t, lv);
        if (FULL) {
            mm_pack<IO, VEC, mm_mode(FINITE)>(in[u], v.mn, v.mx, unordered);
        } else {
            // ragged tile: lanes without a vector contribute the identity (the ballot inside sees only live lanes'
            // values because the others hold zeros)
            Pack<IO, VEC> pk = in[u];
            if (!live)
#pragma unroll
                for (int k = 0; k < VEC; ++k) pk.v[k] = IO{};
            float mn = __builtin_inff(), mx = -__builtin_inff();
            mm_pack<IO, VEC, mm_mode(FINITE)>(pk, mn, mx, unordered);
            if (live) {
                v.mn = mn;
                v.mx = mx;
            }
        }
        if (RED == kRedTile) {
            // a NaN anywhere in the wave marks the whole wave's contribution: the tile has one encoding
            v.nan = unordered != 0 ? 1 : 0;
            acc = mm_merge(acc, v);
        } else if (RED == kRedSeg) {
            v.nan = (unordered & run_lanes) != 0 ? 1 : 0;
            const int kv = (int)a.Kv;
            v.mn = segment_reduce(v.mn, kv, OpMinF());
            v.mx = segment_reduce(v.mx, kv, OpMaxF());
            if (live && (threadIdx.x & (kv - 1)) == 0) mm_write<IO>(a, t.e0 + si, v);
        } else if (RED == kRedAtomic) {
            v.nan = (unordered & my_lane) != 0 ? 1 : 0;
            // first into the tile's own table in LDS (one entry per run the tile touches); the table goes to the
            // global keys once per run and tile instead of once per vector
            if (live) {
                atomicMin(&stage_keys[si], f32_key(v.mn));
                atomicMax(&stage_keys[kMmStage + si], f32_key(v.mx));
                if (v.nan) atomicOr(&stage_keys[2 * kMmStage + si], 1u);
            }
        }
    }
}

template <typename IO, int VEC, int RED, bool FINITE>
__global__ __launch_bounds__(kBlock) void minmax_kernel(const MmArgs a) {
    __shared__ MinMax red_smem[kBlock / kWave];
    __shared__ unsigned int stage_keys[RED == kRedAtomic ? 3 * kMmStage : 1];  // min keys | max keys | NaN flags
    const Tile t = make_tile(a, blockIdx.x);
    if (RED == kRedAtomic) {
        for (int i = threadIdx.x; i < t.nstage; i += kBlock) {
            stage_keys[i] = f32_key(__builtin_inff());
            stage_keys[kMmStage + i] = f32_key(-__builtin_inff());
            stage_keys[2 * kMmStage + i] = 0u;
        }
        __syncthreads();
    }
    MinMax acc = mm_identity();
    if (t.nv == kTileVec) mm_tile<IO, VEC, RED, FINITE, true>(a, t, acc, stage_keys);
    else mm_tile<IO, VEC, RED, FINITE, false>(a, t, acc, stage_keys);
    if (RED == kRedAtomic) {
        __syncthreads();
        for (int i = threadIdx.x; i < t.nstage; i += kBlock) {
            int64_t e = t.e0 + i;
            if (e >= a.J) e %= a.J;
            atomicMin(&a.key_min[e], stage_keys[i]);
            atomicMax(&a.key_max[e], stage_keys[kMmStage + i]);
            if (stage_keys[2 * kMmStage + i]) atomicOr(&a.part_nan[e], 1);
        }
    }
    if (RED == kRedTile) {
        const MinMax b = mm_block_reduce(acc, red_smem);
        const int64_t per_enc = a.mode == kRows ? a.I * (int64_t)a.tpr : (int64_t)a.nblocks;
        if (per_enc == 1) {
            if (threadIdx.x == 0) mm_write<IO>(a, t.e0, b);
            return;
        }
        if (threadIdx.x == 0) {
            a.part_min[blockIdx.x] = b.mn;
            a.part_max[blockIdx.x] = b.mx;
            a.part_nan[blockIdx.x] = b.nan;
        }
    }
}

// Single encoding (per-tensor statistics): a lean streaming kernel without any encoding lookup.  Workgroups of 512
// threads walk the tensor with a grid stride, kFlatUnroll 16-byte vectors per lane in flight, and leave one partial
// each; at most kFlatMaxBlocks of them run, so the launch that folds the partials has a few hundred to read (measured
// on 103 MB: 15.8 us for the stream alone at any grid size; stream + fold 19.8 us with 6272 workgroups of 256, 17.6 us
// with 512 of 512).
constexpr int kFlatBlock = 512;
constexpr int kFlatUnroll = 4;
constexpr int kFlatTileVec = kFlatBlock * kFlatUnroll;
constexpr int kFlatMaxBlocks = 512;

template <typename IO, int VEC, bool FINITE>
__global__ __launch_bounds__(kFlatBlock) void minmax_flat_kernel(const MmFlatArgs a) {
    __shared__ MinMax red_smem[kFlatBlock / kWave];
    constexpr int MODE = mm_mode(FINITE);
    const IO* __restrict__ x = static_cast<const IO*>(a.x);
    IO* __restrict__ cp = static_cast<IO*>(a.copy);
    MinMax acc = mm_identity();
    uint64_t unordered = 0;
    // accumulate: what this workgroup's slot holds is asked for before the stream starts, so that the load's latency
    // is not left over at the end of a kernel that lasts a few microseconds
    MinMax held = mm_identity();
    if (a.accumulate && !a.first && threadIdx.x == 0)
        held = MinMax{a.part_min[blockIdx.x], a.part_max[blockIdx.x], a.part_nan[blockIdx.x]};
    const int64_t full_tiles = a.nvec / kFlatTileVec;
    for (int64_t tile = blockIdx.x; tile < full_tiles; tile += gridDim.x) {
        const int64_t v0 = tile * kFlatTileVec + threadIdx.x;
        Pack<IO, VEC> in[kFlatUnroll];
#pragma unroll
        for (int u = 0; u < kFlatUnroll; ++u) in[u] = load_pack_stream<IO, VEC>(x + (v0 + u * kFlatBlock) * VEC);
        if (cp) {
#pragma unroll
            for (int u = 0; u < kFlatUnroll; ++u) store_pack<IO, VEC>(cp + (v0 + u * kFlatBlock) * VEC, in[u]);
        }
#pragma unroll
        for (int u = 0; u < kFlatUnroll; ++u) mm_pack<IO, VEC, MODE>(in[u], acc.mn, acc.mx, unordered);
    }
    // the vectors past the last full tile: the workgroup after the one that took that tile
    if (blockIdx.x == a.tail_block) {
        for (int64_t v = full_tiles * kFlatTileVec + threadIdx.x; v < a.nvec; v += kFlatBlock) {
            const Pack<IO, VEC> p = load_pack_stream<IO, VEC>(x + v * VEC);
            if (cp) store_pack<IO, VEC>(cp + v * VEC, p);
#pragma unroll
            for (int k = 0; k < VEC; ++k) mm_add(acc, load_f32(p.v[k]), FINITE);
        }
    }
    if (VEC > 1 && blockIdx.x == 0) {  // elements past the last full vector
        const int64_t i = a.nvec * VEC + threadIdx.x;
        if (i < a.numel) {
            const IO v = x[i];
            if (cp) cp[i] = v;
            mm_add(acc, load_f32(v), FINITE);
        }
    }
    acc.nan |= unordered != 0 ? 1 : 0;
    const MinMax b = mm_block_reduce<kFlatBlock>(acc, red_smem);
    if (a.accumulate) {
        // min / max are idempotent and order-free, so slot b may hold the extrema of everything workgroup b has seen
        // in any batch; whoever wants the statistics folds the slots (minmax_fold_kernel), once
        if (threadIdx.x == 0) {
            const MinMax s = mm_merge(b, held);
            a.part_min[blockIdx.x] = s.mn;
            a.part_max[blockIdx.x] = s.mx;
            a.part_nan[blockIdx.x] = s.nan;
            if (a.batch_min) {
                a.batch_min[blockIdx.x] = b.mn;
                a.batch_max[blockIdx.x] = b.mx;
                a.batch_nan[blockIdx.x] = b.nan;
            }
        }
        if (blockIdx.x == 0) {
            for (int q = gridDim.x + threadIdx.x; q < kFlatMaxBlocks; q += kFlatBlock) {
                if (a.first) {
                    a.part_min[q] = __builtin_inff();
                    a.part_max[q] = -__builtin_inff();
                    a.part_nan[q] = 0;
                }
                if (a.batch_min) {
                    a.batch_min[q] = __builtin_inff();
                    a.batch_max[q] = -__builtin_inff();
                    a.batch_nan[q] = 0;
                }
            }
        }
        return;
    }
    if (threadIdx.x == 0) {
        if (gridDim.x == 1) {
            mm_write<IO>(a, 0, b);
        } else {
            a.part_min[blockIdx.x] = b.mn;
            a.part_max[blockIdx.x] = b.mx;
            a.part_nan[blockIdx.x] = b.nan;
        }
    }
}

// Folds the at most kFlatMaxBlocks partials of minmax_flat_kernel: one workgroup, one or two loads per lane.
constexpr int kFoldThreads = 256;
template <typename IO>
__global__ __launch_bounds__(kFoldThreads) void minmax_fold_kernel(const MmFlatArgs a, int nparts) {
    __shared__ MinMax red_smem[kFoldThreads / kWave];
    MinMax s = mm_identity();
    for (int q = threadIdx.x; q < nparts; q += kFoldThreads) s = mm_merge(s, MinMax{a.part_min[q], a.part_max[q], a.part_nan[q]});
    const MinMax r = mm_block_reduce<kFoldThreads>(s, red_smem);
    if (threadIdx.x == 0) mm_write<IO>(a, 0, r);
}

// Runs on the leading axis, each long enough for a workgroup (BLOCK = 256, runs of 512 vectors or more) or a wave
// (BLOCK = 64, runs of 64 to 511 vectors): the workgroup walks its run and writes the run's result itself -- no
// partials, no second launch, no atomics.  Per-channel weights ([4096, 4096]: one pass of four vectors per lane).
template <typename IO, int VEC, bool FINITE, int BLOCK>
__global__ __launch_bounds__(BLOCK) void minmax_runs_kernel(const MmRunArgs a) {
    __shared__ MinMax red_smem[BLOCK / kWave];
    constexpr int MODE = mm_mode(FINITE);
    const IO* __restrict__ x = static_cast<const IO*>(a.x) + (int64_t)blockIdx.x * a.kv * VEC;
    MinMax acc = mm_identity();
    uint64_t unordered = 0;
    int v = threadIdx.x;
    for (; v + (kUnroll - 1) * BLOCK < a.kv; v += kUnroll * BLOCK) {
        Pack<IO, VEC> in[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) in[u] = load_pack_stream<IO, VEC>(x + (int64_t)(v + u * BLOCK) * VEC);
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) mm_pack<IO, VEC, MODE>(in[u], acc.mn, acc.mx, unordered);
    }
    // what is left of the run: whole waves take part so that the ballots inside see defined values
    for (int v0 = v - threadIdx.x; v0 < a.kv; v0 += BLOCK) {
        const bool live = v0 + (int)threadIdx.x < a.kv;
        Pack<IO, VEC> pk;
        if (live) pk = load_pack_stream<IO, VEC>(x + (int64_t)(v0 + threadIdx.x) * VEC);
        else
#pragma unroll
            for (int k = 0; k < VEC; ++k) pk.v[k] = IO{};
        float mn = __builtin_inff(), mx = -__builtin_inff();
        mm_pack<IO, VEC, MODE>(pk, mn, mx, unordered);
        if (live) {
            acc.mn = fminf(acc.mn, mn);
            acc.mx = fmaxf(acc.mx, mx);
        }
    }
    acc.nan = unordered != 0 ? 1 : 0;
    MinMax b;
    if (BLOCK == kWave) {
        b = mm_wave_reduce(acc);
    } else {
        b = mm_block_reduce<BLOCK>(acc, red_smem);
    }
    if (threadIdx.x == 0) mm_write<IO>(a, blockIdx.x, b);
}

// Runs of a power-of-two number of lanes (up to 64) on the leading axis: blocks of 64 bf16 are 8 lanes.  A tile of
// kSegUnroll vectors per lane; the lanes of a run combine with data-parallel moves, the run leaders leave their
// results in LDS, and after one barrier consecutive lanes write consecutive encodings (whole cache lines instead of
// one 2- or 4-byte store per run leader).
// Loads: non-temporal for tensors of kStreamLoadBytes or more, which come from HBM whatever the caches hold (23.9 ->
// about 20 us on a 117 MB bf16 weight that is not resident); ordinary ones below, where a tensor is often still in
// the last-level cache from the kernel that wrote it and the ordinary load is the faster one (by 9 %).
constexpr int kSegUnroll = 2;
constexpr int kSegTileVec = kBlock * kSegUnroll;

// KV: lanes per run when that is at most 16 (the exchanges are then one instruction each, segment_min_f32), else 0
// (the general butterfly over a.kv lanes).  A full tile issues all its loads before it looks at any of them.
template <typename IO, int VEC, bool FINITE, int KV>
__global__ __launch_bounds__(kBlock) void minmax_seg_kernel(const MmRunArgs a) {
    __shared__ float s_mn[kSegTileVec], s_mx[kSegTileVec];
    __shared__ unsigned char s_nan[kSegTileVec];
    constexpr int MODE = mm_mode(FINITE);
    const int64_t v0 = (int64_t)blockIdx.x * kSegTileVec;
    const int64_t left = a.nvec - v0;
    const IO* __restrict__ x = static_cast<const IO*>(a.x) + v0 * VEC;
    const int kv = KV ? KV : a.kv;
    const int kv_shift = KV ? __builtin_ctz(KV ? KV : 1) : a.kv_shift;
    const int lane = threadIdx.x & (kWave - 1);
    const uint64_t run_lanes = kv >= kWave ? ~0ull : ((1ull << kv) - 1) << (lane & ~(kv - 1));
    Pack<IO, VEC> in[kSegUnroll];
    if (left >= kSegTileVec) {
        if (a.stream_loads) {
#pragma unroll
            for (int u = 0; u < kSegUnroll; ++u) in[u] = load_pack_stream<IO, VEC>(x + (int64_t)(u * kBlock + threadIdx.x) * VEC);
        } else {
#pragma unroll
            for (int u = 0; u < kSegUnroll; ++u) in[u] = load_pack<IO, VEC>(x + (int64_t)(u * kBlock + threadIdx.x) * VEC);
        }
    } else {
#pragma unroll
        for (int u = 0; u < kSegUnroll; ++u) {
            const int lv = u * kBlock + threadIdx.x;
            if (lv < left) in[u] = load_pack<IO, VEC>(x + (int64_t)lv * VEC);
            else
#pragma unroll
                for (int k = 0; k < VEC; ++k) in[u].v[k] = IO{};
        }
    }
#pragma unroll
    for (int u = 0; u < kSegUnroll; ++u) {
        const int lv = u * kBlock + threadIdx.x;
        float mn = __builtin_inff(), mx = -__builtin_inff();
        uint64_t unordered = 0;
        mm_pack<IO, VEC, MODE>(in[u], mn, mx, unordered);
        if constexpr (KV != 0) {
            mn = segment_min_f32<KV>(mn);
            mx = segment_max_f32<KV>(mx);
        } else {
            mn = segment_reduce(mn, kv, OpMinF());
            mx = segment_reduce(mx, kv, OpMaxF());
        }
        if ((lane & (kv - 1)) == 0 && lv < left) {  // runs are whole inside the tensor: a live leader means a live run
            const int slot = lv >> kv_shift;
            s_mn[slot] = mn;
            s_mx[slot] = mx;
            s_nan[slot] = (unordered & run_lanes) != 0 ? 1 : 0;
        }
    }
    __syncthreads();
    const int nslots = (int)((left < kSegTileVec ? left : (int64_t)kSegTileVec) >> kv_shift);
    const int64_t e0 = v0 >> kv_shift;
    for (int t = threadIdx.x; t < nslots; t += kBlock) mm_write<IO>(a, e0 + t, MinMax{s_mn[t], s_mx[t], (int)s_nan[t]});
}

// Folds the per-tile partials of every encoding (second launch; see the note on fences in qdq.hip).
constexpr int kFinishThreads = 1024;
template <typename IO>
__global__ __launch_bounds__(kFinishThreads) void minmax_finish_kernel(const MmArgs a, int64_t nparts) {
    __shared__ MinMax red_smem[kFinishThreads / kWave];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    if (a.mode != kRows) {
        MinMax s = mm_identity();
#pragma unroll 4
        for (int64_t q = threadIdx.x; q < nparts; q += kFinishThreads) s = mm_merge(s, MinMax{a.part_min[q], a.part_max[q], a.part_nan[q]});
#pragma unroll
        for (int m = kWave / 2; m >= 1; m >>= 1) s = mm_merge(s, mm_shfl_xor(s, m));
        if (lane == 0) red_smem[wave] = s;
        __syncthreads();
        if (threadIdx.x == 0) {
            MinMax r = red_smem[0];
            for (int w = 1; w < kFinishThreads / kWave; ++w) r = mm_merge(r, red_smem[w]);
            mm_write<IO>(a, 0, r);
        }
        return;
    }
    const int64_t per_enc = a.I * (int64_t)a.tpr;
    const int64_t wave0 = (int64_t)blockIdx.x * (kFinishThreads / kWave) + wave;
    for (int64_t j = wave0; j < a.J; j += (int64_t)gridDim.x * (kFinishThreads / kWave)) {
        MinMax s = mm_identity();
        for (int64_t q = lane; q < per_enc; q += kWave) {
            const int64_t i = q / a.tpr, tt = q - i * a.tpr;
            const int64_t blk = (i * a.J + j) * a.tpr + tt;
            s = mm_merge(s, MinMax{a.part_min[blk], a.part_max[blk], a.part_nan[blk]});
        }
#pragma unroll
        for (int m = kWave / 2; m >= 1; m >>= 1) s = mm_merge(s, mm_shfl_xor(s, m));
        if (lane == 0) mm_write<IO>(a, j, s);
    }
}

template <typename IO>
__global__ __launch_bounds__(kBlock) void minmax_generic_kernel(const MmArgs a) {
    const IO* __restrict__ x = static_cast<const IO*>(a.x);
    const bool fo = a.finite_only == 1;
    const int lane = threadIdx.x & (kWave - 1);
    // every lane of a wave runs the same number of iterations (inactive ones carry the identity), so the wave-level
    // exchanges below are executed by whole waves
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    const int64_t first = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    for (int64_t base = first - lane; base < a.numel; base += stride) {
        const int64_t i = base + lane;
        const bool active = i < a.numel;
        const int64_t e = active ? generic_enc_index(a, i) : -1;
        MinMax v = mm_identity();
        if (active) mm_add(v, load_f32(x[i]), fo);
        // neighbouring elements mostly share an encoding: the lanes of each distinct encoding are combined first and
        // one lane issues the atomics (64 times fewer of them when the whole wave lies in one block)
        uint64_t todo = __builtin_amdgcn_ballot_w64(active);
        while (todo != 0) {
            const int lead = __builtin_ctzll(todo);
            const int64_t el = __shfl(e, lead, kWave);
            const bool mine = active && e == el;
            MinMax m = mine ? v : mm_identity();
#pragma unroll
            for (int k = kWave / 2; k >= 1; k >>= 1) m = mm_merge(m, mm_shfl_xor(m, k));
            if (lane == lead) {
                atomicMin(&a.key_min[el], f32_key(m.mn));
                atomicMax(&a.key_max[el], f32_key(m.mx));
                if (m.nan) atomicOr(&a.part_nan[el], 1);
            }
            todo &= ~__builtin_amdgcn_ballot_w64(mine);
        }
    }
}

// Encodings that change with every element (run length 1, e.g. per-channel along the fastest axis): a lane owns VEC
// neighbouring encodings and walks down rows, so loads stay coalesced 16-byte vectors.  A workgroup is 64 lanes
// across x kMmColWaves waves down; the waves take rows in turn, kMmColUnroll loads in flight each, and the grid's y
// axis splits the rows into row groups.  The waves' extrema meet in LDS, the workgroup's go to its row of the
// partials ([row group][encoding]: no atomics, nothing to clear) and minmax_cols_finish_kernel folds the row groups.
constexpr int kMmColWaves = 16;
constexpr int kMmColUnroll = 4;  // even: rows are taken in pairs
template <typename IO, int VEC, bool FINITE>
__global__ __launch_bounds__(kMmColWaves * kWave) void minmax_cols_kernel(const MmArgs a, int stream_loads) {
    constexpr int kHalf = kMmColWaves / 2;  // the upper half of the waves hands over to the lower half first
    __shared__ float smn[kHalf][kWave * VEC], smx[kHalf][kWave * VEC];
    __shared__ unsigned char snan[kHalf][kWave * VEC];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int64_t cbase = (int64_t)blockIdx.x * kWave * VEC;  // first column of the workgroup
    const int64_t c0 = cbase + (int64_t)lane * VEC;
    // stacked columns: problem blockIdx.z has its own I x J elements, J encodings and gridDim.y rows of partials
    const IO* __restrict__ x = static_cast<const IO*>(a.x) + (int64_t)blockIdx.z * a.I * a.J;
    MinMax m[VEC];
#pragma unroll
    for (int k = 0; k < VEC; ++k) m[k] = mm_identity();
    if (c0 < a.J) {
        // NaN is looked for with one unordered comparison per pair of rows; the comparison's lane mask is OR-ed on the
        // scalar unit, one mask per encoding of the lane (see mm_pack)
        uint64_t unordered[VEC];
#pragma unroll
        for (int k = 0; k < VEC; ++k) unordered[k] = 0;
        const int64_t step = (int64_t)gridDim.y * kMmColWaves * kMmColUnroll;
        for (int64_t r0 = ((int64_t)blockIdx.y * kMmColWaves + wave) * kMmColUnroll; r0 < a.I; r0 += step) {
            Pack<IO, VEC> pk[kMmColUnroll];
#pragma unroll
            for (int u = 0; u < kMmColUnroll; ++u) {
                // rows past the end are read as the step's first row again: extrema do not mind
                const int64_t r = r0 + u < a.I ? r0 + u : r0;
                pk[u] = stream_loads ? load_pack_stream<IO, VEC>(x + r * a.J + c0) : load_pack<IO, VEC>(x + r * a.J + c0);
            }
#pragma unroll
            for (int u = 0; u < kMmColUnroll; u += 2) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    const float f0 = load_f32(pk[u].v[k]), f1 = load_f32(pk[u + 1].v[k]);
                    if (FINITE) {
                        mm_add(m[k], f0, true);
                        mm_add(m[k], f1, true);
                    } else {
                        m[k].mn = fminf(fminf(m[k].mn, f0), f1);
                        m[k].mx = fmaxf(fmaxf(m[k].mx, f0), f1);
                        unordered[k] |= __builtin_amdgcn_ballot_w64(__builtin_isunordered(f0, f1));
                    }
                }
            }
        }
#pragma unroll
        for (int k = 0; k < VEC; ++k) m[k].nan = (int)((unordered[k] >> lane) & 1);
    }
    if (wave >= kHalf) {
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            smn[wave - kHalf][lane * VEC + k] = m[k].mn;
            smx[wave - kHalf][lane * VEC + k] = m[k].mx;
            snan[wave - kHalf][lane * VEC + k] = (unsigned char)m[k].nan;
        }
    }
    __syncthreads();
    if (wave < kHalf) {
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            const int c = lane * VEC + k;
            m[k] = mm_merge(m[k], MinMax{smn[wave][c], smx[wave][c], snan[wave][c]});
            smn[wave][c] = m[k].mn;
            smx[wave][c] = m[k].mx;
            snan[wave][c] = (unsigned char)m[k].nan;
        }
    }
    __syncthreads();
    // a thread per column of the workgroup: neighbouring threads read neighbouring LDS words and store neighbouring
    // partials
    for (int c = threadIdx.x; c < kWave * VEC; c += kMmColWaves * kWave) {
        if (cbase + c >= a.J) break;
        MinMax r = mm_identity();
#pragma unroll
        for (int w = 0; w < kHalf; ++w) r = mm_merge(r, MinMax{smn[w][c], smx[w][c], snan[w][c]});
        if (gridDim.y == 1) {  // a single row group: these are the extrema themselves, no finish launch follows
            mm_write<IO>(a, (int64_t)blockIdx.z * a.J + cbase + c, r);
            continue;
        }
        const int64_t slot = ((int64_t)blockIdx.z * gridDim.y + blockIdx.y) * a.J + cbase + c;
        a.part_min[slot] = r.mn;
        a.part_max[slot] = r.mx;
        a.part_nan[slot] = r.nan;
    }
}

// Folds the row groups of minmax_cols_kernel: a lane per encoding (coalesced reads), the waves of a workgroup take
// the row groups in turn and meet in LDS.
constexpr int kMmColFinishWaves = 4;
template <typename IO>
__global__ __launch_bounds__(kMmColFinishWaves * kWave) void minmax_cols_finish_kernel(const MmArgs a, int groups) {
    __shared__ MinMax shares[kMmColFinishWaves][kWave];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int64_t e = (int64_t)blockIdx.x * kWave + lane;
    MinMax r = mm_identity();
    if (e < a.J) {
#pragma unroll 4
        for (int q = wave; q < groups; q += kMmColFinishWaves) {
            const int64_t slot = ((int64_t)blockIdx.y * groups + q) * a.J + e;
            r = mm_merge(r, MinMax{a.part_min[slot], a.part_max[slot], a.part_nan[slot]});
        }
    }
    shares[wave][lane] = r;
    __syncthreads();
    if (wave == 0 && e < a.J) {
#pragma unroll
        for (int w = 1; w < kMmColFinishWaves; ++w) r = mm_merge(r, shares[w][lane]);
        mm_write<IO>(a, (int64_t)blockIdx.y * a.J + e, r);  // blockIdx.y: the stacked problem
    }
}

__global__ void minmax_keys_init_kernel(unsigned int* kmn, unsigned int* kmx, int* nan, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        kmn[i] = 0xff800000u;  // key of +inf
        kmx[i] = 0x007fffffu;  // key of -inf
        nan[i] = 0;
    }
}

template <typename IO>
__global__ void minmax_keys_finish_kernel(const MmArgs a, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        mm_write<IO>(a, i, MinMax{key_f32(a.key_min[i]), key_f32(a.key_max[i]), a.part_nan[i]});
}

template <typename IO, int RED, bool FINITE>
static void launch_mm_red(const Plan& p, const MmArgs& a, hipStream_t st) {
    if (p.vec == 1) hipLaunchKernelGGL((minmax_kernel<IO, 1, RED, FINITE>), dim3(p.nblocks), dim3(kBlock), 0, st, a);
    else hipLaunchKernelGGL((minmax_kernel<IO, IoTraits<IO>::kVec, RED, FINITE>), dim3(p.nblocks), dim3(kBlock), 0, st, a);
}

static int64_t flat_blocks(const Plan& p) {
    const int64_t tiles = p.nvec > 0 ? (p.nvec + kFlatTileVec - 1) / kFlatTileVec : 1;
    return tiles < kFlatMaxBlocks ? tiles : kFlatMaxBlocks;
}

// Partial triples (min, max, saw-NaN: 12 bytes) a reduction keeps in its workspace: one per workgroup of the
// single-encoding kernel (at most kFlatMaxBlocks, whatever the tensor's size), else what the plan says (one per tile
// or per encoding).
static size_t mm_ws_elems(const Plan& p) {
    if (p.cl.kind == kIJK && p.cl.J == 1) return (size_t)flat_blocks(p);
    return p.ws_elems;
}

// Elements per lane of the column-walking kernel, 0 where it does not apply.
static int mm_cols_lane_elems(int io_dtype, const Plan& p) {
    return p.red == kRedAtomic ? cols_lane_elems(io_dtype, p, p.ptr_aligned) : 0;
}

// Row groups the column-walking kernel would like (about 256 workgroups of sixteen waves, four waves per SIMD of 256
// CUs, every wave at least one step of rows: 8192 x 4096 bf16 17.9 us, 18.6 us with 512 workgroups, 21.4 us with 1024;
// fp32 25.9 / 27.5 / 27.7 us) and the partial triples they need.  The workspace every reduction of this layout needs
// is one row of partials (12 bytes per encoding); with less than the preferred size the kernel runs with as many row
// groups as fit.
static int64_t mm_cols_row_groups(int io_dtype, const Plan& p) {
    const int n = mm_cols_lane_elems(io_dtype, p);
    const int64_t gx = ((p.cl.J + n - 1) / n + kWave - 1) / kWave;
    const int64_t most = (p.cl.I + kMmColWaves * kMmColUnroll - 1) / (kMmColWaves * kMmColUnroll);
    int64_t gy = (256 + gx * p.cl.A - 1) / (gx * p.cl.A);
    gy = gy > most ? most : gy;
    return gy < 1 ? 1 : (gy > 65535 ? 65535 : gy);
}

static MmFlatArgs flat_args(const Plan& p, const MmArgs& a) {
    MmFlatArgs f{};
    static_cast<MmOut&>(f) = static_cast<const MmOut&>(a);
    f.x = a.x;
    f.copy = a.copy;
    f.numel = p.cl.numel;
    f.nvec = p.nvec;
    f.tail_block = (uint32_t)((p.nvec / kFlatTileVec) % flat_blocks(p));
    f.part_min = a.part_min;
    f.part_max = a.part_max;
    f.part_nan = a.part_nan;
    return f;
}

template <typename IO, bool FINITE>
static void launch_mm(const Plan& p, const MmArgs& a, hipStream_t st, int cols_groups) {
    const int64_t ne = p.cl.num_enc;
    const unsigned gb = (unsigned)((ne + 255) / 256 > 1024 ? 1024 : (ne + 255) / 256);
    if (p.cl.kind == kIJK && p.cl.J == 1) {
        const int64_t nb = flat_blocks(p);
        const MmFlatArgs f = flat_args(p, a);
        if (p.vec == 1) hipLaunchKernelGGL((minmax_flat_kernel<IO, 1, FINITE>), dim3((unsigned)nb), dim3(kFlatBlock), 0, st, f);
        else hipLaunchKernelGGL((minmax_flat_kernel<IO, IoTraits<IO>::kVec, FINITE>), dim3((unsigned)nb), dim3(kFlatBlock), 0, st, f);
        if (nb > 1) hipLaunchKernelGGL((minmax_fold_kernel<IO>), dim3(1), dim3(kFoldThreads), 0, st, f, (int)nb);
        return;
    }
    // runs on the leading axis that a workgroup, a wave or a group of lanes can own: lean kernels, one launch
    if (p.cl.kind == kIJK && p.cl.I == 1 && p.cl.J > 1 && p.vec > 1 && p.cl.J <= 0x7fffffff && p.Kv <= 0x7fffffff) {
        MmRunArgs r{};
        static_cast<MmOut&>(r) = static_cast<const MmOut&>(a);
        r.x = a.x;
        r.nvec = p.nvec;
        r.runs = p.cl.J;
        r.kv = (int32_t)p.Kv;
        r.kv_shift = 0;
        while ((1 << r.kv_shift) < r.kv) ++r.kv_shift;
        r.stream_loads = p.cl.numel * (int64_t)sizeof(IO) >= kStreamLoadBytes ? 1 : 0;
        constexpr int V = IoTraits<IO>::kVec;
        // a workgroup per run needs enough runs to fill the GPU, or runs short enough not to matter; a few very long
        // runs keep the tiled kernel with its partials
        if (p.Kv >= 2 * kBlock && (p.cl.J >= 512 || p.Kv <= 8 * kTileVec)) {
            hipLaunchKernelGGL((minmax_runs_kernel<IO, V, FINITE, kBlock>), dim3((unsigned)p.cl.J), dim3(kBlock), 0, st, r);
            return;
        }
        if (p.Kv >= kWave && p.Kv < 2 * kBlock) {
            hipLaunchKernelGGL((minmax_runs_kernel<IO, V, FINITE, kWave>), dim3((unsigned)p.cl.J), dim3(kWave), 0, st, r);
            return;
        }
        if (p.Kv < kWave && is_pow2(p.Kv)) {
            const int64_t nb = (p.nvec + kSegTileVec - 1) / kSegTileVec;
            const dim3 g((unsigned)nb), b(kBlock);
            switch (r.kv) {
                case 1: hipLaunchKernelGGL((minmax_seg_kernel<IO, V, FINITE, 1>), g, b, 0, st, r); break;
                case 2: hipLaunchKernelGGL((minmax_seg_kernel<IO, V, FINITE, 2>), g, b, 0, st, r); break;
                case 4: hipLaunchKernelGGL((minmax_seg_kernel<IO, V, FINITE, 4>), g, b, 0, st, r); break;
                case 8: hipLaunchKernelGGL((minmax_seg_kernel<IO, V, FINITE, 8>), g, b, 0, st, r); break;
                case 16: hipLaunchKernelGGL((minmax_seg_kernel<IO, V, FINITE, 16>), g, b, 0, st, r); break;
                default: hipLaunchKernelGGL((minmax_seg_kernel<IO, V, FINITE, 0>), g, b, 0, st, r); break;
            }
            return;
        }
    }
    if (cols_groups > 0) {
        constexpr int V = IoTraits<IO>::kVec;
        const int n = mm_cols_lane_elems(IoTraits<IO>::kDtype, p);
        const dim3 g((unsigned)(((p.cl.J + n - 1) / n + kWave - 1) / kWave), (unsigned)cols_groups, (unsigned)p.cl.A);
        const int stream_loads = p.cl.numel * (int64_t)sizeof(IO) >= kStreamLoadBytes ? 1 : 0;
        if (n == V) hipLaunchKernelGGL((minmax_cols_kernel<IO, V, FINITE>), g, dim3(kMmColWaves * kWave), 0, st, a, stream_loads);
        else hipLaunchKernelGGL((minmax_cols_kernel<IO, 1, FINITE>), g, dim3(kMmColWaves * kWave), 0, st, a, stream_loads);
        if (cols_groups > 1)
            hipLaunchKernelGGL((minmax_cols_finish_kernel<IO>), dim3((unsigned)((p.cl.J + kWave - 1) / kWave), (unsigned)p.cl.A),
                           dim3(kMmColFinishWaves * kWave), 0, st, a, cols_groups);
        return;
    }
    if (p.red == kRedAtomic) hipLaunchKernelGGL(minmax_keys_init_kernel, dim3(gb), dim3(256), 0, st, a.key_min, a.key_max, a.part_nan, ne);
    if (p.cl.kind == kGeneric) {
        hipLaunchKernelGGL((minmax_generic_kernel<IO>), dim3(p.nblocks), dim3(kBlock), 0, st, a);
    } else if (p.red == kRedTile) {
        launch_mm_red<IO, kRedTile, FINITE>(p, a, st);
        const int64_t per_enc = p.cl.I * (int64_t)p.tpr;
        if (per_enc > 1) {
            const int64_t waves = kFinishThreads / kWave;
            const int64_t nb = (p.cl.J + waves - 1) / waves;
            hipLaunchKernelGGL((minmax_finish_kernel<IO>), dim3((unsigned)(nb > 4096 ? 4096 : nb)), dim3(kFinishThreads), 0, st, a, per_enc);
        }
    } else if (p.red == kRedSeg) {
        launch_mm_red<IO, kRedSeg, FINITE>(p, a, st);
    } else {
        launch_mm_red<IO, kRedAtomic, FINITE>(p, a, st);
    }
    if (p.red == kRedAtomic) hipLaunchKernelGGL((minmax_keys_finish_kernel<IO>), dim3(gb), dim3(256), 0, st, a, ne);
}

}  // namespace ahq

using namespace ahq;

extern "C" int ahq_minmax(int32_t dtype, const ahq_layout* layout, const void* x, void* out_min, void* out_max,
                          void* run_min, void* run_max, int finite_only, void* workspace, size_t workspace_bytes,
                          void* stream);

// Library-internal: the finite-only extrema for a caller that will fold the per-workgroup partials itself.  For a
// single encoding over more than one workgroup only the streaming kernel is launched and the partial arrays are
// handed back (*nparts > 0, out_min / out_max untouched); every other layout runs the complete reduction into
// out_min / out_max (*nparts == 0).
extern "C" __attribute__((visibility("hidden"))) int ahq_minmax_finite_partials(
    int32_t dtype, const ahq_layout* layout, const void* x, void* out_min, void* out_max, void* workspace,
    size_t workspace_bytes, void* stream, const float** part_min, const float** part_max, int64_t* nparts) {
    *nparts = 0;
    Plan p;
    if (dtype < AHQ_F32 || dtype > AHQ_BF16 || !layout || !make_plan(dtype, *layout, aligned16(x), true, &p) ||
        !(p.cl.kind == kIJK && p.cl.J == 1) || flat_blocks(p) <= 1 || !x || !workspace ||
        workspace_bytes < mm_ws_elems(p) * 12)
        return ahq_minmax(dtype, layout, x, out_min, out_max, nullptr, nullptr, 1, workspace, workspace_bytes, stream);
    MmArgs a{};
    fill_geom(p, &a);
    a.x = x;
    a.red = p.red;
    a.finite_only = 1;
    char* w = static_cast<char*>(workspace);
    a.part_min = reinterpret_cast<float*>(w);
    a.part_max = reinterpret_cast<float*>(w + mm_ws_elems(p) * 4);
    a.part_nan = reinterpret_cast<int*>(w + mm_ws_elems(p) * 8);
    const int64_t nb = flat_blocks(p);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const MmFlatArgs f = flat_args(p, a);
#define AHQ_FLAT(IO)                                                                                                  \
    do {                                                                                                              \
        if (p.vec == 1) hipLaunchKernelGGL((minmax_flat_kernel<IO, 1, true>), dim3((unsigned)nb), dim3(kFlatBlock), 0, st, f); \
        else hipLaunchKernelGGL((minmax_flat_kernel<IO, IoTraits<IO>::kVec, true>), dim3((unsigned)nb), dim3(kFlatBlock), 0, st, f); \
    } while (0)
    switch (dtype) {
        case AHQ_F32: AHQ_FLAT(float); break;
        case AHQ_F16: AHQ_FLAT(f16_t); break;
        default: AHQ_FLAT(bf16_t); break;
    }
#undef AHQ_FLAT
    *part_min = a.part_min;
    *part_max = a.part_max;
    *nparts = nb;
    return check_launch("ahq_minmax");
}

extern "C" size_t ahq_minmax_workspace_bytes(const ahq_layout* layout) {
    if (!layout) return 0;
    // the widest plan over dtypes and alignments decides; 12 bytes per tile or per encoding
    size_t need = 0;
    for (int dt = AHQ_F32; dt <= AHQ_BF16; ++dt)
        for (int al = 0; al < 2; ++al) {
            Plan p;
            if (!make_plan(dt, *layout, al != 0, true, &p)) continue;
            size_t n = mm_ws_elems(p) * 12;
            if (mm_cols_lane_elems(dt, p) > 0) n = (size_t)p.cl.A * (size_t)mm_cols_row_groups(dt, p) * (size_t)p.cl.J * 12;  // the preferred size
            if (n > need) need = n;
        }
    return need;
}

static int minmax_impl(int32_t dtype, const ahq_layout* layout, const void* x, void* copy, void* out_min, void* out_max,
                       void* run_min, void* run_max, int finite_only, void* workspace, size_t workspace_bytes,
                       void* stream) {
    if (dtype < AHQ_F32 || dtype > AHQ_BF16) return set_error("bad dtype"), AHQ_ERR_INVALID;
    if (!layout) return set_error("layout is null"), AHQ_ERR_INVALID;
    if (!out_min || !out_max) return set_error("out_min or out_max is null"), AHQ_ERR_INVALID;
    if ((run_min == nullptr) != (run_max == nullptr)) return set_error("run_min and run_max must be given together"), AHQ_ERR_INVALID;
    Plan p;
    if (!make_plan(dtype, *layout, aligned16(x) && aligned16(copy), true, &p)) return AHQ_ERR_INVALID;
    if (p.cl.numel == 0) return set_error("cannot reduce an empty tensor"), AHQ_ERR_INVALID;
    if (!x) return set_error("x is null"), AHQ_ERR_INVALID;
    const size_t ws_elems = mm_ws_elems(p);
    const size_t need = ws_elems * 12;
    const int64_t per_enc = p.red == kRedTile ? (p.mode == kRows ? p.cl.I * (int64_t)p.tpr : (int64_t)p.nblocks) : 0;
    const bool uses_ws = p.red == kRedAtomic || (p.red == kRedTile && per_enc > 1);
    if (uses_ws && (!workspace || workspace_bytes < need)) return set_error("workspace too small"), AHQ_ERR_WORKSPACE;
    MmArgs a{};
    fill_geom(p, &a);
    a.x = x;
    a.out_min = out_min;
    a.out_max = out_max;
    a.red = p.red;
    a.run_min = run_min;
    a.run_max = run_max;
    a.finite_only = finite_only;
    int cols_groups = 0;  // > 0: the column-walking kernel with that many row groups
    if (uses_ws) {
        size_t slots = ws_elems;
        if (mm_cols_lane_elems(dtype, p) > 0) {
            const int64_t fit = (int64_t)(workspace_bytes / ((size_t)p.cl.A * (size_t)p.cl.J * 12));
            const int64_t want = mm_cols_row_groups(dtype, p);
            cols_groups = (int)(fit < want ? fit : want);
            slots = (size_t)p.cl.A * (size_t)cols_groups * (size_t)p.cl.J;
        }
        char* w = static_cast<char*>(workspace);
        a.part_min = reinterpret_cast<float*>(w);
        a.part_max = reinterpret_cast<float*>(w + slots * 4);
        a.part_nan = reinterpret_cast<int*>(w + slots * 8);
        a.key_min = reinterpret_cast<unsigned int*>(w);
        a.key_max = reinterpret_cast<unsigned int*>(w + slots * 4);
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (copy) {
        // the streaming kernel of the single-encoding case writes the copy itself; other layouts copy separately
        if (p.cl.kind == kIJK && p.cl.J == 1) {
            a.copy = copy;
        } else if (hipMemcpyAsync(copy, x, (size_t)p.cl.numel * io_size(dtype), hipMemcpyDeviceToDevice, st) != hipSuccess) {
            return set_error("device-to-device copy failed"), AHQ_ERR_LAUNCH;
        }
    }
#define AHQ_MM(IO) do { if (finite_only == 1) launch_mm<IO, true>(p, a, st, cols_groups); else launch_mm<IO, false>(p, a, st, cols_groups); } while (0)
    switch (dtype) {
        case AHQ_F32: AHQ_MM(float); break;
        case AHQ_F16: AHQ_MM(f16_t); break;
        default: AHQ_MM(bf16_t); break;
    }
#undef AHQ_MM
    return check_launch("ahq_minmax");
}

extern "C" int ahq_minmax(int32_t dtype, const ahq_layout* layout, const void* x, void* out_min, void* out_max,
                          void* run_min, void* run_max, int finite_only, void* workspace, size_t workspace_bytes,
                          void* stream) {
    return minmax_impl(dtype, layout, x, nullptr, out_min, out_max, run_min, run_max, finite_only, workspace,
                       workspace_bytes, stream);
}

extern "C" int ahq_minmax_copy(int32_t dtype, const ahq_layout* layout, const void* x, void* y, void* out_min,
                               void* out_max, void* run_min, void* run_max, int finite_only, void* workspace,
                               size_t workspace_bytes, void* stream) {
    if (!y) return set_error("y is null"), AHQ_ERR_INVALID;
    if (y == x) return set_error("y must not alias x"), AHQ_ERR_INVALID;
    return minmax_impl(dtype, layout, x, y, out_min, out_max, run_min, run_max, finite_only, workspace, workspace_bytes,
                       stream);
}

// ------------------------------------------------------------------- running extrema as one slot per workgroup --
static_assert(AHQ_MINMAX_SLOTS == kFlatMaxBlocks, "the slots are the partials of the single-encoding kernel");
static_assert(AHQ_MINMAX_SLOTS_BYTES == 12 * kFlatMaxBlocks, "two floats and a flag per slot");

static MmFlatArgs slot_args(void* slots) {
    MmFlatArgs f{};
    char* w = static_cast<char*>(slots);
    f.part_min = reinterpret_cast<float*>(w);
    f.part_max = reinterpret_cast<float*>(w + 4 * kFlatMaxBlocks);
    f.part_nan = reinterpret_cast<int*>(w + 8 * kFlatMaxBlocks);
    return f;
}

extern "C" int ahq_minmax_accumulate(int32_t dtype, const void* x, int64_t count, void* copy_to, void* slots,
                                     void* batch_slots, int32_t first, void* stream) {
    if (dtype < AHQ_F32 || dtype > AHQ_BF16) return set_error("bad dtype"), AHQ_ERR_INVALID;
    if (count < 0) return set_error("negative element count"), AHQ_ERR_INVALID;
    if (!slots || (reinterpret_cast<uintptr_t>(slots) & 3u)) return set_error("slots is null or misaligned"), AHQ_ERR_INVALID;
    if (batch_slots && ((reinterpret_cast<uintptr_t>(batch_slots) & 3u) || batch_slots == slots))
        return set_error("batch_slots is misaligned or aliases slots"), AHQ_ERR_INVALID;
    if (count > 0 && !x) return set_error("x is null"), AHQ_ERR_INVALID;
    if (copy_to && copy_to == x) return set_error("copy_to must not alias x"), AHQ_ERR_INVALID;
    if (count == 0 && !first && !batch_slots) return AHQ_OK;  // nothing to add; an empty first batch still clears the slots
    MmFlatArgs f = slot_args(slots);
    if (batch_slots) {
        const MmFlatArgs b = slot_args(batch_slots);
        f.batch_min = b.part_min;
        f.batch_max = b.part_max;
        f.batch_nan = b.part_nan;
    }
    f.x = x;
    f.copy = copy_to;
    f.numel = count;
    const int vec = (aligned16(x) && (!copy_to || aligned16(copy_to))) ? io_vec(dtype) : 1;
    f.nvec = count / vec;
    f.accumulate = 1;
    f.first = first ? 1 : 0;
    const int64_t tiles = f.nvec > 0 ? (f.nvec + kFlatTileVec - 1) / kFlatTileVec : 1;
    const unsigned nb = (unsigned)(tiles < kFlatMaxBlocks ? tiles : kFlatMaxBlocks);
    f.tail_block = (uint32_t)((f.nvec / kFlatTileVec) % nb);
    hipStream_t st = static_cast<hipStream_t>(stream);
#define AHQ_LAUNCH_ACC(IO)                                                                                              \
    do {                                                                                                                \
        if (vec == 1) hipLaunchKernelGGL((minmax_flat_kernel<IO, 1, false>), dim3(nb), dim3(kFlatBlock), 0, st, f);        \
        else hipLaunchKernelGGL((minmax_flat_kernel<IO, IoTraits<IO>::kVec, false>), dim3(nb), dim3(kFlatBlock), 0, st, f); \
    } while (0)
    switch (dtype) {
        case AHQ_F32: AHQ_LAUNCH_ACC(float); break;
        case AHQ_F16: AHQ_LAUNCH_ACC(f16_t); break;
        default: AHQ_LAUNCH_ACC(bf16_t); break;
    }
#undef AHQ_LAUNCH_ACC
    return check_launch("ahq_minmax_accumulate");
}

extern "C" int ahq_minmax_slots_read(int32_t dtype, const void* slots, void* out_min, void* out_max, void* stream) {
    if (dtype < AHQ_F32 || dtype > AHQ_BF16) return set_error("bad dtype"), AHQ_ERR_INVALID;
    if (!slots || !out_min || !out_max) return set_error("null argument"), AHQ_ERR_INVALID;
    MmFlatArgs f = slot_args(const_cast<void*>(slots));
    f.out_min = out_min;
    f.out_max = out_max;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case AHQ_F32: hipLaunchKernelGGL((minmax_fold_kernel<float>), dim3(1), dim3(kFoldThreads), 0, st, f, kFlatMaxBlocks); break;
        case AHQ_F16: hipLaunchKernelGGL((minmax_fold_kernel<f16_t>), dim3(1), dim3(kFoldThreads), 0, st, f, kFlatMaxBlocks); break;
        default: hipLaunchKernelGGL((minmax_fold_kernel<bf16_t>), dim3(1), dim3(kFoldThreads), 0, st, f, kFlatMaxBlocks); break;
    }
    return check_launch("ahq_minmax_slots_read");
}

// ------------------------------------------------------------------------------------ entry point without allocation --
namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {nullptr};  // device address of `scratch` on each device, looked up on first use

// Address of the current device's copy of `scratch`.
int static_scratch(void** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
        return set_error("ahq_minmax_static: cannot identify the current device"), AHQ_ERR_LAUNCH;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            std::snprintf(error_buffer(), 512, "ahq_minmax_static: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
            return AHQ_ERR_LAUNCH;
        }
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return AHQ_OK;
}

}  // namespace

extern "C" int ahq_minmax_static(int32_t dtype, const ahq_layout* layout, const void* x, void* out_min, void* out_max,
                                 void* run_min, void* run_max, int finite_only, void* stream) {
    if (dtype < AHQ_F32 || dtype > AHQ_BF16) return set_error("bad dtype"), AHQ_ERR_INVALID;
    if (!layout) return set_error("layout is null"), AHQ_ERR_INVALID;
    // the size check comes first and needs no device: the plan is host arithmetic
    Plan p;
    if (!make_plan(dtype, *layout, aligned16(x), true, &p)) return AHQ_ERR_INVALID;
    const size_t need = mm_ws_elems(p) * 12;
    if (need > kStaticScratchBytes) {
        std::snprintf(error_buffer(), 512,
                      "ahq_minmax_static: this reduction needs %zu bytes of scratch, the static buffer holds %zu; "
                      "use ahq_minmax with a caller-provided workspace",
                      need, kStaticScratchBytes);
        return AHQ_ERR_WORKSPACE;
    }
    if (!x || !out_min || !out_max) return set_error("x, out_min or out_max is null"), AHQ_ERR_INVALID;
    void* ws = nullptr;
    const int rc = static_scratch(&ws);
    if (rc != AHQ_OK) return rc;
    return minmax_impl(dtype, layout, x, nullptr, out_min, out_max, run_min, run_max, finite_only, ws,
                       kStaticScratchBytes, stream);
}
