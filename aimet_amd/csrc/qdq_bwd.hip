// Fake-quantization backward kernels: straight-through input gradient and the per-encoding scale / offset gradients
// (arithmetic and arguments: qdq_common.h).

#include "qdq_common.h"

namespace ahq {

__device__ __forceinline__ float finish_sum_rt(double s, int cd) {
    if (cd == AHQ_BF16) return rnd<AHQ_BF16>((float)s);
    if (cd == AHQ_F16) return rnd<AHQ_F16>((float)s);
    return (float)s;
}

template <typename IO, int VEC, typename M, int RED, bool FULL, bool FAST>
__device__ __forceinline__ void bwd_math(const QdqArgs& a, const Tile& t, float (*sp)[kStage], const Pack<IO, VEC>* xin,
                                         const Pack<IO, VEC>* gin, IO* __restrict__ gxp, double& acc_s, double& acc_o,
                                         double* stage_sums, float* vec_sums, int base) {
#pragma unroll
    for (int u = 0; u < kBwdUnroll; ++u) {
        const int lv = base + u * kBlock + threadIdx.x;
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
                vec_sums[kBwdTileVec + lv] = vo;
            }
        }
    }
}

template <typename IO, int VEC, typename M, int RED, bool FULL, int ROUNDS>
__device__ __forceinline__ void bwd_tile(const QdqArgs& a, const Tile& t, float (*sp)[kStage], double& acc_s, double& acc_o,
                                         double* stage_sums, float* vec_sums) {
    const IO* __restrict__ x = static_cast<const IO*>(a.x) + t.v0 * VEC;
    const IO* __restrict__ g = static_cast<const IO*>(a.g) + t.v0 * VEC;
    IO* __restrict__ gxp = a.gx ? static_cast<IO*>(a.gx) + t.v0 * VEC : nullptr;
    Pack<IO, VEC> xin[kBwdUnroll], gin[kBwdUnroll];
    const EncRaw pre = preload_encoding(a, t);  // ahead of the elements: see preload_encoding
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
        const int base = r * kBlock * kBwdUnroll;
        if (!FULL && r > 0 && base >= t.nv) break;
#pragma unroll
        for (int u = 0; u < kBwdUnroll; ++u) {
            const int lv = base + u * kBlock + threadIdx.x;
            if (FULL || lv < t.nv) {
                xin[u] = load_pack_hinted<IO, VEC>(x + (int64_t)lv * VEC, a.stream_loads != 0);
                gin[u] = load_pack_hinted<IO, VEC>(g + (int64_t)lv * VEC, a.stream_loads != 0);
            }
        }
        if (r == 0) {
            // the encodings are staged while the first loads are in flight
            stage_encodings<M>(a, t, sp, pre);
            if (RED == kRedAtomic)
                for (int i = threadIdx.x; i < 2 * t.nstage; i += kBlock) stage_sums[i] = 0.0;
            __syncthreads();
        }
        if (!M::kDiv || __builtin_amdgcn_ballot_w64(!lane_can_divide_fast<IO, VEC, M, FULL, kBwdUnroll>(a, t, sp, xin, base)) == 0)
            bwd_math<IO, VEC, M, RED, FULL, true>(a, t, sp, xin, gin, gxp, acc_s, acc_o, stage_sums, vec_sums, base);
        else
            bwd_math<IO, VEC, M, RED, FULL, false>(a, t, sp, xin, gin, gxp, acc_s, acc_o, stage_sums, vec_sums, base);
    }
}

template <typename IO, int VEC, typename M, int RED, int ROUNDS>
__global__ __launch_bounds__(kBlock) void qdq_bwd_kernel(const QdqArgs a) {
    __shared__ float sp[M::kNP + (M::kDiv ? 1 : 0)][kStage];
    __shared__ double red_smem[2][kBlock / kWave];
    __shared__ double stage_sums[RED == kRedAtomic ? 2 * kStage : 1];  // kRedAtomic: (scale, offset) sums per run
    __shared__ float vec_sums[RED == kRedRuns ? 2 * kBwdTileVec : 1];     // kRedRuns: (scale, offset) terms per vector
    const Tile t = make_tile(a, blockIdx.x);
    double acc_s = 0.0, acc_o = 0.0;  // kRedTile: per-thread totals
    if (t.nv == kBlock * kBwdUnroll * ROUNDS) bwd_tile<IO, VEC, M, RED, true, ROUNDS>(a, t, sp, acc_s, acc_o, stage_sums, vec_sums);
    else bwd_tile<IO, VEC, M, RED, false, ROUNDS>(a, t, sp, acc_s, acc_o, stage_sums, vec_sums);
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
                    o += (double)vec_sums[kBwdTileVec + run * kv + k];
                }
                emit(run, s, o);
            }
        } else {
            const int lane = threadIdx.x & (kWave - 1);
            for (int run = threadIdx.x / kWave; run < t.nstage; run += kBlock / kWave) {
                double s = 0.0, o = 0.0;
                for (int k = lane; k < kv; k += kWave) {
                    s += (double)vec_sums[run * kv + k];
                    o += (double)vec_sums[kBwdTileVec + run * kv + k];
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
        // both sums through one barrier (the waves' results are added in wave order by thread 0, which alone needs
        // them; red_smem is not used before this point)
        const double ws = wave_reduce(acc_s, OpAddD());
        const double wo = wave_reduce(acc_o, OpAddD());
        if ((threadIdx.x & (kWave - 1)) == 0) {
            red_smem[0][threadIdx.x / kWave] = ws;
            red_smem[1][threadIdx.x / kWave] = wo;
        }
        __syncthreads();
        double bs = 0.0, bo = 0.0;
        if (threadIdx.x == 0) {
            bs = red_smem[0][0];
            bo = red_smem[1][0];
#pragma unroll
            for (int w = 1; w < kBlock / kWave; ++w) {
                bs += red_smem[0][w];
                bo += red_smem[1][w];
            }
        }
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
constexpr int kFinishLoads = 16;
__global__ __launch_bounds__(kFinishThreads) void qdq_bwd_finish_kernel(const QdqArgs a) {
    __shared__ double red_smem[2][kFinishThreads / kWave];
    const int64_t per_enc = a.mode == kRows ? a.I * (int64_t)a.tpr : (int64_t)a.nblocks;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    if (a.mode != kRows) {
        // single encoding: every thread issues the loads of up to kFinishLoads pairs before it adds the first (the
        // launch is a chain of memory latencies and little else), front to back, then one tree
        double s = 0.0, o = 0.0;
        const double2* __restrict__ pairs = reinterpret_cast<const double2*>(a.partials);
        for (int64_t q0 = threadIdx.x; q0 < per_enc; q0 += (int64_t)kFinishThreads * kFinishLoads) {
            double2 v[kFinishLoads];
#pragma unroll
            for (int u = 0; u < kFinishLoads; ++u) {
                const int64_t q = q0 + (int64_t)u * kFinishThreads;
                v[u] = q < per_enc ? pairs[q] : double2{0.0, 0.0};
            }
#pragma unroll
            for (int u = 0; u < kFinishLoads; ++u) {
                s += v[u].x;
                o += v[u].y;
            }
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

// The same sums for many encodings (at least half a wave of them): a lane per encoding, so that a wave reads 64
// neighbouring pairs, one kilobyte, per load (a wave per encoding reads 64 pairs that lie `stride` apart: a cache line
// fetched for every 16 bytes used).  The waves of a workgroup take contiguous shares of the `count` rows, a few loads
// in flight each, and wave 0 adds the shares up in wave order.
constexpr int kRowsFinishWaves = 16;
constexpr int kRowsFinishLoads = 4;
__global__ __launch_bounds__(kRowsFinishWaves * kWave) void qdq_bwd_rows_finish_kernel(const double* __restrict__ partials,
                                                                                       int64_t count, int64_t num_enc,
                                                                                       float* gscale, float* goffset, int cd) {
    __shared__ double shares[kRowsFinishWaves][2][kWave];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int64_t e = (int64_t)blockIdx.x * kWave + lane;
    // stacked problems (the grid's y axis): each has its own `count` rows of partials and its own num_enc results
    partials += 2 * (int64_t)blockIdx.y * count * num_enc;
    gscale += (int64_t)blockIdx.y * num_enc;
    goffset += (int64_t)blockIdx.y * num_enc;
    const int64_t share = (count + kRowsFinishWaves - 1) / kRowsFinishWaves;
    const int64_t q0 = wave * share, q1 = q0 + share < count ? q0 + share : count;
    double s = 0.0, o = 0.0;
    if (e < num_enc) {
        const double2* __restrict__ pairs = reinterpret_cast<const double2*>(partials) + e;
        for (int64_t q = q0; q < q1; q += kRowsFinishLoads) {
            double2 v[kRowsFinishLoads];
#pragma unroll
            for (int u = 0; u < kRowsFinishLoads; ++u) v[u] = q + u < q1 ? pairs[(q + u) * num_enc] : double2{0.0, 0.0};
#pragma unroll
            for (int u = 0; u < kRowsFinishLoads; ++u) {
                s += v[u].x;
                o += v[u].y;
            }
        }
    }
    shares[wave][0][lane] = s;
    shares[wave][1][lane] = o;
    __syncthreads();
    if (wave == 0 && e < num_enc) {
        s = o = 0.0;
#pragma unroll
        for (int w = 0; w < kRowsFinishWaves; ++w) {
            s += shares[w][0][lane];
            o += shares[w][1][lane];
        }
        gscale[e] = finish_sum_rt(s, cd);
        goffset[e] = finish_sum_rt(o, cd);
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

// Backward for run length 1 (see qdq_fwd_cols_kernel).  A lane keeps the sums of its VEC encodings over the rows it
// walks: in single precision in registers for kColFlushSteps steps (kColFlushSteps * kColUnroll terms per encoding,
// about what the tiled kernel adds in single precision per vector), then added to double-precision sums that live in
// LDS, a table per wave (sixteen double accumulators per lane in registers leave the 16-bit kernels two waves per
// SIMD).  At the end the first waves add the tables up in wave order and the workgroup's sums go to its own row of the
// partials ([row group][encoding]), which qdq_bwd_rows_finish_kernel adds up in order.
constexpr int kColFlushSteps = 4;

// One step of a wave: kColUnroll rows of VEC elements per lane.  Like the tiled kernel, the division-free form looks
// at a whole row of the wave before it spends work on out-of-range terms: when every element is inside the grid the
// input gradient is the output gradient as loaded and the offset gradient gets no term.  r0 is the same for all lanes
// of a wave, so the row test is wave-uniform.  Returns whether vo received terms (wave-uniform).
template <typename IO, int VEC, typename M, bool FAST>
__device__ __forceinline__ bool bwd_cols_rows(const QdqArgs& a, const Pack<IO, VEC>* xin, const Pack<IO, VEC>* gin,
                                              const EncP* e, IO* __restrict__ gxp, int64_t r0, int64_t c0, float* vs,
                                              float* vo) {
    bool offset_terms = false;
#pragma unroll
    for (int u = 0; u < kColUnroll; ++u) {
        if (r0 + u >= a.I) continue;
        IO* const out_row = gxp ? gxp + (r0 + u) * a.J + c0 : nullptr;
        if constexpr (FAST && M::kSplitBwd) {
            float tq[VEC], xr[VEC], m[VEC];
            bool all_in = true;
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                M::bwd_pre(load_f32(xin[u].v[k]), e[k], e[k].p1 + a.gc.qmin, e[k].p1 + a.gc.qmax, tq[k], xr[k], m[k]);
                all_in &= (m[k] == xr[k]);
            }
            if (__builtin_amdgcn_ballot_w64(!all_in) == 0) {
#pragma unroll
                for (int k = 0; k < VEC; ++k) vs[k] += M::bwd_gs_in(load_f32(gin[u].v[k]), tq[k], xr[k]);
                if (out_row) store_pack_stream<IO, VEC>(out_row, gin[u]);
            } else {
                offset_terms = true;
                Pack<IO, VEC> out;
#pragma unroll
                for (int k = 0; k < VEC; ++k) {
                    const float gr = load_f32(gin[u].v[k]);
                    const bool in = (m[k] == xr[k]);
                    out.v[k] = store_cast<IO>(in ? gr : 0.f);
                    vs[k] += in ? M::bwd_gs_in(gr, tq[k], xr[k]) : M::bwd_gs_out(gr, m[k]);
                    vo[k] += in ? 0.f : M::bwd_goff_out(gr, e[k]);
                }
                if (out_row) store_pack_stream<IO, VEC>(out_row, out);
            }
        } else {
            offset_terms = true;
            Pack<IO, VEC> out;
#pragma unroll
            for (int k = 0; k < VEC; ++k) {
                float gx, gs, go;
                M::template bwd<FAST>(load_f32(gin[u].v[k]), load_f32(xin[u].v[k]), e[k], a.gc, gx, gs, go);
                out.v[k] = store_cast<IO>(gx);
                vs[k] += gs;
                vo[k] += go;
            }
            if (out_row) store_pack_stream<IO, VEC>(out_row, out);
        }
    }
    return offset_terms;
}

// adds a lane's single-precision sums to its double-precision ones in the wave's table and clears them
template <int VEC>
__device__ __forceinline__ void flush_col_sums(double (*table)[kWave], int lane, float* vs, float* vo, bool offset_terms) {
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
        table[2 * k][lane] += (double)vs[k];
        vs[k] = 0.f;
    }
    if (offset_terms) {
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
            table[2 * k + 1][lane] += (double)vo[k];
            vo[k] = 0.f;
        }
    }
}

template <typename IO, int VEC, typename M, int WAVES>
__global__ __launch_bounds__(WAVES * kWave) void qdq_bwd_cols_kernel(const QdqArgs a) {
    __shared__ double sums[WAVES][2 * VEC][kWave];  // [wave][2 * k: scale sum, 2 * k + 1: offset sum][lane]
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int64_t c0 = ((int64_t)blockIdx.x * kWave + lane) * VEC;
    const bool live = c0 < a.J;
    const bool want_pg = a.partials != nullptr;
    if (want_pg) {  // a wave clears its own table: nobody else touches it before the barrier below
#pragma unroll
        for (int i = 0; i < 2 * VEC; ++i) sums[wave][i][lane] = 0.0;
    }
    if (live) {
        const int64_t zoff = (int64_t)blockIdx.z * a.I * a.J;  // stacked columns: problem z has its own I x J elements
        const IO* __restrict__ x = static_cast<const IO*>(a.x) + zoff;
        const IO* __restrict__ g = static_cast<const IO*>(a.g) + zoff;
        IO* __restrict__ gxp = a.gx ? static_cast<IO*>(a.gx) + zoff : nullptr;
        EncP e[VEC];
        bool enc_fast = true;
        load_col_encodings<M, VEC>(a, (int64_t)blockIdx.z * a.J + c0, e);
#pragma unroll
        for (int k = 0; k < VEC; ++k) enc_fast &= !M::kDiv || e[k].rs != 0.f;
        float vs[VEC], vo[VEC];
#pragma unroll
        for (int k = 0; k < VEC; ++k) vs[k] = vo[k] = 0.f;
        bool offset_terms = false;
        int pending = 0;
        const int64_t step = (int64_t)gridDim.y * WAVES * kColUnroll;
        for (int64_t r0 = ((int64_t)blockIdx.y * WAVES + wave) * kColUnroll; r0 < a.I; r0 += step) {
            Pack<IO, VEC> xin[kColUnroll], gin[kColUnroll];
            bool ok = enc_fast;
#pragma unroll
            for (int u = 0; u < kColUnroll; ++u)
                if (r0 + u < a.I) {
                    xin[u] = load_pack_hinted<IO, VEC>(x + (r0 + u) * a.J + c0, a.stream_loads != 0);
                    gin[u] = load_pack_hinted<IO, VEC>(g + (r0 + u) * a.J + c0, a.stream_loads != 0);
                }
#pragma unroll
            for (int u = 0; u < kColUnroll; ++u)
                if (M::kDiv && r0 + u < a.I) ok &= row_can_divide_fast<IO, VEC>(xin[u]);
            // one wave-uniform branch per step, each side a straight run of arithmetic over all its elements
            if (!M::kDiv || __builtin_amdgcn_ballot_w64(!ok) == 0)
                offset_terms |= bwd_cols_rows<IO, VEC, M, true>(a, xin, gin, e, gxp, r0, c0, vs, vo);
            else
                offset_terms |= bwd_cols_rows<IO, VEC, M, false>(a, xin, gin, e, gxp, r0, c0, vs, vo);
            if (want_pg && ++pending == kColFlushSteps) {
                flush_col_sums<VEC>(sums[wave], lane, vs, vo, offset_terms);
                pending = 0;
                offset_terms = false;
            }
        }
        if (want_pg && pending) flush_col_sums<VEC>(sums[wave], lane, vs, vo, offset_terms);
    }
    if (!want_pg) return;
    __syncthreads();
    // the tables are added up in wave order, whichever wave finished first; the 2 * VEC sums of a lane are shared out
    // over the waves, and a lane's pair of sums for one encoding is one 16-byte store
    double* row = a.partials + 2 * ((int64_t)blockIdx.z * gridDim.y + blockIdx.y) * a.J;
    for (int k = wave; k < VEC; k += WAVES) {
        if (!live) break;
        double ps = 0.0, po = 0.0;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            ps += sums[w][2 * k][lane];
            po += sums[w][2 * k + 1][lane];
        }
        if (gridDim.y == 1) {  // a single row group: these are the sums themselves, no finish launch follows
            const int64_t enc = (int64_t)blockIdx.z * a.J + c0 + k;
            a.gscale[enc] = finish_sum_rt(ps, a.out_cd);
            a.goffset[enc] = finish_sum_rt(po, a.out_cd);
        } else {
            store_pack<double, 2>(row + 2 * (c0 + k), Pack<double, 2>{{ps, po}});
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


// Elements per lane of the column-walking backward kernel, 0 where it does not apply.  It takes run length 1 whatever
// reduction the plan would otherwise use for it.  On a 16-bit tensor a lane takes four encodings (8-byte vectors), not
// eight: with eight, the encodings, the two rows of two tensors and the temporaries of the split form need about 170
// registers, two or three waves per SIMD (8192 x 4096 bf16 with learned encodings: 47.6 us against 42 us, same tensors
// every launch).
static int bwd_cols_lane_elems(int io_dtype, const Plan& p, bool aligned) {
    if (!(p.red == kRedAtomic || p.red == kRedRuns || p.red == kRedNone)) return 0;
    const int n = cols_lane_elems(io_dtype, p, aligned);
    return n > 4 ? 4 : n;
}

// Workgroups of eight waves, about as many as the chip holds at once, for the reason given at the forward launch
// (bf16: 42.0 us with 1024 workgroups, 45.0 us with 2048; float32: 72.8 us with 256, 74.9 us with 512, 75.9 us with 1024).
constexpr int kBwdColWaves = 8;
static dim3 bwd_cols_grid(int io_dtype, const Plan& p, int lane_elems) {
    const int64_t target = io_dtype == AHQ_F32 ? 256 : 1024;
    return lane_elems == 4 ? cols_grid<4>(p, target, kBwdColWaves) : cols_grid<1>(p, target, kBwdColWaves);
}

// pairs of doubles the backward pass needs as scratch for its parameter gradients
static size_t bwd_scratch_pairs(int io_dtype, const Plan& p, bool aligned, bool want_pg) {
    if (!want_pg) return 0;
    const int lane_elems = bwd_cols_lane_elems(io_dtype, p, aligned);
    if (lane_elems > 0) return (size_t)p.cl.A * (size_t)bwd_cols_grid(io_dtype, p, lane_elems).y * (size_t)p.cl.J;
    return p.ws_elems;
}

template <typename IO, typename M, int RED>
static void launch_bwd_red(const Plan& p, const QdqArgs& a, hipStream_t st) {
    if constexpr (RED == kRedTile) {
        if (p.tile_vec == kBwdTileVec) {  // a whole row per tile, in kBwdRounds rounds (plan_bwd)
            if (p.vec == 1) hipLaunchKernelGGL((qdq_bwd_kernel<IO, 1, M, RED, kBwdRounds>), dim3(p.nblocks), dim3(kBlock), 0, st, a);
            else hipLaunchKernelGGL((qdq_bwd_kernel<IO, IoTraits<IO>::kVec, M, RED, kBwdRounds>), dim3(p.nblocks), dim3(kBlock), 0, st, a);
            return;
        }
    }
    if (p.vec == 1) {
        hipLaunchKernelGGL((qdq_bwd_kernel<IO, 1, M, RED, 1>), dim3(p.nblocks), dim3(kBlock), 0, st, a);
    } else {
        hipLaunchKernelGGL((qdq_bwd_kernel<IO, IoTraits<IO>::kVec, M, RED, 1>), dim3(p.nblocks), dim3(kBlock), 0, st, a);
    }
}

template <typename IO, typename M>
static void launch_bwd(const Plan& p, const QdqArgs& a, hipStream_t st, bool aligned) {
    const int lane_elems = bwd_cols_lane_elems(IoTraits<IO>::kDtype, p, aligned);
    if (lane_elems > 0) {
        constexpr int W = kBwdColWaves;
        dim3 g = bwd_cols_grid(IoTraits<IO>::kDtype, p, lane_elems);
        // arithmetic without a division and no sums to keep: few registers, eight waves per SIMD, so the chip holds
        // more workgroups at once (8192 x 4096 fp32: 70.3 us against 81.8 us)
        const int64_t light = IoTraits<IO>::kVec > 4 ? 2048 : 1024;
        if (lane_elems == 4) {
            if (!M::kDiv && !a.partials) g = cols_grid<4>(p, light, W);
            hipLaunchKernelGGL((qdq_bwd_cols_kernel<IO, 4, M, W>), g, dim3(W * kWave), 0, st, a);
        } else {
            if (!M::kDiv && !a.partials) g = cols_grid<1>(p, light, W);
            hipLaunchKernelGGL((qdq_bwd_cols_kernel<IO, 1, M, W>), g, dim3(W * kWave), 0, st, a);
        }
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

// The input gradient alone (no sums): the kernels of launch_bwd that need no reduction.
template <typename IO, typename M>
static void launch_bwd_input_only(const Plan& p, const QdqArgs& a, hipStream_t st, bool aligned) {
    const int lane_elems = bwd_cols_lane_elems(IoTraits<IO>::kDtype, p, aligned);
    if (lane_elems > 0) {
        constexpr int W = kBwdColWaves;
        const dim3 g = bwd_cols_grid(IoTraits<IO>::kDtype, p, lane_elems);
        if (lane_elems == 4) hipLaunchKernelGGL((qdq_bwd_cols_kernel<IO, 4, M, W>), g, dim3(W * kWave), 0, st, a);
        else hipLaunchKernelGGL((qdq_bwd_cols_kernel<IO, 1, M, W>), g, dim3(W * kWave), 0, st, a);
        return;
    }
    if (p.cl.kind == kGeneric) {
        hipLaunchKernelGGL((qdq_bwd_generic_kernel<IO, M>), dim3(p.nblocks), dim3(kBlock), 0, st, a);
        return;
    }
    launch_bwd_red<IO, M, kRedNone>(p, a, st);
}

}  // namespace ahq

using namespace ahq;

extern "C" int ahq_float_qdq_backward(int32_t dtype, const ahq_layout* layout, const void* g, const void* x, void* gx,
                                      const float* scale, int32_t mantissa_bits, int32_t exponent_min, float max_value,
                                      int32_t overflow_to_nan, int32_t unsigned_zero, void* stream) {
    if (dtype < AHQ_F32 || dtype > AHQ_BF16) return set_error("bad dtype"), AHQ_ERR_INVALID;
    if (!layout) return set_error("layout is null"), AHQ_ERR_INVALID;
    if (!scale) return set_error("scale is null"), AHQ_ERR_INVALID;
    if (mantissa_bits < 0 || mantissa_bits > 23 || exponent_min < -126 || exponent_min > 127 || !(max_value > 0.f))
        return set_error("bad float format description"), AHQ_ERR_INVALID;
    Plan p;
    const bool al = aligned16(x) && aligned16(g) && aligned16(gx);
    if (!make_plan(dtype, *layout, al, false, &p, kBwdUnroll, true)) return AHQ_ERR_INVALID;
    if (p.cl.numel == 0) return AHQ_OK;
    if (!x || !g || !gx) return set_error("x, g or gx is null"), AHQ_ERR_INVALID;
    QdqArgs a{};
    a.x = x;
    a.g = g;
    a.gx = gx;
    a.scale = scale;
    ahq_grid grid{};
    grid.io_dtype = dtype;
    grid.compute_dtype = dtype;
    fill_args(grid, p, &a);
    a.gc.qmin = (float)exponent_min;
    a.gc.qmax = max_value;
    a.gc.zps = (float)mantissa_bits;
    a.gc.flags = (overflow_to_nan ? kCastOverflowNaN : 0) | (unsigned_zero ? kCastUnsignedZero : 0);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == AHQ_F32) launch_bwd_input_only<float, MathFloatCast<AHQ_F32>>(p, a, st, al);
    else if (dtype == AHQ_F16) launch_bwd_input_only<f16_t, MathFloatCast<AHQ_F16>>(p, a, st, al);
    else launch_bwd_input_only<bf16_t, MathFloatCast<AHQ_BF16>>(p, a, st, al);
    return check_launch("ahq_float_qdq_backward");
}

// The tiling of the backward pass: tiles of one round, of kBwdRounds rounds where a row then is one tile instead of two.
static bool plan_bwd(int io_dtype, const ahq_layout& layout, bool aligned, bool want_pg, Plan* p) {
    if (!make_plan(io_dtype, layout, aligned, want_pg, p, kBwdUnroll, true)) return false;
    if (p->red == kRedTile && p->mode == kRows && p->tpr > 1 && p->tpr <= kBwdRounds) {
        Plan q;
        if (make_plan(io_dtype, layout, aligned, want_pg, &q, kBwdTileUnroll, true) && q.red == kRedTile &&
            q.mode == kRows && q.tpr == 1)
            *p = q;
    }
    return true;
}

extern "C" size_t ahq_qdq_backward_workspace_bytes(const ahq_grid* grid, const ahq_layout* layout, int want_param_grads) {
    if (!grid || !layout) return 0;
    const bool pg = want_param_grads != 0;
    Plan p;
    if (!plan_bwd(grid->io_dtype, *layout, true, pg, &p)) return 0;
    size_t a = bwd_scratch_pairs(grid->io_dtype, p, true, pg) * 2 * sizeof(double);
    // an unaligned tensor falls back to the scalar path whose strategy may need a different amount
    Plan q;
    if (plan_bwd(grid->io_dtype, *layout, false, pg, &q)) {
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
    if (!plan_bwd(grid->io_dtype, *layout, al, want_pg, &p)) return AHQ_ERR_INVALID;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (p.cl.numel == 0) return AHQ_OK;  // nothing to read: outputs are left untouched
    if (!x || !g) return set_error("x or g is null"), AHQ_ERR_INVALID;
    if (!gx && !want_pg) return AHQ_OK;
    const int col_lane_elems = bwd_cols_lane_elems(grid->io_dtype, p, al);
    const bool cols = col_lane_elems > 0;
    const size_t ws_need = bwd_scratch_pairs(grid->io_dtype, p, al, want_pg) * 2 * sizeof(double);
    if (ws_need > 0 && (!workspace || workspace_bytes < ws_need)) return set_error("workspace too small"), AHQ_ERR_WORKSPACE;
    if (ws_need > 0 && !aligned16(workspace)) return set_error("workspace must be 16-byte aligned"), AHQ_ERR_INVALID;
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
    const int64_t col_groups = cols ? (int64_t)bwd_cols_grid(grid->io_dtype, p, col_lane_elems).y : 0;
    if (want_pg && ((cols && col_groups > 1) || (!cols && p.red == kRedRuns && p.cl.I > 1))) {
        // one slot per (row group, encoding) or per run: added up per encoding in a fixed order (the column kernel
        // with a single row group has stored the sums itself)
        const int64_t count = cols ? col_groups : p.cl.I;
        if (p.cl.J >= kWave / 2 && (p.cl.J + kWave - 1) / kWave <= 0x7fffffff) {
            hipLaunchKernelGGL(qdq_bwd_rows_finish_kernel, dim3((unsigned)((p.cl.J + kWave - 1) / kWave), cols ? (unsigned)p.cl.A : 1u),
                               dim3(kRowsFinishWaves * kWave), 0, st, (const double*)a.partials, count, p.cl.J, gscale, goffset,
                               (int)grid->compute_dtype);
        } else {
            const int64_t nb = (p.cl.J + kBlock / kWave - 1) / (kBlock / kWave);
            hipLaunchKernelGGL(qdq_bwd_strided_finish_kernel, dim3((unsigned)(nb > 4096 ? 4096 : nb)), dim3(kBlock), 0, st,
                               (const double*)a.partials, count, p.cl.J, p.cl.J, gscale, goffset, (int)grid->compute_dtype);
        }
    }
    return check_launch("ahq_qdq_backward");
}
