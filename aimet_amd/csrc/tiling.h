// How a flat tensor is cut into workgroup tiles and how a tile finds the encodings it touches.
// Shared by the fake-quantization kernels and the statistics kernels.
#pragma once

#include "ahq_device.h"
#include "ahq_host.h"
#include "layout.h"

namespace ahq {

// kFlat: tiles of tile_vec vectors over the flat tensor; kRows: tiles never leave a run (runs of at least half a tile);
// kRuns: a tile is a whole number of neighbouring runs (runs shorter than half a tile)
enum TileMode : int { kFlat = 0, kRows = 1, kRuns = 2 };
// How per-encoding reductions leave the kernel:
//   kRedTile    every tile lies inside one run; workgroup totals go straight to the output when one tile covers the
//               whole encoding, else to a partials array that a second small launch adds in a fixed order
//   kRedSeg     a run is a power-of-two number (<= 64) of neighbouring lanes: shuffle reduction, direct store
//   kRedAtomic  anything else: atomics into a per-encoding scratch array, finished by a second tiny kernel
//   kRedRuns    (only on request, for sums whose order must not vary) tiles of whole runs: every run is summed inside
//               its tile in a fixed order and stored -- straight to the output when each encoding has one run, else to
//               one slot per run that a second launch adds up per encoding in a fixed order
enum RedMode : int { kRedNone = 0, kRedTile = 1, kRedSeg = 2, kRedAtomic = 3, kRedRuns = 4 };

// Geometry every tiled kernel receives (flat index = (i*J + j)*K + k, encoding index = j).
struct Geom {
    int64_t numel;
    int64_t nvec;  // numel / VEC
    int64_t I, J, K;
    int64_t Kv;    // vectors per run of one encoding (K / VEC); 2^62 when J == 1
    int32_t kv_shift;  // log2(Kv) when Kv is a power of two below 2^31, else -1
    int32_t tile_vec;  // vectors per tile: kBlock x (vectors per thread, at most kUnroll)
    int32_t mode;
    int32_t tpr;   // tiles per row (kRows); runs per tile (kRuns)
    uint32_t nblocks;
    int64_t ntiles;  // tiles in total (== nblocks: one tile per workgroup)
    // generic layout (per-element coordinate walk)
    int32_t nseg;
    int64_t seg_extent[2 * AHQ_MAX_DIMS];
    int64_t seg_flat_stride[2 * AHQ_MAX_DIMS];
    int64_t seg_enc_stride[2 * AHQ_MAX_DIMS];
};

struct Tile {
    int64_t v0;    // first vector of the tile
    int nv;        // vectors in the tile
    int64_t rem0;  // position of v0 inside its run, in vectors
    int64_t e0;    // encoding index of the first run
    int nstage;    // runs touched
};

__device__ __forceinline__ Tile make_tile(const Geom& a, int64_t tile) {
    Tile t;
    if (a.mode == kRows) {
        const int64_t row = a.tpr == 1 ? tile : tile / a.tpr;  // (a 64-bit division costs a workgroup a few hundred instructions)
        const int64_t tt = tile - row * a.tpr;
        t.v0 = row * a.Kv + tt * a.tile_vec;
        const int64_t left = a.Kv - tt * a.tile_vec;
        t.nv = (int)(left < a.tile_vec ? left : a.tile_vec);
        t.rem0 = tt * a.tile_vec;
        t.e0 = a.I == 1 ? row : row % a.J;
        t.nstage = 1;
    } else if (a.mode == kRuns) {
        const int64_t run0 = tile * a.tpr;
        const int64_t left = a.I * a.J - run0;
        const int n = (int)(left < a.tpr ? left : a.tpr);
        t.v0 = run0 * a.Kv;
        t.nv = n > 0 ? n * (int)a.Kv : 0;
        t.rem0 = 0;
        t.e0 = a.I == 1 ? run0 : run0 % a.J;
        t.nstage = n > 0 ? n : 0;
    } else {
        t.v0 = tile * a.tile_vec;
        const int64_t left = a.nvec - t.v0;
        t.nv = (int)(left < a.tile_vec ? left : a.tile_vec);
        if (t.nv < 0) t.nv = 0;
        if (a.J == 1) {
            t.rem0 = 0;
            t.e0 = 0;
            t.nstage = 1;
        } else {
            // (the usual block sizes are powers of two: shifts instead of 64-bit divisions, which cost a workgroup a
            // few hundred instructions each)
            const int64_t row0 = a.kv_shift >= 0 ? t.v0 >> a.kv_shift : t.v0 / a.Kv;
            t.rem0 = t.v0 - row0 * a.Kv;
            t.e0 = a.I == 1 ? row0 : row0 % a.J;
            const int64_t last = t.rem0 + t.nv - 1;
            t.nstage = t.nv > 0 ? (int)(a.kv_shift >= 0 ? last >> a.kv_shift : last / a.Kv) + 1 : 0;
        }
    }
    return t;
}

// index of local vector lv's run among the runs the tile touches
__device__ __forceinline__ int stage_index(const Geom& a, const Tile& t, int lv) {
    if (t.nstage == 1) return 0;
    const int64_t p = t.rem0 + lv;
    if (a.Kv >= a.tile_vec) return p >= a.Kv ? 1 : 0;
    if (a.kv_shift >= 0) return (int)((uint32_t)p >> a.kv_shift);  // the usual block sizes: no per-lane division
    return (int)((uint32_t)p / (uint32_t)a.Kv);
}

__device__ __forceinline__ int64_t generic_enc_index(const Geom& a, int64_t idx) {
    int64_t e = 0;
    for (int s = 0; s < a.nseg; ++s) {
        const int64_t c = (idx / a.seg_flat_stride[s]) % a.seg_extent[s];
        e += c * a.seg_enc_stride[s];
    }
    return e;
}

// ------------------------------------------------------------------------------------------------------ host side --
struct Plan {
    CanonLayout cl;
    int vec;       // element vector width used (16 bytes worth, or 1)
    int mode;
    int tpr;       // kRows: tiles per row; kRuns: runs per tile
    int red;
    uint32_t nblocks;
    int64_t Kv, nvec;
    int tile_vec;  // vectors per tile
    int64_t ntiles;
    size_t ws_elems;  // kRedTile: number of tiles; kRedAtomic: number of encodings; kRedRuns: runs if I > 1; else 0
    bool ptr_aligned; // what the caller said of its pointers: all 16-byte aligned
};

inline int io_vec(int dtype) { return dtype == AHQ_F32 ? 4 : 8; }
inline size_t io_size(int dtype) { return dtype == AHQ_F32 ? 4 : 2; }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool is_pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }

// Decide tiling and reduction strategy.  `ptr_aligned`: every tensor pointer is 16-byte aligned; `unroll`: vectors per
// thread and tile the kernel family works with (its register arrays hold that many).  `ordered`: the reduction is a
// floating-point sum whose result must not depend on the order workgroups finish in: short runs get kRedRuns instead
// of kRedAtomic, unless that needs more scratch (one slot per run) than the tensor itself occupies.
inline bool make_plan(int io_dtype, const ahq_layout& layout, bool ptr_aligned, bool want_red, Plan* p,
                      int unroll = kUnroll, bool ordered = false) {
    const int tile_vec = kBlock * unroll;
    p->tile_vec = tile_vec;
    p->ptr_aligned = ptr_aligned;
    const char* err = nullptr;
    if (!canonicalize(layout, &p->cl, &err)) {
        set_error(err);
        return false;
    }
    const CanonLayout& c = p->cl;
    p->mode = kFlat;
    p->tpr = 0;
    p->red = kRedNone;
    p->ws_elems = 0;
    if (c.kind == kGeneric) {
        p->vec = 1;
        p->Kv = 1;
        p->nvec = c.numel;
        int64_t nb = (c.numel + kBlock - 1) / kBlock;
        if (nb > 65536) nb = 65536;
        p->nblocks = (uint32_t)(nb < 1 ? 1 : nb);
        p->ntiles = p->nblocks;
        if (want_red) {
            p->red = kRedAtomic;
            p->ws_elems = (size_t)c.num_enc;
        }
        return true;
    }
    const int V = io_vec(io_dtype);
    const bool shared = ptr_aligned && (c.J == 1 || c.K % V == 0);
    p->vec = shared ? V : 1;
    p->nvec = c.numel / p->vec;
    p->Kv = c.J == 1 ? ((int64_t)1 << 62) : c.K / p->vec;
    int64_t nb = (p->nvec + tile_vec - 1) / tile_vec;
    if (want_red) {
        if (c.J == 1) {
            p->red = kRedTile;
        } else if (c.I == 1 && is_pow2(p->Kv) && p->Kv <= kWave) {
            p->red = kRedSeg;
        } else if (p->Kv > tile_vec / 2 || (p->Kv == tile_vec / 2 && !(ordered && c.I == 1))) {
            // (runs of exactly half a tile go two to a tile when the sum is ordered anyway: full tiles, no finish)
            p->red = kRedTile;
            p->mode = kRows;
            p->tpr = (int)((p->Kv + tile_vec - 1) / tile_vec);
            nb = c.I * c.J * (int64_t)p->tpr;
        } else if (ordered && (c.I == 1 || c.K * (int64_t)io_size(io_dtype) >= 16)) {
            p->red = kRedRuns;
            p->mode = kRuns;
            p->tpr = (int)(tile_vec / p->Kv);
            nb = (c.I * c.J + p->tpr - 1) / p->tpr;
            p->ws_elems = c.I > 1 ? (size_t)(c.I * c.J) : 0;
        } else {
            p->red = kRedAtomic;
        }
        if (p->red == kRedTile) p->ws_elems = (size_t)(nb < 1 ? 1 : nb);
        if (p->red == kRedAtomic) p->ws_elems = (size_t)c.num_enc;
    }
    if (nb < 1) nb = 1;
    if (nb > 0x7fffffff) {
        set_error("tensor too large for one launch");
        return false;
    }
    p->ntiles = nb;
    p->nblocks = (uint32_t)nb;
    return true;
}

// Elements a lane of the column-walking kernels owns per row of this layout: a 16-byte vector where the rows allow
// it, one element where they do not (row length no multiple of the vector, tensors off 16-byte alignment), 0 where
// those kernels do not apply (run length above 1, a single row, fewer than half a wave of columns: there the tiled
// kernel's full waves win).  Stacked columns (A > 1) are A such problems side by side, the grid's z axis.
inline int cols_lane_elems(int io_dtype, const Plan& p, bool aligned) {
    const CanonLayout& c = p.cl;
    const bool form = c.kind == kIJK || (c.kind == kGeneric && c.A > 1 && c.A <= 65535);
    if (!form || c.K != 1 || c.I <= 1) return 0;
    const int V = io_vec(io_dtype);
    if (aligned && c.J % V == 0 && c.J / V >= kWave / 2 && (c.J / V + kWave - 1) / kWave <= 0x7fffffff) return V;
    return (c.J >= kWave / 2 && (c.J + kWave - 1) / kWave <= 0x7fffffff) ? 1 : 0;
}

inline void fill_geom(const Plan& p, Geom* g) {
    const CanonLayout& c = p.cl;
    g->numel = c.numel;
    g->nvec = p.nvec;
    g->I = c.I;
    g->J = c.J;
    g->K = c.K;
    g->Kv = p.Kv;
    g->kv_shift = -1;
    g->tile_vec = p.tile_vec;
    if (p.Kv < ((int64_t)1 << 31) && is_pow2(p.Kv))
        for (int b = 0; b < 31; ++b)
            if (((int64_t)1 << b) == p.Kv) g->kv_shift = b;
    g->mode = p.mode;
    g->tpr = p.tpr;
    g->nblocks = p.nblocks;
    g->ntiles = p.ntiles;
    g->nseg = c.kind == kGeneric ? c.nseg : 0;
    for (int i = 0; i < g->nseg; ++i) {
        g->seg_extent[i] = c.seg_extent[i];
        g->seg_flat_stride[i] = c.seg_flat_stride[i];
        g->seg_enc_stride[i] = c.seg_enc_stride[i];
    }
}

}  // namespace ahq
