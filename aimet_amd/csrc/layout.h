// Host-side canonicalisation of an ahq_layout into the forms the kernels understand.
//
// Every layout is first rewritten as a list of (extent, encoding-stride) "segments" over the flat element index
// (a blocked dimension of size d with block b becomes two segments: (d/b, stride) and (b, 0)), size-1 segments are
// dropped and neighbouring segments that describe one linear run are merged.  What is left is classified:
//
//   IJK      flat index = (i*J + j)*K + k  and encoding index = j      (I, J, K >= 1)
//            per-tensor is J == 1; per-channel on the leading axis is I == 1; blocks along the fastest axis
//            with one row of blocks per leading coordinate collapse to I == 1, J = #blocks, K = block size
//   GENERIC  anything else (2-D blocks, several channel axes): per-element coordinate walk.  One generic form is also
//            described as STACKED COLUMNS: flat index = (a*I + i)*J + j and encoding index = a*J + j  (A > 1: blocks
//            along a leading axis with one encoding per element of the fastest axis), which the column-walking
//            kernels take as A problems of the IJK form with K == 1
#pragma once

#include <cstdint>
#include <vector>

#include "../../include/aimet_amd.h"

namespace ahq {

enum LayoutKind : int32_t { kIJK = 0, kGeneric = 1 };

struct Segment {
    int64_t extent;
    int64_t enc_stride;  // 0 = broadcast
};

struct CanonLayout {
    int32_t kind = kIJK;
    int64_t numel = 0;
    int64_t num_enc = 1;
    // IJK form
    int64_t I = 1, J = 1, K = 1;
    // stacked columns (kind == kGeneric and A > 1): I, J as above, K == 1
    int64_t A = 1;
    // generic form: segments outermost first, with the flat stride of each
    int32_t nseg = 0;
    int64_t seg_extent[2 * AHQ_MAX_DIMS];
    int64_t seg_flat_stride[2 * AHQ_MAX_DIMS];
    int64_t seg_enc_stride[2 * AHQ_MAX_DIMS];
};

// Returns false (and leaves *err pointing at a static message) if the layout is malformed.
inline bool canonicalize(const ahq_layout& in, CanonLayout* out, const char** err) {
    if (in.ndim < 0 || in.ndim > AHQ_MAX_DIMS) {
        *err = "layout.ndim out of range";
        return false;
    }
    std::vector<Segment> segs;
    int64_t numel = 1;
    for (int d = 0; d < in.ndim; ++d) {
        const int64_t dim = in.dims[d], blk = in.block[d], es = in.enc_stride[d];
        if (dim < 0) {
            *err = "negative dimension";
            return false;
        }
        if (dim == 0) {
            numel = 0;
            continue;
        }
        if (blk <= 0 || dim % blk != 0) {
            *err = "block size must be positive and divide the dimension";
            return false;
        }
        if (es < 0) {
            *err = "negative encoding stride";
            return false;
        }
        numel *= dim;
        const int64_t nblk = dim / blk;
        if (nblk > 1) segs.push_back({nblk, es});
        if (blk > 1) segs.push_back({blk, 0});
    }
    out->numel = numel;
    // An encoding stride on an extent-1 segment is irrelevant; normalise broadcast segments to stride 0 and merge.
    std::vector<Segment> merged;
    for (const Segment& s : segs) {
        if (!merged.empty()) {
            Segment& p = merged.back();
            const bool both_bcast = p.enc_stride == 0 && s.enc_stride == 0;
            const bool linear = p.enc_stride != 0 && s.enc_stride != 0 && p.enc_stride == s.enc_stride * s.extent;
            if (both_bcast || linear) {
                p.extent *= s.extent;
                p.enc_stride = s.enc_stride;
                continue;
            }
        }
        merged.push_back(s);
    }
    // number of encodings = 1 + sum (extent-1)*stride  (dense encodings assumed: this is the max index + 1)
    int64_t max_idx = 0;
    for (const Segment& s : merged) max_idx += (s.extent - 1) * s.enc_stride;
    out->num_enc = max_idx + 1;

    // classify
    auto is_b = [&](size_t i) { return merged[i].enc_stride == 0; };
    const size_t m = merged.size();
    out->kind = kIJK;
    out->I = out->J = out->K = 1;
    bool ijk = true;
    if (m == 0) {
        // scalar / single element
    } else if (m == 1) {
        if (is_b(0)) out->K = merged[0].extent;
        else if (merged[0].enc_stride == 1) out->J = merged[0].extent;
        else ijk = false;
    } else if (m == 2) {
        if (!is_b(0) && is_b(1) && merged[0].enc_stride == 1) {
            out->J = merged[0].extent;
            out->K = merged[1].extent;
        } else if (is_b(0) && !is_b(1) && merged[1].enc_stride == 1) {
            out->I = merged[0].extent;
            out->J = merged[1].extent;
        } else {
            ijk = false;
        }
    } else if (m == 3 && is_b(0) && !is_b(1) && is_b(2) && merged[1].enc_stride == 1) {
        out->I = merged[0].extent;
        out->J = merged[1].extent;
        out->K = merged[2].extent;
    } else {
        ijk = false;
    }
    if (!ijk) {
        out->kind = kGeneric;
        if (merged.size() > 2 * AHQ_MAX_DIMS) {
            *err = "too many layout segments";
            return false;
        }
        out->nseg = (int32_t)merged.size();
        int64_t stride = 1;
        for (int i = out->nseg - 1; i >= 0; --i) {
            out->seg_extent[i] = merged[i].extent;
            out->seg_enc_stride[i] = merged[i].enc_stride;
            out->seg_flat_stride[i] = stride;
            stride *= merged[i].extent;
        }
        if (m == 3 && !is_b(0) && is_b(1) && !is_b(2) && merged[2].enc_stride == 1 &&
            merged[0].enc_stride == merged[2].extent) {
            out->A = merged[0].extent;
            out->I = merged[1].extent;
            out->J = merged[2].extent;
        }
    }
    if (numel == 0) {
        out->kind = kIJK;
        out->A = out->I = out->J = 1;
        out->K = 0;
    }
    return true;
}

}  // namespace ahq
