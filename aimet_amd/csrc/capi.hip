// Entry points that do not belong to one kernel family.
#include <cstdio>

#include "ahq_host.h"
#include "layout.h"

extern "C" const char* ahq_last_error(void) { return ahq::error_buffer(); }
extern "C" int ahq_version(void) { return 1; }

namespace {

constexpr size_t kAlign = 256;
inline size_t align_up(size_t v) { return (v + kAlign - 1) / kAlign * kAlign; }

inline size_t dtype_bytes(int32_t dtype) { return dtype == AHQ_F32 ? 4 : 2; }

// statistics (minimum, then maximum, each aligned) in front of the reduction's own workspace
bool calibrate_qdq_offsets(int32_t dtype, const ahq_layout* layout, ahq::CanonLayout* canon, size_t* off_max,
                           size_t* off_reduce, size_t* total) {
    ahq::CanonLayout& c = *canon;
    const char* err = nullptr;
    if (!ahq::canonicalize(*layout, &c, &err)) return ahq::set_error(err), false;
    const size_t stats = align_up((size_t)c.num_enc * dtype_bytes(dtype));
    *off_max = stats;
    *off_reduce = 2 * stats;
    *total = 2 * stats + ahq_minmax_workspace_bytes(layout);
    return true;
}

}  // namespace

extern "C" size_t ahq_minmax_calibrate_qdq_workspace_bytes(int32_t dtype, const ahq_layout* layout) {
    if (!layout || dtype < AHQ_F32 || dtype > AHQ_BF16) return 0;
    ahq::CanonLayout c;
    size_t off_max, off_reduce, total;
    return calibrate_qdq_offsets(dtype, layout, &c, &off_max, &off_reduce, &total) ? total : 0;
}

extern "C" int ahq_minmax_calibrate_qdq(const ahq_grid* grid, const ahq_layout* layout, const void* x, void* y,
                                        int64_t num_steps, int32_t symmetric, float minimum_scale_in_dtype,
                                        float minimum_scale, float dtype_max, float near_max_threshold, int32_t* flags,
                                        int32_t param_dtype, void* param_min, void* param_max,
                                        double grid_minimum_scale, float* scale, float* offset, void* workspace,
                                        size_t workspace_bytes, void* stream) {
    using ahq::set_error;
    if (!grid || !layout || !x || !y || !offset) return set_error("null argument"), AHQ_ERR_INVALID;
    const int32_t dtype = grid->io_dtype;
    if (dtype < AHQ_F32 || dtype > AHQ_BF16) return set_error("bad dtype"), AHQ_ERR_INVALID;
    if (grid->op != AHQ_OP_QDQ || grid->arith == AHQ_ARITH_DLQ)
        return set_error("a quantize-dequantize grid of the ATen or autograd arithmetic is expected"), AHQ_ERR_INVALID;
    ahq::CanonLayout c;
    size_t off_max, off_reduce, total;
    if (!calibrate_qdq_offsets(dtype, layout, &c, &off_max, &off_reduce, &total)) return AHQ_ERR_INVALID;
    if (!workspace || workspace_bytes < total) return set_error("workspace too small"), AHQ_ERR_WORKSPACE;
    if (c.numel == 0) return set_error("cannot calibrate on an empty tensor"), AHQ_ERR_INVALID;
    char* w = static_cast<char*>(workspace);
    void* stat_min = w;
    void* stat_max = w + off_max;
    int rc = ahq_minmax(dtype, layout, x, stat_min, stat_max, nullptr, nullptr, 0, w + off_reduce, total - off_reduce,
                        stream);
    if (rc != AHQ_OK) return rc;
    rc = ahq_minmax_finalize(dtype, stat_min, stat_max, c.num_enc, num_steps, symmetric, minimum_scale_in_dtype,
                             minimum_scale, dtype_max, near_max_threshold, flags, param_dtype, param_min, param_max,
                             grid->qmin, grid->qmax, grid_minimum_scale, scale, symmetric ? nullptr : offset, stream);
    if (rc != AHQ_OK) return rc;
    return ahq_qdq_forward(grid, layout, x, y, nullptr, scale, offset, nullptr, nullptr, stream);
}

extern "C" int ahq_grid_probe_many(const ahq_grid_probe_item* items, int64_t count, uint8_t* verdicts,
                                   uint8_t* unsupported, void* stream) {
    using ahq::set_error;
    if (count < 0 || (count > 0 && (!items || !verdicts))) return set_error("null argument"), AHQ_ERR_INVALID;
    for (int64_t i = 0; i < count; ++i) {
        const ahq_grid_probe_item& it = items[i];
        if (unsupported) unsupported[i] = 0;
        const int rc = ahq_grid_probe(it.dtype, &it.layout, it.x, it.num_levels, verdicts + i, stream);
        if (rc == AHQ_ERR_UNSUPPORTED && unsupported) {
            unsupported[i] = 1;
            continue;
        }
        if (rc != AHQ_OK) {
            char msg[512];
            std::snprintf(msg, sizeof msg, "item %lld: %s", (long long)i, ahq::error_buffer());
            set_error(msg);
            return rc;
        }
    }
    return AHQ_OK;
}

extern "C" int ahq_minmax_calibrate_qdq_many(const ahq_calibrate_qdq_item* items, int64_t count, int32_t* flags,
                                             void* stream) {
    using ahq::set_error;
    if (count < 0 || (count > 0 && !items)) return set_error("null argument"), AHQ_ERR_INVALID;
    for (int64_t i = 0; i < count; ++i) {
        const ahq_calibrate_qdq_item& it = items[i];
        const int rc = ahq_minmax_calibrate_qdq(&it.grid, &it.layout, it.x, it.y, it.num_steps, it.symmetric,
                                                it.minimum_scale_in_dtype, it.minimum_scale, it.dtype_max,
                                                it.near_max_threshold, flags, it.param_dtype, it.param_min,
                                                it.param_max, it.grid_minimum_scale, it.scale, it.offset, it.workspace,
                                                it.workspace_bytes, stream);
        if (rc != AHQ_OK) {
            char msg[512];
            std::snprintf(msg, sizeof msg, "item %lld: %s", (long long)i, ahq::error_buffer());
            set_error(msg);
            return rc;
        }
    }
    return AHQ_OK;
}
