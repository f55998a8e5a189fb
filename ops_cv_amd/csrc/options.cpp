// Process-wide switches: see options.hpp.
#include "options.hpp"

#include <atomic>
#include <cstdlib>
#include <cstring>
#include <mutex>

namespace opscv {

namespace {

struct Store {
    std::atomic<int64_t> gs_variant{kGsAuto};
    std::atomic<int64_t> resize_variant{kResizeAuto};
    std::atomic<int64_t> nearest_variant{kNearestAuto};
    // the core count of the reference's tiling unit test (test_resize_bilinear_v2_tiling.cpp: {64, 245760})
    std::atomic<int64_t> reference_cores{64};
    // the unified buffer of the reference's tiling unit test (test_resize_nearest_neighbor_v2_tiling.cpp: {64, 253952})
    std::atomic<int64_t> reference_ub_bytes{253952};
    std::atomic<int64_t> grid_sampler2d_rule{kRuleGridSampler2D};
    std::atomic<int64_t> gs3d_grad_variant{kGs3dGradAuto};
};

long long positive_env(const char* name)
{
    const char* v = getenv(name);
    if (v == nullptr) {
        return 0;
    }
    const long long n = strtoll(v, nullptr, 10);
    return n > 0 ? n : 0;
}

Store& store()
{
    static Store s;
    static std::once_flag once;
    std::call_once(once, [] {
        if (const char* v = getenv("OPSCV_GS_VARIANT")) {
            s.gs_variant = (v[0] == 'd') ? kGsDirect : (v[0] == 'r' ? kGsRing : (v[0] == 's' ? kGsRingSingle : kGsAuto));
        }
        if (const char* v = getenv("OPSCV_RESIZE_VARIANT")) {
            s.resize_variant = (v[0] == 'g') ? kResizeGeneric
                               : (v[0] == 'r') ? kResizeRegisterBand
                               : (v[0] == 'b') ? kResizeLdsBand
                                               : kResizeAuto;
        }
        if (const char* v = getenv("OPSCV_NEAREST_VARIANT")) {
            s.nearest_variant = (v[0] == 'g') ? kNearestGather : kNearestAuto;
        }
        if (const long long n = positive_env("OPSCV_REFERENCE_CORES")) {
            s.reference_cores = n;
        }
        if (const long long n = positive_env("OPSCV_REFERENCE_UB_BYTES")) {
            s.reference_ub_bytes = n;
        }
        if (const char* v = getenv("OPSCV_GS3D_GRAD_VARIANT")) {
            s.gs3d_grad_variant = (v[0] == 'o') ? kGs3dGradOrdered : (v[0] == 'g' ? kGs3dGradGather : kGs3dGradAuto);
        }
        if (const char* v = getenv("OPSCV_GRID_SAMPLER2D_RULE")) {
            s.grid_sampler2d_rule = (strcmp(v, "arch35") == 0 || strcmp(v, "1") == 0) ? kRuleGridSampleArch35
                                                                                       : kRuleGridSampler2D;
        }
    });
    return s;
}

struct Entry {
    const char* name;
    std::atomic<int64_t> Store::*field;
    int64_t lo, hi;
};

const Entry kEntries[] = {
    {"gs_variant", &Store::gs_variant, kGsAuto, kGsRingSingle},
    {"resize_variant", &Store::resize_variant, kResizeAuto, kResizeLdsBand},
    {"nearest_variant", &Store::nearest_variant, kNearestAuto, kNearestGather},
    {"reference_cores", &Store::reference_cores, 1, INT64_MAX},
    {"reference_ub_bytes", &Store::reference_ub_bytes, 1, INT64_MAX},
    {"grid_sampler2d_rule", &Store::grid_sampler2d_rule, kRuleGridSampler2D, kRuleGridSampleArch35},
    {"gs3d_grad_variant", &Store::gs3d_grad_variant, kGs3dGradAuto, kGs3dGradGather},
};

const Entry* find(const char* name)
{
    if (name == nullptr) {
        return nullptr;
    }
    for (const Entry& e : kEntries) {
        if (strcmp(e.name, name) == 0) {
            return &e;
        }
    }
    return nullptr;
}

}  // namespace

Options current_options()
{
    Store& s = store();
    Options o;
    o.gs_variant = (int32_t)s.gs_variant.load(std::memory_order_relaxed);
    o.resize_variant = (int32_t)s.resize_variant.load(std::memory_order_relaxed);
    o.nearest_variant = (int32_t)s.nearest_variant.load(std::memory_order_relaxed);
    o.reference_cores = s.reference_cores.load(std::memory_order_relaxed);
    o.reference_ub_bytes = s.reference_ub_bytes.load(std::memory_order_relaxed);
    o.grid_sampler2d_rule = (int32_t)s.grid_sampler2d_rule.load(std::memory_order_relaxed);
    o.gs3d_grad_variant = (int32_t)s.gs3d_grad_variant.load(std::memory_order_relaxed);
    return o;
}

bool set_option(const char* name, int64_t value)
{
    const Entry* e = find(name);
    if (e == nullptr || value < e->lo || value > e->hi) {
        return false;
    }
    (store().*(e->field)).store(value, std::memory_order_relaxed);
    return true;
}

bool get_option(const char* name, int64_t* value)
{
    const Entry* e = find(name);
    if (e == nullptr || value == nullptr) {
        return false;
    }
    *value = (store().*(e->field)).load(std::memory_order_relaxed);
    return true;
}

}  // namespace opscv
