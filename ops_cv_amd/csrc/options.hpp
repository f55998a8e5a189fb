// Process-wide switches of the library: kernel-variant overrides for tests and benchmarks, the properties of the
// reference's device that some of its template choices read, and the coordinate rule of aclnnGridSampler2D.
//
// The values live in atomics.  They start from the environment, read once when the first of them is asked for, and
// change only through set_option() (opscvSetOption).  Every first phase copies what it needs into its executor, so a
// second phase runs with the values of its first phase whatever happens in between, and nothing on the launch path
// looks at the environment.
#pragma once

#include <cstdint>

namespace opscv {

// (kGsRingSingle: the ring kernel with one channel per stage, where two interleaved channels would be the choice)
enum GsVariant : int32_t { kGsAuto = 0, kGsDirect = 1, kGsRing = 2, kGsRingSingle = 3 };
enum ResizeVariant : int32_t { kResizeAuto = 0, kResizeGeneric = 1, kResizeRegisterBand = 2, kResizeLdsBand = 3 };
enum NearestVariant : int32_t { kNearestAuto = 0, kNearestGather = 1 };
enum GsRule : int32_t { kRuleGridSampler2D = 0, kRuleGridSampleArch35 = 1 };
enum Gs3dGradVariant : int32_t { kGs3dGradAuto = 0, kGs3dGradOrdered = 1, kGs3dGradGather = 2 };

struct Options {
    int32_t gs_variant = kGsAuto;            // OPSCV_GS_VARIANT = direct | ring | single
    int32_t resize_variant = kResizeAuto;    // OPSCV_RESIZE_VARIANT = generic | register | band
    int32_t nearest_variant = kNearestAuto;  // OPSCV_NEAREST_VARIANT = gather
    int64_t reference_cores = 64;            // OPSCV_REFERENCE_CORES
    int64_t reference_ub_bytes = 253952;     // OPSCV_REFERENCE_UB_BYTES
    int32_t grid_sampler2d_rule = kRuleGridSampler2D;  // OPSCV_GRID_SAMPLER2D_RULE = arch35
    int32_t gs3d_grad_variant = kGs3dGradAuto;         // OPSCV_GS3D_GRAD_VARIANT = ordered | gather
};

// the current values (a consistent enough snapshot: each field is one atomic load)
Options current_options();

// names: "gs_variant", "resize_variant", "nearest_variant", "reference_cores", "reference_ub_bytes",
// "grid_sampler2d_rule", "gs3d_grad_variant"; false for an unknown name or a value outside the option's range
bool set_option(const char* name, int64_t value);
bool get_option(const char* name, int64_t* value);

}  // namespace opscv
