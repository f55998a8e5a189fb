// Shared pieces of the two-phase API: planning of view packing and the second-phase runner.
#pragma once

#include <hip/hip_runtime_api.h>

#include <memory>

#include "acl_types.hpp"

namespace opscv {

// Chooses where the kernel operand for the tensor `t` (at most five dimensions) lives: the tensor's own memory
// when the view is contiguous, else a 256-byte aligned slice of the workspace; in that case a gather (input) or
// scatter (output) step is queued on the executor and its workspace requirement grows.  With `perm`, the
// operand's dimension i is the view's dimension perm[i] (a transposed operand: contiguity is judged and the
// packing done in the permuted order).
PlannedPtr plan_view(aclOpExecutor* ex, const aclTensor* t, int elem_bytes, bool is_output,
                     const int* perm = nullptr);

// alignment the second phase asks of the caller's workspace pointer (hipMalloc returns 256-byte aligned memory; a
// byte-offset slice of a larger buffer may not be)
constexpr uintptr_t kWorkspaceAlignment = 16;

// What every first phase returns when planning went wrong inside the library (today: more strided views than the
// packing lists hold).
aclnnStatus plan_status(const aclOpExecutor* ex, const char* api);

inline void* resolve(const PlannedPtr& p, void* workspace)
{
    return p.in_workspace ? (void*)((char*)workspace + p.ws_offset) : p.direct;
}

// Second phase common to every operator: checks the executor and the workspace, gathers packed inputs,
// launches the operator, scatters the packed output, frees the executor (always, also on failure).
aclnnStatus run_executor(void* workspace, uint64_t workspace_size, aclOpExecutor* ex, aclrtStream stream,
                         OpKind expected, const char* api);

// The work of the second phase for a planned executor that stays the caller's (nothing is freed): gathers packed
// inputs into `workspace`, launches the operator, scatters the packed output.  `workspace` must hold
// ex->workspace_bytes bytes.
aclnnStatus execute_plan(void* workspace, const aclOpExecutor* ex, aclrtStream stream, const char* api);

// File-scope device array that stands in for the caller's workspace in the entry points that must not allocate
// (static_scratch.hip): address of this device's copy and its size in bytes.
hipError_t static_scratch(void** ptr, uint64_t* bytes);

}  // namespace opscv
