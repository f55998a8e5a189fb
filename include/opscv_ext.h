/*
 * Entry points of the MI355X library that have no counterpart in the reference: introspection used by the
 * parity tests and the benchmark.  They are not part of the drop-in surface.
 */
#ifndef OPSCV_EXT_H_
#define OPSCV_EXT_H_

#include "opscv_acl_base.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Per-pixel decision record written by opscvGridSampler2DTaps (28 bytes, packed). */
typedef struct {
    int32_t x0;   /* bilinear: north-west tap column; nearest: selected column */
    int32_t y0;   /* bilinear: north-west tap row;    nearest: selected row    */
    float w[4];   /* bilinear weights nw, ne, sw, se; zeros for nearest          */
    int32_t flag; /* 1 when the pixel is written as NaN (non-finite source coordinate, bilinear only) */
} opscvTapRecord;

/*
 * Runs only the coordinate stage of the grid sampler (the code the sampling kernels share) and writes one
 * record per output pixel to `taps` (device memory, N*Hout*Wout records).  `grid` is contiguous
 * (N,Hout,Wout,2) device memory of type `dataType` (ACL_FLOAT, ACL_FLOAT16 or ACL_BF16).  Asynchronous on
 * `stream`.  Lets a test compare every integer corner index and weight with the CPU oracle bit for bit.
 */
ACLNN_API aclnnStatus opscvGridSampler2DTaps(const void* grid, aclDataType dataType, int64_t N, int64_t Hin,
                                             int64_t Win, int64_t Hout, int64_t Wout, int64_t interpolationMode,
                                             int64_t paddingMode, bool alignCorners, opscvTapRecord* taps,
                                             aclrtStream stream);

/* Per-pixel record of the bicubic mode written by opscvGridSampler2DBicubicTaps (68 bytes, packed). */
typedef struct {
    int32_t bx[4]; /* tap columns after padding, -1 = outside the image */
    int32_t by[4]; /* tap rows after padding, -1 = outside the image */
    float cx[4];   /* column coefficients */
    float cy[4];   /* row coefficients */
    int32_t flag;  /* 1 when the pixel is written as NaN (non-finite source coordinate) */
} opscvBicubicTapRecord;

/* Same as opscvGridSampler2DTaps for interpolationMode 2 (bicubic). */
ACLNN_API aclnnStatus opscvGridSampler2DBicubicTaps(const void* grid, aclDataType dataType, int64_t N, int64_t Hin,
                                                    int64_t Win, int64_t Hout, int64_t Wout, int64_t paddingMode,
                                                    bool alignCorners, opscvBicubicTapRecord* taps,
                                                    aclrtStream stream);

/*
 * Name of the kernel variant phase 2 would launch for an executor returned by a GetWorkspaceSize call
 * ("" for a no-op executor).  The string is static.
 */
ACLNN_API const char* opscvExecutorVariant(const aclOpExecutor* executor);

/*
 * Size in bytes of the library-owned scratch array behind opscvGridSampler2DNoAlloc: the most that the non-contiguous
 * views of one call may need for packing (each packed view takes its size rounded up to 256 bytes).
 */
#define OPSCV_NOALLOC_SCRATCH_BYTES (16u << 20)

/*
 * aclnnGridSampler2DGetWorkspaceSize + aclnnGridSampler2D as one call that allocates nothing, neither on the device
 * nor on the host.  It has no counterpart in the reference; it is for callers that cannot allocate a workspace
 * between the two phases: code under HIP graph capture, serving loops with a fixed memory plan, harnesses that
 * forbid allocation.  Same arguments, validation, status codes and results as the two-phase pair.  Where that pair
 * packs non-contiguous views into the caller's workspace (and scatters a non-contiguous output from it), this entry
 * point uses a file-scope device array of OPSCV_NOALLOC_SCRATCH_BYTES bytes that every device holds from library load
 * to process end.  A call whose views would need more returns ACLNN_ERR_PARAM_INVALID (161002) and launches nothing.
 * Contiguous tensors and channels-last views use no scratch at all.  All calls on one device share the array: calls
 * that overlap in time on one device (different streams, different threads) race on it and must be serialised by the
 * caller; calls on one stream are ordered by the stream.  Asynchronous on `stream` like aclnnGridSampler2D.
 *
 * Under stream capture: the first call on a device asks the runtime for the address of that device's copy of the
 * array, and the first launch of a kernel variant on a device sets that kernel's shared-memory attribute; neither may
 * be recorded.  Make one ordinary (uncaptured) call with the same dtype, modes and shapes on the device before the
 * capture begins; every later call, captured or not, only launches kernels.  The packing and clearing steps are
 * kernels (no memset node is recorded).
 */
ACLNN_API aclnnStatus opscvGridSampler2DNoAlloc(const aclTensor* input, const aclTensor* grid,
                                                int64_t interpolationMode, int64_t paddingMode, bool alignCorners,
                                                aclTensor* out, aclrtStream stream);

/*
 * Process-wide options.  They start from the environment, read once when the library first needs one of them, and
 * change only through opscvSetOption afterwards; every GetWorkspaceSize call copies the values it needs into its
 * executor, so a second phase runs with the options of its first phase and never looks at the environment.
 *
 *   name                    environment (initial value)      values
 *   "grid_sampler2d_rule"   OPSCV_GRID_SAMPLER2D_RULE=arch35  0 (default): bilinear coordinates as in the reference's
 *                                                            GridSampler2D kernel (grid_sampler2_d_simt.h);
 *                                                            1: as in the kernel its aclnnGridSampler2D launches on
 *                                                            its newest part (see aclnn_grid_sampler2d.h)
 *   "reference_cores"       OPSCV_REFERENCE_CORES            vector cores of the reference's device (default 64): its
 *                                                            choice between two resize templates and the chunk phase
 *                                                            of the 3-D sampler gradient read it
 *   "reference_ub_bytes"    OPSCV_REFERENCE_UB_BYTES         unified buffer of the reference's device (default
 *                                                            253952): gates its replicating nearest-resize template
 *   "gs_variant"            OPSCV_GS_VARIANT=direct|ring|single   0 automatic, 1 direct kernel, 2 no pair-layout variant,
 *                                                            3 as 2 and single-channel stages in the ring kernel
 *   "resize_variant"        OPSCV_RESIZE_VARIANT=generic|register|band   0 automatic, 1 per-element kernels,
 *                                                            2 register-band kernel, 3 no flat LDS kernel
 *   "nearest_variant"       OPSCV_NEAREST_VARIANT=gather     0 automatic, 1 gather from memory
 *   "gs3d_grad_variant"     OPSCV_GS3D_GRAD_VARIANT=ordered|gather   0 automatic, 1 ordered kernel, 2 gather variant
 *                                                            wherever it can run (input gradient of the 3-D sampler)
 * The last four pick among kernels with identical results (tests and benchmarks use them); the first three can
 * change result bits.  Returns ACLNN_ERR_PARAM_INVALID for an unknown name or a value out of range.
 */
ACLNN_API aclnnStatus opscvSetOption(const char* name, int64_t value);
ACLNN_API aclnnStatus opscvGetOption(const char* name, int64_t* value);

/*
 * Revision of the data movement of a kernel variant (the names opscvExecutorVariant returns): a small integer that
 * goes up whenever a change to the variant's kernels changes which bytes they move or how (loads, stores, staging,
 * work split).  A counter measurement of memory traffic is valid for the revision it was taken on; the benchmark
 * reports such a figure only while the revision matches.  Unknown names return 0.
 */
ACLNN_API int32_t opscvVariantRevision(const char* variant);

/* Library version string, e.g. "opscv-amd 0.1 (gfx950)". */
ACLNN_API const char* opscvVersion(void);

#ifdef __cplusplus
}
#endif

#endif /* OPSCV_EXT_H_ */
