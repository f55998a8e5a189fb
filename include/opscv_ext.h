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

/* Library version string, e.g. "opscv-amd 0.1 (gfx950)". */
ACLNN_API const char* opscvVersion(void);

#ifdef __cplusplus
}
#endif

#endif /* OPSCV_EXT_H_ */
