/*
 * Minimal ACL-compatible base types for the MI355X build of the ops-cv bilinear path.
 *
 * The reference gets these from the CANN toolkit (acl/acl.h, aclnn/aclnn_base.h), which is not part of
 * the reference tree.  They are re-declared here from the public CANN API so that code written against
 * the reference's aclnn headers links against this library unchanged:
 *   - opaque handle names and aclrtStream: docs/zh/context/data_structure.md:7-79
 *   - status codes:                        docs/zh/context/aclnn_return_code.md:8-32
 *   - aclCreateTensor argument order:      image/grid_sample/examples/test_aclnn_grid_sample2_d.cpp:68-69,
 *                                          tests/ut/op_api/op_api_ut_common/src/tensor_desc.cpp:65-67
 *   - aclCreateIntArray:                   image/upsample_bilinear2d/examples/test_aclnn_upsample_bilinear2d.cpp:99
 *   - aclCreateFloatArray / aclGetFloatArraySize: image/resize_bilinear_v2/op_api/aclnn_resize.cpp:69
 * Enum values are CANN's published ones; they are kept in this single header.
 *
 * On this platform aclrtStream carries a hipStream_t and every tensorData pointer is a HIP device pointer.
 */
#ifndef OPSCV_ACL_BASE_H_
#define OPSCV_ACL_BASE_H_

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#ifndef ACLNN_API
#define ACLNN_API __attribute__((visibility("default")))
#endif

typedef int32_t aclnnStatus;
typedef int aclError;

#define ACL_SUCCESS 0
#define ACLNN_SUCCESS 0
#define ACLNN_ERR_PARAM_NULLPTR 161001
#define ACLNN_ERR_PARAM_INVALID 161002
#define ACLNN_ERR_RUNTIME_ERROR 361001
#define ACLNN_ERR_INNER 561000
#define ACLNN_ERR_INNER_TILING_ERROR 561002
#define ACLNN_ERR_INNER_CREATE_EXECUTOR 561101
#define ACLNN_ERR_INNER_NULLPTR 561103

typedef enum {
    ACL_DT_UNDEFINED = -1,
    ACL_FLOAT = 0,
    ACL_FLOAT16 = 1,
    ACL_INT8 = 2,
    ACL_INT32 = 3,
    ACL_UINT8 = 4,
    ACL_INT16 = 6,
    ACL_UINT16 = 7,
    ACL_UINT32 = 8,
    ACL_INT64 = 9,
    ACL_UINT64 = 10,
    ACL_DOUBLE = 11,
    ACL_BOOL = 12,
    ACL_STRING = 13,
    ACL_COMPLEX64 = 16,
    ACL_COMPLEX128 = 17,
    ACL_BF16 = 27
} aclDataType;

typedef enum {
    ACL_FORMAT_UNDEFINED = -1,
    ACL_FORMAT_NCHW = 0,
    ACL_FORMAT_NHWC = 1,
    ACL_FORMAT_ND = 2,
    ACL_FORMAT_NC1HWC0 = 3,
    ACL_FORMAT_FRACTAL_Z = 4,
    ACL_FORMAT_NC1HWC0_C04 = 12,
    ACL_FORMAT_HWCN = 16,
    ACL_FORMAT_NDHWC = 27,
    ACL_FORMAT_FRACTAL_NZ = 29,
    ACL_FORMAT_NCDHW = 30,
    ACL_FORMAT_NDC1HWC0 = 32,
    ACL_FRACTAL_Z_3D = 33
} aclFormat;

typedef struct aclTensor aclTensor;
typedef struct aclIntArray aclIntArray;
typedef struct aclFloatArray aclFloatArray;
typedef struct aclBoolArray aclBoolArray;
typedef struct aclOpExecutor aclOpExecutor;
typedef void* aclrtStream;

/*
 * Tensor descriptor over caller-owned device memory.  viewDims/stride/offset describe the logical view
 * (stride and offset in elements; stride == NULL means contiguous), storageDims the underlying buffer.
 * tensorData may be NULL for descriptors that are only passed to a GetWorkspaceSize call.
 * At most 8 dimensions.  Returns NULL on invalid arguments.
 */
ACLNN_API aclTensor* aclCreateTensor(const int64_t* viewDims, uint64_t viewDimsNum, aclDataType dataType,
                                     const int64_t* stride, int64_t offset, aclFormat format,
                                     const int64_t* storageDims, uint64_t storageDimsNum, void* tensorData);
ACLNN_API aclnnStatus aclDestroyTensor(const aclTensor* tensor);

ACLNN_API aclIntArray* aclCreateIntArray(const int64_t* value, uint64_t size);
ACLNN_API aclnnStatus aclDestroyIntArray(const aclIntArray* array);
ACLNN_API aclnnStatus aclGetIntArraySize(const aclIntArray* array, uint64_t* size);

ACLNN_API aclFloatArray* aclCreateFloatArray(const float* value, uint64_t size);
ACLNN_API aclnnStatus aclDestroyFloatArray(const aclFloatArray* array);
ACLNN_API aclnnStatus aclGetFloatArraySize(const aclFloatArray* array, uint64_t* size);

ACLNN_API aclBoolArray* aclCreateBoolArray(const bool* value, uint64_t size);
ACLNN_API aclnnStatus aclDestroyBoolArray(const aclBoolArray* array);
ACLNN_API aclnnStatus aclGetBoolArraySize(const aclBoolArray* array, uint64_t* size);

/*
 * Releases an executor whose second-phase call will never be made (the second-phase call itself frees
 * the executor it is given, docs/zh/context/data_structure.md:63-69).
 */
ACLNN_API aclnnStatus aclDestroyAclOpExecutor(aclOpExecutor* executor);

/* Text of the most recent failure on the calling thread ("" when none); valid until the next failure. */
ACLNN_API const char* aclGetRecentErrMsg(void);

#ifdef __cplusplus
}
#endif

#endif /* OPSCV_ACL_BASE_H_ */
