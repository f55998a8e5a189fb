// Handle constructors/destructors and the thread-local error text behind aclGetRecentErrMsg.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <new>

#include "acl_types.hpp"

namespace opscv {

static thread_local char g_err[1024] = {0};

void set_error(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    const char* log = getenv("OPSCV_LOG");
    if (log != nullptr && log[0] == '1') {
        fprintf(stderr, "[opscv] %s\n", g_err);
    }
}

void clear_error() { g_err[0] = '\0'; }

}  // namespace opscv

extern "C" {

aclTensor* aclCreateTensor(const int64_t* viewDims, uint64_t viewDimsNum, aclDataType dataType,
                           const int64_t* stride, int64_t offset, aclFormat format, const int64_t* storageDims,
                           uint64_t storageDimsNum, void* tensorData)
{
    if (viewDimsNum > kMaxDims || storageDimsNum > kMaxDims || (viewDimsNum > 0 && viewDims == nullptr) ||
        offset < 0) {
        opscv::set_error("aclCreateTensor: invalid dims (view %llu, storage %llu) or offset %lld",
                         (unsigned long long)viewDimsNum, (unsigned long long)storageDimsNum, (long long)offset);
        return nullptr;
    }
    for (uint64_t i = 0; i < viewDimsNum; i++) {
        if (viewDims[i] < 0) {
            opscv::set_error("aclCreateTensor: negative view dim");
            return nullptr;
        }
    }
    aclTensor* t = new (std::nothrow) aclTensor();
    if (t == nullptr) {
        return nullptr;
    }
    t->ndim = (int64_t)viewDimsNum;
    int64_t run = 1;
    for (int64_t i = t->ndim - 1; i >= 0; i--) {
        t->dims[i] = viewDims[i];
        t->strides[i] = (stride != nullptr) ? stride[i] : run;
        run *= viewDims[i];
    }
    t->offset = offset;
    t->dtype = dataType;
    t->format = format;
    if (storageDims != nullptr) {
        t->storage_ndim = (int64_t)storageDimsNum;
        for (uint64_t i = 0; i < storageDimsNum; i++) {
            t->storage_dims[i] = storageDims[i];
        }
    } else {
        t->storage_ndim = t->ndim;
        memcpy(t->storage_dims, t->dims, sizeof(t->dims));
    }
    t->data = tensorData;
    return t;
}

aclnnStatus aclDestroyTensor(const aclTensor* tensor)
{
    delete tensor;
    return ACLNN_SUCCESS;
}

aclIntArray* aclCreateIntArray(const int64_t* value, uint64_t size)
{
    if (size > 0 && value == nullptr) {
        return nullptr;
    }
    aclIntArray* a = new (std::nothrow) aclIntArray();
    if (a != nullptr) {
        a->v.assign(value, value + size);
    }
    return a;
}

aclnnStatus aclDestroyIntArray(const aclIntArray* array)
{
    delete array;
    return ACLNN_SUCCESS;
}

aclnnStatus aclGetIntArraySize(const aclIntArray* array, uint64_t* size)
{
    if (array == nullptr || size == nullptr) {
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    *size = array->v.size();
    return ACLNN_SUCCESS;
}

aclFloatArray* aclCreateFloatArray(const float* value, uint64_t size)
{
    if (size > 0 && value == nullptr) {
        return nullptr;
    }
    aclFloatArray* a = new (std::nothrow) aclFloatArray();
    if (a != nullptr) {
        a->v.assign(value, value + size);
    }
    return a;
}

aclnnStatus aclDestroyFloatArray(const aclFloatArray* array)
{
    delete array;
    return ACLNN_SUCCESS;
}

aclnnStatus aclGetFloatArraySize(const aclFloatArray* array, uint64_t* size)
{
    if (array == nullptr || size == nullptr) {
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    *size = array->v.size();
    return ACLNN_SUCCESS;
}

aclBoolArray* aclCreateBoolArray(const bool* value, uint64_t size)
{
    if (size > 0 && value == nullptr) {
        return nullptr;
    }
    aclBoolArray* a = new (std::nothrow) aclBoolArray();
    if (a != nullptr) {
        a->v.assign(value, value + size);
    }
    return a;
}

aclnnStatus aclDestroyBoolArray(const aclBoolArray* array)
{
    delete array;
    return ACLNN_SUCCESS;
}

aclnnStatus aclGetBoolArraySize(const aclBoolArray* array, uint64_t* size)
{
    if (array == nullptr || size == nullptr) {
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    *size = array->v.size();
    return ACLNN_SUCCESS;
}

aclnnStatus aclDestroyAclOpExecutor(aclOpExecutor* executor)
{
    if (executor == nullptr) {
        return ACLNN_ERR_PARAM_NULLPTR;
    }
    if (executor->magic != kExecutorMagic) {
        opscv::set_error("aclDestroyAclOpExecutor: not a live executor");
        return ACLNN_ERR_PARAM_INVALID;
    }
    executor->magic = 0;
    delete executor;
    return ACLNN_SUCCESS;
}

const char* aclGetRecentErrMsg(void) { return opscv::g_err; }

}  // extern "C"
