// Handle life cycle, stream, workspace, pointer mode, version.
// Behaviour follows sparse/common/aclsparse_auxiliary.cpp:64-198, :253-279 of
// the reference; device memory comes from hipMalloc instead of aclrtMalloc.
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <new>

#include "internal.h"

namespace opsparse {

void LogError(const char *fmt, ...)
{
    static const bool enabled = std::getenv("OPS_SPARSE_LOG") != nullptr;
    if (!enabled) {
        return;
    }
    va_list ap;
    va_start(ap, fmt);
    std::fputs("[ops_sparse] ", stderr);
    std::vfprintf(stderr, fmt, ap);
    std::fputc('\n', stderr);
    va_end(ap);
}

OpsparseScalar MakeScalar(const void *p, aclDataType computeType, aclsparsePointerMode_t mode, double dflt)
{
    OpsparseScalar s{};
    s.isInt = (computeType == ACL_INT32) ? 1 : 0;
    s.value = dflt;
    s.devicePtr = nullptr;
    if (p == nullptr) {
        return s;
    }
    if (mode == ACL_SPARSE_POINTER_MODE_DEVICE) {
        s.devicePtr = p;
        return s;
    }
    s.value = s.isInt ? static_cast<double>(*static_cast<const int32_t *>(p))
                      : static_cast<double>(*static_cast<const float *>(p));
    return s;
}

aclsparseStatus_t EnsureWorkspace(aclsparseContext *h)
{
    if (h->useUserWorkspace || h->defaultWorkspace != nullptr) {
        return ACL_SPARSE_STATUS_SUCCESS;
    }
    void *ws = nullptr;
    if (hipMalloc(&ws, kDefaultWorkspaceBytes) != hipSuccess) {
        (void)hipGetLastError();
        LogError("hipMalloc of the %zu-byte default workspace failed", kDefaultWorkspaceBytes);
        return ACL_SPARSE_STATUS_ALLOC_FAILED;
    }
    h->defaultWorkspace = ws;
    h->defaultWorkspaceBytes = kDefaultWorkspaceBytes;
    return ACL_SPARSE_STATUS_SUCCESS;
}

}  // namespace opsparse

extern "C" {

aclsparseStatus_t aclsparseCreate(aclsparseHandle_t *handle)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    if (*handle != nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;  // refuse to overwrite a live handle
    }
    auto *h = new (std::nothrow) aclsparseContext();
    if (h == nullptr) {
        return ACL_SPARSE_STATUS_ALLOC_FAILED;
    }
    // The 4 MiB default workspace is allocated on first use (EnsureWorkspace),
    // so creating a handle never touches the device.
    *handle = h;
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseDestroy(aclsparseHandle_t handle)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    // Work queued by this handle may still be using the default workspace.
    if (handle->defaultWorkspace != nullptr) {
        if (handle->stream != nullptr) {
            (void)hipStreamSynchronize(handle->stream);
        } else {
            (void)hipDeviceSynchronize();
        }
        (void)hipFree(handle->defaultWorkspace);
    }
    delete handle;
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseSetStream(aclsparseHandle_t handle, aclrtStream stream)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    handle->stream = static_cast<hipStream_t>(stream);
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseGetStream(aclsparseHandle_t handle, aclrtStream *stream)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    if (stream == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    *stream = handle->stream;
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseSetWorkspace(aclsparseHandle_t handle, void *workspace, size_t workspaceSize)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    if (workspace == nullptr) {
        handle->useUserWorkspace = false;  // back to the library's own workspace
        return ACL_SPARSE_STATUS_SUCCESS;
    }
    if (workspaceSize == 0) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    // Grow-only: a request that is not larger than the workspace in use is a no-op.
    if (handle->useUserWorkspace && workspaceSize <= handle->userWorkspaceBytes) {
        return ACL_SPARSE_STATUS_SUCCESS;
    }
    handle->userWorkspace = workspace;
    handle->userWorkspaceBytes = workspaceSize;
    handle->useUserWorkspace = true;
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseGetWorkspace(aclsparseHandle_t handle, void **workspace, size_t *workspaceSize)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    if (workspace == nullptr || workspaceSize == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    const aclsparseStatus_t st = opsparse::EnsureWorkspace(handle);
    if (st != ACL_SPARSE_STATUS_SUCCESS) {
        return st;
    }
    *workspace = handle->workspace();
    *workspaceSize = handle->workspaceBytes();
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseGetVersion(aclsparseHandle_t /*handle*/, int *version)
{
    if (version == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    *version = opsparse::kVersionMajor * 10000 + opsparse::kVersionMinor * 100 + opsparse::kVersionPatch;
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseSetPointerMode(aclsparseHandle_t handle, aclsparsePointerMode_t mode)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    if (mode != ACL_SPARSE_POINTER_MODE_HOST && mode != ACL_SPARSE_POINTER_MODE_DEVICE) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    handle->pointerMode = mode;
    return ACL_SPARSE_STATUS_SUCCESS;
}

aclsparseStatus_t aclsparseGetPointerMode(aclsparseHandle_t handle, aclsparsePointerMode_t *mode)
{
    if (handle == nullptr) {
        return ACL_SPARSE_STATUS_HANDLE_IS_NULLPTR;
    }
    if (mode == nullptr) {
        return ACL_SPARSE_STATUS_INVALID_VALUE;
    }
    *mode = handle->pointerMode;
    return ACL_SPARSE_STATUS_SUCCESS;
}

}  // extern "C"
