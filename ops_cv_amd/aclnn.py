"""ctypes binding of the aclnn C-ABI exported by libopscv_amd.so.

The raw entry points keep the reference's names and argument order
(image/grid_sample/op_api/aclnn_grid_sampler2d.h:53-82,
image/upsample_bilinear2d/op_host/op_api/aclnn_upsample_bilinear_2d.h:25-34).  The helpers at the bottom
run both phases on torch tensors the way the reference's examples do on device buffers
(image/grid_sample/examples/test_aclnn_grid_sample2_d.cpp:102-135).

There is no CPU fallback: when the library is missing or no GPU is present the compute helpers raise.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libopscv_amd.so")

# aclDataType / aclFormat values (include/opscv_acl_base.h)
ACL_DT_UNDEFINED = -1
ACL_FLOAT = 0
ACL_FLOAT16 = 1
ACL_INT8 = 2
ACL_INT32 = 3
ACL_UINT8 = 4
ACL_INT16 = 6
ACL_UINT16 = 7
ACL_UINT32 = 8
ACL_INT64 = 9
ACL_UINT64 = 10
ACL_DOUBLE = 11
ACL_BOOL = 12
ACL_COMPLEX64 = 16
ACL_COMPLEX128 = 17
ACL_BF16 = 27

ACL_FORMAT_NCHW = 0
ACL_FORMAT_NHWC = 1
ACL_FORMAT_ND = 2
ACL_FORMAT_HWCN = 16
ACL_FORMAT_NDHWC = 27
ACL_FORMAT_NCDHW = 30

ACLNN_SUCCESS = 0
ACLNN_ERR_PARAM_NULLPTR = 161001
ACLNN_ERR_PARAM_INVALID = 161002
ACLNN_ERR_RUNTIME_ERROR = 361001
ACLNN_ERR_INNER_CREATE_EXECUTOR = 561101
ACLNN_ERR_INNER_NULLPTR = 561103

INTERP_BILINEAR, INTERP_NEAREST, INTERP_BICUBIC = 0, 1, 2
PAD_ZEROS, PAD_BORDER, PAD_REFLECTION = 0, 1, 2


class TapRecord(ctypes.Structure):
    _fields_ = [("x0", ctypes.c_int32), ("y0", ctypes.c_int32), ("w", ctypes.c_float * 4),
                ("flag", ctypes.c_int32)]


_lib = None


def library_path():
    return _LIB_PATH


def load_library():
    """Loads libopscv_amd.so (built beforehand by ops_cv_amd.build / __graft_entry__.build)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise RuntimeError("libopscv_amd.so is not built: run `python -m ops_cv_amd.build`")
    L = ctypes.CDLL(_LIB_PATH)
    vp, i64, u64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_uint64, ctypes.c_int32
    p_i64, p_u64, p_vp = ctypes.POINTER(i64), ctypes.POINTER(u64), ctypes.POINTER(vp)
    L.aclCreateTensor.restype = vp
    L.aclCreateTensor.argtypes = [p_i64, u64, ctypes.c_int, p_i64, i64, ctypes.c_int, p_i64, u64, vp]
    L.aclDestroyTensor.restype = i32
    L.aclDestroyTensor.argtypes = [vp]
    L.aclCreateIntArray.restype = vp
    L.aclCreateIntArray.argtypes = [p_i64, u64]
    L.aclDestroyIntArray.restype = i32
    L.aclDestroyIntArray.argtypes = [vp]
    L.aclGetIntArraySize.restype = i32
    L.aclGetIntArraySize.argtypes = [vp, p_u64]
    L.aclCreateFloatArray.restype = vp
    L.aclCreateFloatArray.argtypes = [ctypes.POINTER(ctypes.c_float), u64]
    L.aclDestroyFloatArray.restype = i32
    L.aclDestroyFloatArray.argtypes = [vp]
    L.aclGetFloatArraySize.restype = i32
    L.aclGetFloatArraySize.argtypes = [vp, p_u64]
    L.aclDestroyAclOpExecutor.restype = i32
    L.aclDestroyAclOpExecutor.argtypes = [vp]
    L.aclGetRecentErrMsg.restype = ctypes.c_char_p
    L.aclGetRecentErrMsg.argtypes = []
    L.aclnnGridSampler2DGetWorkspaceSize.restype = i32
    L.aclnnGridSampler2DGetWorkspaceSize.argtypes = [vp, vp, i64, i64, ctypes.c_bool, vp, p_u64, p_vp]
    L.aclnnGridSampler2D.restype = i32
    L.aclnnGridSampler2D.argtypes = [vp, u64, vp, vp]
    L.aclCreateBoolArray.restype = vp
    L.aclCreateBoolArray.argtypes = [ctypes.POINTER(ctypes.c_bool), u64]
    L.aclDestroyBoolArray.restype = i32
    L.aclDestroyBoolArray.argtypes = [vp]
    L.aclnnGridSampler2DBackwardGetWorkspaceSize.restype = i32
    L.aclnnGridSampler2DBackwardGetWorkspaceSize.argtypes = [vp, vp, vp, i64, i64, ctypes.c_bool, vp, vp, vp, p_u64,
                                                             p_vp]
    L.aclnnGridSampler2DBackward.restype = i32
    L.aclnnGridSampler2DBackward.argtypes = [vp, u64, vp, vp]
    L.aclnnGridSampler3DBackwardGetWorkspaceSize.restype = i32
    L.aclnnGridSampler3DBackwardGetWorkspaceSize.argtypes = L.aclnnGridSampler2DBackwardGetWorkspaceSize.argtypes
    L.aclnnGridSampler3DBackward.restype = i32
    L.aclnnGridSampler3DBackward.argtypes = [vp, u64, vp, vp]
    L.aclnnGridSampler3DGetWorkspaceSize.restype = i32
    L.aclnnGridSampler3DGetWorkspaceSize.argtypes = [vp, vp, i64, i64, ctypes.c_bool, vp, p_u64, p_vp]
    L.aclnnGridSampler3D.restype = i32
    L.aclnnGridSampler3D.argtypes = [vp, u64, vp, vp]
    L.aclnnUpsampleBilinear2dGetWorkspaceSize.restype = i32
    L.aclnnUpsampleBilinear2dGetWorkspaceSize.argtypes = [vp, vp, ctypes.c_bool, ctypes.c_double, ctypes.c_double,
                                                         vp, p_u64, p_vp]
    L.aclnnUpsampleBilinear2d.restype = i32
    L.aclnnUpsampleBilinear2d.argtypes = [vp, u64, vp, vp]
    L.aclnnResizeGetWorkspaceSize.restype = i32
    L.aclnnResizeGetWorkspaceSize.argtypes = [vp, vp, ctypes.c_char_p, vp, ctypes.POINTER(u64), ctypes.POINTER(vp)]
    L.aclnnResize.restype = i32
    L.aclnnResize.argtypes = [vp, u64, vp, vp]
    L.aclnnUpsampleBilinear2dBackwardGetWorkspaceSize.restype = i32
    L.aclnnUpsampleBilinear2dBackwardGetWorkspaceSize.argtypes = [vp, vp, vp, ctypes.c_bool, ctypes.c_double,
                                                                  ctypes.c_double, vp, ctypes.POINTER(u64),
                                                                  ctypes.POINTER(vp)]
    L.aclnnUpsampleBilinear2dBackward.restype = i32
    L.aclnnUpsampleBilinear2dBackward.argtypes = [vp, u64, vp, vp]
    L.opscvGridSampler2DTaps.restype = i32
    L.opscvGridSampler2DTaps.argtypes = [vp, ctypes.c_int, i64, i64, i64, i64, i64, i64, i64, ctypes.c_bool, vp, vp]
    L.opscvGridSampler2DBicubicTaps.restype = i32
    L.opscvGridSampler2DBicubicTaps.argtypes = [vp, ctypes.c_int, i64, i64, i64, i64, i64, i64, ctypes.c_bool, vp, vp]
    L.opscvExecutorVariant.restype = ctypes.c_char_p
    L.opscvExecutorVariant.argtypes = [vp]
    L.opscvGridSampler2DNoAlloc.restype = i32
    L.opscvGridSampler2DNoAlloc.argtypes = [vp, vp, i64, i64, ctypes.c_bool, vp, vp]
    L.opscvVersion.restype = ctypes.c_char_p
    L.opscvVersion.argtypes = []
    L.opscvSetOption.restype = ctypes.c_int
    L.opscvSetOption.argtypes = [ctypes.c_char_p, ctypes.c_int64]
    L.opscvGetOption.restype = ctypes.c_int
    L.opscvGetOption.argtypes = [ctypes.c_char_p, ctypes.POINTER(ctypes.c_int64)]
    L.opscvVariantRevision.restype = ctypes.c_int32
    L.opscvVariantRevision.argtypes = [ctypes.c_char_p]
    _lib = L
    return L


class AclnnError(RuntimeError):
    def __init__(self, api, status):
        msg = load_library().aclGetRecentErrMsg().decode("utf-8", "replace")
        super().__init__("%s failed with status %d: %s" % (api, status, msg))
        self.status = status


def _i64_array(values):
    if values is None:
        return None
    return (ctypes.c_int64 * len(values))(*[int(v) for v in values])


def create_tensor(view_dims, dtype, fmt=ACL_FORMAT_ND, strides=None, offset=0, storage_dims=None, data=None):
    """aclCreateTensor with the reference's argument meaning; returns the opaque handle (int) or None."""
    L = load_library()
    dims = _i64_array(view_dims)
    st = _i64_array(strides)
    sd = _i64_array(storage_dims if storage_dims is not None else view_dims)
    n_sd = len(storage_dims) if storage_dims is not None else len(view_dims)
    return L.aclCreateTensor(dims, len(view_dims), dtype, st, offset, fmt, sd, n_sd, data)


def destroy_tensor(handle):
    if handle:
        load_library().aclDestroyTensor(handle)


def create_int_array(values):
    return load_library().aclCreateIntArray(_i64_array(values), len(values))


def destroy_int_array(handle):
    if handle:
        load_library().aclDestroyIntArray(handle)


def get_workspace_size_grid_sampler2d(inp, grid, interpolation_mode, padding_mode, align_corners, out):
    """Phase 1 on raw handles; returns (status, workspace_bytes, executor_handle)."""
    L = load_library()
    ws = ctypes.c_uint64(0)
    ex = ctypes.c_void_p(None)
    st = L.aclnnGridSampler2DGetWorkspaceSize(inp, grid, interpolation_mode, padding_mode, bool(align_corners), out,
                                              ctypes.byref(ws), ctypes.byref(ex))
    return st, ws.value, ex.value


def create_bool_array(values):
    L = load_library()
    arr = (ctypes.c_bool * len(values))(*[bool(v) for v in values])
    return L.aclCreateBoolArray(arr, len(values))


def destroy_bool_array(handle):
    if handle:
        load_library().aclDestroyBoolArray(handle)


def get_workspace_size_grid_sampler2d_backward(grad_out, inp, grid, interpolation_mode, padding_mode, align_corners,
                                               output_mask, input_grad, grid_grad):
    """Phase 1 of aclnnGridSampler2DBackward on raw handles; returns (status, workspace_bytes, executor_handle)."""
    L = load_library()
    ws = ctypes.c_uint64(0)
    ex = ctypes.c_void_p(None)
    st = L.aclnnGridSampler2DBackwardGetWorkspaceSize(grad_out, inp, grid, interpolation_mode, padding_mode,
                                                      bool(align_corners), output_mask, input_grad, grid_grad,
                                                      ctypes.byref(ws), ctypes.byref(ex))
    return st, ws.value, ex.value


def get_workspace_size_grid_sampler3d_backward(grad_out, inp, grid, interpolation_mode, padding_mode, align_corners,
                                               output_mask, input_grad, grid_grad):
    """Phase 1 of aclnnGridSampler3DBackward on raw handles; returns (status, workspace_bytes, executor_handle)."""
    L = load_library()
    ws = ctypes.c_uint64(0)
    ex = ctypes.c_void_p(None)
    st = L.aclnnGridSampler3DBackwardGetWorkspaceSize(grad_out, inp, grid, interpolation_mode, padding_mode,
                                                      bool(align_corners), output_mask, input_grad, grid_grad,
                                                      ctypes.byref(ws), ctypes.byref(ex))
    return st, ws.value, ex.value


def get_workspace_size_grid_sampler3d(inp, grid, interpolation_mode, padding_mode, align_corners, out):
    """Phase 1 of aclnnGridSampler3D on raw handles; returns (status, workspace_bytes, executor_handle)."""
    L = load_library()
    ws = ctypes.c_uint64(0)
    ex = ctypes.c_void_p(None)
    st = L.aclnnGridSampler3DGetWorkspaceSize(inp, grid, interpolation_mode, padding_mode, bool(align_corners), out,
                                              ctypes.byref(ws), ctypes.byref(ex))
    return st, ws.value, ex.value


def get_workspace_size_upsample_bilinear2d(self_t, output_size, align_corners, scales_h, scales_w, out):
    L = load_library()
    ws = ctypes.c_uint64(0)
    ex = ctypes.c_void_p(None)
    st = L.aclnnUpsampleBilinear2dGetWorkspaceSize(self_t, output_size, bool(align_corners), float(scales_h),
                                                   float(scales_w), out, ctypes.byref(ws), ctypes.byref(ex))
    return st, ws.value, ex.value


def create_float_array(values):
    arr = (ctypes.c_float * len(values))(*[float(v) for v in values])
    return load_library().aclCreateFloatArray(arr, len(values))


def destroy_float_array(handle):
    if handle:
        load_library().aclDestroyFloatArray(handle)


def get_workspace_size_resize(self_t, scales, mode, out):
    """Phase 1 of aclnnResize on raw handles; `mode` is bytes or None."""
    L = load_library()
    ws = ctypes.c_uint64(0)
    ex = ctypes.c_void_p(None)
    st = L.aclnnResizeGetWorkspaceSize(self_t, scales, mode, out, ctypes.byref(ws), ctypes.byref(ex))
    return st, ws.value, ex.value


def get_workspace_size_upsample_bilinear2d_backward(grad_out, output_size, input_size, align_corners, scales_h,
                                                    scales_w, out):
    L = load_library()
    ws = ctypes.c_uint64(0)
    ex = ctypes.c_void_p(None)
    st = L.aclnnUpsampleBilinear2dBackwardGetWorkspaceSize(grad_out, output_size, input_size, bool(align_corners),
                                                           float(scales_h), float(scales_w), out, ctypes.byref(ws),
                                                           ctypes.byref(ex))
    return st, ws.value, ex.value


def destroy_executor(handle):
    if handle:
        return load_library().aclDestroyAclOpExecutor(handle)
    return ACLNN_ERR_PARAM_NULLPTR


def executor_variant(handle):
    return load_library().opscvExecutorVariant(handle).decode()


def set_option(name, value):
    """opscvSetOption; raises on an unknown name or a value out of range."""
    st = load_library().opscvSetOption(name.encode(), int(value))
    if st != ACLNN_SUCCESS:
        raise AclnnError("opscvSetOption(%r, %r)" % (name, value), st)


def get_option(name):
    v = ctypes.c_int64(0)
    st = load_library().opscvGetOption(name.encode(), ctypes.byref(v))
    if st != ACLNN_SUCCESS:
        raise AclnnError("opscvGetOption(%r)" % name, st)
    return v.value


class option:
    """Context manager: an option set for the block and restored afterwards."""

    def __init__(self, name, value):
        self.name, self.value = name, value

    def __enter__(self):
        self.saved = get_option(self.name)
        set_option(self.name, self.value)
        return self

    def __exit__(self, *exc):
        set_option(self.name, self.saved)
        return False


def variant_revision(name):
    """Revision of the data movement of a kernel variant (opscvVariantRevision)."""
    return int(load_library().opscvVariantRevision(name.encode()))


# ----------------------------------------------------------------------------------------------------
# torch-tensor helpers (device memory + stream come from torch; everything else is the C-ABI)
# ----------------------------------------------------------------------------------------------------

def _torch():
    import torch
    return torch


def acl_dtype_of(t):
    torch = _torch()
    table = {torch.float32: ACL_FLOAT, torch.float16: ACL_FLOAT16, torch.bfloat16: ACL_BF16,
             torch.float64: ACL_DOUBLE, torch.int32: ACL_INT32, torch.int64: ACL_INT64, torch.uint8: ACL_UINT8,
             torch.int8: ACL_INT8, torch.int16: ACL_INT16, torch.bool: ACL_BOOL}
    return table[t.dtype]


def tensor_handle(t, fmt=ACL_FORMAT_ND):
    """aclTensor over a torch CUDA tensor's memory; strides and storage offset of the view are honoured."""
    if not t.is_cuda:
        raise RuntimeError("ops_cv_amd needs device tensors: there is no CPU path")
    base = t.untyped_storage().data_ptr()
    nstorage = t.untyped_storage().nbytes() // t.element_size()
    return create_tensor(list(t.shape), acl_dtype_of(t), fmt, list(t.stride()), t.storage_offset(), [nstorage],
                         ctypes.c_void_p(base))


def _stream_handle(stream):
    torch = _torch()
    s = torch.cuda.current_stream() if stream is None else stream
    return ctypes.c_void_p(s.cuda_stream)


def grid_sampler2d(inp, grid, interpolation_mode=0, padding_mode=0, align_corners=False, out=None, stream=None,
                   workspace=None):
    """Both phases of aclnnGridSampler2D on torch CUDA tensors; returns `out` (N,C,Hout,Wout)."""
    torch = _torch()
    L = load_library()
    if out is None:
        out = torch.empty((inp.shape[0], inp.shape[1], grid.shape[1], grid.shape[2]), dtype=inp.dtype,
                          device=inp.device)
    hs = [tensor_handle(inp), tensor_handle(grid), tensor_handle(out)]
    try:
        st, ws, ex = get_workspace_size_grid_sampler2d(hs[0], hs[1], interpolation_mode, padding_mode,
                                                       align_corners, hs[2])
        if st != ACLNN_SUCCESS:
            raise AclnnError("aclnnGridSampler2DGetWorkspaceSize", st)
        if ws > 0 and (workspace is None or workspace.numel() * workspace.element_size() < ws):
            workspace = torch.empty(ws, dtype=torch.uint8, device=inp.device)
        wptr = ctypes.c_void_p(workspace.data_ptr()) if ws > 0 else None
        wsize = workspace.numel() * workspace.element_size() if ws > 0 else 0
        st = L.aclnnGridSampler2D(wptr, wsize, ex, _stream_handle(stream))
        if st != ACLNN_SUCCESS:
            raise AclnnError("aclnnGridSampler2D", st)
    finally:
        for h in hs:
            destroy_tensor(h)
    return out


NOALLOC_SCRATCH_BYTES = 16 << 20  # OPSCV_NOALLOC_SCRATCH_BYTES (include/opscv_ext.h)


def grid_sampler2d_noalloc(inp, grid, out, interpolation_mode=0, padding_mode=0, align_corners=False, stream=None):
    """opscvGridSampler2DNoAlloc on torch CUDA tensors: one call, no workspace; `out` is the caller's.  Returns the
    status code (0 on success) so that a test can look at the refusals as well."""
    L = load_library()
    hs = [tensor_handle(inp), tensor_handle(grid), tensor_handle(out)]
    try:
        return L.opscvGridSampler2DNoAlloc(hs[0], hs[1], interpolation_mode, padding_mode, align_corners, hs[2],
                                           _stream_handle(stream))
    finally:
        for h in hs:
            destroy_tensor(h)


def grid_sampler2d_backward(grad_out, inp, grid, interpolation_mode=0, padding_mode=0, align_corners=False,
                            output_mask=(True, True), input_grad=None, grid_grad=None, stream=None, workspace=None):
    """Both phases of aclnnGridSampler2DBackward on torch CUDA tensors; returns (input_grad, grid_grad).  A gradient
    whose mask flag is false is left untouched."""
    torch = _torch()
    L = load_library()
    if input_grad is None:
        input_grad = torch.empty_like(inp)
    if grid_grad is None:
        grid_grad = torch.empty_like(grid)
    hs = [tensor_handle(t) for t in (grad_out, inp, grid, input_grad, grid_grad)]
    mask = create_bool_array(list(output_mask))
    try:
        st, ws, ex = get_workspace_size_grid_sampler2d_backward(hs[0], hs[1], hs[2], interpolation_mode, padding_mode,
                                                                align_corners, mask, hs[3], hs[4])
        if st != ACLNN_SUCCESS:
            raise AclnnError("aclnnGridSampler2DBackwardGetWorkspaceSize", st)
        if ws > 0 and (workspace is None or workspace.numel() * workspace.element_size() < ws):
            workspace = torch.empty(ws, dtype=torch.uint8, device=inp.device)
        wptr = ctypes.c_void_p(workspace.data_ptr()) if ws > 0 else None
        wsize = workspace.numel() * workspace.element_size() if ws > 0 else 0
        st = L.aclnnGridSampler2DBackward(wptr, wsize, ex, _stream_handle(stream))
        if st != ACLNN_SUCCESS:
            raise AclnnError("aclnnGridSampler2DBackward", st)
    finally:
        for h in hs:
            destroy_tensor(h)
        destroy_bool_array(mask)
    return input_grad, grid_grad


def grid_sampler3d_backward(grad_out, inp, grid, interpolation_mode=0, padding_mode=0, align_corners=False,
                            output_mask=(True, True), input_grad=None, grid_grad=None, stream=None, workspace=None,
                            channels_last=False):
    """Both phases of aclnnGridSampler3DBackward on torch CUDA tensors; returns (input_grad, grid_grad).  A gradient
    whose mask flag is false is left untouched.  With channels_last, grad_out, inp and input_grad are (N,D,H,W,C)."""
    torch = _torch()
    L = load_library()
    if input_grad is None:
        input_grad = torch.empty_like(inp)
    if grid_grad is None:
        grid_grad = torch.empty_like(grid)
    fmt = ACL_FORMAT_NDHWC if channels_last else ACL_FORMAT_NCDHW
    hs = [tensor_handle(grad_out, fmt), tensor_handle(inp, fmt), tensor_handle(grid), tensor_handle(input_grad, fmt),
          tensor_handle(grid_grad)]
    mask = create_bool_array(list(output_mask))
    try:
        st, ws, ex = get_workspace_size_grid_sampler3d_backward(hs[0], hs[1], hs[2], interpolation_mode, padding_mode,
                                                                align_corners, mask, hs[3], hs[4])
        if st != ACLNN_SUCCESS:
            raise AclnnError("aclnnGridSampler3DBackwardGetWorkspaceSize", st)
        if ws > 0 and (workspace is None or workspace.numel() * workspace.element_size() < ws):
            workspace = torch.empty(ws, dtype=torch.uint8, device=inp.device)
        wptr = ctypes.c_void_p(workspace.data_ptr()) if ws > 0 else None
        wsize = workspace.numel() * workspace.element_size() if ws > 0 else 0
        st = L.aclnnGridSampler3DBackward(wptr, wsize, ex, _stream_handle(stream))
        if st != ACLNN_SUCCESS:
            raise AclnnError("aclnnGridSampler3DBackward", st)
    finally:
        for h in hs:
            destroy_tensor(h)
        destroy_bool_array(mask)
    return input_grad, grid_grad


def grid_sampler3d(inp, grid, interpolation_mode=0, padding_mode=0, align_corners=False, out=None, stream=None,
                   channels_last=False, workspace=None):
    """Both phases of aclnnGridSampler3D on torch CUDA tensors.

    inp is (N,C,D,H,W) and the result (N,C,Do,Ho,Wo); with channels_last inp is (N,D,H,W,C) and the result
    (N,Do,Ho,Wo,C) (format NDHWC).  grid is (N,Do,Ho,Wo,3).
    """
    torch = _torch()
    L = load_library()
    fmt = ACL_FORMAT_NDHWC if channels_last else ACL_FORMAT_NCDHW
    if out is None:
        if channels_last:
            shape = (inp.shape[0], grid.shape[1], grid.shape[2], grid.shape[3], inp.shape[4])
        else:
            shape = (inp.shape[0], inp.shape[1], grid.shape[1], grid.shape[2], grid.shape[3])
        out = torch.empty(shape, dtype=inp.dtype, device=inp.device)
    hs = [tensor_handle(inp, fmt), tensor_handle(grid), tensor_handle(out, fmt)]
    try:
        st, ws, ex = get_workspace_size_grid_sampler3d(hs[0], hs[1], interpolation_mode, padding_mode,
                                                       align_corners, hs[2])
        if st != ACLNN_SUCCESS:
            raise AclnnError("aclnnGridSampler3DGetWorkspaceSize", st)
        if ws > 0 and (workspace is None or workspace.numel() * workspace.element_size() < ws):
            workspace = torch.empty(ws, dtype=torch.uint8, device=inp.device)
        wptr = ctypes.c_void_p(workspace.data_ptr()) if ws > 0 else None
        wsize = workspace.numel() * workspace.element_size() if ws > 0 else 0
        st = L.aclnnGridSampler3D(wptr, wsize, ex, _stream_handle(stream))
        if st != ACLNN_SUCCESS:
            raise AclnnError("aclnnGridSampler3D", st)
    finally:
        for h in hs:
            destroy_tensor(h)
    return out


def upsample_bilinear2d(self_t, output_size, align_corners=False, scales_h=0.0, scales_w=0.0, out=None, stream=None,
                        channels_last=False, workspace=None):
    """Both phases of aclnnUpsampleBilinear2d; tensors are NCHW views, or NHWC views when channels_last."""
    torch = _torch()
    L = load_library()
    fmt = ACL_FORMAT_NHWC if channels_last else ACL_FORMAT_NCHW
    if out is None:
        if channels_last:
            shape = (self_t.shape[0], output_size[0], output_size[1], self_t.shape[3])
        else:
            shape = (self_t.shape[0], self_t.shape[1], output_size[0], output_size[1])
        out = torch.empty(shape, dtype=self_t.dtype, device=self_t.device)
    hs = [tensor_handle(self_t, fmt), tensor_handle(out, fmt)]
    size = create_int_array(list(output_size))
    try:
        st, ws, ex = get_workspace_size_upsample_bilinear2d(hs[0], size, align_corners, scales_h, scales_w, hs[1])
        if st != ACLNN_SUCCESS:
            raise AclnnError("aclnnUpsampleBilinear2dGetWorkspaceSize", st)
        if ws > 0 and (workspace is None or workspace.numel() * workspace.element_size() < ws):
            workspace = torch.empty(ws, dtype=torch.uint8, device=self_t.device)
        wptr = ctypes.c_void_p(workspace.data_ptr()) if ws > 0 else None
        wsize = workspace.numel() * workspace.element_size() if ws > 0 else 0
        st = L.aclnnUpsampleBilinear2d(wptr, wsize, ex, _stream_handle(stream))
        if st != ACLNN_SUCCESS:
            raise AclnnError("aclnnUpsampleBilinear2d", st)
    finally:
        for h in hs:
            destroy_tensor(h)
        destroy_int_array(size)
    return out


def resize(self_t, scales, mode="bilinear", out=None, stream=None, channels_last=False, workspace=None):
    """Both phases of aclnnResize.  `scales` holds four floats in the order of the tensor's dimensions; the output
    extents are trunc(in * scale).  Tensors are NCHW views, or NHWC views when channels_last."""
    torch = _torch()
    L = load_library()
    fmt = ACL_FORMAT_NHWC if channels_last else ACL_FORMAT_NCHW
    if out is None:
        shape = list(self_t.shape)
        for d in ((1, 2) if channels_last else (2, 3)):
            shape[d] = int(float(self_t.shape[d]) * float(scales[d]))
        out = torch.empty(shape, dtype=self_t.dtype, device=self_t.device)
    hs = [tensor_handle(self_t, fmt), tensor_handle(out, fmt)]
    sc = create_float_array(list(scales))
    try:
        st, ws, ex = get_workspace_size_resize(hs[0], sc, mode.encode(), hs[1])
        if st != ACLNN_SUCCESS:
            raise AclnnError("aclnnResizeGetWorkspaceSize", st)
        if ws > 0 and (workspace is None or workspace.numel() * workspace.element_size() < ws):
            workspace = torch.empty(ws, dtype=torch.uint8, device=self_t.device)
        wptr = ctypes.c_void_p(workspace.data_ptr()) if ws > 0 else None
        wsize = workspace.numel() * workspace.element_size() if ws > 0 else 0
        st = L.aclnnResize(wptr, wsize, ex, _stream_handle(stream))
        if st != ACLNN_SUCCESS:
            raise AclnnError("aclnnResize", st)
    finally:
        for h in hs:
            destroy_tensor(h)
        destroy_float_array(sc)
    return out


def upsample_bilinear2d_backward(grad_out, input_size, align_corners=False, scales_h=0.0, scales_w=0.0, out=None,
                                 stream=None, channels_last=False, out_dtype=None, workspace=None):
    """Both phases of aclnnUpsampleBilinear2dBackward.  `input_size` holds the four extents of the tensor that was
    upsampled, in the order of the tensors' layout (NCHW, or NHWC when channels_last)."""
    torch = _torch()
    L = load_library()
    fmt = ACL_FORMAT_NHWC if channels_last else ACL_FORMAT_NCHW
    if out is None:
        out = torch.empty(tuple(input_size), dtype=grad_out.dtype if out_dtype is None else out_dtype,
                          device=grad_out.device)
    hw = (1, 2) if channels_last else (2, 3)
    hs = [tensor_handle(grad_out, fmt), tensor_handle(out, fmt)]
    osz = create_int_array([grad_out.shape[hw[0]], grad_out.shape[hw[1]]])
    isz = create_int_array(list(input_size))
    try:
        st, ws, ex = get_workspace_size_upsample_bilinear2d_backward(hs[0], osz, isz, align_corners, scales_h,
                                                                     scales_w, hs[1])
        if st != ACLNN_SUCCESS:
            raise AclnnError("aclnnUpsampleBilinear2dBackwardGetWorkspaceSize", st)
        if ws > 0 and (workspace is None or workspace.numel() * workspace.element_size() < ws):
            workspace = torch.empty(ws, dtype=torch.uint8, device=grad_out.device)
        wptr = ctypes.c_void_p(workspace.data_ptr()) if ws > 0 else None
        wsize = workspace.numel() * workspace.element_size() if ws > 0 else 0
        st = L.aclnnUpsampleBilinear2dBackward(wptr, wsize, ex, _stream_handle(stream))
        if st != ACLNN_SUCCESS:
            raise AclnnError("aclnnUpsampleBilinear2dBackward", st)
    finally:
        for h in hs:
            destroy_tensor(h)
        destroy_int_array(osz)
        destroy_int_array(isz)
    return out


def grid_sampler2d_taps(grid, h_in, w_in, interpolation_mode=0, padding_mode=0, align_corners=False, stream=None):
    """Per-pixel tap records (numpy structured array) computed on the device by the kernels' coordinate stage."""
    import numpy as np
    torch = _torch()
    L = load_library()
    grid = grid.contiguous()
    n, ho, wo, _ = grid.shape
    raw = torch.empty((n * ho * wo, ctypes.sizeof(TapRecord)), dtype=torch.uint8, device=grid.device)
    st = L.opscvGridSampler2DTaps(ctypes.c_void_p(grid.data_ptr()), acl_dtype_of(grid), n, h_in, w_in, ho, wo,
                                  interpolation_mode, padding_mode, bool(align_corners),
                                  ctypes.c_void_p(raw.data_ptr()), _stream_handle(stream))
    if st != ACLNN_SUCCESS:
        raise AclnnError("opscvGridSampler2DTaps", st)
    torch.cuda.synchronize()
    dt = np.dtype([("ix0", "<i4"), ("iy0", "<i4"), ("w", "<f4", (4,)), ("flag", "<i4")])
    return raw.cpu().numpy().view(dt).reshape(n, ho, wo)


def grid_sampler2d_bicubic_taps(grid, h_in, w_in, padding_mode=0, align_corners=False, stream=None):
    """Per-pixel records of the bicubic mode: tap columns/rows after padding, coefficients, NaN flag."""
    import numpy as np
    torch = _torch()
    L = load_library()
    grid = grid.contiguous()
    n, ho, wo, _ = grid.shape
    dt = np.dtype([("bx", "<i4", (4,)), ("by", "<i4", (4,)), ("cx", "<f4", (4,)), ("cy", "<f4", (4,)),
                   ("flag", "<i4")])
    raw = torch.empty((n * ho * wo, dt.itemsize), dtype=torch.uint8, device=grid.device)
    st = L.opscvGridSampler2DBicubicTaps(ctypes.c_void_p(grid.data_ptr()), acl_dtype_of(grid), n, h_in, w_in, ho, wo,
                                         padding_mode, bool(align_corners), ctypes.c_void_p(raw.data_ptr()),
                                         _stream_handle(stream))
    if st != ACLNN_SUCCESS:
        raise AclnnError("opscvGridSampler2DBicubicTaps", st)
    torch.cuda.synchronize()
    return raw.cpu().numpy().view(dt).reshape(n, ho, wo)
