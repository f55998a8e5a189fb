"""ctypes view of the CPU oracle (oracle/libcv_oracle.so).

Test infrastructure: imported by tests/, the smoke entry and the benchmark's cpu_baseline leg only.
The shipped package never imports this module.
"""
import ctypes
import os
import subprocess

import numpy as np

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_ORACLE_DIR = os.path.join(_ROOT, "oracle")
_LIB_PATH = os.path.join(_ORACLE_DIR, "libcv_oracle.so")

F32, F16, BF16 = 0, 1, 2


class GsTap(ctypes.Structure):
    _fields_ = [("ix0", ctypes.c_int32), ("iy0", ctypes.c_int32), ("w", ctypes.c_float * 4),
                ("flag", ctypes.c_int32)]


TAP_DTYPE = np.dtype([("ix0", "<i4"), ("iy0", "<i4"), ("w", "<f4", (4,)), ("flag", "<i4")])
BICUBIC_TAP_DTYPE = np.dtype([("bx", "<i4", (4,)), ("by", "<i4", (4,)), ("cx", "<f4", (4,)), ("cy", "<f4", (4,)),
                              ("flag", "<i4")])


def build(force=False):
    """Compile the oracle with gcc when the shared object is missing (or when forced)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _ORACLE_DIR, "-B" if force else "-s", "libcv_oracle.so"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    build()
    L = ctypes.CDLL(_LIB_PATH)
    i64, i32, f32, vp = ctypes.c_int64, ctypes.c_int32, ctypes.c_float, ctypes.c_void_p
    L.oracle_half_to_float.restype = f32
    L.oracle_half_to_float.argtypes = [ctypes.c_uint16]
    L.oracle_float_to_half.restype = ctypes.c_uint16
    L.oracle_float_to_half.argtypes = [f32]
    L.oracle_bf16_to_float.restype = f32
    L.oracle_bf16_to_float.argtypes = [ctypes.c_uint16]
    L.oracle_float_to_bf16.restype = ctypes.c_uint16
    L.oracle_float_to_bf16.argtypes = [f32]
    L.oracle_unnormalize.restype = f32
    L.oracle_unnormalize.argtypes = [f32, i32, i32]
    L.oracle_clip_coordinates.restype = f32
    L.oracle_clip_coordinates.argtypes = [f32, i32]
    L.oracle_reflect_coordinates.restype = f32
    L.oracle_reflect_coordinates.argtypes = [f32, f32, f32]
    L.oracle_compute_source_index.restype = f32
    L.oracle_compute_source_index.argtypes = [f32, i32, i32, i32]
    L.oracle_safe_downgrade.restype = f32
    L.oracle_safe_downgrade.argtypes = [f32]
    L.oracle_banker_round.restype = i32
    L.oracle_banker_round.argtypes = [f32]
    L.oracle_grid_sampler2d.restype = ctypes.c_int
    L.oracle_grid_sampler2d.argtypes = [vp, vp, vp, ctypes.c_int, i64, i64, i64, i64, i64, i64, ctypes.c_int,
                                        ctypes.c_int, ctypes.c_int, ctypes.c_int]
    L.oracle_grid_sampler2d_taps.restype = ctypes.c_int
    L.oracle_grid_sampler2d_taps.argtypes = [vp, vp, ctypes.c_int, i64, i64, i64, i64, i64, ctypes.c_int,
                                             ctypes.c_int, ctypes.c_int]
    L.oracle_compute_coordinates.restype = f32
    L.oracle_compute_coordinates.argtypes = [f32, i32, i32, i32]
    L.oracle_cubic_convolution1.restype = f32
    L.oracle_cubic_convolution1.argtypes = [f32, f32]
    L.oracle_cubic_convolution2.restype = f32
    L.oracle_cubic_convolution2.argtypes = [f32, f32]
    L.oracle_grid_sampler2d_bicubic_taps.restype = ctypes.c_int
    L.oracle_grid_sampler2d_bicubic_taps.argtypes = [vp, vp, ctypes.c_int, i64, i64, i64, i64, i64, ctypes.c_int,
                                                     ctypes.c_int]
    L.oracle_resize_nearest.restype = ctypes.c_int
    L.oracle_resize_nearest.argtypes = [vp, vp, ctypes.c_int, i64, i64, i64, i64, i64, i64, ctypes.c_int]
    L.oracle_upsample_bilinear2d_backward.restype = ctypes.c_int
    L.oracle_upsample_bilinear2d_backward.argtypes = [vp, vp, ctypes.c_int, ctypes.c_int, i64, i64, i64, i64, i64,
                                                      i64, ctypes.c_int, ctypes.c_int, ctypes.c_double, ctypes.c_double]
    L.oracle_resize_scale.restype = f32
    L.oracle_resize_scale.argtypes = [i64, i64, ctypes.c_int, f32]
    L.oracle_upsample_bilinear2d.restype = ctypes.c_int
    L.oracle_upsample_bilinear2d.argtypes = [vp, vp, ctypes.c_int, i64, i64, i64, i64, i64, i64, ctypes.c_int,
                                             ctypes.c_double, ctypes.c_double, ctypes.c_int]
    L.oracle_upsample_axis_taps.restype = ctypes.c_int
    L.oracle_upsample_axis_taps.argtypes = [i64, i64, ctypes.c_int, f32, vp, vp, vp]
    L.oracle_grid_sampler3d.restype = ctypes.c_int
    L.oracle_grid_sampler3d.argtypes = [vp, vp, vp, ctypes.c_int] + [i64] * 8 + [ctypes.c_int] * 4
    L.oracle_gs3d_unnormalize.restype = f32
    L.oracle_gs3d_unnormalize.argtypes = [f32, ctypes.c_int32, ctypes.c_int32]
    L.oracle_gs3d_clip.restype = f32
    L.oracle_gs3d_clip.argtypes = [f32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32]
    L.oracle_grid_sampler2d_backward.restype = ctypes.c_int
    L.oracle_grid_sampler2d_backward.argtypes = [vp] * 5 + [ctypes.c_int] + [i64] * 6 + [ctypes.c_int] * 3
    L.oracle_grid_sampler3d_backward.restype = ctypes.c_int
    L.oracle_grid_sampler3d_backward.argtypes = [vp] * 5 + [ctypes.c_int] + [i64] * 8 + [ctypes.c_int] * 3
    L.oracle_set_reference_cores.restype = None
    L.oracle_set_reference_cores.argtypes = [i64]
    L.oracle_set_reference_ub_bytes.restype = None
    L.oracle_set_reference_ub_bytes.argtypes = [i64]
    L.oracle_nearest_nhwc_schedule.restype = ctypes.c_int
    L.oracle_nearest_nhwc_schedule.argtypes = [ctypes.c_int, i64, i64, i64, i64, i64, i64]
    L.oracle_resize_uses_hw_split.restype = ctypes.c_int
    L.oracle_resize_uses_hw_split.argtypes = [i64] * 6
    L.oracle_upsample_bilinear2d_nhwc.restype = ctypes.c_int
    L.oracle_upsample_bilinear2d_nhwc.argtypes = [vp, vp, ctypes.c_int] + [i64] * 6 + [ctypes.c_int, ctypes.c_double,
                                                                                         ctypes.c_double]
    L.oracle_resize_point_copy.restype = ctypes.c_int
    L.oracle_resize_point_copy.argtypes = [vp, vp, ctypes.c_int] + [i64] * 6 + [ctypes.c_int, ctypes.c_double,
                                                                            ctypes.c_double]
    L.oracle_max_threads.restype = ctypes.c_int
    L.oracle_max_threads.argtypes = []
    L.oracle_grid_sampler2d_arch35.restype = ctypes.c_int
    L.oracle_grid_sampler2d_arch35.argtypes = [vp, vp, vp, ctypes.c_int] + [i64] * 6 + [ctypes.c_int, ctypes.c_int]
    L.oracle_upsample_a2_axis_taps.restype = ctypes.c_int
    L.oracle_upsample_a2_axis_taps.argtypes = [i64, i64, ctypes.c_int, ctypes.c_float, vp, vp, vp, vp]
    L.oracle_upsample_bilinear2d_a2.restype = ctypes.c_int
    L.oracle_upsample_bilinear2d_a2.argtypes = [vp, vp] + [i64] * 6 + [ctypes.c_int]
    _lib = L
    return L


def _code_of(arr):
    """Element code for a numpy array: float32 -> F32, float16 -> F16; uint16 needs an explicit code."""
    if arr.dtype == np.float32:
        return F32
    if arr.dtype == np.float16:
        return F16
    raise TypeError("pass dtype= explicitly for %s arrays (bf16 travels as uint16)" % arr.dtype)


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def grid_sampler2d(x, grid, interp=0, pad=0, align=False, dtype=None, threads=0):
    """x (N,C,H,W), grid (N,Ho,Wo,2) -> y (N,C,Ho,Wo); arrays are float32, float16, or uint16 holding bf16 bits."""
    x = np.ascontiguousarray(x)
    grid = np.ascontiguousarray(grid)
    code = _code_of(x) if dtype is None else dtype
    N, C, H, W = x.shape
    _, Ho, Wo, two = grid.shape
    assert two == 2 and grid.shape[0] == N and grid.dtype == x.dtype
    y = np.empty((N, C, Ho, Wo), dtype=x.dtype)
    rc = lib().oracle_grid_sampler2d(_ptr(x), _ptr(grid), _ptr(y), code, N, C, H, W, Ho, Wo, interp, pad,
                                     int(bool(align)), threads)
    if rc != 0:
        raise ValueError("oracle_grid_sampler2d rc=%d" % rc)
    return y


def grid_sampler2d_taps(grid, H, W, interp=0, pad=0, align=False, dtype=None):
    grid = np.ascontiguousarray(grid)
    code = _code_of(grid) if dtype is None else dtype
    N, Ho, Wo, _ = grid.shape
    taps = np.zeros((N, Ho, Wo), dtype=TAP_DTYPE)
    rc = lib().oracle_grid_sampler2d_taps(_ptr(grid), _ptr(taps), code, N, H, W, Ho, Wo, interp, pad,
                                          int(bool(align)))
    if rc != 0:
        raise ValueError("oracle_grid_sampler2d_taps rc=%d" % rc)
    return taps


def grid_sampler2d_bicubic_taps(grid, H, W, pad=0, align=False, dtype=None):
    grid = np.ascontiguousarray(grid)
    code = _code_of(grid) if dtype is None else dtype
    N, Ho, Wo, _ = grid.shape
    taps = np.zeros((N, Ho, Wo), dtype=BICUBIC_TAP_DTYPE)
    rc = lib().oracle_grid_sampler2d_bicubic_taps(_ptr(grid), _ptr(taps), code, N, H, W, Ho, Wo, pad,
                                                  int(bool(align)))
    if rc != 0:
        raise ValueError("oracle_grid_sampler2d_bicubic_taps rc=%d" % rc)
    return taps


def resize_nearest(x, out_hw, channels_last=False, dtype=None):
    """x (N,C,H,W) or, with channels_last, (N,H,W,C) -> the same layout at out_hw"""
    x = np.ascontiguousarray(x)
    code = _code_of(x) if dtype is None else dtype
    if channels_last:
        N, Hs, Ws, C = x.shape
        y = np.empty((N, out_hw[0], out_hw[1], C), dtype=x.dtype)
    else:
        N, C, Hs, Ws = x.shape
        y = np.empty((N, C, out_hw[0], out_hw[1]), dtype=x.dtype)
    rc = lib().oracle_resize_nearest(_ptr(x), _ptr(y), code, N, C, Hs, Ws, out_hw[0], out_hw[1], int(channels_last))
    if rc != 0:
        raise ValueError("oracle_resize_nearest rc=%d" % rc)
    return y


def upsample_bilinear2d_backward(grads, in_hw, align=False, channels_last=False, dtype=None, out_dtype=None,
                                 out_numpy_dtype=None, scales_h=0.0, scales_w=0.0):
    """grads (N,C,Hd,Wd) or channels_last (N,Hd,Wd,C) -> gradient of the (.., in_hw) tensor that was upsampled"""
    grads = np.ascontiguousarray(grads)
    code = _code_of(grads) if dtype is None else dtype
    ocode = code if out_dtype is None else out_dtype
    if channels_last:
        N, Hd, Wd, C = grads.shape
        shape = (N, in_hw[0], in_hw[1], C)
    else:
        N, C, Hd, Wd = grads.shape
        shape = (N, C, in_hw[0], in_hw[1])
    y = np.empty(shape, dtype=grads.dtype if out_numpy_dtype is None else out_numpy_dtype)
    rc = lib().oracle_upsample_bilinear2d_backward(_ptr(grads), _ptr(y), code, ocode, N, C, in_hw[0], in_hw[1], Hd, Wd,
                                                   int(bool(align)), int(channels_last), float(scales_h),
                                                   float(scales_w))
    if rc != 0:
        raise ValueError("oracle_upsample_bilinear2d_backward rc=%d" % rc)
    return y


def resize_point_copy(x_nhwc, out_hw, align=False, scales_h=0.0, scales_w=0.0, dtype=None):
    """x (N,H,W,C) -> y (N,Ho,Wo,C) when the reference's point-copy template applies, else None"""
    x = np.ascontiguousarray(x_nhwc)
    code = _code_of(x) if dtype is None else dtype
    N, Hs, Ws, C = x.shape
    y = np.empty((N, out_hw[0], out_hw[1], C), dtype=x.dtype)
    rc = lib().oracle_resize_point_copy(_ptr(x), _ptr(y), code, N, C, Hs, Ws, out_hw[0], out_hw[1], int(bool(align)),
                                        float(scales_h), float(scales_w))
    return y if rc == 1 else None


def grid_sampler2d_backward(gout, x, grid, interp=0, pad=0, align=False, dtype=None, want=(True, True)):
    """gout (N,C,Ho,Wo), x (N,C,H,W), grid (N,Ho,Wo,2) -> (dx or None, dgrid or None)"""
    gout, x, grid = (np.ascontiguousarray(a) for a in (gout, x, grid))
    code = _code_of(x) if dtype is None else dtype
    N, C, H, W = x.shape
    _, Ho, Wo, _ = grid.shape
    assert gout.shape == (N, C, Ho, Wo)
    dx = np.empty_like(x) if want[0] else None
    dg = np.empty_like(grid) if want[1] else None
    rc = lib().oracle_grid_sampler2d_backward(_ptr(gout), _ptr(x), _ptr(grid), _ptr(dx) if want[0] else None,
                                              _ptr(dg) if want[1] else None, code, N, C, H, W, Ho, Wo, interp, pad,
                                              int(bool(align)))
    if rc != 0:
        raise ValueError("oracle_grid_sampler2d_backward rc=%d" % rc)
    return dx, dg


def grid_sampler3d_backward(gout, x, grid, interp=0, pad=0, align=False, dtype=None, want=(True, True)):
    """gout (N,C,Do,Ho,Wo), x (N,C,D,H,W), grid (N,Do,Ho,Wo,3) -> (dx or None, dgrid or None)"""
    gout, x, grid = (np.ascontiguousarray(a) for a in (gout, x, grid))
    code = _code_of(x) if dtype is None else dtype
    N, C, D, H, W = x.shape
    _, Do, Ho, Wo, _ = grid.shape
    assert gout.shape == (N, C, Do, Ho, Wo)
    dx = np.empty_like(x) if want[0] else None
    dg = np.empty_like(grid) if want[1] else None
    rc = lib().oracle_grid_sampler3d_backward(_ptr(gout), _ptr(x), _ptr(grid), _ptr(dx) if want[0] else None,
                                              _ptr(dg) if want[1] else None, code, N, C, D, H, W, Do, Ho, Wo, interp,
                                              pad, int(bool(align)))
    if rc != 0:
        raise ValueError("oracle_grid_sampler3d_backward rc=%d" % rc)
    return dx, dg


def grid_sampler3d(x, grid, interp=0, pad=0, align=False, dtype=None, threads=0):
    """x (N,C,D,H,W), grid (N,Do,Ho,Wo,3) -> y (N,C,Do,Ho,Wo); float32, float16, or uint16 holding bf16 bits."""
    x = np.ascontiguousarray(x)
    grid = np.ascontiguousarray(grid)
    code = _code_of(x) if dtype is None else dtype
    N, C, D, H, W = x.shape
    _, Do, Ho, Wo, three = grid.shape
    assert three == 3 and grid.shape[0] == N and grid.dtype == x.dtype
    y = np.empty((N, C, Do, Ho, Wo), dtype=x.dtype)
    rc = lib().oracle_grid_sampler3d(_ptr(x), _ptr(grid), _ptr(y), code, N, C, D, H, W, Do, Ho, Wo, interp, pad,
                                     int(bool(align)), threads)
    if rc != 0:
        raise ValueError("oracle_grid_sampler3d rc=%d" % rc)
    return y


def upsample_bilinear2d(x, out_hw, align=False, scales_h=0.0, scales_w=0.0, dtype=None, threads=0):
    x = np.ascontiguousarray(x)
    code = _code_of(x) if dtype is None else dtype
    N, C, Hs, Ws = x.shape
    Hd, Wd = out_hw
    y = np.empty((N, C, Hd, Wd), dtype=x.dtype)
    rc = lib().oracle_upsample_bilinear2d(_ptr(x), _ptr(y), code, N, C, Hs, Ws, Hd, Wd, int(bool(align)),
                                          float(scales_h), float(scales_w), threads)
    if rc != 0:
        raise ValueError("oracle_upsample_bilinear2d rc=%d" % rc)
    return y


def grid_sampler2d_arch35(x, grid, pad=0, align=False, dtype=None):
    """bilinear 2-D sampling by the rule of the reference's GridSample operator on its newest part (what the library
    computes under option grid_sampler2d_rule = 1)"""
    x = np.ascontiguousarray(x)
    grid = np.ascontiguousarray(grid)
    code = _code_of(x) if dtype is None else dtype
    N, C, H, W = x.shape
    _, Ho, Wo, _ = grid.shape
    y = np.empty((N, C, Ho, Wo), dtype=x.dtype)
    rc = lib().oracle_grid_sampler2d_arch35(_ptr(x), _ptr(grid), _ptr(y), code, N, C, H, W, Ho, Wo, pad,
                                            int(bool(align)))
    if rc != 0:
        raise ValueError("oracle_grid_sampler2d_arch35 rc=%d" % rc)
    return y


def upsample_a2_axis_taps(len_src, len_dst, align=False, scale=0.0):
    """(i0, i1, l0, l1) of the reference's matmul upsample kernel for one axis"""
    i0 = np.zeros(len_dst, dtype=np.int32)
    i1 = np.zeros(len_dst, dtype=np.int32)
    l0 = np.zeros(len_dst, dtype=np.float32)
    l1 = np.zeros(len_dst, dtype=np.float32)
    lib().oracle_upsample_a2_axis_taps(len_src, len_dst, int(bool(align)), float(scale), _ptr(i0), _ptr(i1), _ptr(l0),
                                       _ptr(l1))
    return i0, i1, l0, l1


def upsample_bilinear2d_a2(x, out_hw, align=False):
    x = np.ascontiguousarray(x, dtype=np.float32)
    N, C, Hs, Ws = x.shape
    y = np.empty((N, C, out_hw[0], out_hw[1]), dtype=np.float32)
    rc = lib().oracle_upsample_bilinear2d_a2(_ptr(x), _ptr(y), N, C, Hs, Ws, out_hw[0], out_hw[1], int(bool(align)))
    if rc != 0:
        raise ValueError("oracle_upsample_bilinear2d_a2 rc=%d" % rc)
    return y


def set_reference_cores(cores):
    """vector cores of the device the reference would run on (its NCHW template choice depends on it); 0 -> default"""
    lib().oracle_set_reference_cores(int(cores))


def set_reference_ub_bytes(n):
    """unified-buffer bytes of the device the reference would run on (gates its replicating nearest template); 0 -> default"""
    lib().oracle_set_reference_ub_bytes(int(n))


def nearest_nhwc_schedule(dtype_code, N, C, Hs, Ws, Hd, Wd):
    """schedule id the reference's tiling picks for a channels-last nearest resize (6-8: the replicating template)"""
    return int(lib().oracle_nearest_nhwc_schedule(dtype_code, N, C, Hs, Ws, Hd, Wd))


def resize_uses_hw_split(N, C, Hs, Ws, Hd, Wd):
    return bool(lib().oracle_resize_uses_hw_split(N, C, Hs, Ws, Hd, Wd))


NHWC_TEMPLATES = ("per_element", "copy", "broadcast", "first_pixel", "point_copy", "channel_parallel")


def upsample_bilinear2d_nhwc(x_nhwc, out_hw, align=False, scales_h=0.0, scales_w=0.0, dtype=None, with_template=False):
    """x (N,H,W,C) -> y (N,Ho,Wo,C) with the reference's template choice for channels-last tensors"""
    x = np.ascontiguousarray(x_nhwc)
    code = _code_of(x) if dtype is None else dtype
    N, Hs, Ws, C = x.shape
    y = np.empty((N, out_hw[0], out_hw[1], C), dtype=x.dtype)
    rc = lib().oracle_upsample_bilinear2d_nhwc(_ptr(x), _ptr(y), code, N, C, Hs, Ws, out_hw[0], out_hw[1],
                                               int(bool(align)), float(scales_h), float(scales_w))
    if rc < 0:
        raise ValueError("oracle_upsample_bilinear2d_nhwc rc=%d" % rc)
    return (y, NHWC_TEMPLATES[rc]) if with_template else y


def upsample_axis_taps(len_src, len_dst, align=False, user_scale=0.0):
    i0 = np.zeros(len_dst, dtype=np.int32)
    i1 = np.zeros(len_dst, dtype=np.int32)
    lam = np.zeros(len_dst, dtype=np.float32)
    lib().oracle_upsample_axis_taps(len_src, len_dst, int(bool(align)), float(user_scale), _ptr(i0), _ptr(i1),
                                    _ptr(lam))
    return i0, i1, lam


def f32_to_bf16_bits(a):
    """Round-to-nearest-even float32 -> bf16 bit patterns (uint16), NaN kept quiet."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    u = a.view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + (0x7FFF + ((u >> 16) & 1))) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def bf16_bits_to_f32(b):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32)
