"""The C-ABI boundary without a GPU: exported symbols, phase-1 validation order and status codes.

The cases mirror the reference's op_api unit tests, which build descriptors with NULL data pointers and call only
the GetWorkspaceSize phase: image/grid_sample/tests/ut/op_host/op_api/test_aclnn_grid_sampler2d.cpp and
image/upsample_bilinear2d/tests/ut/op_host/op_api/test_aclnn_upsample_bilinear_2d.cpp,
image/resize_bilinear_v2/tests/ut/op_host/op_api/test_aclnn_resize.cpp,
image/resize_bilinear_v2_grad/tests/ut/op_host/op_api/test_aclnn_upsample_bilineard_2d_backward.cpp,
image/grid_sample/tests/ut/op_host/op_api/test_aclnn_grid_sampler3d.cpp,
image/grid_sampler2_d_grad/tests/ut/op_host/op_api/test_aclnn_grid_sampler2d_backward.cpp.
"""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol(aclnn):
    L = aclnn.load_library()
    declared = set()
    for name in os.listdir(os.path.join(ROOT, "include")):
        text = open(os.path.join(ROOT, "include", name)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        declared |= set(re.findall(r"ACLNN_API\s+[\w\s\*]+?\b(\w+)\s*\(", text))
    assert {"aclnnGridSampler2DGetWorkspaceSize", "aclnnGridSampler2D", "aclnnUpsampleBilinear2dGetWorkspaceSize",
            "aclnnUpsampleBilinear2d", "aclCreateTensor", "aclGetRecentErrMsg"} <= declared
    for sym in sorted(declared):
        assert hasattr(L, sym), "libopscv_amd.so does not export %s" % sym
    assert b"gfx950" in L.opscvVersion()


class Desc:
    """Descriptor builder in the spirit of the reference's TensorDesc (NULL data pointer)."""

    def __init__(self, aclnn):
        self.a = aclnn
        self.handles = []

    def t(self, dims, dtype, fmt=None, strides=None, offset=0, storage=None):
        if dims is None:
            return None
        fmt = self.a.ACL_FORMAT_ND if fmt is None else fmt
        h = self.a.create_tensor(dims, dtype, fmt, strides, offset, storage)
        assert h
        self.handles.append(h)
        return h

    def close(self):
        for h in self.handles:
            self.a.destroy_tensor(h)


@pytest.fixture
def desc(aclnn):
    d = Desc(aclnn)
    yield d
    d.close()


def _gs(aclnn, desc, inp=(1, 1, 5, 8), grid=(1, 3, 3, 2), out=(1, 1, 3, 3), dt=None, gdt=None, odt=None, interp=0, pad=0,
        align=False, fmts=(None, None, None), **kw):
    dt = aclnn.ACL_FLOAT if dt is None else dt
    i = desc.t(inp, dt, fmts[0], **kw)
    g = desc.t(grid, dt if gdt is None else gdt, fmts[1])
    o = desc.t(out, dt if odt is None else odt, fmts[2])
    st, ws, ex = aclnn.get_workspace_size_grid_sampler2d(i, g, interp, pad, align, o)
    if ex:
        assert aclnn.destroy_executor(ex) == 0
    return st, ws, bool(ex)


def test_grid_sampler_success_cases(aclnn, desc):
    for dt in (aclnn.ACL_FLOAT, aclnn.ACL_FLOAT16, aclnn.ACL_BF16):  # reference cases 1, 5, 6
        st, ws, ex = _gs(aclnn, desc, dt=dt)
        assert (st, ws, ex) == (0, 0, True)
    # formats are ignored (cases "nchw nhwc", "hwcn nchw", "nhwc nhwc" with nearest/border)
    assert _gs(aclnn, desc, fmts=(aclnn.ACL_FORMAT_NCHW, aclnn.ACL_FORMAT_NHWC, aclnn.ACL_FORMAT_ND))[0] == 0
    assert _gs(aclnn, desc, fmts=(aclnn.ACL_FORMAT_HWCN, aclnn.ACL_FORMAT_NCHW, aclnn.ACL_FORMAT_ND))[0] == 0
    assert _gs(aclnn, desc, interp=1, pad=1, fmts=(aclnn.ACL_FORMAT_NCHW, aclnn.ACL_FORMAT_NHWC, None))[0] == 0
    for interp in (0, 1, 2):
        for pad in (0, 1, 2):
            for align in (False, True):
                assert _gs(aclnn, desc, interp=interp, pad=pad, align=align)[0] == 0


def test_grid_sampler_null_pointers(aclnn, desc):
    assert _gs(aclnn, desc, inp=None)[0] == aclnn.ACLNN_ERR_PARAM_NULLPTR
    assert _gs(aclnn, desc, grid=None)[0] == aclnn.ACLNN_ERR_PARAM_NULLPTR
    assert _gs(aclnn, desc, out=None)[0] == aclnn.ACLNN_ERR_PARAM_NULLPTR
    L = aclnn.load_library()
    i, g, o = desc.t((1, 1, 5, 8), 0), desc.t((1, 3, 3, 2), 0), desc.t((1, 1, 3, 3), 0)
    ex = ctypes.c_void_p()
    assert L.aclnnGridSampler2DGetWorkspaceSize(i, g, 0, 0, False, o, None, ctypes.byref(ex)) == 161001
    assert b"NULL" in L.aclGetRecentErrMsg()


def test_grid_sampler_dtype_checks(aclnn, desc):
    bad = [aclnn.ACL_UINT8, aclnn.ACL_INT8, aclnn.ACL_INT16, aclnn.ACL_INT32, aclnn.ACL_INT64, aclnn.ACL_BOOL,
           aclnn.ACL_COMPLEX64, aclnn.ACL_COMPLEX128]
    for dt in bad:  # reference cases 8-15
        assert _gs(aclnn, desc, dt=dt)[0] == aclnn.ACLNN_ERR_PARAM_INVALID
    # mismatching dtypes (reference case "format not same": DOUBLE input with FLOAT grid/out)
    assert _gs(aclnn, desc, dt=aclnn.ACL_DOUBLE, gdt=aclnn.ACL_FLOAT, odt=aclnn.ACL_FLOAT)[0] == 161002
    assert _gs(aclnn, desc, odt=aclnn.ACL_FLOAT16)[0] == 161002
    # DOUBLE passes the reference's checks but has no kernel here: documented gap, same status class
    assert _gs(aclnn, desc, dt=aclnn.ACL_DOUBLE)[0] == 161002


def test_grid_sampler_attr_and_shape_checks(aclnn, desc):
    assert _gs(aclnn, desc, interp=3)[0] == 161002
    assert _gs(aclnn, desc, interp=-1)[0] == 161002
    assert _gs(aclnn, desc, pad=3)[0] == 161002
    assert _gs(aclnn, desc, grid=(2, 3, 3, 2))[0] == 161002          # batch mismatch
    assert _gs(aclnn, desc, grid=(1, 3, 3, 3))[0] == 161002          # last grid dim must be 2
    assert _gs(aclnn, desc, inp=(1, 1, 0, 8))[0] == 161002           # empty spatial input
    assert _gs(aclnn, desc, inp=(1, 1, 5))[0] == 161002              # not 4-D
    assert _gs(aclnn, desc, out=(1, 2, 3, 3))[0] == 161002           # channel mismatch
    assert _gs(aclnn, desc, out=(1, 1, 3, 2))[0] == 161002           # grid/out W mismatch
    # validation order: dtype is reported before attributes and shapes, attributes before shapes
    L = aclnn.load_library()
    _gs(aclnn, desc, dt=aclnn.ACL_INT32, interp=7, grid=(2, 3, 3, 2))
    assert b"dtype" in L.aclGetRecentErrMsg()
    _gs(aclnn, desc, interp=7, grid=(2, 3, 3, 2))
    assert b"interpolationMode" in L.aclGetRecentErrMsg()
    # bicubic is the third supported mode
    assert _gs(aclnn, desc, interp=2)[0] == 0


def test_grid_sampler_empty_and_views(aclnn, desc):
    # empty batch / empty grid: success, no workspace, an executor is still handed out
    assert _gs(aclnn, desc, inp=(0, 1, 5, 8), grid=(0, 3, 3, 2), out=(0, 1, 3, 3)) == (0, 0, True)
    assert _gs(aclnn, desc, grid=(1, 0, 3, 2), out=(1, 1, 0, 3)) == (0, 0, True)
    # non-contiguous input view (reference case "not contiguous"): accepted, packed through the workspace
    st, ws, ex = _gs(aclnn, desc, strides=(40, 40, 1, 5), storage=(1, 1, 8, 5))
    assert st == 0 and ex and ws >= 40 * 4
    # contiguous with an offset needs no workspace
    st, ws, ex = _gs(aclnn, desc, offset=16, storage=(100,))
    assert (st, ws) == (0, 0)


def test_executor_lifecycle(aclnn, desc):
    L = aclnn.load_library()
    i, g, o = desc.t((0, 1, 5, 8), 0), desc.t((0, 3, 3, 2), 0), desc.t((0, 1, 3, 3), 0)
    st, ws, ex = aclnn.get_workspace_size_grid_sampler2d(i, g, 0, 0, False, o)
    assert st == 0 and ex
    # phase 2 on a no-op executor touches no device and consumes the executor
    assert L.aclnnGridSampler2D(None, 0, ex, None) == 0
    assert L.aclnnGridSampler2D(None, 0, None, None) == aclnn.ACLNN_ERR_PARAM_NULLPTR
    assert L.aclDestroyAclOpExecutor(None) == aclnn.ACLNN_ERR_PARAM_NULLPTR
    # an executor of one operator is refused by the other operator's phase 2 (and is consumed by the call)
    i2, g2, o2 = desc.t((1, 1, 5, 8), 0), desc.t((1, 3, 3, 2), 0), desc.t((1, 1, 3, 3), 0)
    st, ws, ex = aclnn.get_workspace_size_grid_sampler2d(i2, g2, 0, 0, False, o2)
    assert st == 0
    assert L.aclnnUpsampleBilinear2d(None, 0, ex, None) == aclnn.ACLNN_ERR_PARAM_INVALID
    # NULL data pointers are only rejected when something has to run
    st, ws, ex = aclnn.get_workspace_size_grid_sampler2d(i2, g2, 0, 0, False, o2)
    assert L.aclnnGridSampler2D(None, 0, ex, None) == aclnn.ACLNN_ERR_PARAM_NULLPTR
    # workspace smaller than requested
    v = desc.t((1, 1, 5, 8), 0, None, (40, 40, 1, 5), 0, (1, 1, 8, 5))
    st, ws, ex = aclnn.get_workspace_size_grid_sampler2d(v, g2, 0, 0, False, o2)
    assert st == 0 and ws > 0
    assert L.aclnnGridSampler2D(None, 0, ex, None) == aclnn.ACLNN_ERR_PARAM_NULLPTR
    st, ws, ex = aclnn.get_workspace_size_grid_sampler2d(v, g2, 0, 0, False, o2)
    buf = ctypes.create_string_buffer(8)
    assert L.aclnnGridSampler2D(buf, 8, ex, None) == aclnn.ACLNN_ERR_PARAM_INVALID


def _up(aclnn, desc, inp=(1, 1, 3, 3), out=(1, 1, 6, 6), size=(6, 6), dt=None, odt=None, fmt=None, ofmt=None, align=False,
        sh=2.0, sw=2.0):
    dt = aclnn.ACL_FLOAT if dt is None else dt
    fmt = aclnn.ACL_FORMAT_NCHW if fmt is None else fmt
    s = desc.t(inp, dt, fmt)
    o = desc.t(out, dt if odt is None else odt, fmt if ofmt is None else ofmt)
    arr = aclnn.create_int_array(list(size)) if size is not None else None
    st, ws, ex = aclnn.get_workspace_size_upsample_bilinear2d(s, arr, align, sh, sw, o)
    variant = aclnn.executor_variant(ex) if ex else None
    if ex:
        aclnn.destroy_executor(ex)
    aclnn.destroy_int_array(arr)
    return st, ws, variant


def test_upsample_status_codes(aclnn, desc):
    INV, INNER = aclnn.ACLNN_ERR_PARAM_INVALID, aclnn.ACLNN_ERR_INNER_NULLPTR
    # test_001: empty tensors but outputSize {2,2} != out H,W -> the size check comes before the empty check
    assert _up(aclnn, desc, inp=(1, 1, 0, 0), out=(1, 1, 0, 0), size=(2, 2))[0] == INV
    # test_002: same size
    st, ws, variant = _up(aclnn, desc, out=(1, 1, 3, 3), size=(3, 3), sh=1.0, sw=1.0)
    assert (st, ws, variant) == (0, 0, "copy")
    # nullptr self / out -> inner nullptr (this operator, unlike the grid sampler)
    assert _up(aclnn, desc, inp=None)[0] == INNER
    assert _up(aclnn, desc, out=None)[0] == INNER
    # dtype mismatch, unsupported dtype
    assert _up(aclnn, desc, odt=aclnn.ACL_FLOAT16)[0] == INV
    assert _up(aclnn, desc, dt=aclnn.ACL_INT32)[0] == INV
    # N/C checks (ncdim001..004)
    assert _up(aclnn, desc, out=(1, 1, 2, 2), size=(2, 2), dt=aclnn.ACL_FLOAT16, sh=1.0, sw=1.0)[0] == 0
    assert _up(aclnn, desc, inp=(1, 2, 3, 3), out=(1, 1, 2, 2), size=(2, 2), dt=aclnn.ACL_FLOAT16)[0] == INV
    assert _up(aclnn, desc, inp=(1, 1, 3, 3), out=(1, 1, 3, 3), size=(2, 2), fmt=aclnn.ACL_FORMAT_NHWC)[0] == INV
    assert _up(aclnn, desc, inp=(1, 1, 3, 4), out=(1, 1, 2, 3), size=(2, 2), fmt=aclnn.ACL_FORMAT_NHWC)[0] == INV
    # negative scales
    assert _up(aclnn, desc, sh=-2.0, sw=-2.0)[0] == INV
    assert _up(aclnn, desc, sh=1.0, sw=-2.0)[0] == INV
    # formats
    assert _up(aclnn, desc, ofmt=aclnn.ACL_FORMAT_NHWC)[0] == INV
    assert _up(aclnn, desc, fmt=aclnn.ACL_FORMAT_ND)[0] == INV
    assert _up(aclnn, desc, inp=(1, 3, 3), out=(1, 6, 6))[0] == INV
    assert _up(aclnn, desc, dt=aclnn.ACL_DOUBLE)[0] == INV  # DOUBLE only with NHWC in the reference
    # outputSize checks (Ascend910B2 cases 1001-1004)
    assert _up(aclnn, desc)[0] == 0
    assert _up(aclnn, desc, size=(0, 0))[0] == INV
    assert _up(aclnn, desc, size=None)[0] == INV
    assert _up(aclnn, desc, size=(6, 6, 6))[0] == INV
    # empty tensors with consistent sizes: success, nothing to run
    st, ws, variant = _up(aclnn, desc, inp=(0, 1, 3, 3), out=(0, 1, 6, 6))
    assert (st, ws, variant) == (0, 0, "")


def test_upsample_template_selection(aclnn, desc):
    """kernel-template choice for the shapes of the reference tiling UT (keys 40000 copy, 40002 broadcast, 3000x
    bilinear): image/resize_bilinear_v2/tests/ut/op_host/arch35/test_resize_bilinear_v2_tiling.cpp"""
    f16, f32 = aclnn.ACL_FLOAT16, aclnn.ACL_FLOAT
    # case12/13: 1x1 -> 11x21 is the broadcast template for both align_corners and half-pixel
    assert _up(aclnn, desc, inp=(1, 1, 1, 1), out=(1, 1, 11, 21), size=(11, 21), align=True, sh=0, sw=0)[2] == "broadcast"
    assert _up(aclnn, desc, inp=(1, 1, 1, 1), out=(1, 1, 11, 21), size=(11, 21), dt=f16, sh=0, sw=0)[2] == "broadcast"
    # below 128 output bytes per plane the half-pixel case stays on the bilinear template
    v = _up(aclnn, desc, inp=(1, 1, 1, 1), out=(1, 1, 4, 4), size=(4, 4), dt=f16, sh=0, sw=0)[2]
    assert v.startswith("nchw")
    assert _up(aclnn, desc, inp=(1, 1, 1, 1), out=(1, 1, 4, 4), size=(4, 4), dt=f16, align=True, sh=0, sw=0)[2] == "broadcast"
    # 1x1 destination with align_corners -> first pixel; case16: equal sizes -> copy
    assert _up(aclnn, desc, inp=(1, 1, 5, 5), out=(1, 1, 1, 1), size=(1, 1), align=True, sh=0, sw=0)[2] == "first_pixel"
    assert _up(aclnn, desc, inp=(3, 5, 11, 21), out=(3, 5, 11, 21), size=(11, 21), dt=aclnn.ACL_BF16, sh=0, sw=0)[2] == "copy"
    # case01/02/06: ordinary NCHW bilinear; NHWC has its own kernel
    assert _up(aclnn, desc, inp=(2, 256, 12, 12), out=(2, 256, 18, 18), size=(18, 18), dt=f32, sh=1.5, sw=1.5)[2].startswith("nchw")
    assert _up(aclnn, desc, inp=(2, 128, 128, 256), out=(2, 192, 192, 256), size=(192, 192), dt=f32,
               fmt=aclnn.ACL_FORMAT_NHWC, align=True)[2] == "nhwc_vec"
    assert _up(aclnn, desc, inp=(2, 12, 12, 5), out=(2, 18, 18, 5), size=(18, 18), dt=f32,
               fmt=aclnn.ACL_FORMAT_NHWC, align=True)[2] == "nhwc_band_lds"
    assert _up(aclnn, desc, inp=(2, 12, 12, 5), out=(2, 14, 14, 5), size=(14, 14), dt=f32,
               fmt=aclnn.ACL_FORMAT_NHWC, align=True)[2] == "nhwc_unit"


def test_upsample_template_selection_channels_last(aclnn, desc):
    """the channels-last cases of the reference tiling UT whose attributes this entry point can express
    (image/resize_bilinear_v2/tests/ut/op_host/arch35/test_resize_bilinear_v2_tiling.cpp case04, 05, 07, 09, 10, 11,
    15, 16): keys 30000/30002 per-element, 40001 point copy, 10000 channel-parallel (four weights), 40003 broadcast,
    40000 copy"""
    f16, f32, nhwc = aclnn.ACL_FLOAT16, aclnn.ACL_FLOAT, aclnn.ACL_FORMAT_NHWC

    def variant(inp, out, dt, align, sh=0.0, sw=0.0):
        st, ws, v = _up(aclnn, desc, inp=inp, out=out, size=out[1:3], dt=dt, fmt=nhwc, align=align, sh=sh, sw=sw)
        assert st == 0 and ws == 0
        return v

    assert variant((2, 128, 128, 256), (2, 192, 192, 256), f32, True, 1.5, 1.5) == "nhwc_vec"                 # case04
    assert variant((128, 14, 16, 256), (128, 5, 8, 256), f32, False, 3.0, 3.0) == "nhwc_vec"                  # case05
    assert variant((128, 14, 16, 256), (128, 5, 8, 256), f32, False) == "nhwc_four_weights"   # size ratios 2.8 and 2
    assert variant((1, 36, 15, 128), (1, 12, 5, 128), f32, False) == "point_copy"                             # case07
    assert variant((1, 36, 15, 128), (1, 12, 5, 128), f32, False, 0.2, 0.2) == "point_copy"                   # case09
    assert variant((190, 22, 79, 128), (190, 13, 43, 128), f16, False, 0.31269457412229545,
                   0.27077088627767687) == "nhwc_four_weights"                                                # case10
    assert variant((190, 22, 79, 128), (190, 13, 43, 128), f16, False) == "nhwc_vec"          # 22 / 13 is under two
    assert variant((1, 1, 1, 64), (1, 59, 32, 64), f32, True) == "broadcast"                                  # case11
    assert variant((12768, 128, 128, 256), (12768, 192, 192, 256), f32, True, 1.5, 1.5) == "nhwc_vec"         # case15
    assert variant((3, 11, 21, 5), (3, 11, 21, 5), aclnn.ACL_BF16, False) == "copy"                           # case16
    # runs under 128 bytes never take the four-weights template; a 1x1 source of such runs is interpolated with
    # half-pixel centres and broadcast with align_corners
    assert variant((1, 8, 8, 32), (1, 3, 3, 32), f32, False) == "nhwc_four_weights"
    assert variant((1, 8, 8, 32), (1, 3, 3, 32), f16, False) == "nhwc_vec"
    # pixels that are not whole 16-byte vectors: images that at least double in area are staged in LDS as rows of
    # W * C elements, the others move units of 12, 8, 6, 4 or 2 bytes
    assert variant((1, 1, 1, 14), (1, 13, 7, 14), f32, False) == "nhwc_band_lds"
    assert variant((1, 4, 4, 3), (1, 13, 7, 3), f16, False) == "nhwc_band_lds"
    assert variant((1, 9, 9, 14), (1, 10, 8, 14), f32, False) == "nhwc_unit"      # 56-byte pixels: 8-byte units
    assert variant((1, 9, 9, 7), (1, 10, 8, 7), f32, False) == "nhwc_unit"        # one element per unit
    assert variant((1, 9, 9, 3), (1, 10, 8, 3), f32, False) == "nhwc_unit"        # three-channel images: 12 bytes
    assert variant((1, 9, 9, 3), (1, 10, 8, 3), f16, False) == "nhwc_unit"        # ... and 6 bytes
    assert variant((1, 1, 1, 14), (1, 13, 7, 14), f32, True) == "broadcast"
    assert variant((1, 8, 8, 8), (1, 1, 1, 8), f32, True) == "first_pixel"
    assert variant((1, 8, 8, 32), (1, 1, 1, 32), f32, True) == "point_copy"
    assert variant((1, 8, 8, 32), (1, 1, 3, 32), f32, True) == "nhwc_four_weights"


def _rs(aclnn, desc, inp=(1, 1, 2, 2), out=(1, 1, 4, 4), scales=(1, 1, 2, 2), mode=b"nearest", dt=None, odt=None,
        fmt=None, ofmt=None):
    dt = aclnn.ACL_FLOAT if dt is None else dt
    fmt = aclnn.ACL_FORMAT_NCHW if fmt is None else fmt
    s = desc.t(inp, dt, fmt)
    o = desc.t(out, dt if odt is None else odt, fmt if ofmt is None else ofmt)
    arr = aclnn.create_float_array(list(scales)) if scales is not None else None
    st, ws, ex = aclnn.get_workspace_size_resize(s, arr, mode, o)
    variant = aclnn.executor_variant(ex) if ex else None
    if ex:
        aclnn.destroy_executor(ex)
    aclnn.destroy_float_array(arr)
    return st, ws, variant


def test_resize_status_codes(aclnn, desc):
    """test_aclnn_resize.cpp case_1 .. case_11 and the element checks of aclnn_resize.cpp:82-121"""
    INV, NULL = aclnn.ACLNN_ERR_PARAM_INVALID, aclnn.ACLNN_ERR_PARAM_NULLPTR
    for dt in (aclnn.ACL_FLOAT, aclnn.ACL_FLOAT16, aclnn.ACL_BF16):
        assert _rs(aclnn, desc, dt=dt, mode=b"nearest") == (0, 0, "nearest_nchw")          # case_1, case_2
        st, ws, variant = _rs(aclnn, desc, dt=dt, mode=b"bilinear")                        # case_3, case_4
        assert st == 0 and ws == 0 and variant.startswith("nchw")
    assert _rs(aclnn, desc, scales=(1, 1, 2))[0] == INV                                    # case_5
    assert _rs(aclnn, desc, inp=None)[0] == NULL                                           # case_6
    assert _rs(aclnn, desc, scales=None)[0] == NULL                                        # case_7
    assert _rs(aclnn, desc, out=None)[0] == NULL                                           # case_8
    assert _rs(aclnn, desc, mode=None)[0] == NULL
    assert _rs(aclnn, desc, mode=b"trilinear")[0] == INV                                   # case_9
    assert _rs(aclnn, desc, odt=aclnn.ACL_FLOAT16)[0] == INV                               # case_10
    assert _rs(aclnn, desc, out=(1, 2, 4, 4))[0] == INV                                    # case_11
    # the mode is matched by prefix
    assert _rs(aclnn, desc, mode=b"nearest-exact")[0] == 0
    assert _rs(aclnn, desc, mode=b"bilinear_v2")[0] == 0
    # unsupported dtype, unequal / unsupported formats
    assert _rs(aclnn, desc, dt=aclnn.ACL_DOUBLE)[0] == INV
    assert _rs(aclnn, desc, ofmt=aclnn.ACL_FORMAT_NHWC)[0] == INV
    assert _rs(aclnn, desc, fmt=aclnn.ACL_FORMAT_ND)[0] == INV
    # output extents must equal trunc(in * scale) within scale +- 1e-5
    assert _rs(aclnn, desc, out=(1, 1, 5, 4))[0] == INV
    assert _rs(aclnn, desc, out=(1, 1, 4, 2))[0] == INV
    # ... where the lower bound truncates 2 * (2 - 1e-5) = 3.99998 to 3, so 3 passes as it does in the reference
    assert _rs(aclnn, desc, out=(1, 1, 4, 3))[0] == 0
    assert _rs(aclnn, desc, inp=(1, 1, 3, 3), out=(1, 1, 4, 7), scales=(1, 1, 1.5, 2.5))[0] == 0
    # NHWC: dimensions and scales are read in N,H,W,C order
    st, ws, variant = _rs(aclnn, desc, inp=(1, 2, 2, 8), out=(1, 4, 4, 8), scales=(1, 2, 2, 1), fmt=aclnn.ACL_FORMAT_NHWC)
    assert (st, variant) == (0, "nearest_nhwc")
    assert _rs(aclnn, desc, inp=(1, 2, 2, 8), out=(1, 4, 4, 8), scales=(1, 1, 2, 2), fmt=aclnn.ACL_FORMAT_NHWC)[0] == INV
    # rank
    assert _rs(aclnn, desc, inp=(1, 2, 2), out=(1, 4, 4), scales=(1, 2, 2, 1))[0] == INV
    # same size -> copy; 1x1 source -> broadcast; empty -> no-op
    assert _rs(aclnn, desc, out=(1, 1, 2, 2), scales=(1, 1, 1, 1))[2] == "copy"
    assert _rs(aclnn, desc, inp=(1, 1, 1, 1), out=(1, 1, 4, 4), scales=(1, 1, 4, 4))[2] == "broadcast"
    assert _rs(aclnn, desc, inp=(0, 1, 2, 2), out=(0, 1, 4, 4))[:2] == (0, 0)


def _ub(aclnn, desc, grad=(1, 1, 2, 2), out=(1, 1, 3, 3), osize=(2, 2), isize=(1, 1, 3, 3), dt=None, odt=None, fmt=None,
        ofmt=None, align=False, sh=2.0, sw=2.0):
    dt = aclnn.ACL_FLOAT if dt is None else dt
    fmt = aclnn.ACL_FORMAT_NCHW if fmt is None else fmt
    g = desc.t(grad, dt, fmt)
    o = desc.t(out, dt if odt is None else odt, fmt if ofmt is None else ofmt)
    a1 = aclnn.create_int_array(list(osize)) if osize is not None else None
    a2 = aclnn.create_int_array(list(isize)) if isize is not None else None
    st, ws, ex = aclnn.get_workspace_size_upsample_bilinear2d_backward(g, a1, a2, align, sh, sw, o)
    variant = aclnn.executor_variant(ex) if ex else None
    if ex:
        aclnn.destroy_executor(ex)
    aclnn.destroy_int_array(a1)
    aclnn.destroy_int_array(a2)
    return st, ws, variant


def test_upsample_backward_status_codes(aclnn, desc):
    """test_aclnn_upsample_bilineard_2d_backward.cpp cases 001-017 and the checks of
    aclnn_upsample_bilinear_2d_backward.cpp:48-230"""
    INV, NULL = aclnn.ACLNN_ERR_PARAM_INVALID, aclnn.ACLNN_ERR_PARAM_NULLPTR
    # 001/002 (+ bf16, supported on the newest parts): scales 2.0 with sizes 2x2 <- 3x3 do not match the size ratio:
    # accepted, the user-scale template runs
    for dt in (aclnn.ACL_FLOAT, aclnn.ACL_FLOAT16, aclnn.ACL_BF16):
        assert _ub(aclnn, desc, dt=dt) == (0, 0, "resize_grad_gather_scales")
    assert _ub(aclnn, desc, sh=0.0, sw=0.0)[2] == "resize_grad_lds"
    assert _ub(aclnn, desc, align=True)[2] == "resize_grad_lds"
    # 003-012: unsupported dtypes
    for dt in (aclnn.ACL_DOUBLE, aclnn.ACL_INT32):
        assert _ub(aclnn, desc, dt=dt)[0] == INV
    # 013: empty tensor
    assert _ub(aclnn, desc, grad=(0, 1, 2, 2), out=(0, 1, 3, 3), isize=(0, 1, 3, 3))[:2] == (0, 0)
    # 014/015: rank
    assert _ub(aclnn, desc, grad=(2, 2))[0] == INV
    assert _ub(aclnn, desc, grad=(1, 1, 1, 2, 2))[0] == INV
    # 016: null arguments
    assert _ub(aclnn, desc, grad=None)[0] == NULL
    assert _ub(aclnn, desc, out=None)[0] == NULL
    assert _ub(aclnn, desc, osize=None)[0] == NULL
    assert _ub(aclnn, desc, isize=None)[0] == NULL
    # 017: out dtype; a FLOAT gradient may be reduced into a 16-bit out, a 16-bit one may not change type
    assert _ub(aclnn, desc, odt=aclnn.ACL_FLOAT16)[0] == 0
    assert _ub(aclnn, desc, dt=aclnn.ACL_FLOAT16, odt=aclnn.ACL_FLOAT)[0] == INV
    # sizes: array lengths, positive extents, gradOut == (N,C,outputSize), out == inputSize
    assert _ub(aclnn, desc, osize=(2, 2, 2))[0] == INV
    assert _ub(aclnn, desc, isize=(1, 3, 3))[0] == INV
    assert _ub(aclnn, desc, osize=(0, 2), grad=(1, 1, 0, 2))[0] == INV
    assert _ub(aclnn, desc, osize=(3, 2))[0] == INV
    assert _ub(aclnn, desc, out=(1, 1, 3, 4))[0] == INV
    assert _ub(aclnn, desc, out=(1, 2, 3, 3))[0] == INV
    # formats: equal, NCHW or NHWC; NHWC reads the four extents as N,H,W,C
    assert _ub(aclnn, desc, ofmt=aclnn.ACL_FORMAT_NHWC)[0] == INV
    assert _ub(aclnn, desc, grad=(1, 2, 2, 5), out=(1, 3, 3, 5), isize=(1, 3, 3, 5), fmt=aclnn.ACL_FORMAT_NHWC,
               sh=0, sw=0) == (0, 0, "resize_grad_lds")
    # 16-bit rows of an odd number of elements are not whole 4-byte words: the per-element gather
    assert _ub(aclnn, desc, grad=(1, 2, 3, 5), out=(1, 3, 3, 5), osize=(2, 3), isize=(1, 3, 3, 5),
               fmt=aclnn.ACL_FORMAT_NHWC, dt=aclnn.ACL_FLOAT16, sh=0, sw=0) == (0, 0, "resize_grad_gather")
    # equal sizes: a copy
    assert _ub(aclnn, desc, grad=(1, 1, 3, 3), osize=(3, 3), sh=1.0, sw=1.0)[2] == "copy"


def _gs3(aclnn, desc, inp=(2, 1, 1, 3, 3), grid=(2, 1, 2, 2, 3), out=(2, 1, 1, 2, 2), dt=None, gdt=None, odt=None,
         interp=0, pad=0, align=False, fmt=None, ofmt=None, **kw):
    dt = aclnn.ACL_FLOAT if dt is None else dt
    fmt = aclnn.ACL_FORMAT_NCDHW if fmt is None else fmt
    i = desc.t(inp, dt, fmt, **kw)
    g = desc.t(grid, dt if gdt is None else gdt, aclnn.ACL_FORMAT_NCDHW)
    o = desc.t(out, dt if odt is None else odt, fmt if ofmt is None else ofmt)
    st, ws, ex = aclnn.get_workspace_size_grid_sampler3d(i, g, interp, pad, align, o)
    variant = aclnn.executor_variant(ex) if ex else None
    if ex:
        assert aclnn.destroy_executor(ex) == 0
    return st, ws, variant


def test_grid_sampler3d_status_codes(aclnn, desc):
    """test_aclnn_grid_sampler3d.cpp:33-289 and the check order of aclnn_grid_sampler3d.cpp:194-208"""
    INV, NULL = aclnn.ACLNN_ERR_PARAM_INVALID, aclnn.ACLNN_ERR_PARAM_NULLPTR
    # input_nullptr, grid_nullptr, out_nullptr
    assert _gs3(aclnn, desc, inp=None)[0] == NULL
    assert _gs3(aclnn, desc, grid=None)[0] == NULL
    assert _gs3(aclnn, desc, out=None)[0] == NULL
    # input_empty: success, no workspace, an executor that does nothing
    assert _gs3(aclnn, desc, inp=(2, 0, 1, 3, 3), out=(2, 0, 1, 2, 2)) == (0, 0, "")
    # dtype_float16 / float32 / bf16 accepted, int8 rejected; DOUBLE passes the reference's list but has no kernel here
    for dt in (aclnn.ACL_FLOAT16, aclnn.ACL_FLOAT, aclnn.ACL_BF16):
        assert _gs3(aclnn, desc, dt=dt) == (0, 0, "gs3d_bilinear")
    assert _gs3(aclnn, desc, dt=aclnn.ACL_INT8)[0] == INV
    assert _gs3(aclnn, desc, dt=aclnn.ACL_DOUBLE)[0] == INV
    assert _gs3(aclnn, desc, gdt=aclnn.ACL_FLOAT16)[0] == INV
    assert _gs3(aclnn, desc, odt=aclnn.ACL_FLOAT16)[0] == INV
    # shape_n_input1_grid2, shape_c_input1_out2, shape_h_grid2_out3, shape_w_grid2_out4, shape_grid_not_3
    assert _gs3(aclnn, desc, inp=(1, 1, 1, 3, 3), out=(1, 1, 1, 2, 2))[0] == INV
    assert _gs3(aclnn, desc, out=(2, 3, 1, 2, 2))[0] == INV
    assert _gs3(aclnn, desc, out=(2, 1, 1, 3, 2))[0] == INV
    assert _gs3(aclnn, desc, out=(2, 1, 1, 2, 4))[0] == INV
    assert _gs3(aclnn, desc, grid=(2, 1, 2, 2, 4))[0] == INV
    # rank and empty spatial extents
    assert _gs3(aclnn, desc, inp=(2, 1, 3, 3))[0] == INV
    assert _gs3(aclnn, desc, inp=(2, 1, 1, 0, 3))[0] == INV
    # mode_3, padding_mode_3 (interpolation is 0 or 1 only; there is no volumetric bicubic)
    assert _gs3(aclnn, desc, interp=3)[0] == INV
    assert _gs3(aclnn, desc, interp=2)[0] == INV
    assert _gs3(aclnn, desc, pad=3)[0] == INV
    assert _gs3(aclnn, desc, interp=1, pad=2, align=True) == (0, 0, "gs3d_nearest")
    # input_format_invalid, out_format_invalid
    assert _gs3(aclnn, desc, fmt=aclnn.ACL_FORMAT_NCHW, ofmt=aclnn.ACL_FORMAT_NCDHW)[0] == INV
    assert _gs3(aclnn, desc, ofmt=aclnn.ACL_FORMAT_NCHW)[0] == INV
    assert _gs3(aclnn, desc, fmt=aclnn.ACL_FORMAT_ND)[0] == 0
    # format errors come before attribute errors, dtype errors before both
    msg = aclnn.load_library().aclGetRecentErrMsg
    _gs3(aclnn, desc, fmt=aclnn.ACL_FORMAT_NCHW, interp=7)
    assert b"format" in msg()
    _gs3(aclnn, desc, dt=aclnn.ACL_INT8, fmt=aclnn.ACL_FORMAT_NCHW)
    assert b"dtype" in msg()
    # isNCDHW_special_case: an ordinary shape here
    assert _gs3(aclnn, desc, inp=(22, 4, 16, 64, 64), grid=(22, 16, 64, 64, 3), out=(22, 4, 16, 64, 64))[0] == 0
    # ascend910B2_NDHWC_case_01: channels-last extents (N,D,H,W,C); the operand is a permuted view, so a channel
    # count above one needs workspace for the input and for the output
    assert _gs3(aclnn, desc, inp=(2, 1, 3, 3, 1), out=(2, 1, 2, 2, 1), fmt=aclnn.ACL_FORMAT_NDHWC)[:2] == (0, 0)
    # dense channels-last tensors are sampled in place; a strided one is packed as a permuted view
    assert _gs3(aclnn, desc, inp=(2, 1, 3, 3, 4), out=(2, 1, 2, 2, 4), fmt=aclnn.ACL_FORMAT_NDHWC) == \
        (0, 0, "gs3d_ndhwc_bilinear")
    st, ws, variant = _gs3(aclnn, desc, inp=(2, 1, 3, 3, 4), out=(2, 1, 2, 2, 4), fmt=aclnn.ACL_FORMAT_NDHWC,
                           strides=(72, 72, 24, 8, 1), storage=(144,))
    assert st == 0 and variant == "gs3d_bilinear" and ws >= 2 * 9 * 4 * 4
    # a strided NCDHW view is packed too
    st, ws, _ = _gs3(aclnn, desc, strides=(18, 18, 18, 6, 2), storage=(36,))
    assert st == 0 and ws >= 2 * 9 * 4


_KEEP = object()


def _gsb(aclnn, desc, gout=(1, 1, 3, 3), inp=(1, 1, 5, 8), grid=(1, 3, 3, 2), dx=_KEEP, dgrid=_KEEP, dt=None,
         dts=None, interp=0, pad=0, align=False, mask=(True, True), **kw):
    dt = aclnn.ACL_FLOAT if dt is None else dt
    dts = dts or {}
    dx = inp if dx is _KEEP else dx
    dgrid = grid if dgrid is _KEEP else dgrid
    hs = [desc.t(shape, dts.get(name, dt), **(kw if name == "inp" else {}))
          for name, shape in (("gout", gout), ("inp", inp), ("grid", grid), ("dx", dx), ("dgrid", dgrid))]
    m = aclnn.create_bool_array(list(mask)) if mask is not None else None
    st, ws, ex = aclnn.get_workspace_size_grid_sampler2d_backward(hs[0], hs[1], hs[2], interp, pad, align, m, hs[3],
                                                                  hs[4])
    variant = aclnn.executor_variant(ex) if ex else None
    if ex:
        assert aclnn.destroy_executor(ex) == 0
    aclnn.destroy_bool_array(m)
    return st, ws, variant


def test_grid_sampler2d_backward_status_codes(aclnn, desc):
    """test_aclnn_grid_sampler2d_backward.cpp and the check order of aclnn_grid_sampler2d_backward.cpp:195-243"""
    INV, NULL = aclnn.ACLNN_ERR_PARAM_INVALID, aclnn.ACLNN_ERR_PARAM_NULLPTR
    # case_1: the example shapes, float; 16-bit types as on the newest parts
    for dt in (aclnn.ACL_FLOAT, aclnn.ACL_FLOAT16, aclnn.ACL_BF16):
        assert _gsb(aclnn, desc, dt=dt) == (0, 0, "gs2d_grad_ordered")
    # case_2..case_6: each tensor missing in turn
    for missing in ("gout", "inp", "grid", "dx", "dgrid"):
        assert _gsb(aclnn, desc, **{missing: None})[0] == NULL, missing
    # a missing mask succeeds as a no-op before anything else is looked at, even with tensors missing
    assert _gsb(aclnn, desc, mask=None, inp=None) == (0, 0, "")
    # both flags false: a no-op; one flag: that gradient only
    assert _gsb(aclnn, desc, mask=(False, False)) == (0, 0, "")
    assert _gsb(aclnn, desc, mask=(True, False))[0] == 0 and _gsb(aclnn, desc, mask=(False, True))[0] == 0
    assert _gsb(aclnn, desc, mask=(True,))[0] == INV
    assert _gsb(aclnn, desc, mask=(True, True, True))[0] == INV
    # dtypes: all five equal, from the list; DOUBLE passes the list but has no kernel here
    for name in ("gout", "grid", "dx", "dgrid"):
        assert _gsb(aclnn, desc, dts={name: aclnn.ACL_FLOAT16})[0] == INV, name
    assert _gsb(aclnn, desc, dt=aclnn.ACL_INT32)[0] == INV
    assert _gsb(aclnn, desc, dt=aclnn.ACL_DOUBLE)[0] == INV
    # attributes
    assert _gsb(aclnn, desc, interp=3)[0] == INV and _gsb(aclnn, desc, interp=-1)[0] == INV
    assert _gsb(aclnn, desc, pad=3)[0] == INV
    assert _gsb(aclnn, desc, interp=2, pad=2, align=True)[0] == 0
    # shapes
    assert _gsb(aclnn, desc, inp=(1, 5, 8), dx=(1, 5, 8))[0] == INV
    assert _gsb(aclnn, desc, gout=(2, 1, 3, 3))[0] == INV          # batch
    assert _gsb(aclnn, desc, gout=(1, 2, 3, 3))[0] == INV          # channels
    assert _gsb(aclnn, desc, inp=(1, 1, 0, 8), dx=(1, 1, 0, 8))[0] == INV
    assert _gsb(aclnn, desc, gout=(1, 1, 3, 4))[0] == INV          # grid vs gradOutput
    assert _gsb(aclnn, desc, grid=(1, 3, 3, 3), dgrid=(1, 3, 3, 3))[0] == INV
    assert _gsb(aclnn, desc, dx=(1, 1, 5, 7))[0] == INV
    assert _gsb(aclnn, desc, dgrid=(1, 3, 2, 2))[0] == INV
    # empty tensors: success without work
    assert _gsb(aclnn, desc, gout=(0, 1, 3, 3), inp=(0, 1, 5, 8), grid=(0, 3, 3, 2)) == (0, 0, "")
    # case_9_BIGC: 4096 channels are fine
    assert _gsb(aclnn, desc, gout=(1, 4096, 3, 3), inp=(1, 4096, 5, 8))[0] == 0
    # a strided input view needs workspace
    st, ws, _ = _gsb(aclnn, desc, strides=(80, 80, 16, 2), storage=(80,))
    assert st == 0 and ws >= 40 * 4


def _gsb3(aclnn, desc, gout=(1, 1, 1, 2, 2), inp=(1, 1, 1, 3, 3), grid=(1, 1, 2, 2, 3), dx=_KEEP, dgrid=_KEEP, dt=None,
          dts=None, interp=0, pad=0, align=False, mask=(True, True), fmt=None, **kw):
    dt = aclnn.ACL_FLOAT if dt is None else dt
    fmt = aclnn.ACL_FORMAT_NCDHW if fmt is None else fmt
    dts = dts or {}
    dx = inp if dx is _KEEP else dx
    dgrid = grid if dgrid is _KEEP else dgrid
    hs = [desc.t(shape, dts.get(name, dt), fmt=fmt, **(kw if name == "inp" else {}))
          for name, shape in (("gout", gout), ("inp", inp), ("grid", grid), ("dx", dx), ("dgrid", dgrid))]
    m = aclnn.create_bool_array(list(mask)) if mask is not None else None
    st, ws, ex = aclnn.get_workspace_size_grid_sampler3d_backward(hs[0], hs[1], hs[2], interp, pad, align, m, hs[3],
                                                                  hs[4])
    variant = aclnn.executor_variant(ex) if ex else None
    if ex:
        assert aclnn.destroy_executor(ex) == 0
    aclnn.destroy_bool_array(m)
    return st, ws, variant


def test_grid_sampler3d_backward_status_codes(aclnn, desc):
    """image/grid_sampler3_d_grad/tests/ut/op_host/op_api/test_aclnn_grid_sampler3d_backward.cpp and the check order
    of aclnn_grid_sampler3d_backward.cpp:174-238"""
    INV, NULL = aclnn.ACLNN_ERR_PARAM_INVALID, aclnn.ACLNN_ERR_PARAM_NULLPTR
    # dtype_float16 / dtype_float32 / dtype_bf16: the unit test's shapes
    # bilinear asks for the scratch of the gather variant: per batch item four flag words, a count and eight 16-bit slots
    # per cell of the (D+1) x (H+1) x (W+1) lattice of low corners (2 x 4 x 4 here), an overflow list of 1024 (cell,
    # point) pairs, eight weights per grid point (4) and gradOutput once more, in groups of four channels
    for dt, esz in ((aclnn.ACL_FLOAT, 4), (aclnn.ACL_FLOAT16, 2), (aclnn.ACL_BF16, 2)):
        assert _gsb3(aclnn, desc, dt=dt) == (0, (4 + 32 + 4 * 32 + 2048) * 4 + 4 * 8 * esz + 4 * 4 * esz,
                                             "gs3d_grad_lists")
        assert _gsb3(aclnn, desc, dt=dt, interp=1) == (0, 0, "gs3d_grad_ordered")
    # gradOutput_nullptr .. gridGrad_nullptr
    for missing in ("gout", "inp", "grid", "dx", "dgrid"):
        assert _gsb3(aclnn, desc, **{missing: None})[0] == NULL, missing
    # a missing mask succeeds as a no-op before anything else is looked at
    assert _gsb3(aclnn, desc, mask=None, inp=None) == (0, 0, "")
    # output_mask_false_false: success, no work; a mask of another length is checked after the shapes
    assert _gsb3(aclnn, desc, mask=(False, False)) == (0, 0, "")
    assert _gsb3(aclnn, desc, mask=(True, False))[0] == 0 and _gsb3(aclnn, desc, mask=(False, True))[0] == 0
    assert _gsb3(aclnn, desc, mask=(True,))[0] == INV
    assert _gsb3(aclnn, desc, mask=(True, True, True))[0] == INV
    # dtypes
    for name in ("gout", "grid", "dx", "dgrid"):
        assert _gsb3(aclnn, desc, dts={name: aclnn.ACL_FLOAT16})[0] == INV, name
    assert _gsb3(aclnn, desc, dt=aclnn.ACL_INT32)[0] == INV
    assert _gsb3(aclnn, desc, dt=aclnn.ACL_DOUBLE)[0] == INV
    # mode_3, padding_mode_3; bicubic does not exist in three dimensions
    assert _gsb3(aclnn, desc, interp=3)[0] == INV and _gsb3(aclnn, desc, interp=2)[0] == INV
    assert _gsb3(aclnn, desc, interp=-1)[0] == INV
    assert _gsb3(aclnn, desc, pad=3)[0] == INV
    assert _gsb3(aclnn, desc, interp=1, pad=2, align=True)[0] == 0
    # shape_n_input1_grid2, shape_c_input1_output2, shape_h_grid2_output3, shape_w_grid2_output4
    assert _gsb3(aclnn, desc, grid=(2, 1, 2, 2, 3), dgrid=(2, 1, 2, 2, 3))[0] == INV
    assert _gsb3(aclnn, desc, gout=(1, 2, 1, 2, 2))[0] == INV
    assert _gsb3(aclnn, desc, gout=(1, 1, 1, 3, 2))[0] == INV
    assert _gsb3(aclnn, desc, gout=(1, 1, 1, 2, 4))[0] == INV
    assert _gsb3(aclnn, desc, gout=(1, 1, 2, 2, 2))[0] == INV
    assert _gsb3(aclnn, desc, inp=(1, 1, 3, 3), dx=(1, 1, 3, 3))[0] == INV
    assert _gsb3(aclnn, desc, grid=(1, 1, 2, 2, 2), dgrid=(1, 1, 2, 2, 2))[0] == INV
    assert _gsb3(aclnn, desc, dx=(1, 1, 1, 3, 4))[0] == INV
    assert _gsb3(aclnn, desc, dgrid=(1, 1, 2, 1, 3))[0] == INV
    # empty tensors: success without work
    assert _gsb3(aclnn, desc, gout=(0, 1, 1, 2, 2), inp=(0, 1, 1, 3, 3), grid=(0, 1, 2, 2, 3)) == (0, 0, "")
    # channels-last: the format of input says where the channels are; such tensors are packed through the workspace
    nd = aclnn.ACL_FORMAT_NDHWC
    st, ws, v = _gsb3(aclnn, desc, gout=(1, 1, 2, 2, 5), inp=(1, 1, 3, 3, 5), fmt=nd)
    assert st == 0 and v == "gs3d_grad_lists" and ws >= (20 + 45 + 45) * 4
    assert _gsb3(aclnn, desc, gout=(1, 1, 2, 2, 4), inp=(1, 1, 3, 3, 5), fmt=nd)[0] == INV
    # volumes of more than one LDS band ask for scratch: two words per chunk of 256 grid points and batch item, only
    # when the input gradient is wanted; the gather variant's scratch follows from the next 256-byte boundary
    big = dict(gout=(3, 1, 2, 30, 10), inp=(3, 1, 10, 30, 30), grid=(3, 2, 30, 10, 3))
    assert _gsb3(aclnn, desc, interp=1, **big)[:2] == (0, 3 * 3 * 2 * 4)
    cells, points = 11 * 31 * 31, 600
    per_item = ((4 + cells + 3) // 4 * 4 + 4 * cells + 2048) * 4 + points * 8 * 4 + points * 4 * 4
    # (fifteen voxels per grid point: the ordered kernel by itself, the gather when asked for)
    assert _gsb3(aclnn, desc, **big) == (0, 3 * 3 * 2 * 4, "gs3d_grad_ordered")
    with aclnn.option("gs3d_grad_variant", 2):
        assert _gsb3(aclnn, desc, **big) == (0, 256 + 3 * per_item, "gs3d_grad_lists")
    assert _gsb3(aclnn, desc, mask=(False, True), **big)[:2] == (0, 0)


def test_resize_template_selection_point_copy(aclnn, desc):
    """resize_bilinear_v2_tiling_arch35.cpp:254-303: channels-last runs of 128 bytes and more, shrunk by whole factors
    (odd ones with half-pixel centres), are copied instead of interpolated"""
    nhwc = aclnn.ACL_FORMAT_NHWC
    kw = dict(mode=b"bilinear", fmt=nhwc)
    assert _rs(aclnn, desc, inp=(1, 9, 15, 32), out=(1, 3, 5, 32), scales=(1, 1 / 3, 1 / 3, 1), **kw)[2] == "point_copy"
    # factor 2 with half-pixel centres samples between pixels; 31 channels of fp32 are under 128 bytes
    assert _rs(aclnn, desc, inp=(1, 8, 8, 32), out=(1, 4, 4, 32), scales=(1, 0.5, 0.5, 1), **kw)[2] != "point_copy"
    assert _rs(aclnn, desc, inp=(1, 9, 15, 31), out=(1, 3, 5, 31), scales=(1, 1 / 3, 1 / 3, 1), **kw)[2] != "point_copy"
    # NCHW never takes the template
    assert _rs(aclnn, desc, inp=(1, 32, 9, 15), out=(1, 32, 3, 5), scales=(1, 1, 1 / 3, 1 / 3), mode=b"bilinear")[2] != \
        "point_copy"


def test_options_api_and_rule_captured_at_phase_one(aclnn):
    """opscvSetOption / opscvGetOption: names, ranges, defaults; the bilinear coordinate rule goes into the executor at
    phase 1 (the variant name of a shape beyond LDS shows it) and applies to the bilinear mode only"""
    defaults = {"gs_variant": 0, "resize_variant": 0, "nearest_variant": 0, "reference_cores": 64,
                "reference_ub_bytes": 253952, "grid_sampler2d_rule": 0, "gs3d_grad_variant": 0}
    for name, value in defaults.items():
        assert aclnn.get_option(name) == value, name
    L = aclnn.load_library()
    assert L.opscvSetOption(b"no_such_option", 1) == 161002
    assert L.opscvSetOption(b"grid_sampler2d_rule", 2) == 161002
    assert L.opscvSetOption(b"reference_cores", 0) == 161002
    assert L.opscvSetOption(None, 0) == 161001
    assert aclnn.get_option("grid_sampler2d_rule") == 0
    f16 = aclnn.ACL_FLOAT16

    def variant(interp):
        hs = [aclnn.create_tensor((1, 2, 300, 310), f16), aclnn.create_tensor((1, 20, 24, 2), f16),
              aclnn.create_tensor((1, 2, 20, 24), f16)]
        st, ws, ex = aclnn.get_workspace_size_grid_sampler2d(hs[0], hs[1], interp, 0, False, hs[2])
        assert st == 0 and ws == 0
        v = aclnn.executor_variant(ex)
        aclnn.destroy_executor(ex)
        for h in hs:
            aclnn.destroy_tensor(h)
        return v

    assert variant(0) == "direct"
    with aclnn.option("grid_sampler2d_rule", 1):
        assert variant(0) == "direct_arch35"
        assert variant(1) == "direct"  # nearest: the rule does not apply
    assert variant(0) == "direct"
    with aclnn.option("gs_variant", 1):
        assert aclnn.get_option("gs_variant") == 1
    assert aclnn.get_option("gs_variant") == 0


def test_grid_sampler3d_backward_gather_variant_is_gated_on_point_density(aclnn):
    """the gather variant of the 3-D sampler's input gradient pays per voxel, the ordered kernel per grid point: phase 1
    takes the gather (and its scratch) only up to eight voxels per grid point, and option gs3d_grad_variant overrides"""
    f16 = aclnn.ACL_FLOAT16

    def plan(vol, pts, N=2, C=4):
        D, H, W = vol
        Do, Ho, Wo = pts
        hs = [aclnn.create_tensor((N, C, Do, Ho, Wo), f16, aclnn.ACL_FORMAT_NCDHW),
              aclnn.create_tensor((N, C, D, H, W), f16, aclnn.ACL_FORMAT_NCDHW),
              aclnn.create_tensor((N, Do, Ho, Wo, 3), f16),
              aclnn.create_tensor((N, C, D, H, W), f16, aclnn.ACL_FORMAT_NCDHW),
              aclnn.create_tensor((N, Do, Ho, Wo, 3), f16)]
        mask = aclnn.create_bool_array([True, True])
        st, ws, ex = aclnn.get_workspace_size_grid_sampler3d_backward(hs[0], hs[1], hs[2], 0, 0, False, mask, hs[3],
                                                                      hs[4])
        assert st == 0
        v = aclnn.executor_variant(ex)
        aclnn.destroy_executor(ex)
        for h in hs:
            aclnn.destroy_tensor(h)
        aclnn.destroy_bool_array(mask)
        return v, ws

    dense = plan((16, 32, 32), (16, 32, 32))        # one voxel per point
    edge_in = plan((16, 32, 32), (4, 16, 32))       # eight voxels per point: still the gather
    edge_out = plan((16, 32, 32), (4, 16, 31))      # a little over eight
    sparse = plan((64, 64, 64), (4, 16, 16))        # 256 voxels per point
    assert dense[0] == "gs3d_grad_lists" and edge_in[0] == "gs3d_grad_lists"
    assert edge_out[0] == "gs3d_grad_ordered" and sparse[0] == "gs3d_grad_ordered"
    # the ordered kernel asks for the chunk spans only: kilobytes, where the gather of the sparse case would want
    # five words per lattice cell (several megabytes per batch item)
    assert sparse[1] < 64 * 1024 < (1 << 20) < plan((16, 64, 64), (16, 64, 64))[1]
    with aclnn.option("gs3d_grad_variant", 1):
        assert plan((16, 32, 32), (16, 32, 32))[0] == "gs3d_grad_ordered"
    with aclnn.option("gs3d_grad_variant", 2):
        forced = plan((64, 64, 64), (4, 16, 16))
        assert forced[0] == "gs3d_grad_lists" and forced[1] > 5 * 4 * 65 ** 3


def test_second_phase_refuses_a_misaligned_workspace(aclnn):
    """the kernels read and write their workspace slices with 16-byte accesses and 32-bit atomics: a workspace that
    does not start on a 16-byte boundary is refused before anything is launched (and the executor is consumed)"""
    import ctypes
    f32 = aclnn.ACL_FLOAT
    L = aclnn.load_library()
    # a transposed input view needs packing, hence a workspace
    hs = [aclnn.create_tensor((1, 2, 4, 6), f32, strides=(48, 24, 1, 4)), aclnn.create_tensor((1, 3, 3, 2), f32),
          aclnn.create_tensor((1, 2, 3, 3), f32)]
    st, ws, ex = aclnn.get_workspace_size_grid_sampler2d(hs[0], hs[1], 0, 0, False, hs[2])
    assert st == 0 and ws >= 48 * 4
    assert L.aclnnGridSampler2D(ctypes.c_void_p(0x7f0000001008), ws, ex, None) == 161002
    assert b"16-byte boundary" in L.aclGetRecentErrMsg()
    # the executor is gone: a second use is refused as not live
    st, ws, ex = aclnn.get_workspace_size_grid_sampler2d(hs[0], hs[1], 0, 0, False, hs[2])
    assert L.aclnnGridSampler2D(None, ws, ex, None) == 161001
    for h in hs:
        aclnn.destroy_tensor(h)
