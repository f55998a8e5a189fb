"""Tensors of 2^31 elements and more (byte offsets beyond 4 GiB): the paths where the reference switches to 64-bit
indexing (grid_sampler2_d_simt.h:535-556; resize tiling keys 30003/30005, resize_bilinear_v2_tiling_arch35.cpp:606-615).

The GPU runs the full tensors, generated on the device; the oracle checks the first and the last few channels / planes
only (channels are independent of each other), the last ones being where element and byte offsets exceed 32 bits.
"""
import numpy as np
import pytest

import inputs as I

pytestmark = pytest.mark.gpu

TWO31 = 1 << 31


def _bits(t):
    import torch
    return t.detach().contiguous().cpu().view(torch.int16).numpy().view(np.uint16)


def _f16(bits):
    return bits.view(np.float16)


def _check_sampler_channels(oracle, x, g, y, interp, pad, align, channels, variant_prefix, aclnn):
    """x, y (N,C,..) fp16 device tensors (any memory layout), g (N,Ho,Wo,2); compares the given channel slices."""
    import torch
    g_np = _f16(_bits(g))
    for sl in channels:
        xs = _f16(_bits(x[:, sl]))
        ref = oracle.grid_sampler2d(xs, g_np, interp, pad, align, dtype=I.oracle_code("fp16"))
        got = _f16(_bits(y[:, sl]))
        nan = np.isnan(ref)
        assert np.array_equal(np.isnan(got), nan)
        assert np.array_equal(np.where(nan, 0, got.view(np.uint16)), np.where(nan, 0, ref.view(np.uint16))), \
            "channels %s differ" % (sl,)


def _variant(aclnn, x, g, y, interp, pad, align):
    hs = [aclnn.tensor_handle(t) for t in (x, g, y)]
    st, _, ex = aclnn.get_workspace_size_grid_sampler2d(hs[0], hs[1], interp, pad, align, hs[2])
    assert st == 0, aclnn.load_library().aclGetRecentErrMsg()
    v = aclnn.executor_variant(ex)
    aclnn.destroy_executor(ex)
    for h in hs:
        aclnn.destroy_tensor(h)
    return v


@pytest.mark.parametrize("case", ["lds_ring", "lds_pair", "direct", "box_lds", "box_lds_scattered", "nhwc"])
def test_grid_sampler_beyond_2_31_elements(oracle, device, aclnn, case):
    import torch
    torch.manual_seed(11)
    if case == "lds_ring":      # input and output both beyond 2^31 elements, planes staged in LDS
        N, C, H, W, Ho, Wo, interp, pad, align = 2, 140000, 128, 64, 128, 64, 0, 0, False
    elif case == "lds_pair":    # output beyond 2^31 elements through the pair-layout kernel
        N, C, H, W, Ho, Wo, interp, pad, align = 1, 40000, 64, 32, 240, 240, 0, 1, True
    elif case == "direct":      # planes far beyond LDS: the direct kernel (output rows of odd length; fp32 too)
        N, C, H, W, Ho, Wo, interp, pad, align = 1, 2100, 1024, 1024, 1023, 1025, 1, 2, False  # rows of odd length
    elif case.startswith("box_lds"):  # planes far beyond LDS, bilinear: a tile's box of the input through LDS
        N, C, H, W, Ho, Wo, interp, pad, align = 1, 2100, 1024, 1024, 1024, 1024, 0, 2, False
    else:                       # channels-last views of NHWC memory
        N, C, H, W, Ho, Wo, interp, pad, align = 1, 2100, 1024, 1024, 1024, 1024, 1, 0, False
    assert N * C * Ho * Wo >= TWO31
    x = torch.randn((N, C, H, W), device=device, dtype=torch.float16)
    g = (torch.rand((N, Ho, Wo, 2), device=device) * 2.3 - 1.15).to(torch.float16)
    if case == "box_lds":
        # a smooth warp, so that the tiles' boxes fit (scattered points, the case after this one, take the kernel's
        # pair loads instead)
        g = torch.from_numpy(I.affine_grid(np.random.default_rng(11), N, Ho, Wo)).to(device).to(torch.float16)
    y = torch.empty((N, C, Ho, Wo), device=device, dtype=torch.float16)
    if case == "nhwc":
        x = x.contiguous(memory_format=torch.channels_last)
        y = y.contiguous(memory_format=torch.channels_last)
    v = _variant(aclnn, x, g, y, interp, pad, align)
    assert v.startswith("box_lds" if case.startswith("box_lds") else case), v
    aclnn.grid_sampler2d(x, g, interp, pad, align, out=y)
    torch.cuda.synchronize()
    _check_sampler_channels(oracle, x, g, y, interp, pad, align, [slice(0, 2), slice(C // 2, C // 2 + 2),
                                                                  slice(C - 3, C)], case, aclnn)


@pytest.mark.parametrize("layout", ["nchw", "nhwc"])
@pytest.mark.parametrize("align", [False, True])
def test_upsample_beyond_2_31_output_elements(oracle, device, aclnn, layout, align):
    """fp16 1024x1024 planes doubled: 600 planes make 2.5e9 output elements (5 GB); NCHW and channels-last"""
    import torch
    torch.manual_seed(12)
    N, C, H, W, Ho, Wo = 1, 600, 1024, 1024, 2048, 2048
    assert N * C * Ho * Wo >= TWO31
    x = torch.randn((N, C, H, W), device=device, dtype=torch.float16)
    if layout == "nhwc":
        xm = x.permute(0, 2, 3, 1).contiguous()  # (N,H,W,C) memory
        y = aclnn.upsample_bilinear2d(xm, (Ho, Wo), align, 0.0, 0.0, channels_last=True)
        torch.cuda.synchronize()
        pick = lambda t, sl: t[..., sl].permute(0, 3, 1, 2)
        src = xm
    else:
        y = aclnn.upsample_bilinear2d(x, (Ho, Wo), align, 0.0, 0.0)
        torch.cuda.synchronize()
        pick = lambda t, sl: t[:, sl]
        src = x
    # The oracle sees a few planes at a time; its template choice follows the sizes it is given, so it is asked with
    # what holds for the full tensor too: 4 M output pixels per plane lie beyond the H*W-split threshold with 32-bit
    # and with 64-bit indices alike, and the channels-last per-element template does not depend on the channel count
    assert oracle.resize_uses_hw_split(N, C, H, W, Ho, Wo) == oracle.resize_uses_hw_split(N, 2, H, W, Ho, Wo)
    for sl in (slice(0, 1), slice(C - 2, C)):
        xs = _f16(_bits(pick(src, sl)))
        if layout == "nhwc":
            ref, template = oracle.upsample_bilinear2d_nhwc(np.ascontiguousarray(xs.transpose(0, 2, 3, 1)), (Ho, Wo),
                                                            align, 0.0, 0.0, dtype=I.oracle_code("fp16"),
                                                            with_template=True)
            assert template == "per_element"
            got = _f16(_bits(y[..., sl]))
        else:
            ref = oracle.upsample_bilinear2d(xs, (Ho, Wo), align, 0.0, 0.0, dtype=I.oracle_code("fp16"))
            got = _f16(_bits(pick(y, sl)))
        assert np.array_equal(got.view(np.uint16), ref.view(np.uint16)), "planes %s differ (%s, align=%s)" % (
            sl, layout, align)


def test_upsample_idx64_moves_the_template_threshold(oracle, device, aclnn):
    """Beyond 2^32 - 1 elements the reference indexes with 64 bits and halves the plane size from which it picks its
    H*W-split template (cores * 512 instead of cores * 1024 output pixels, resize_bilinear_v2_tiling_arch35.cpp:606-615),
    whose first rows and columns blend the border pixel with itself.  201 x 199 output planes lie between the two
    thresholds for the default 64 cores: 110000 of them (4.4e9 elements, fp32) take the split template, a few do not."""
    import torch
    torch.manual_seed(13)
    N, C, H, W, Ho, Wo = 1, 110000, 100, 100, 201, 199
    assert N * C * Ho * Wo > 0xFFFFFFFF
    assert oracle.resize_uses_hw_split(N, C, H, W, Ho, Wo) and not oracle.resize_uses_hw_split(N, 2, H, W, Ho, Wo)
    x = torch.randn((N, C, H, W), device=device, dtype=torch.float32)
    y = aclnn.upsample_bilinear2d(x, (Ho, Wo), False, 0.0, 0.0)
    torch.cuda.synchronize()
    try:
        for sl in (slice(0, 2), slice(C - 2, C)):
            xs = x[:, sl].contiguous().cpu().numpy()
            got = y[:, sl].contiguous().cpu().numpy()
            oracle.set_reference_cores(32)  # 32 * 1024 = 64 * 512: the few planes decide like the full tensor
            ref = oracle.upsample_bilinear2d(xs, (Ho, Wo), False, 0.0, 0.0)
            oracle.set_reference_cores(0)
            other = oracle.upsample_bilinear2d(xs, (Ho, Wo), False, 0.0, 0.0)
            assert not np.array_equal(ref.view(np.uint32), other.view(np.uint32))  # the templates differ on this data
            assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), "planes %s differ" % (sl,)
    finally:
        oracle.set_reference_cores(0)


def test_grid_sampler_backward_beyond_2_31_elements(oracle, device, aclnn):
    """aclnnGridSampler2DBackward with input, gradOutput and input gradient of more than 2^31 elements each, through the
    list variant of the input gradient and the LDS-ring variant of the grid gradient.  The input gradient is checked on
    the first and the last channels (a channel's gradient depends on that channel of gradOutput and on the grid only),
    the grid gradient on the last batch item, whose sums run over planes that start beyond 2^31 elements."""
    import torch
    torch.manual_seed(17)
    N, C, H, W, Ho, Wo = 9, 65535, 64, 64, 64, 64
    assert N * C * H * W > TWO31 and N * C * Ho * Wo > TWO31
    x = torch.randn((N, C, H, W), device=device, dtype=torch.float16)
    go = torch.randn((N, C, Ho, Wo), device=device, dtype=torch.float16)
    g = (torch.rand((N, Ho, Wo, 2), device=device) * 2.3 - 1.15).to(torch.float16)
    dx = torch.empty_like(x)
    dg = torch.empty_like(g)
    hs = [aclnn.tensor_handle(t) for t in (go, x, g, dx, dg)]
    m = aclnn.create_bool_array([True, True])
    st, ws, ex = aclnn.get_workspace_size_grid_sampler2d_backward(hs[0], hs[1], hs[2], 0, 0, False, m, hs[3], hs[4])
    assert st == 0 and aclnn.executor_variant(ex) == "gs2d_grad_lists_lds"
    aclnn.destroy_executor(ex)
    aclnn.destroy_bool_array(m)
    for h in hs:
        aclnn.destroy_tensor(h)
    aclnn.grid_sampler2d_backward(go, x, g, 0, 0, False, (True, True), dx, dg)
    torch.cuda.synchronize()
    g_np = _f16(_bits(g))
    code = I.oracle_code("fp16")
    for sl in (slice(0, 3), slice(C - 3, C)):
        rdx, _ = oracle.grid_sampler2d_backward(_f16(_bits(go[:, sl])), _f16(_bits(x[:, sl])), g_np, 0, 0, False,
                                                dtype=code, want=(True, False))
        assert np.array_equal(_bits(dx[:, sl]), rdx.view(np.uint16)), "input gradient, channels %s" % (sl,)
    n = N - 1
    _, rdg = oracle.grid_sampler2d_backward(_f16(_bits(go[n:])), _f16(_bits(x[n:])), g_np[n:], 0, 0, False, dtype=code,
                                            want=(False, True))
    assert np.array_equal(_bits(dg[n:]), rdg.view(np.uint16)), "grid gradient of the last batch item"
