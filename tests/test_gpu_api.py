"""GPU tests of the boundary behaviour: strided views, offsets, NHWC, fallback variants, full-size configurations."""
import ctypes

import numpy as np
import pytest

import inputs as I

pytestmark = pytest.mark.gpu


def _torch():
    import torch
    return torch


def test_noncontiguous_views_are_honoured(oracle, device, aclnn):
    torch = _torch()
    rng = np.random.default_rng(21)
    x32 = rng.standard_normal((2, 3, 9, 12)).astype(np.float32)
    g32 = rng.uniform(-1.2, 1.2, (2, 7, 5, 2)).astype(np.float32)
    ref = oracle.grid_sampler2d(x32, g32, 0, 0, False)
    # input as a transposed view of an (N,C,W,H) buffer, grid as a slice of a larger buffer, out as a strided slice
    xt = torch.from_numpy(np.ascontiguousarray(x32.transpose(0, 1, 3, 2))).to(device).transpose(2, 3)
    assert not xt.is_contiguous()
    gbig = torch.zeros((2, 7, 10, 2), device=device)
    gbig[:, :, ::2, :] = torch.from_numpy(g32).to(device)
    gv = gbig[:, :, ::2, :]
    obig = torch.full((2, 3, 7, 9), -7.0, device=device)
    ov = obig[:, :, :, 2:7]
    out = aclnn.grid_sampler2d(xt, gv, 0, 0, False, out=ov)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), ref)
    rest = obig.cpu().numpy()
    assert (rest[..., :2] == -7.0).all() and (rest[..., 7:] == -7.0).all()  # nothing outside the view is touched
    # upsample on a view with a storage offset
    u32 = rng.standard_normal((2, 2, 6, 8)).astype(np.float32)
    ubig = torch.zeros((3, 2, 6, 8), device=device)
    ubig[1:] = torch.from_numpy(u32).to(device)
    y = aclnn.upsample_bilinear2d(ubig[1:], (12, 16), False, 2.0, 2.0)
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy(), oracle.upsample_bilinear2d(u32, (12, 16), False, 2.0, 2.0))


@pytest.mark.parametrize("dtype", I.DTYPES)
@pytest.mark.parametrize("align", [False, True])
def test_upsample_nhwc(oracle, device, aclnn, dtype, align):
    torch = _torch()
    rng = np.random.default_rng(22)
    seen = set()
    for (N, C, H, W), size in [((2, 5, 7, 9), (14, 18)), ((1, 64, 1, 1), (6, 6)), ((1, 3, 8, 8), (8, 8)),
                               ((2, 3, 6, 6), (1, 1)), ((1, 130, 3, 3), (5, 7)), ((2, 16, 9, 11), (20, 17)),
                               ((1, 64, 12, 10), (5, 23)), ((1, 8, 1, 6), (4, 4)), ((1, 14, 1, 1), (13, 7)),
                               # long channel runs shrunk to half or less: the four-weights template, with channel
                               # counts for every vector width of its kernel (16 bytes, 8 bytes, one element)
                               ((2, 64, 12, 10), (5, 4)), ((1, 68, 23, 17), (7, 8)), ((1, 67, 9, 31), (4, 3)),
                               ((2, 128, 16, 16), (1, 1)), ((1, 72, 40, 6), (3, 3)),
                               # pixels that are not whole 16-byte vectors: units of 12, 8, 6 and 4 bytes
                               ((2, 3, 9, 11), (20, 17)), ((1, 6, 5, 7), (11, 13)), ((1, 10, 6, 4), (9, 9)),
                               ((1, 9, 6, 4), (5, 10)), ((1, 2, 6, 4), (9, 7)), ((1, 20, 5, 5), (12, 12)),
                               ((3, 3, 33, 47), (70, 129))]:
        x32 = rng.standard_normal((N, C, H, W)).astype(np.float32)
        x = I.cast_np(x32, dtype)
        xh = np.ascontiguousarray(x.transpose(0, 2, 3, 1))
        ref, template = oracle.upsample_bilinear2d_nhwc(xh, size, align, dtype=I.oracle_code(dtype), with_template=True)
        seen.add(template)
        y = aclnn.upsample_bilinear2d(I.to_torch(xh, dtype, device), size, align, channels_last=True)
        torch.cuda.synchronize()
        got = I.from_torch(y, dtype)
        assert np.array_equal(_bits(got, dtype), _bits(ref, dtype)), \
            "nhwc %s %s align=%s template %s" % (dtype, (N, C, H, W), align, template)
        # the same tensors one element into their allocations: dense, but off the 16-byte grid
        xo = torch.zeros(xh.size + 1, device=device, dtype=y.dtype)
        xo[1:] = I.to_torch(xh, dtype, device).reshape(-1)
        yo = torch.zeros(y.numel() + 2, device=device, dtype=y.dtype)
        aclnn.upsample_bilinear2d(xo[1:].view(xh.shape), size, align, out=yo[1:-1].view(y.shape), channels_last=True)
        torch.cuda.synchronize()
        assert torch.equal(yo[1:-1].view(y.shape), y) and yo[0] == 0 and yo[-1] == 0, \
            "nhwc offset %s %s align=%s" % (dtype, (N, C, H, W), align)
    assert {"per_element", "copy", "broadcast", "channel_parallel"} <= seen


@pytest.mark.parametrize("dtype", I.DTYPES)
@pytest.mark.parametrize("forced", ["generic", "register"])
def test_upsample_nhwc_kernels_behind_the_lds_variant(oracle, device, aclnn, dtype, forced, monkeypatch):
    """Option resize_variant = generic reaches the per-element channels-last kernel (kept for band counts beyond the grid
    limit), = register the unit kernel on shapes that the LDS-staged variant would take; both match the oracle"""
    torch = _torch()
    aclnn.set_option("resize_variant", {"generic": 1, "register": 2}[forced])
    rng = np.random.default_rng(29)
    seen = set()
    for (N, C, H, W), size, align in [((2, 5, 7, 9), (14, 18), False), ((1, 3, 9, 6), (4, 11), True),
                                      ((1, 7, 12, 10), (5, 23), False), ((2, 3, 9, 11), (20, 17), False),
                                      ((1, 6, 5, 7), (11, 13), True), ((1, 10, 6, 4), (9, 9), False),
                                      ((1, 9, 6, 4), (5, 10), False), ((1, 2, 6, 4), (9, 7), True),
                                      ((1, 20, 5, 5), (12, 12), False)]:
        x = I.cast_np(rng.standard_normal((N, H, W, C)).astype(np.float32), dtype)
        ref = oracle.upsample_bilinear2d_nhwc(x, size, align, dtype=I.oracle_code(dtype))
        xt = I.to_torch(x, dtype, device)
        y = torch.empty((N,) + tuple(size) + (C,), dtype=xt.dtype, device=device)
        hs = [aclnn.tensor_handle(xt, aclnn.ACL_FORMAT_NHWC), aclnn.tensor_handle(y, aclnn.ACL_FORMAT_NHWC)]
        arr = aclnn.create_int_array(list(size))
        st, _, ex = aclnn.get_workspace_size_upsample_bilinear2d(hs[0], arr, align, 0.0, 0.0, hs[1])
        assert st == 0
        seen.add(aclnn.executor_variant(ex))
        aclnn.destroy_executor(ex)
        aclnn.destroy_int_array(arr)
        for h in hs:
            aclnn.destroy_tensor(h)
        aclnn.upsample_bilinear2d(xt, size, align, out=y, channels_last=True)
        torch.cuda.synchronize()
        assert np.array_equal(_bits(I.from_torch(y, dtype), dtype), _bits(ref, dtype)), (dtype, N, C, H, W, align)
    # 20 channels of fp32 are whole 16-byte vectors, which have a kernel of their own
    assert seen - {"nhwc_vec"} == ({"nhwc_generic"} if forced == "generic" else {"nhwc_unit"})


@pytest.mark.parametrize("dtype", I.DTYPES)
def test_grid_sampler_variants_agree(oracle, device, aclnn, dtype):
    """every kernel variant (LDS ring classes, direct fallback for odd or oversized planes) matches the oracle"""
    torch = _torch()
    rng = np.random.default_rng(23)
    L = aclnn.load_library()
    seen = set()
    shapes = [(2, 5, 13, 17, 19, 23),    # odd byte count for 16-bit types -> direct
              (2, 9, 16, 16, 40, 40),    # small planes
              (1, 6, 64, 64, 64, 64),    # 8 KiB planes (16-bit)
              (1, 5, 128, 128, 50, 70),  # 32 KiB planes (16-bit)
              (1, 3, 160, 200, 33, 65),  # 64-128 KiB planes
              (1, 2, 300, 320, 31, 33)]  # beyond LDS -> direct
    for (N, C, H, W, Ho, Wo) in shapes:
        x = I.cast_np(rng.standard_normal((N, C, H, W)).astype(np.float32), dtype)
        g = I.cast_np(rng.uniform(-1.2, 1.2, (N, Ho, Wo, 2)).astype(np.float32), dtype)
        xt, gt = I.to_torch(x, dtype, device), I.to_torch(g, dtype, device)
        out = torch.empty((N, C, Ho, Wo), dtype=xt.dtype, device=device)
        hs = [aclnn.tensor_handle(t) for t in (xt, gt, out)]
        for interp in (0, 1):
            for pad in (0, 2):
                st, ws, ex = aclnn.get_workspace_size_grid_sampler2d(hs[0], hs[1], interp, pad, False, hs[2])
                assert st == 0
                seen.add(aclnn.executor_variant(ex))
                assert L.aclnnGridSampler2D(None, 0, ex, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
                torch.cuda.synchronize()
                ref = oracle.grid_sampler2d(x, g, interp, pad, False, dtype=I.oracle_code(dtype))
                assert np.array_equal(I.from_torch(out, dtype).view(np.uint8), ref.view(np.uint8)), (
                    dtype, (N, C, H, W, Ho, Wo), interp, pad)
        for h in hs:
            aclnn.destroy_tensor(h)
    assert "direct" in seen and len(seen) >= 4, seen


def test_full_size_grid_sampler_fp16_n16_c256(oracle, device, aclnn):
    """the headline configuration at full size, all six mode/padding variants, against the oracle"""
    torch = _torch()
    rng = np.random.default_rng(31)
    x = I.cast_np(rng.standard_normal((16, 256, 64, 64), dtype=np.float32), "fp16")
    g32 = I.affine_grid(rng, 16, 64, 64)
    outside = (np.abs(g32) > 1).any(-1).mean()
    assert 0.01 <= outside <= 0.15, outside
    g = I.cast_np(g32, "fp16")
    xt, gt = I.to_torch(x, "fp16", device), I.to_torch(g, "fp16", device)
    for interp in (0, 1):
        for pad in (0, 1, 2):
            y = aclnn.grid_sampler2d(xt, gt, interp, pad, False)
            torch.cuda.synchronize()
            ref = oracle.grid_sampler2d(x, g, interp, pad, False)
            assert np.array_equal(I.from_torch(y, "fp16").view(np.uint16), ref.view(np.uint16)), (interp, pad)


@pytest.mark.parametrize("shape", [(32, 64, 64, 64, 64, 64), (16, 128, 64, 64, 64, 128), (64, 32, 32, 128, 64, 64),
                                   (8, 136, 48, 64, 128, 64)])
def test_grid_sampler_launches_of_two_workgroups_per_cu(oracle, device, aclnn, shape):
    """shapes whose launch is exactly two workgroups per CU of a 256-CU part, where the ring kernel and the bicubic
    pair-layout kernel give the channel blocks that are handed out first more channels than the others (22 and 10 of
    32, 11 and 5 of 16, ...) and deal the channels out in turn: every channel must still be sampled once, in bilinear,
    nearest, bicubic and the second bilinear rule; the last shape has a channel count that does not divide (no uneven
    split there)"""
    torch = _torch()
    N, C, H, W, Ho, Wo = shape
    rng = np.random.default_rng(4100 + N + C)
    for dtype in ("fp16", "fp32"):
        x = I.cast_np(rng.standard_normal((N, C, H, W), dtype=np.float32), dtype)
        # every channel different from its neighbours by a constant, so that a channel taken twice or skipped shows
        x += I.cast_np(np.arange(C, dtype=np.float32).reshape(1, C, 1, 1) / 4, dtype)
        g = I.cast_np(I.affine_grid(rng, N, Ho, Wo), dtype)
        xt, gt = I.to_torch(x, dtype, device), I.to_torch(g, dtype, device)
        for interp, pad in ((0, 0), (1, 2), (0, 1), (2, 0), (2, 1)):
            y = aclnn.grid_sampler2d(xt, gt, interp, pad, False)
            torch.cuda.synchronize()
            ref = oracle.grid_sampler2d(x, g, interp, pad, False, dtype=I.oracle_code(dtype))
            got = I.from_torch(y, dtype)
            if interp == 2:
                same = (got.view(np.uint8).reshape(got.shape + (-1,)) == ref.view(np.uint8).reshape(ref.shape + (-1,))).all(-1)
                assert np.all(same | (np.isnan(got.astype(np.float32)) & np.isnan(ref.astype(np.float32)))), (dtype, interp, pad)
            else:
                assert np.array_equal(got.view(np.uint8), ref.view(np.uint8)), (dtype, interp, pad)
        with aclnn.option("grid_sampler2d_rule", 1):
            y = aclnn.grid_sampler2d(xt, gt, 0, 0, False)
            torch.cuda.synchronize()
        ref = oracle.grid_sampler2d_arch35(x, g, 0, False, dtype=I.oracle_code(dtype))
        assert np.array_equal(I.from_torch(y, dtype).view(np.uint8), ref.view(np.uint8)), (dtype, "second rule")


def test_full_size_random_gather_bf16(oracle, device, aclnn):
    torch = _torch()
    rng = np.random.default_rng(32)
    x = I.cast_np(rng.standard_normal((8, 128, 128, 128), dtype=np.float32), "bf16")
    g = I.cast_np(rng.uniform(-1.1, 1.1, (8, 256, 256, 2)).astype(np.float32), "bf16")
    y = aclnn.grid_sampler2d(I.to_torch(x, "bf16", device), I.to_torch(g, "bf16", device), 0, 1, True)
    torch.cuda.synchronize()
    ref = oracle.grid_sampler2d(x, g, 0, 1, True, dtype=oracle.BF16)
    assert np.array_equal(I.from_torch(y, "bf16"), ref)


def test_full_size_4k_upscale_properties(oracle, device, aclnn):
    """(4,16,1080,1920) -> (2160,3840) fp16 align_corners: oracle on a few planes, invariants on everything"""
    torch = _torch()
    rng = np.random.default_rng(33)
    x = torch.from_numpy(rng.random((4, 16, 1080, 1920), dtype=np.float32)).to(torch.float16)
    x[1, 3] = 0.625  # a constant plane stays constant
    xt = x.to(device)
    y = aclnn.upsample_bilinear2d(xt, (2160, 3840), True)
    torch.cuda.synchronize()
    yc = y.cpu()
    assert (yc[1, 3] == 0.625).all()
    # align_corners keeps the four corner samples of every plane
    for (a, b) in [((0, 0), (0, 0)), ((0, 3839), (0, 1919)), ((2159, 0), (1079, 0)), ((2159, 3839), (1079, 1919))]:
        assert torch.equal(yc[:, :, a[0], a[1]], x[:, :, b[0], b[1]])
    # convexity: every output lies within the range of its plane
    assert (yc.amax((2, 3)) <= x.amax((2, 3))).all() and (yc.amin((2, 3)) >= x.amin((2, 3))).all()
    planes = [(0, 0), (2, 7), (3, 15)]
    xs = np.stack([x[n, c].numpy() for n, c in planes])[:, None]
    ref = oracle.upsample_bilinear2d(xs, (2160, 3840), True)
    got = np.stack([yc[n, c].numpy() for n, c in planes])[:, None]
    assert np.array_equal(got.view(np.uint16), ref.view(np.uint16))


def test_full_size_upsample_fp32_56_to_112(oracle, device, aclnn):
    torch = _torch()
    rng = np.random.default_rng(34)
    x = rng.standard_normal((8, 64, 56, 56), dtype=np.float32)
    y = aclnn.upsample_bilinear2d(torch.from_numpy(x).to(device), (112, 112), False, 2.0, 2.0)
    torch.cuda.synchronize()
    ref = oracle.upsample_bilinear2d(x, (112, 112), False, 2.0, 2.0)
    assert np.array_equal(y.cpu().numpy().view(np.uint32), ref.view(np.uint32))


@pytest.mark.parametrize("dtype", I.DTYPES)
@pytest.mark.parametrize("channels_last", [False, True])
def test_resize_entry_point(oracle, device, aclnn, dtype, channels_last):
    """aclnnResize: bilinear is the upsample kernel with align_corners=False and scale = in/out; nearest is
    floor(dst * in/out).  Both bit-exact against the oracle, NCHW and NHWC, vector and scalar shapes."""
    import torch
    rng = np.random.default_rng(300 + int(channels_last))
    cases = [((1, 1, 2, 2), (2.0, 2.0)), ((2, 8, 9, 12), (2.0, 2.0)), ((1, 16, 7, 5), (1.5, 2.5)),
             ((2, 3, 16, 16), (0.5, 0.75)), ((1, 4, 1, 1), (4.0, 8.0)), ((1, 2, 6, 6), (1.0, 1.0)),
             ((1, 8, 33, 64), (3.0, 2.0)), ((1, 64, 20, 18), (0.25, 0.5)), ((2, 66, 9, 14), (0.4, 0.3))]
    for shape, (sh, sw) in cases:
        N, C, H, W = shape
        Ho, Wo = int(float(H) * sh), int(float(W) * sw)
        x = I.cast_np(rng.standard_normal(shape).astype(np.float32), dtype)
        xin = np.ascontiguousarray(x.transpose(0, 2, 3, 1)) if channels_last else x
        scales = (1.0, sh, sw, 1.0) if channels_last else (1.0, 1.0, sh, sw)
        xt = I.to_torch(xin, dtype, device)
        for mode in ("nearest", "bilinear"):
            y = I.from_torch(aclnn.resize(xt, scales, mode, channels_last=channels_last), dtype)
            torch.cuda.synchronize()
            if mode == "nearest":
                ref = oracle.resize_nearest(xin, (Ho, Wo), channels_last=channels_last, dtype=I.oracle_code(dtype))
            elif channels_last:
                ref = oracle.upsample_bilinear2d_nhwc(xin, (Ho, Wo), False, 0.0, 0.0, dtype=I.oracle_code(dtype))
            else:
                ref = oracle.upsample_bilinear2d(x, (Ho, Wo), False, 0.0, 0.0, dtype=I.oracle_code(dtype))
            view = np.uint32 if dtype == "fp32" else np.uint16
            assert y.shape == ref.shape
            assert np.array_equal(y.view(view), ref.view(view)), (mode, shape, sh, sw, dtype, channels_last)


def test_resize_strided_views(oracle, device, aclnn):
    """aclnnResize honours non-contiguous self and out views (packed through the workspace)"""
    import torch
    rng = np.random.default_rng(301)
    big = torch.from_numpy(rng.standard_normal((2, 4, 10, 24)).astype(np.float32)).to(device)
    xv = big[:, 1:3, 2:9, 3:19:2]
    outbig = torch.zeros((2, 2, 14, 40), device=device)
    ov = outbig[:, :, :, ::2][..., :16]
    aclnn.resize(xv, (1.0, 1.0, 2.0, 2.0), "nearest", out=ov)
    torch.cuda.synchronize()
    ref = oracle.resize_nearest(xv.contiguous().cpu().numpy(), (14, 16))
    assert np.array_equal(ov.cpu().numpy(), ref)
    assert float(outbig[:, :, :, 1::2].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", I.DTYPES)
@pytest.mark.parametrize("interp", [0, 1, 2])
def test_grid_sampler_channels_last_views(oracle, device, aclnn, dtype, interp):
    """input and out handed over as channels_last views (N,C,H,W dims, NHWC memory): sampled in place by the
    channels-last kernel, bit-exact against the oracle; vector (C % 8 or 4 == 0) and scalar channel counts"""
    import torch
    rng = np.random.default_rng(400 + interp)
    for (N, C, H, W, Ho, Wo, pad, align) in [(2, 16, 9, 11, 13, 7, 0, False), (1, 64, 32, 32, 40, 24, 1, True),
                                             (2, 5, 7, 6, 9, 9, 2, False), (1, 24, 5, 8, 4, 33, 0, True),
                                             (1, 3, 1, 1, 5, 5, 1, False)]:
        x = I.cast_np(rng.standard_normal((N, C, H, W)).astype(np.float32), dtype)
        g = I.cast_np(rng.uniform(-1.3, 1.3, (N, Ho, Wo, 2)).astype(np.float32), dtype)
        if C >= 16:
            g[0, 0, 0] = np.array([np.nan, 0.0]).astype(np.float32).view(np.float32) if dtype == "fp32" else g[0, 0, 0]
        ref = oracle.grid_sampler2d(x, g, interp, pad, align, dtype=I.oracle_code(dtype))
        xt = I.to_torch(x, dtype, device).contiguous(memory_format=torch.channels_last)
        gt = I.to_torch(g, dtype, device)
        out = torch.empty((N, C, Ho, Wo), dtype=xt.dtype, device=device).contiguous(memory_format=torch.channels_last)
        hs = [aclnn.tensor_handle(xt), aclnn.tensor_handle(gt), aclnn.tensor_handle(out)]
        st, ws, ex = aclnn.get_workspace_size_grid_sampler2d(hs[0], hs[1], interp, pad, align, hs[2])
        assert st == 0
        expect_inplace = C > 1 and (H * W > 1) and (Ho * Wo > 1)
        if expect_inplace:
            assert ws == 0 and aclnn.executor_variant(ex) == "nhwc"
        aclnn.destroy_executor(ex)
        for h in hs:
            aclnn.destroy_tensor(h)
        y = aclnn.grid_sampler2d(xt, gt, interp, pad, align, out=out)
        torch.cuda.synchronize()
        got = I.from_torch(y.contiguous(), dtype)
        nan = np.isnan(I.as_f32(ref, dtype))
        assert np.array_equal(np.isnan(I.as_f32(got, dtype)), nan)
        view = np.uint32 if dtype == "fp32" else np.uint16
        assert np.array_equal(np.where(nan, 0, got.view(view)), np.where(nan, 0, ref.view(view))), (N, C, H, W, pad, align)
        # mixed layouts fall back to packing and give the same result
        out2 = aclnn.grid_sampler2d(xt, gt, interp, pad, align)
        torch.cuda.synchronize()
        got2 = I.from_torch(out2, dtype)
        assert np.array_equal(np.where(nan, 0, got2.view(view)), np.where(nan, 0, ref.view(view)))


@pytest.mark.parametrize("dtype", I.DTYPES)
@pytest.mark.parametrize("channels_last", [False, True])
def test_upsample_backward(oracle, device, aclnn, dtype, channels_last):
    """aclnnUpsampleBilinear2dBackward: bit-exact against the oracle's restatement of the reference's deterministic
    templates (size-ratio and user scales), NCHW and NHWC, and reproducible from run to run"""
    import torch
    rng = np.random.default_rng(500 + int(channels_last))
    cases = [((2, 3, 5, 7), (10, 14), False, 0.0, 0.0), ((1, 4, 8, 8), (3, 5), True, 0.0, 0.0),
             ((2, 2, 16, 16), (33, 47), False, 0.0, 0.0), ((1, 5, 1, 5), (4, 10), True, 0.0, 0.0),
             ((1, 2, 4, 6), (10, 10), False, 2.5, 1.7), ((2, 1, 8, 8), (4, 3), False, 0.6, 0.45),
             ((1, 3, 6, 6), (6, 6), False, 0.0, 0.0), ((1, 8, 56, 56), (112, 112), False, 2.0, 2.0),
             # several column tiles and ragged row tiles of the LDS variant; an odd incoming width (16-bit types
             # then take the gather kernel); a x20 upscale whose tile exceeds the LDS capacity; a strong downscale
             ((1, 2, 37, 300), (75, 610), True, 0.0, 0.0), ((2, 1, 19, 131), (40, 263), False, 0.0, 0.0),
             ((1, 1, 9, 130), (180, 2600), False, 0.0, 0.0), ((1, 2, 90, 260), (11, 40), True, 0.0, 0.0),
             # channel counts whose channels-last rows span several column tiles with taps 3, 16 and 40 elements apart
             ((2, 3, 21, 131), (40, 262), False, 0.0, 0.0), ((1, 16, 9, 40), (20, 85), True, 0.0, 0.0),
             ((1, 40, 6, 12), (13, 30), False, 0.0, 0.0)]
    for in_shape, (Ho, Wo), align, sh, sw in cases:
        N, C, H, W = in_shape
        g = I.cast_np(rng.standard_normal((N, C, Ho, Wo)).astype(np.float32), dtype)
        gin = np.ascontiguousarray(g.transpose(0, 2, 3, 1)) if channels_last else g
        isz = (N, H, W, C) if channels_last else (N, C, H, W)
        ref = oracle.upsample_bilinear2d_backward(gin, (H, W), align, channels_last=channels_last,
                                                  dtype=I.oracle_code(dtype), scales_h=sh, scales_w=sw)
        gt = I.to_torch(gin, dtype, device)
        y1 = I.from_torch(aclnn.upsample_bilinear2d_backward(gt, isz, align, sh, sw, channels_last=channels_last), dtype)
        y2 = I.from_torch(aclnn.upsample_bilinear2d_backward(gt, isz, align, sh, sw, channels_last=channels_last), dtype)
        torch.cuda.synchronize()
        view = np.uint32 if dtype == "fp32" else np.uint16
        assert np.array_equal(y1.view(view), ref.view(view)), (in_shape, Ho, Wo, align, sh, sw, dtype, channels_last)
        assert np.array_equal(y1.view(view), y2.view(view))


def test_upsample_backward_fp32_into_fp16(oracle, device, aclnn):
    """a FLOAT gradient reduced into a FLOAT16 result, and a strided gradient view"""
    import torch
    rng = np.random.default_rng(510)
    g = rng.standard_normal((2, 3, 12, 10)).astype(np.float32)
    ref = oracle.upsample_bilinear2d_backward(g, (6, 5), False, dtype=oracle.F32, out_dtype=oracle.F16,
                                              out_numpy_dtype=np.float16)
    y = aclnn.upsample_bilinear2d_backward(torch.from_numpy(g).to(device), (2, 3, 6, 5), False, out_dtype=torch.float16)
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy().view(np.uint16), ref.view(np.uint16))
    big = torch.from_numpy(rng.standard_normal((2, 3, 12, 20)).astype(np.float32)).to(device)
    gv = big[:, :, :, ::2]
    y = aclnn.upsample_bilinear2d_backward(gv, (2, 3, 6, 5), False)
    torch.cuda.synchronize()
    ref = oracle.upsample_bilinear2d_backward(gv.contiguous().cpu().numpy(), (6, 5), False)
    assert np.array_equal(y.cpu().numpy(), ref)


def _bits(a, dtype):
    return a.view(np.uint32 if dtype == "fp32" else np.uint16)


@pytest.mark.parametrize("dtype", I.DTYPES)
@pytest.mark.parametrize("interp", [0, 1])
def test_grid_sampler3d(oracle, device, aclnn, dtype, interp):
    """aclnnGridSampler3D against the oracle, bit for bit: every padding and alignment, grids reaching well outside
    the volume, special values (NaN, infinities, huge and tie coordinates), single-voxel axes"""
    torch = _torch()
    rng = np.random.default_rng(500 + interp)
    shapes = [(2, 3, 5, 6, 7, 4, 5, 9), (1, 8, 1, 1, 1, 2, 2, 2), (1, 2, 9, 3, 1, 3, 7, 5), (2, 1, 2, 17, 33, 6, 3, 70),
              (1, 20, 4, 4, 4, 1, 1, 3)]
    for (N, C, D, H, W, Do, Ho, Wo) in shapes:
        x = I.cast_np(rng.standard_normal((N, C, D, H, W)).astype(np.float32), dtype)
        g32 = rng.uniform(-2.5, 2.5, (N, Do, Ho, Wo, 3)).astype(np.float32)
        flat = g32.reshape(-1, 3)
        special = np.array([np.nan, np.inf, -np.inf, 1e30, -1e30, 1.0, -1.0, 0.0, 3e9, 0.5], np.float32)
        k = min(len(special), flat.shape[0])
        for j in range(k):
            flat[j, j % 3] = special[j]
        g = I.cast_np(g32, dtype)
        for pad in range(3):
            for align in (False, True):
                ref = oracle.grid_sampler3d(x, g, interp, pad, align, dtype=I.oracle_code(dtype))
                y = aclnn.grid_sampler3d(I.to_torch(x, dtype, device), I.to_torch(g, dtype, device), interp, pad, align)
                torch.cuda.synchronize()
                got = I.from_torch(y, dtype)
                rn = np.isnan(I.as_f32(ref, dtype))
                assert np.array_equal(np.isnan(I.as_f32(got, dtype)), rn), (N, C, D, H, W, pad, align)
                assert np.array_equal(np.where(rn, 0, _bits(got, dtype)), np.where(rn, 0, _bits(ref, dtype))), \
                    (N, C, D, H, W, Do, Ho, Wo, pad, align)


@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_grid_sampler2d_box_variant(oracle, device, aclnn, dtype, interp):
    """Samples of 16-bit elements on planes beyond the LDS variants (80 KB), every interpolation mode: a tile of 32 x 16 output pixels copies
    the box of input pixels it reads into LDS.  Smooth warps (boxes that fit), scattered points and strong
    minification (boxes that do not: pair loads from global memory), a batch item whose points all lie outside the
    image, special grid values, tiles cut by the right and lower edge, channel counts that are not whole groups of
    four, few tiles (runs of channels to different workgroups); every padding and alignment; bit for bit the oracle"""
    torch = _torch()
    rng = np.random.default_rng(640 + interp)
    cases = [
        # N, C, H, W, Ho, Wo, kind
        (2, 5, 208, 200, 70, 100, "affine"),
        (1, 9, 256, 168, 48, 64, "affine"),
        (2, 3, 208, 200, 64, 66, "scattered"),
        (1, 4, 600, 136, 40, 96, "minify"),
        (3, 6, 208, 208, 33, 70, "mixed"),
    ]
    for (N, C, H, W, Ho, Wo, kind) in cases:
        x = I.cast_np(rng.standard_normal((N, C, H, W)).astype(np.float32), dtype)
        if kind == "scattered":
            g32 = rng.uniform(-1.2, 1.2, (N, Ho, Wo, 2)).astype(np.float32)
        elif kind == "minify":
            g32 = I.affine_grid(rng, N, Ho, Wo, max_deg=80.0, scale=(0.9, 1.1))  # a tile spans hundreds of input rows
        else:
            g32 = I.affine_grid(rng, N, Ho, Wo)
        if kind == "mixed":
            g32[1] = rng.uniform(-1.2, 1.2, (Ho, Wo, 2)).astype(np.float32)  # one item scattered
            g32[2] = 3.0 + g32[2]                                            # one item outside the image altogether
        flat = g32.reshape(-1, 2)
        special = I.special_grid_values()
        at = rng.integers(0, flat.shape[0], len(special))
        flat[at, rng.integers(0, 2, len(special))] = special
        g = I.cast_np(g32, dtype)
        for pad in range(3):
            for align in (False, True):
                tx, tg = I.to_torch(x, dtype, device), I.to_torch(g, dtype, device)
                ty = torch.empty((N, C, Ho, Wo), dtype=tx.dtype, device=device)
                hs = [aclnn.tensor_handle(t) for t in (tx, tg, ty)]
                st, _, ex = aclnn.get_workspace_size_grid_sampler2d(hs[0], hs[1], interp, pad, align, hs[2])
                assert st == 0 and aclnn.executor_variant(ex) == "box_lds", (N, C, H, W, Ho, Wo)
                aclnn.destroy_executor(ex)
                for h in hs:
                    aclnn.destroy_tensor(h)
                ref = oracle.grid_sampler2d(x, g, interp, pad, align, dtype=I.oracle_code(dtype))
                y = aclnn.grid_sampler2d(tx, tg, interp, pad, align)
                torch.cuda.synchronize()
                got = I.from_torch(y, dtype)
                rn = np.isnan(I.as_f32(ref, dtype))
                assert np.array_equal(np.isnan(I.as_f32(got, dtype)), rn), (kind, interp, N, C, H, W, pad, align)
                assert np.array_equal(np.where(rn, 0, _bits(got, dtype)), np.where(rn, 0, _bits(ref, dtype))), \
                    (kind, interp, N, C, H, W, Ho, Wo, pad, align)
    # shapes the variant leaves to the direct kernel: rows of odd length, rows that are not whole 16-byte units
    for (H, W, Ho, Wo) in [(208, 200, 64, 65), (208, 204, 64, 64)]:
        tx = I.to_torch(I.cast_np(rng.standard_normal((1, 2, H, W)).astype(np.float32), dtype), dtype, device)
        tg = I.to_torch(I.cast_np(I.affine_grid(rng, 1, Ho, Wo), dtype), dtype, device)
        ty = torch.empty((1, 2, Ho, Wo), dtype=tx.dtype, device=device)
        hs = [aclnn.tensor_handle(t) for t in (tx, tg, ty)]
        st, _, ex = aclnn.get_workspace_size_grid_sampler2d(hs[0], hs[1], interp, 0, False, hs[2])
        assert st == 0 and aclnn.executor_variant(ex) == "direct", (H, W, Ho, Wo)
        aclnn.destroy_executor(ex)
        for h in hs:
            aclnn.destroy_tensor(h)


def test_grid_sampler3d_layouts_and_views(oracle, device, aclnn):
    """NDHWC tensors (permuted operands), strided NCDHW views, the reference's own example shape"""
    torch = _torch()
    rng = np.random.default_rng(510)
    N, C, D, H, W, Do, Ho, Wo = 2, 5, 4, 6, 7, 3, 5, 8
    x = rng.standard_normal((N, C, D, H, W)).astype(np.float32)
    g = rng.uniform(-1.3, 1.3, (N, Do, Ho, Wo, 3)).astype(np.float32)
    for interp, pad, align in [(0, 0, False), (0, 2, True), (1, 1, False)]:
        ref = oracle.grid_sampler3d(x, g, interp, pad, align)
        # channels-last extents (N,D,H,W,C) in and out
        xl = torch.from_numpy(np.ascontiguousarray(x.transpose(0, 2, 3, 4, 1))).to(device)
        y = aclnn.grid_sampler3d(xl, torch.from_numpy(g).to(device), interp, pad, align, channels_last=True)
        torch.cuda.synchronize()
        assert y.shape == (N, Do, Ho, Wo, C)
        assert np.array_equal(y.cpu().numpy().transpose(0, 4, 1, 2, 3), ref)
        # NCDHW views: input a transposed view, grid a slice with a storage offset, out a strided slice
        xv = torch.from_numpy(np.ascontiguousarray(x.transpose(0, 1, 2, 4, 3))).to(device).transpose(3, 4)
        assert not xv.is_contiguous()
        gbig = torch.zeros((N + 1, Do, Ho, Wo, 3), device=device)
        gbig[1:] = torch.from_numpy(g).to(device)
        obig = torch.full((N, C, Do, Ho, Wo + 4), -3.0, device=device)
        out = aclnn.grid_sampler3d(xv, gbig[1:], interp, pad, align, out=obig[..., 2:2 + Wo])
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy(), ref)
        rest = obig.cpu().numpy()
        assert (rest[..., :2] == -3.0).all() and (rest[..., 2 + Wo:] == -3.0).all()
    # the shape of the reference's special case (aclnn_grid_sampler3d.cpp:277-312): 22 x 4 x 16 x 64 x 64, fp16,
    # against live torch on the host through the oracle at a tolerance-free comparison with the oracle only
    x = I.cast_np(rng.standard_normal((22, 4, 16, 64, 64)).astype(np.float32), "fp16")
    g = I.cast_np(rng.uniform(-1.1, 1.1, (22, 16, 64, 64, 3)).astype(np.float32), "fp16")
    ref = oracle.grid_sampler3d(x, g, 0, 0, False)
    y = aclnn.grid_sampler3d(I.to_torch(x, "fp16", device), I.to_torch(g, "fp16", device), 0, 0, False)
    torch.cuda.synchronize()
    assert np.array_equal(I.from_torch(y, "fp16").view(np.uint16), ref.view(np.uint16))


@pytest.mark.parametrize("dtype", I.DTYPES)
@pytest.mark.parametrize("interp", [0, 1, 2])
def test_grid_sampler2d_backward(oracle, device, aclnn, dtype, interp):
    """aclnnGridSampler2DBackward against the oracle, bit for bit, both gradients: every padding and alignment,
    several chunks of 256 points, planes larger than one LDS band, points piling up on few texels, special grid
    values"""
    torch = _torch()
    rng = np.random.default_rng(600 + interp)
    shapes = [(2, 3, 5, 8, 3, 3), (1, 2, 9, 11, 23, 29), (2, 1, 70, 80, 20, 30), (1, 4, 1, 1, 17, 31),
              (1, 2, 3, 2, 40, 40)]
    for (N, C, H, W, Ho, Wo) in shapes:
        x = I.cast_np(rng.standard_normal((N, C, H, W)).astype(np.float32), dtype)
        g32 = rng.uniform(-1.5, 1.5, (N, Ho, Wo, 2)).astype(np.float32)
        flat = g32.reshape(-1, 2)
        special = np.array([np.nan, np.inf, -np.inf, 1e30, -1e30, 1.0, -1.0, 0.0], np.float32)
        for j in range(min(len(special), flat.shape[0])):
            flat[j, j % 2] = special[j]
        g = I.cast_np(g32, dtype)
        go = I.cast_np(rng.standard_normal((N, C, Ho, Wo)).astype(np.float32), dtype)
        for pad in range(3):
            for align in (False, True):
                rdx, rdg = oracle.grid_sampler2d_backward(go, x, g, interp, pad, align, dtype=I.oracle_code(dtype))
                dx, dg = aclnn.grid_sampler2d_backward(I.to_torch(go, dtype, device), I.to_torch(x, dtype, device),
                                                       I.to_torch(g, dtype, device), interp, pad, align)
                torch.cuda.synchronize()
                for got, ref, what in ((I.from_torch(dx, dtype), rdx, "dx"), (I.from_torch(dg, dtype), rdg, "dgrid")):
                    rn = np.isnan(I.as_f32(ref, dtype))
                    assert np.array_equal(np.isnan(I.as_f32(got, dtype)), rn), (what, N, C, H, W, pad, align)
                    assert np.array_equal(np.where(rn, 0, _bits(got, dtype)), np.where(rn, 0, _bits(ref, dtype))), \
                        (what, N, C, H, W, Ho, Wo, pad, align)


@pytest.mark.parametrize("dtype", I.DTYPES)
def test_grid_sampler2d_backward_grid_gradient_lds_variant(oracle, device, aclnn, dtype):
    """The grid gradient with the input planes staged through LDS (enough workgroups of 256 points, 16 channels or
    more, planes of whole 4 KiB): bit for bit the oracle's channel-ordered sums, every padding and alignment, partial last tile, batch counts
    that are and are not a multiple of 8, corners outside the image next to non-finite gradOutput values, special
    grid values, every ring class"""
    torch = _torch()
    rng = np.random.default_rng(620)
    # planes of 4, 8, 12 and 32 KiB for 16-bit elements, twice that for fp32 (the 32 KiB shape is halved): every ring
    # class and several copy counts per loader
    shapes = [(8, 16, 32, 64, 64, 64), (3, 17, 64, 64, 108, 104), (8, 19, 64, 96, 64, 64),
              (2, 16, 64 if dtype == "fp32" else 128, 128, 128, 128)]
    for (N, C, H, W, Ho, Wo) in shapes:
        x = I.cast_np(rng.standard_normal((N, C, H, W)).astype(np.float32), dtype)
        g32 = rng.uniform(-1.3, 1.3, (N, Ho, Wo, 2)).astype(np.float32)
        flat = g32.reshape(-1, 2)
        special = np.array([np.nan, np.inf, -np.inf, 1e30, -1e30, 1.0, -1.0, 0.0], np.float32)
        for j in range(len(special)):
            flat[j, j % 2] = special[j]
        g = I.cast_np(g32, dtype)
        go32 = rng.standard_normal((N, C, Ho, Wo)).astype(np.float32)
        # non-finite incoming gradients, some at points whose corners fall outside the image
        gof = go32.reshape(N, C, -1)
        outside = np.argwhere(np.abs(g32.reshape(N, -1, 2)).max(axis=2) > 1.0)
        for j, (n_, p_) in enumerate(outside[:12]):
            gof[n_, j % C, p_] = (np.inf, -np.inf, np.nan)[j % 3]
        gof[0, 1, 5] = np.inf
        go = I.cast_np(go32, dtype)
        for pad in range(3):
            for align in (False, True):
                tensors = [I.to_torch(v, dtype, device) for v in (go, x, g)]
                hs = [aclnn.tensor_handle(t) for t in tensors + [tensors[1], tensors[2]]]
                m = aclnn.create_bool_array([True, True])
                st, ws, ex = aclnn.get_workspace_size_grid_sampler2d_backward(hs[0], hs[1], hs[2], 0, pad, align, m,
                                                                              hs[3], hs[4])
                # the input gradient takes its list variant where an item's points fit one sorting workgroup and a
                # gradOutput plane fits a slot of the ring
                lists = Ho * Wo <= 16384 and Ho * Wo * (4 if dtype == "fp32" else 2) <= 32768
                assert st == 0 and aclnn.executor_variant(ex) == ("gs2d_grad_lists_lds" if lists
                                                                   else "gs2d_grad_ordered_lds")
                assert aclnn.destroy_executor(ex) == 0
                aclnn.destroy_bool_array(m)
                for h in hs:
                    aclnn.destroy_tensor(h)
                rdx, rdg = oracle.grid_sampler2d_backward(go, x, g, 0, pad, align, dtype=I.oracle_code(dtype))
                dx, dg = aclnn.grid_sampler2d_backward(I.to_torch(go, dtype, device), I.to_torch(x, dtype, device),
                                                       I.to_torch(g, dtype, device), 0, pad, align)
                torch.cuda.synchronize()
                for got, ref, what in ((I.from_torch(dx, dtype), rdx, "dx"), (I.from_torch(dg, dtype), rdg, "dgrid")):
                    rn = np.isnan(I.as_f32(ref, dtype))
                    assert np.array_equal(np.isnan(I.as_f32(got, dtype)), rn), (what, N, C, H, W, pad, align)
                    assert np.array_equal(np.where(rn, 0, _bits(got, dtype)), np.where(rn, 0, _bits(ref, dtype))), \
                        (what, N, C, H, W, Ho, Wo, pad, align)


@pytest.mark.parametrize("dtype", I.DTYPES)
def test_grid_sampler2d_backward_grid_gradient_box_variant(oracle, device, aclnn, dtype):
    """The grid gradient with two lanes per grid point and only the box of each plane staged that a 16 x 16 block of
    grid points reaches (even channel counts, outputs of whole 16 x 16 blocks): smooth grids whose boxes are a small
    part of the plane, a batch item whose points all lie outside the image (empty boxes), blocks that straddle the
    image's edge, random grids (the box is the whole plane), special grid values, both plane size classes, channel
    counts that leave a partial turn of the unrolled loop, every padding and alignment"""
    torch = _torch()
    rng = np.random.default_rng(650)
    shapes = [(8, 16, 64, 64, 64, 64), (8, 22, 32, 64, 48, 96), (4, 36, 64, 128 if dtype != "fp32" else 64, 64, 128)]
    for (N, C, H, W, Ho, Wo) in shapes:
        x = I.cast_np(rng.standard_normal((N, C, H, W)).astype(np.float32), dtype)
        g32 = I.affine_grid(rng, N, Ho, Wo)
        g32[1] = g32[1] * 0.2 + 3.0                                   # every point outside the image
        g32[2] = rng.uniform(-1.2, 1.2, (Ho, Wo, 2)).astype(np.float32)  # the box is the whole plane
        g32[3] = g32[3] * 0.3 + 0.85                                  # a small patch across the image's corner
        flat = g32[0].reshape(-1, 2)
        special = np.array([np.nan, np.inf, -np.inf, 1e30, -1e30, 1.0, -1.0, 0.0], np.float32)
        for j in range(len(special)):
            flat[17 * j + 3, j % 2] = special[j]
        g = I.cast_np(g32, dtype)
        go32 = rng.standard_normal((N, C, Ho, Wo)).astype(np.float32)
        go32 += np.arange(C, dtype=np.float32).reshape(1, C, 1, 1) / 8
        go32[0, 1, 0, 5] = np.inf
        go32[3, C - 1, Ho - 1, Wo - 1] = np.nan
        go = I.cast_np(go32, dtype)
        for pad in range(3):
            for align in (False, True):
                rdx, rdg = oracle.grid_sampler2d_backward(go, x, g, 0, pad, align, dtype=I.oracle_code(dtype))
                dx, dg = aclnn.grid_sampler2d_backward(I.to_torch(go, dtype, device), I.to_torch(x, dtype, device),
                                                       I.to_torch(g, dtype, device), 0, pad, align)
                torch.cuda.synchronize()
                for got, ref, what in ((I.from_torch(dx, dtype), rdx, "dx"), (I.from_torch(dg, dtype), rdg, "dgrid")):
                    rn = np.isnan(I.as_f32(ref, dtype))
                    assert np.array_equal(np.isnan(I.as_f32(got, dtype)), rn), (what, N, C, H, W, pad, align)
                    assert np.array_equal(np.where(rn, 0, _bits(got, dtype)), np.where(rn, 0, _bits(ref, dtype))), \
                        (what, N, C, H, W, Ho, Wo, pad, align)


@pytest.mark.parametrize("dtype", ("fp16", "fp32"))
def test_grid_sampler2d_backward_launch_of_two_workgroups_per_cu(oracle, device, aclnn, dtype):
    """a shape whose last kernel (the gather over the contribution lists) is launched as exactly two workgroups per CU
    of a 256-CU part: the channel blocks handed out first take 10 channels, the others 6, in units dealt out in turn;
    every channel's gradient must still be written once"""
    torch = _torch()
    rng = np.random.default_rng(640)
    N, C, H, W, Ho, Wo = 16, 64, 64, 64, 64, 64
    x = I.cast_np(rng.standard_normal((N, C, H, W)).astype(np.float32), dtype)
    g = I.cast_np(I.affine_grid(rng, N, Ho, Wo), dtype)
    go32 = rng.standard_normal((N, C, Ho, Wo)).astype(np.float32)
    # every channel different from its neighbours by a constant, so that a channel taken twice or skipped shows
    go32 += np.arange(C, dtype=np.float32).reshape(1, C, 1, 1) / 4
    go = I.cast_np(go32, dtype)
    tensors = [I.to_torch(v, dtype, device) for v in (go, x, g)]
    rdx, rdg = oracle.grid_sampler2d_backward(go, x, g, 0, 0, False, dtype=I.oracle_code(dtype))
    dx, dg = aclnn.grid_sampler2d_backward(*tensors, 0, 0, False)
    torch.cuda.synchronize()
    for got, ref, what in ((I.from_torch(dx, dtype), rdx, "dx"), (I.from_torch(dg, dtype), rdg, "dgrid")):
        assert np.array_equal(_bits(got, dtype), _bits(ref, dtype)), what


@pytest.mark.parametrize("dtype", I.DTYPES)
def test_grid_sampler2d_backward_input_gradient_list_variant(oracle, device, aclnn, dtype):
    """The input gradient as a gather over per-element contribution lists (8 channels or more, up to 16384 grid
    points per item and 32 KiB per gradOutput plane): bit for bit the oracle's chunk / corner / point order, with points piling up on few elements
    (lists far longer than the eight entries a lane holds), elements nobody reaches, points outside the image,
    non-finite gradOutput next to corners outside the image, every padding and alignment, channel counts that are not
    a multiple of the planes staged together, plane sizes that leave a partial element tile, batches where one item
    takes the sorted path and the others the slots"""
    torch = _torch()
    rng = np.random.default_rng(630)
    for (N, C, H, W, Ho, Wo, kind) in [(2, 9, 7, 9, 24, 24, "pile"), (3, 8, 30, 40, 64, 64, "random"),
                                        (1, 13, 64, 64, 90, 88, "smooth"), (2, 8, 20, 20, 32, 64, "outside"),
                                        (1, 8, 40, 44, 100, 64 if dtype == "fp32" else 128, "random"),
                                        (3, 8, 48, 48, 40, 40, "mixed"), (8, 16, 64, 64, 64, 64, "mixed")]:
        x = I.cast_np(rng.standard_normal((N, C, H, W)).astype(np.float32), dtype)
        if kind == "pile":
            g32 = rng.choice(np.array([-0.93, -0.31, 0.02, 0.4, 0.77], np.float32), (N, Ho, Wo, 2))
        elif kind == "smooth":
            ys, xs = np.meshgrid(np.linspace(-1.05, 1.05, Ho), np.linspace(-1.05, 1.05, Wo), indexing="ij")
            g32 = np.broadcast_to(np.stack([xs * 0.9 + ys * 0.1, ys * 0.95 - xs * 0.05], -1), (N, Ho, Wo, 2))
            g32 = np.ascontiguousarray(g32, dtype=np.float32)
        elif kind == "outside":
            g32 = rng.uniform(-2.5, 2.5, (N, Ho, Wo, 2)).astype(np.float32)
        elif kind == "mixed":
            # one item whose points pile up (its cells overflow their slots, the item is sorted) among items whose
            # cells hold a few points each (lists straight from the slots); several workgroups of points per item
            g32 = rng.uniform(-1.0, 1.0, (N, Ho, Wo, 2)).astype(np.float32)
            g32[N // 2] = rng.choice(np.array([-0.93, -0.31, 0.02, 0.4, 0.77], np.float32), (Ho, Wo, 2))
        else:
            g32 = rng.uniform(-1.2, 1.2, (N, Ho, Wo, 2)).astype(np.float32)
        flat = g32.reshape(-1, 2)
        special = np.array([np.nan, np.inf, -np.inf, 1e30, -1e30, 1.0, -1.0, 0.0], np.float32)
        for j in range(len(special)):
            flat[j, j % 2] = special[j]
        g = I.cast_np(g32, dtype)
        go32 = rng.standard_normal((N, C, Ho, Wo)).astype(np.float32)
        gof = go32.reshape(N, C, -1)
        edge = np.argwhere(np.abs(g32.reshape(N, -1, 2)).max(axis=2) > 0.97)
        for j, (n_, p_) in enumerate(edge[:10]):
            gof[n_, j % C, p_] = (np.inf, -np.inf, np.nan)[j % 3]
        go = I.cast_np(go32, dtype)
        for pad in range(3):
            for align in (False, True):
                tensors = [I.to_torch(v, dtype, device) for v in (go, x, g)]
                hs = [aclnn.tensor_handle(t) for t in tensors + [tensors[1], tensors[2]]]
                m = aclnn.create_bool_array([True, True])
                st, ws, ex = aclnn.get_workspace_size_grid_sampler2d_backward(hs[0], hs[1], hs[2], 0, pad, align, m,
                                                                              hs[3], hs[4])
                assert st == 0 and ws > 0 and aclnn.executor_variant(ex).startswith("gs2d_grad_lists")
                assert aclnn.destroy_executor(ex) == 0
                aclnn.destroy_bool_array(m)
                for h in hs:
                    aclnn.destroy_tensor(h)
                rdx, rdg = oracle.grid_sampler2d_backward(go, x, g, 0, pad, align, dtype=I.oracle_code(dtype))
                dx, dg = aclnn.grid_sampler2d_backward(*tensors, 0, pad, align)
                torch.cuda.synchronize()
                for got, ref, what in ((I.from_torch(dx, dtype), rdx, "dx"), (I.from_torch(dg, dtype), rdg, "dgrid")):
                    rn = np.isnan(I.as_f32(ref, dtype))
                    assert np.array_equal(np.isnan(I.as_f32(got, dtype)), rn), (what, kind, pad, align)
                    assert np.array_equal(np.where(rn, 0, _bits(got, dtype)), np.where(rn, 0, _bits(ref, dtype))), \
                        (what, kind, N, C, H, W, Ho, Wo, pad, align)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_grid_sampler2d_backward_interleaved_planes(oracle, device, aclnn, dtype):
    """16-bit gradOutput planes staged interleaved by the gather over the contribution lists: four channels per step
    (planes of up to 8 KiB) and two (up to 16 KiB), channel counts that leave one, two or three planes for the last
    step, planes that are not whole loads for every loader lane, a plane whose first point holds a non-finite value
    (a contribution that a lane does not have must not read it), lists longer than a lane holds; bit for bit"""
    torch = _torch()
    rng = np.random.default_rng(650)
    for (N, C, H, W, Ho, Wo, kind) in [(2, 9, 20, 24, 24, 40, "random"), (2, 10, 20, 24, 24, 40, "smooth"),
                                        (3, 11, 33, 31, 40, 40, "smooth"), (1, 9, 64, 64, 72, 96, "smooth"),
                                        (2, 12, 48, 40, 64, 128, "random"), (2, 16, 12, 12, 40, 48, "pile"),
                                        (16, 24, 64, 64, 64, 64, "smooth")]:
        x = I.cast_np(rng.standard_normal((N, C, H, W)).astype(np.float32), dtype)
        if kind == "smooth":
            g32 = I.affine_grid(rng, N, Ho, Wo)
        elif kind == "pile":
            g32 = rng.choice(np.array([-0.9, -0.3, 0.05, 0.45, 0.8], np.float32), (N, Ho, Wo, 2))
        else:
            g32 = rng.uniform(-1.1, 1.1, (N, Ho, Wo, 2)).astype(np.float32)
        g = I.cast_np(g32, dtype)
        go32 = rng.standard_normal((N, C, Ho, Wo)).astype(np.float32)
        go32 += np.arange(C, dtype=np.float32).reshape(1, C, 1, 1) / 4
        # the first point of some planes is infinite; its own grid point is moved far outside the image, so that no
        # element takes it and the reference's result stays finite
        go32[:, ::3, 0, 0] = np.inf
        g32[:, 0, 0, :] = 5.0
        g = I.cast_np(g32, dtype)
        go = I.cast_np(go32, dtype)
        tensors = [I.to_torch(v, dtype, device) for v in (go, x, g)]
        rdx, rdg = oracle.grid_sampler2d_backward(go, x, g, 0, 0, False, dtype=I.oracle_code(dtype))
        assert np.isfinite(I.as_f32(rdx, dtype)).all()
        dx, dg = aclnn.grid_sampler2d_backward(*tensors, 0, 0, False)
        torch.cuda.synchronize()
        for got, ref, what in ((I.from_torch(dx, dtype), rdx, "dx"), (I.from_torch(dg, dtype), rdg, "dgrid")):
            assert np.array_equal(_bits(got, dtype), _bits(ref, dtype)), (what, kind, N, C, H, W, Ho, Wo)


def test_grid_sampler2d_backward_mask_views_and_torch(oracle, device, aclnn):
    torch = _torch()
    import torch.nn.functional as F
    rng = np.random.default_rng(610)
    N, C, H, W, Ho, Wo = 2, 3, 12, 10, 9, 14
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    g = rng.uniform(-1.2, 1.2, (N, Ho, Wo, 2)).astype(np.float32)
    go = rng.standard_normal((N, C, Ho, Wo)).astype(np.float32)
    xt, gt, got = (torch.from_numpy(a).to(device) for a in (x, g, go))
    # masked outputs stay untouched
    dx = torch.full((N, C, H, W), 7.0, device=device)
    dg = torch.full((N, Ho, Wo, 2), 7.0, device=device)
    aclnn.grid_sampler2d_backward(got, xt, gt, 0, 0, False, (True, False), dx, dg)
    torch.cuda.synchronize()
    rdx, rdg = oracle.grid_sampler2d_backward(go, x, g, 0, 0, False)
    assert np.array_equal(dx.cpu().numpy(), rdx) and (dg == 7.0).all()
    dx.fill_(7.0)
    aclnn.grid_sampler2d_backward(got, xt, gt, 0, 0, False, (False, True), dx, dg)
    torch.cuda.synchronize()
    assert np.array_equal(dg.cpu().numpy(), rdg) and (dx == 7.0).all()
    # strided views on both sides
    xv = torch.from_numpy(np.ascontiguousarray(x.transpose(0, 1, 3, 2))).to(device).transpose(2, 3)
    dxbig = torch.full((N, C, H, W + 3), -1.0, device=device)
    dgbig = torch.full((N, Ho, Wo, 4), -1.0, device=device)
    aclnn.grid_sampler2d_backward(got, xv, gt, 0, 1, True, (True, True), dxbig[..., 1:1 + W], dgbig[..., 1:3])
    torch.cuda.synchronize()
    rdx, rdg = oracle.grid_sampler2d_backward(go, x, g, 0, 1, True)
    assert np.array_equal(dxbig[..., 1:1 + W].cpu().numpy(), rdx) and np.array_equal(dgbig[..., 1:3].cpu().numpy(), rdg)
    assert (dxbig[..., 0] == -1.0).all() and (dgbig[..., 3] == -1.0).all()
    # live torch autograd on the device (tolerance: another summation order)
    for mode, m in (("bilinear", 0), ("bicubic", 2)):
        xa, ga = xt.clone().requires_grad_(True), gt.clone().requires_grad_(True)
        F.grid_sample(xa, ga, mode=mode, padding_mode="border", align_corners=False).backward(got)
        dx, dg = aclnn.grid_sampler2d_backward(got, xt, gt, m, 1, False)
        torch.cuda.synchronize()
        assert (dx - xa.grad).abs().max().item() <= 1e-4
        assert ((dg - ga.grad).abs() > 1e-3).float().mean().item() <= 0.02


@pytest.mark.parametrize("dtype", I.DTYPES)
@pytest.mark.parametrize("interp", [0, 1])
def test_grid_sampler3d_backward(oracle, device, aclnn, dtype, interp):
    """aclnnGridSampler3DBackward against the oracle, bit for bit, both gradients: every padding and alignment,
    several chunks of 256 points, volumes larger than one LDS band, points piling up on few voxels, special grid
    values, channel counts around the group size"""
    torch = _torch()
    rng = np.random.default_rng(700 + interp)
    shapes = [(2, 3, 2, 5, 8, 2, 3, 3), (1, 2, 4, 9, 11, 5, 7, 9), (2, 1, 30, 20, 17, 6, 20, 10),
              (1, 5, 1, 1, 1, 3, 17, 31), (1, 2, 2, 3, 2, 10, 12, 10), (1, 4, 3, 3, 3, 1, 1, 1)]
    for (N, C, D, H, W, Do, Ho, Wo) in shapes:
        x = I.cast_np(rng.standard_normal((N, C, D, H, W)).astype(np.float32), dtype)
        g32 = rng.uniform(-1.5, 1.5, (N, Do, Ho, Wo, 3)).astype(np.float32)
        flat = g32.reshape(-1, 3)
        special = np.array([np.nan, np.inf, -np.inf, 1e30, -1e30, 1.0, -1.0, 0.0], np.float32)
        for j in range(min(len(special), flat.shape[0])):
            flat[j, j % 3] = special[j]
        g = I.cast_np(g32, dtype)
        go = I.cast_np(rng.standard_normal((N, C, Do, Ho, Wo)).astype(np.float32), dtype)
        for pad in range(3):
            for align in (False, True):
                rdx, rdg = oracle.grid_sampler3d_backward(go, x, g, interp, pad, align, dtype=I.oracle_code(dtype))
                dx, dg = aclnn.grid_sampler3d_backward(I.to_torch(go, dtype, device), I.to_torch(x, dtype, device),
                                                       I.to_torch(g, dtype, device), interp, pad, align)
                torch.cuda.synchronize()
                for got, ref, what in ((I.from_torch(dx, dtype), rdx, "dx"), (I.from_torch(dg, dtype), rdg, "dgrid")):
                    rn = np.isnan(I.as_f32(ref, dtype))
                    assert np.array_equal(np.isnan(I.as_f32(got, dtype)), rn), (what, N, C, D, H, W, pad, align)
                    assert np.array_equal(np.where(rn, 0, _bits(got, dtype)), np.where(rn, 0, _bits(ref, dtype))), \
                        (what, N, C, D, H, W, Do, Ho, Wo, pad, align)


@pytest.mark.parametrize("dtype", I.DTYPES)
def test_grid_sampler3d_backward_gather_variant(oracle, device, aclnn, dtype, monkeypatch):
    """The input gradient of the 3-D sampler as a gather over every voxel's contributions: bit for bit the oracle's
    (chunk, corner, point) order on jittered lattices (about eight contributions per voxel), on denser grids (lists of
    more than sixteen entries, some items handed to the ordered kernel because a voxel has more than 32), with one
    piled-up item among lattice items, with a cell that overflows its slots into the item's overflow list, with
    channel counts around the group of four, and with more items than cores
    (chunk boundaries that move from item to item).  Which items the gather did is read from the flag words it keeps
    in the workspace, which is handed over full of ones."""
    torch = _torch()
    rng = np.random.default_rng(720)
    code = I.oracle_code(dtype)
    esz = 4 if dtype == "fp32" else 2

    def lattice(N, Do, Ho, Wo, spread, jitter):
        ax = [np.linspace(-1 + 1 / n, 1 - 1 / n, n) for n in (Do, Ho, Wo)]
        gz, gy, gx = np.meshgrid(*ax, indexing="ij")
        base = np.stack([gx, gy, gz], -1)[None].astype(np.float32)
        g = base * rng.uniform(1 - spread, 1 + spread, (N, 1, 1, 1, 3)) + rng.uniform(-0.1, 0.1, (N, 1, 1, 1, 3))
        return (g + rng.normal(0, jitter, g.shape)).astype(np.float32)

    cases = [  # N, C, (D, H, W), (Do, Ho, Wo), kind, cores
        (3, 5, (6, 12, 10), (6, 12, 10), "lattice", 2),
        (2, 4, (5, 9, 33), (7, 12, 40), "dense", 64),
        (3, 1, (4, 8, 8), (4, 8, 8), "mixed", 64),
        (2, 3, (4, 8, 8), (4, 8, 8), "crowded", 64),
        (2, 6, (3, 20, 70), (3, 20, 70), "lattice", 64),
        (5, 2, (4, 6, 6), (5, 8, 8), "dense", 2),
        (5, 3, (5, 8, 8), (5, 8, 8), "lattice", 2),
    ]
    seen_gathered = seen_flagged = 0
    try:
        for (N, C, (D, H, W), (Do, Ho, Wo), kind, cores) in cases:
            aclnn.set_option("reference_cores", cores)
            oracle.set_reference_cores(cores)
            g32 = lattice(N, Do, Ho, Wo, 0.1, 0.03)
            if kind == "mixed":
                g32[1] = np.float32(0.1)  # every point of the item on one spot: lists far beyond what a voxel holds
            if kind == "crowded":
                # a lattice with a dozen points moved onto one spot: that cell overflows its eight slots and its voxels
                # find the rest in the item's overflow list; the item is still the gather's
                g32[:, 0, :2, :6] = np.float32(0.3)
            g = I.cast_np(g32, dtype)
            x = I.cast_np(rng.standard_normal((N, C, D, H, W)).astype(np.float32), dtype)
            go = I.cast_np(rng.standard_normal((N, C, Do, Ho, Wo)).astype(np.float32), dtype)
            points, cells, vol = Do * Ho * Wo, (D + 1) * (H + 1) * (W + 1), D * H * W
            for pad, align in ((0, False), (1, True), (2, False)):
                ws = torch.full((64 << 20,), 0xFF, dtype=torch.uint8, device=device)
                rdx, rdg = oracle.grid_sampler3d_backward(go, x, g, 0, pad, align, dtype=code)
                dx, dg = aclnn.grid_sampler3d_backward(I.to_torch(go, dtype, device), I.to_torch(x, dtype, device),
                                                       I.to_torch(g, dtype, device), 0, pad, align, workspace=ws)
                torch.cuda.synchronize()
                for got, ref, what in ((I.from_torch(dx, dtype), rdx, "dx"), (I.from_torch(dg, dtype), rdg, "dgrid")):
                    assert np.array_equal(_bits(got, dtype), _bits(ref, dtype)), (what, kind, N, C, D, H, W, pad, align)
                # the flag word of every item: first word of its scratch, behind the chunk spans (none for one band)
                per_core = (N + cores - 1) // cores if N > cores else 1
                chunks = ((255 if per_core > 1 else 0) + points + 255) // 256
                range_bytes = N * 2 * chunks * 4 if vol > 2048 else 0  # bands of 2048 voxels or more
                item_words = (((4 + cells + 3) // 4 * 4 + 4 * cells + 2048) * 4 + points * 8 * esz +
                              (C + 3) // 4 * points * 4 * esz + 15) // 16 * 4
                words = ws.view(torch.int32)
                flags = [int(words[(range_bytes + 255) // 256 * 64 + n * item_words].item()) for n in range(N)]
                assert all(f in (0, 1) for f in flags), flags
                # (border and reflection padding fold the points beyond the volume onto its faces, edges and corners,
                # which may crowd a cell there: only zeros padding keeps a lattice item's cells sparse for certain)
                if kind == "mixed" and pad == 0:
                    assert flags == [0, 1, 0], flags
                if kind == "lattice" and pad == 0:
                    assert flags == [0] * N, flags
                if kind == "crowded" and pad == 0:
                    assert flags == [0] * N, flags
                    overflowed = [int(words[(range_bytes + 255) // 256 * 64 + n * item_words + 1].item()) for n in range(N)]
                    assert all(o >= 4 for o in overflowed), overflowed
                seen_gathered += flags.count(0)
                seen_flagged += flags.count(1)
    finally:
        oracle.set_reference_cores(64)
        aclnn.set_option("reference_cores", 64)
    assert seen_gathered > 0 and seen_flagged > 0


def test_grid_sampler3d_backward_sparse_volume_takes_the_ordered_kernel(oracle, device, aclnn):
    """a volume sampled at few points (more than eight voxels per grid point) stays with the ordered kernel; forced
    either way the two variants give the oracle's bits"""
    torch = _torch()
    rng = np.random.default_rng(733)
    N, C, (D, H, W), (Do, Ho, Wo) = 2, 5, (12, 20, 24), (3, 9, 10)
    x = rng.standard_normal((N, C, D, H, W)).astype(np.float16)
    g = rng.uniform(-1.05, 1.05, (N, Do, Ho, Wo, 3)).astype(np.float16)
    go = rng.standard_normal((N, C, Do, Ho, Wo)).astype(np.float16)
    rdx, rdg = oracle.grid_sampler3d_backward(go, x, g, 0, 0, False)
    xt, gt, got = (torch.from_numpy(a).to(device) for a in (x, g, go))
    hs = [aclnn.tensor_handle(t, aclnn.ACL_FORMAT_NCDHW) for t in (got, xt)] + [aclnn.tensor_handle(gt)]
    hs += [aclnn.tensor_handle(torch.empty_like(xt), aclnn.ACL_FORMAT_NCDHW), aclnn.tensor_handle(torch.empty_like(gt))]
    mask = aclnn.create_bool_array([True, True])
    st, _, ex = aclnn.get_workspace_size_grid_sampler3d_backward(hs[0], hs[1], hs[2], 0, 0, False, mask, hs[3], hs[4])
    assert st == 0 and aclnn.executor_variant(ex) == "gs3d_grad_ordered"
    aclnn.destroy_executor(ex)
    for h in hs:
        aclnn.destroy_tensor(h)
    aclnn.destroy_bool_array(mask)
    for forced in (0, 1, 2):
        with aclnn.option("gs3d_grad_variant", forced):
            dx, dg = aclnn.grid_sampler3d_backward(got, xt, gt, 0, 0, False)
        torch.cuda.synchronize()
        assert np.array_equal(dx.cpu().numpy().view(np.uint16), rdx.view(np.uint16)), forced
        assert np.array_equal(dg.cpu().numpy().view(np.uint16), rdg.view(np.uint16)), forced


def test_grid_sampler3d_backward_core_split_mask_layouts_and_torch(oracle, device, aclnn, monkeypatch):
    torch = _torch()
    import torch.nn.functional as F
    rng = np.random.default_rng(710)
    # more batch items than cores of the reference device: a core walks several items as one run of points, which
    # moves the chunk boundaries of the later ones (300 points: item 1 of a core starts at thread 44)
    # the second volume spans two LDS bands, which brings in the per-chunk voxel spans
    for (N, C, D, H, W, Do, Ho, Wo) in [(5, 2, 2, 3, 3, 3, 10, 10), (5, 2, 3, 60, 50, 3, 10, 10)]:
        x = rng.standard_normal((N, C, D, H, W)).astype(np.float16)
        g = rng.uniform(-1.1, 1.1, (N, Do, Ho, Wo, 3)).astype(np.float16)
        if D > 2:
            g[..., :2] *= 0.05  # pile the points up on few voxels
        go = rng.standard_normal((N, C, Do, Ho, Wo)).astype(np.float16)
        results = []
        try:
            for cores in (2, 64):
                aclnn.set_option("reference_cores", cores)
                oracle.set_reference_cores(cores)
                rdx, rdg = oracle.grid_sampler3d_backward(go, x, g, 0, 1, False)
                dx, dg = aclnn.grid_sampler3d_backward(*(torch.from_numpy(a).to(device) for a in (go, x, g)), 0, 1,
                                                       False)
                torch.cuda.synchronize()
                assert np.array_equal(dx.cpu().numpy().view(np.uint16), rdx.view(np.uint16)), (cores, D)
                assert np.array_equal(dg.cpu().numpy().view(np.uint16), rdg.view(np.uint16)), (cores, D)
                results.append(rdx)
        finally:
            oracle.set_reference_cores(64)
            aclnn.set_option("reference_cores", 64)
        # the order is visible in fp16
        assert not np.array_equal(results[0].view(np.uint16), results[1].view(np.uint16))
    # masks, strided views, channels-last, torch autograd (fp32)
    N, C, D, H, W, Do, Ho, Wo = 2, 3, 4, 6, 5, 3, 7, 6
    x = rng.standard_normal((N, C, D, H, W)).astype(np.float32)
    g = rng.uniform(-1.2, 1.2, (N, Do, Ho, Wo, 3)).astype(np.float32)
    go = rng.standard_normal((N, C, Do, Ho, Wo)).astype(np.float32)
    xt, gt, got = (torch.from_numpy(a).to(device) for a in (x, g, go))
    rdx, rdg = oracle.grid_sampler3d_backward(go, x, g, 0, 0, False)
    dx = torch.full((N, C, D, H, W), 7.0, device=device)
    dg = torch.full((N, Do, Ho, Wo, 3), 7.0, device=device)
    aclnn.grid_sampler3d_backward(got, xt, gt, 0, 0, False, (True, False), dx, dg)
    torch.cuda.synchronize()
    assert np.array_equal(dx.cpu().numpy(), rdx) and (dg == 7.0).all()
    dx.fill_(7.0)
    aclnn.grid_sampler3d_backward(got, xt, gt, 0, 0, False, (False, True), dx, dg)
    torch.cuda.synchronize()
    assert np.array_equal(dg.cpu().numpy(), rdg) and (dx == 7.0).all()
    dxbig = torch.full((N, C, D, H, W + 3), -1.0, device=device)
    dgbig = torch.full((N, Do, Ho, Wo, 5), -1.0, device=device)
    xv = torch.from_numpy(np.ascontiguousarray(x.transpose(0, 1, 2, 4, 3))).to(device).transpose(3, 4)
    aclnn.grid_sampler3d_backward(got, xv, gt, 0, 0, False, (True, True), dxbig[..., 1:1 + W], dgbig[..., 1:4])
    torch.cuda.synchronize()
    assert np.array_equal(dxbig[..., 1:1 + W].cpu().numpy(), rdx) and np.array_equal(dgbig[..., 1:4].cpu().numpy(), rdg)
    assert (dxbig[..., 0] == -1.0).all() and (dgbig[..., 4] == -1.0).all()
    # channels-last operands give the channels-last gradient
    xl, gol = (t.permute(0, 2, 3, 4, 1).contiguous() for t in (xt, got))
    dxl, dgl = aclnn.grid_sampler3d_backward(gol, xl, gt, 0, 0, False, channels_last=True)
    torch.cuda.synchronize()
    assert np.array_equal(dxl.permute(0, 4, 1, 2, 3).cpu().numpy(), rdx) and np.array_equal(dgl.cpu().numpy(), rdg)
    for mode, m in (("bilinear", 0), ("nearest", 1)):
        xa, ga = xt.clone().requires_grad_(True), gt.clone().requires_grad_(True)
        F.grid_sample(xa, ga, mode=mode, padding_mode="reflection", align_corners=True).backward(got)
        dx, dg = aclnn.grid_sampler3d_backward(got, xt, gt, m, 2, True)
        torch.cuda.synchronize()
        assert (dx - xa.grad).abs().max().item() <= 1e-4
        assert ((dg - ga.grad).abs() > 1e-3).float().mean().item() <= 0.02


@pytest.mark.parametrize("dtype", I.DTYPES)
def test_resize_nearest_wide_rows(oracle, device, aclnn, dtype):
    """nearest NCHW with whole-vector rows (the LDS-staged kernel): several column chunks, bands that straddle
    planes, non-integer factors, down-scaling, and a factor whose source segment exceeds the LDS slots"""
    import torch
    rng = np.random.default_rng(320)
    cases = [((2, 3, 5, 1040), (13, 4160)), ((1, 2, 9, 2560), (7, 1600)), ((3, 1, 4, 64), (11, 8)),
             ((1, 1, 3, 8192), (5, 256)), ((1, 4, 7, 528), (7, 2072)), ((1, 2, 6, 24), (12, 48))]
    for shape, (Ho, Wo) in cases:
        N, C, H, W = shape
        x = I.cast_np(rng.standard_normal(shape).astype(np.float32), dtype)
        ref = oracle.resize_nearest(x, (Ho, Wo), dtype=I.oracle_code(dtype))
        out = torch.empty((N, C, Ho, Wo), dtype=I.to_torch(x[:1, :1, :1, :1], dtype, device).dtype, device=device)
        # scales such that trunc(in * scale) == out and the kernel's scale is in/out
        y = aclnn.resize(I.to_torch(x, dtype, device), (1.0, 1.0, Ho / H, Wo / W), "nearest", out=out)
        torch.cuda.synchronize()
        got = I.from_torch(y, dtype)
        view = np.uint32 if dtype == "fp32" else np.uint16
        assert np.array_equal(got.view(view), ref.view(view)), (shape, Ho, Wo, dtype)


@pytest.mark.parametrize("dtype", I.DTYPES)
def test_resize_nearest_few_channels_last(oracle, device, aclnn, dtype):
    """nearest on channels-last images whose pixels are not whole vectors: growing images with source rows on the
    16-byte grid gather out of LDS (rows of W * C elements), the others from memory; several column chunks, ragged
    row ends, non-integer factors"""
    import torch
    rng = np.random.default_rng(321)
    cases = [((2, 8, 8, 3), (16, 24), True), ((1, 6, 16, 5), (7, 40), True), ((1, 5, 1000, 3), (9, 2100), True),
             ((2, 4, 24, 1), (8, 50), True), ((1, 7, 8, 6), (9, 13), True), ((1, 7, 9, 3), (9, 13), False),
             ((1, 12, 16, 3), (5, 7), False)]
    for shape, (Ho, Wo), lds in cases:
        N, H, W, C = shape
        x = I.cast_np(rng.standard_normal(shape).astype(np.float32), dtype)
        ref = oracle.resize_nearest(x, (Ho, Wo), channels_last=True, dtype=I.oracle_code(dtype))
        xt = I.to_torch(x, dtype, device)
        out = torch.empty((N, Ho, Wo, C), dtype=xt.dtype, device=device)
        sc = aclnn.create_float_array([1.0, Ho / H, Wo / W, 1.0])
        hs = [aclnn.tensor_handle(xt, aclnn.ACL_FORMAT_NHWC), aclnn.tensor_handle(out, aclnn.ACL_FORMAT_NHWC)]
        st, _, ex = aclnn.get_workspace_size_resize(hs[0], sc, b"nearest", hs[1])
        assert st == 0
        variant = aclnn.executor_variant(ex)
        aclnn.destroy_executor(ex)
        aclnn.destroy_float_array(sc)
        for h in hs:
            aclnn.destroy_tensor(h)
        # 16-bit rows of 9 * 3 elements are off the 16-byte grid; fp32 rows of 27 elements too
        assert variant == ("nearest_nhwc_lds" if lds else "nearest_nhwc"), (shape, variant)
        y = aclnn.resize(xt, (1.0, Ho / H, Wo / W, 1.0), "nearest", out=out, channels_last=True)
        torch.cuda.synchronize()
        got = I.from_torch(y, dtype)
        view = np.uint32 if dtype == "fp32" else np.uint16
        assert np.array_equal(got.view(view), ref.view(view)), (shape, Ho, Wo, dtype)


@pytest.mark.parametrize("dtype", I.DTYPES)
def test_resize_nearest_replicating_template(oracle, device, aclnn, dtype, monkeypatch):
    """nearest on channels-last images where the reference takes its replicating template (whole upscale factors,
    128 bytes of channels or more, rows that fit its unified buffer): source = destination / factor, which the float
    rule leaves at factors of 41 and up -- columns 41 and 82 of a 3 -> 123 upscale; next to it shapes that fail one
    gate each and keep the float rule, and the unified-buffer size as an environment switch.  Pixels of whole vectors
    (the gather from memory) and of 66 elements (the gather out of LDS)."""
    import torch
    rng = np.random.default_rng(322)
    code = I.oracle_code(dtype)
    esz = 4 if dtype == "fp32" else 2
    wide = 128 // esz  # channels of 128 bytes
    cases = [((2, 3, 3, wide), (6, 123)), ((1, 2, 3, 2 * wide), (2, 141)),     # x41, x47 along W
             ((1, 1, 4, wide + 2), (41, 8)),                                    # x41 along H, pixels off the vector grid
             ((1, 3, 3, wide // 2), (6, 123)),                                  # 64 bytes of channels: float rule
             ((1, 3, 3, wide), (6, 124)),                                       # a factor that is not whole: float rule
             ((1, 2, 3, 8 * wide), (2, 123))]                                   # rows beyond the buffer: float rule
    replicating = [True, True, True, False, False, False]
    for (shape, (Ho, Wo)), rep in zip(cases, replicating):
        N, H, W, C = shape
        assert (oracle.nearest_nhwc_schedule(code, N, C, H, W, Ho, Wo) in (6, 7, 8)) == rep, shape
        x = I.cast_np(rng.standard_normal(shape).astype(np.float32), dtype)
        ref = oracle.resize_nearest(x, (Ho, Wo), channels_last=True, dtype=code)
        if rep:
            assert np.array_equal(ref, np.repeat(np.repeat(x, Ho // H, axis=1), Wo // W, axis=2))
        xt = I.to_torch(x, dtype, device)
        out = torch.empty((N, Ho, Wo, C), dtype=xt.dtype, device=device)
        y = aclnn.resize(xt, (1.0, Ho / H, Wo / W, 1.0), "nearest", out=out, channels_last=True)
        torch.cuda.synchronize()
        got = I.from_torch(y, dtype)
        view = np.uint32 if dtype == "fp32" else np.uint16
        assert np.array_equal(got.view(view), ref.view(view)), (shape, Ho, Wo, dtype)
    # the same tensor as planes: the float rule, which differs at columns 41 and 82
    x = I.cast_np(rng.standard_normal((1, 2, 3, wide)).astype(np.float32), dtype)
    yl = aclnn.resize(I.to_torch(x, dtype, device), (1.0, 1.0, 41.0, 1.0), "nearest",
                      out=torch.empty((1, 2, 123, wide), dtype=I.to_torch(x, dtype, device).dtype, device=device),
                      channels_last=True)
    xp = np.ascontiguousarray(x.transpose(0, 3, 1, 2))
    yp = aclnn.resize(I.to_torch(xp, dtype, device), (1.0, 1.0, 1.0, 41.0), "nearest",
                      out=torch.empty((1, wide, 2, 123), dtype=I.to_torch(x, dtype, device).dtype, device=device))
    torch.cuda.synchronize()
    gl, gp = I.from_torch(yl, dtype), I.from_torch(yp, dtype)
    differ = [w for w in range(123) if not np.array_equal(gl[0, :, w, :], gp[0, :, :, w].T)]
    assert differ == [41, 82]
    # a larger unified buffer lets the last case above through
    shape, (Ho, Wo) = cases[5]
    N, H, W, C = shape
    x = I.cast_np(rng.standard_normal(shape).astype(np.float32), dtype)
    aclnn.set_option("reference_ub_bytes", 1 << 20)
    oracle.set_reference_ub_bytes(1 << 20)
    try:
        ref = oracle.resize_nearest(x, (Ho, Wo), channels_last=True, dtype=code)
        assert np.array_equal(ref, np.repeat(x, 41, axis=2))
        xt = I.to_torch(x, dtype, device)
        y = aclnn.resize(xt, (1.0, 1.0, 41.0, 1.0), "nearest",
                         out=torch.empty((N, Ho, Wo, C), dtype=xt.dtype, device=device), channels_last=True)
        torch.cuda.synchronize()
        assert np.array_equal(I.from_torch(y, dtype), ref)
    finally:
        oracle.set_reference_ub_bytes(0)


@pytest.mark.parametrize("dtype", I.DTYPES)
def test_resize_point_copy(oracle, device, aclnn, dtype):
    """channels-last shrinks by whole factors take the reference's point-copy template: bit-exact copies, also of
    infinities and NaNs, through aclnnUpsampleBilinear2d and aclnnResize; vector and scalar channel counts"""
    torch = _torch()
    rng = np.random.default_rng(330)
    C_vec, C_odd = 128, 130
    for (N, Hs, Ws, C, Ho, Wo, align) in [(2, 12, 15, C_vec, 4, 5, False), (1, 11, 13, C_vec, 6, 5, True),
                                          (1, 9, 9, C_odd, 3, 3, False), (1, 5, 7, C_vec, 1, 7, False)]:
        x32 = rng.standard_normal((N, Hs, Ws, C)).astype(np.float32)
        x32[0, 1, 1, :4] = [np.inf, -np.inf, np.nan, -0.0]
        x = I.cast_np(x32, dtype)
        ref = oracle.resize_point_copy(x, (Ho, Wo), align=align, dtype=I.oracle_code(dtype))
        assert ref is not None
        xt = I.to_torch(x, dtype, device)
        hs = [aclnn.tensor_handle(xt, aclnn.ACL_FORMAT_NHWC)]
        y = aclnn.upsample_bilinear2d(xt, (Ho, Wo), align, channels_last=True)
        torch.cuda.synchronize()
        aclnn.destroy_tensor(hs[0])
        got = I.from_torch(y, dtype)
        assert np.array_equal(_bits(got, dtype), _bits(ref, dtype)), (N, Hs, Ws, C, Ho, Wo, align, dtype)
        if not align:
            y2 = aclnn.resize(xt, (1.0, Ho / Hs, Wo / Ws, 1.0), "bilinear", channels_last=True)
            torch.cuda.synchronize()
            assert np.array_equal(_bits(I.from_torch(y2, dtype), dtype), _bits(ref, dtype))


@pytest.mark.parametrize("dtype", I.DTYPES)
@pytest.mark.parametrize("interp", [0, 1])
def test_grid_sampler3d_channels_last(oracle, device, aclnn, dtype, interp):
    """dense NDHWC tensors are sampled in place: every vector width of the channel run (16, 8, 4 bytes, one element),
    all paddings, special grid values; bit-exact against the oracle on the transposed data"""
    torch = _torch()
    rng = np.random.default_rng(520 + interp)
    for (N, C, D, H, W, Do, Ho, Wo) in [(2, 4, 5, 6, 7, 4, 5, 9), (1, 8, 3, 4, 5, 2, 3, 33), (1, 1, 4, 4, 4, 3, 3, 3),
                                        (2, 3, 2, 9, 5, 3, 7, 5), (1, 20, 3, 3, 3, 2, 2, 17), (1, 64, 2, 2, 2, 1, 3, 5)]:
        x = I.cast_np(rng.standard_normal((N, C, D, H, W)).astype(np.float32), dtype)
        g32 = rng.uniform(-1.8, 1.8, (N, Do, Ho, Wo, 3)).astype(np.float32)
        flat = g32.reshape(-1, 3)
        special = np.array([np.nan, np.inf, -np.inf, 1e30, 1.0, -1.0, 0.0], np.float32)
        for j in range(min(len(special), flat.shape[0])):
            flat[j, j % 3] = special[j]
        g = I.cast_np(g32, dtype)
        xl = I.to_torch(np.ascontiguousarray(x.transpose(0, 2, 3, 4, 1)), dtype, device)
        gt = I.to_torch(g, dtype, device)
        for pad in range(3):
            for align in (False, True):
                ref = oracle.grid_sampler3d(x, g, interp, pad, align, dtype=I.oracle_code(dtype))
                y = aclnn.grid_sampler3d(xl, gt, interp, pad, align, channels_last=True)
                torch.cuda.synchronize()
                got = I.from_torch(y, dtype).transpose(0, 4, 1, 2, 3)
                rn = np.isnan(I.as_f32(ref, dtype))
                assert np.array_equal(np.isnan(I.as_f32(got, dtype)), rn), (N, C, D, H, W, pad, align)
                assert np.array_equal(np.where(rn, 0, _bits(np.ascontiguousarray(got), dtype)),
                                      np.where(rn, 0, _bits(ref, dtype))), (N, C, D, H, W, Do, Ho, Wo, pad, align)
