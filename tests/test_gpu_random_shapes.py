"""Seeded random shapes and modes for every entry point, bit-exact against the oracle.

The enumerated tests pick shapes by hand around the kernels' size classes; this sweep draws them, so that tile
edges, odd extents and class boundaries nobody thought of are met as well.  Every case prints its parameters first.
"""
import os
import sys

import numpy as np
import pytest

import inputs as I

pytestmark = pytest.mark.gpu

# the committed runs use the fixed seeds below; OPSCV_TEST_SEED shifts them all for an extra hunt
SEED_SHIFT = int(os.environ.get("OPSCV_TEST_SEED", "0"))


def _bits(a, dtype):
    return np.ascontiguousarray(a).view(np.uint32 if dtype == "fp32" else np.uint16)


def _same(got, ref, dtype, what):
    rn = np.isnan(I.as_f32(ref, dtype))
    assert np.array_equal(np.isnan(I.as_f32(got, dtype)), rn), what
    assert np.array_equal(np.where(rn, 0, _bits(got, dtype)), np.where(rn, 0, _bits(ref, dtype))), what


def _say(*what):
    print("case:", *what)
    sys.stdout.flush()


def _dims(rng, lo, hi, n):
    # log-uniform extents: small ones are as likely as large ones
    return [int(round(np.exp(rng.uniform(np.log(lo), np.log(hi))))) for _ in range(n)]


SPECIAL_COORDS = np.array([np.nan, np.inf, -np.inf, 1e30, -1e30, 3e9, -3e9, 1.0, -1.0, 0.0, -0.0, 0.5, -0.5, 2.0, -2.0],
                          np.float32)


def _sprinkle(rng, g32, H, W, align):
    """a few per cent of the coordinates replaced: non-finite and huge values, the borders, and coordinates that
    land exactly on pixel centres and on the ties between them"""
    flat = g32.reshape(-1)
    k = max(1, flat.size // 25)
    idx = rng.integers(0, flat.size, k)
    flat[idx] = SPECIAL_COORDS[rng.integers(0, len(SPECIAL_COORDS), k)]
    idx = rng.integers(0, flat.size, k)
    size = np.where(idx % 2 == 0, W, H).astype(np.float32)   # x coordinates at even positions
    half = rng.integers(0, 2 * int(max(H, W)) + 2, k).astype(np.float32) / 2.0   # pixel centres and half-way points
    half = np.minimum(half, size)
    if align:
        flat[idx] = np.where(size > 1, 2.0 * half / np.maximum(size - 1, 1) - 1.0, 0.0).astype(np.float32)
    else:
        flat[idx] = ((2.0 * half + 1.0) / size - 1.0).astype(np.float32)
    return g32


def test_random_grid_sampler2d(oracle, device, aclnn):
    import torch
    rng = np.random.default_rng(9001 + SEED_SHIFT)
    for case in range(240):
        dtype = I.DTYPES[case % 3]
        N, C = _dims(rng, 1, 5, 1)[0], _dims(rng, 1, 40, 1)[0]
        H, W = _dims(rng, 1, 150, 2)
        Ho, Wo = _dims(rng, 1, 120, 2)
        interp, pad, align = int(rng.integers(0, 3)), int(rng.integers(0, 3)), bool(rng.integers(0, 2))
        cl = case % 4 == 3   # a quarter of the cases: input and out as channels-last views
        _say("gs2d", dtype, N, C, H, W, Ho, Wo, interp, pad, align, cl)
        x = I.cast_np(rng.standard_normal((N, C, H, W)).astype(np.float32), dtype)
        g32 = rng.uniform(-1.4, 1.4, (N, Ho, Wo, 2)).astype(np.float32)
        if case % 2 == 1:
            g32 = _sprinkle(rng, g32, H, W, align)
        g = I.cast_np(g32, dtype)
        ref = oracle.grid_sampler2d(x, g, interp, pad, align, dtype=I.oracle_code(dtype))
        xt, gt = I.to_torch(x, dtype, device), I.to_torch(g, dtype, device)
        if cl:
            xt = xt.contiguous(memory_format=torch.channels_last)
            out = torch.empty((N, C, Ho, Wo), dtype=xt.dtype, device=device).contiguous(memory_format=torch.channels_last)
            y = aclnn.grid_sampler2d(xt, gt, interp, pad, align, out=out).contiguous()
        else:
            y = aclnn.grid_sampler2d(xt, gt, interp, pad, align)
        torch.cuda.synchronize()
        _same(I.from_torch(y, dtype), ref, dtype, (case, dtype, N, C, H, W, Ho, Wo, interp, pad, align, cl))


def test_random_grid_sampler2d_second_rule(oracle, device, aclnn):
    """option grid_sampler2d_rule = 1 over random shapes, padding modes and views, against the oracle's restatement of
    the reference's second bilinear kernel"""
    import torch
    rng = np.random.default_rng(9007 + SEED_SHIFT)
    for case in range(90):
        dtype = I.DTYPES[case % 3]
        N, C = _dims(rng, 1, 5, 1)[0], _dims(rng, 1, 40, 1)[0]
        H, W = _dims(rng, 1, 150, 2)
        Ho, Wo = _dims(rng, 1, 120, 2)
        pad, align = int(rng.integers(0, 3)), bool(rng.integers(0, 2))
        cl = case % 5 == 4
        _say("gs2d rule 1", dtype, N, C, H, W, Ho, Wo, pad, align, cl)
        x = I.cast_np(rng.standard_normal((N, C, H, W)).astype(np.float32), dtype)
        g32 = rng.uniform(-1.4, 1.4, (N, Ho, Wo, 2)).astype(np.float32)
        if case % 2 == 1:
            g32 = _sprinkle(rng, g32, H, W, align)
        g = I.cast_np(g32, dtype)
        ref = oracle.grid_sampler2d_arch35(x, g, pad, align, dtype=I.oracle_code(dtype))
        xt, gt = I.to_torch(x, dtype, device), I.to_torch(g, dtype, device)
        with aclnn.option("grid_sampler2d_rule", 1):
            if cl:
                xt = xt.contiguous(memory_format=torch.channels_last)
                out = torch.empty((N, C, Ho, Wo), dtype=xt.dtype,
                                  device=device).contiguous(memory_format=torch.channels_last)
                y = aclnn.grid_sampler2d(xt, gt, 0, pad, align, out=out).contiguous()
            else:
                y = aclnn.grid_sampler2d(xt, gt, 0, pad, align)
        torch.cuda.synchronize()
        _same(I.from_torch(y, dtype), ref, dtype, (case, dtype, N, C, H, W, Ho, Wo, pad, align, cl))


def test_random_grid_sampler2d_pair_layouts(oracle, device, aclnn):
    """rows of 32, 64, 96 or 128 16-bit elements, where the pair-layout kernels take bilinear samples of large output
    planes and bicubic samples under zeros and border padding: random row counts, channel counts of every remainder,
    odd output widths (which send the case to another variant: checked all the same), smooth and scattered grids with
    special values sprinkled in; the variant that ran is counted so that the sweep cannot miss both kernels"""
    import torch
    rng = np.random.default_rng(9006 + SEED_SHIFT)
    seen = {}
    for case in range(60):
        dtype = ("fp16", "bf16")[case % 2]
        N, C = int(rng.integers(1, 4)), int(rng.integers(1, 20))
        H, W = int(rng.integers(1, 130)), 32 * int(rng.integers(1, 5))
        interp = (0, 2)[case % 3 != 0]
        pad, align = int(rng.integers(0, 3)), bool(rng.integers(0, 2))
        if interp == 0:
            Ho, Wo = int(rng.integers(2 * H, 3 * H + 8)), int(rng.integers(2 * W, 2 * W + 40))  # several pixels per input pixel
        else:
            Ho, Wo = int(rng.integers(1, 140)), int(rng.integers(1, 140))
            if case % 5 != 0:  # mostly what the bicubic pair kernel takes: zeros or border padding, whole pixel pairs
                pad = int(rng.integers(0, 2))
                Wo += Wo % 2
        _say("gs2d pair", dtype, N, C, H, W, Ho, Wo, interp, pad, align)
        x = I.cast_np(rng.standard_normal((N, C, H, W)).astype(np.float32), dtype)
        if case % 4 == 0:
            g32 = I.affine_grid(rng, N, Ho, Wo, max_deg=40.0, scale=(0.6, 1.4), shift=0.4)
        else:
            g32 = rng.uniform(-1.5, 1.5, (N, Ho, Wo, 2)).astype(np.float32)
        if case % 2 == 1:
            g32 = _sprinkle(rng, g32, H, W, align)
        g = I.cast_np(g32, dtype)
        tx, tg = I.to_torch(x, dtype, device), I.to_torch(g, dtype, device)
        ty = torch.empty((N, C, Ho, Wo), dtype=tx.dtype, device=device)
        hs = [aclnn.tensor_handle(t) for t in (tx, tg, ty)]
        st, _, ex = aclnn.get_workspace_size_grid_sampler2d(hs[0], hs[1], interp, pad, align, hs[2])
        assert st == 0
        variant = aclnn.executor_variant(ex)
        seen[variant.split("_w")[0]] = seen.get(variant.split("_w")[0], 0) + 1
        aclnn.destroy_executor(ex)
        for h in hs:
            aclnn.destroy_tensor(h)
        ref = oracle.grid_sampler2d(x, g, interp, pad, align, dtype=I.oracle_code(dtype))
        y = aclnn.grid_sampler2d(tx, tg, interp, pad, align, out=ty)
        torch.cuda.synchronize()
        _same(I.from_torch(y, dtype), ref, dtype, (case, dtype, N, C, H, W, Ho, Wo, interp, pad, align, variant))
    assert seen.get("lds_pair", 0) >= 3 and seen.get("lds_pair_bicubic", 0) >= 5, seen


def test_random_grid_sampler2d_channel_pairs(oracle, device, aclnn):
    """bilinear and (every third case) bicubic samples of 16-bit planes between 2 and 8 KiB with enough batch items and channels that the ring kernel
    gives every channel block several channels: where that count is even it stages two channels at a time
    (interleaved in LDS), where it is odd or the rows get padded it does not -- checked all the same, and the
    variant that ran is counted so that the sweep cannot miss the interleaved stages.  Random row counts and widths,
    every padding, both alignments, smooth and scattered grids with special values sprinkled in."""
    import torch
    rng = np.random.default_rng(9008 + SEED_SHIFT)
    seen = {}
    for case in range(36):
        dtype = ("fp16", "bf16")[case % 2]
        N = int(rng.choice([8, 16, 24, 32]))
        C = int(rng.integers(8, 40)) * (2 if case % 4 != 3 else 1)
        W = 64 if case % 3 != 2 else 8 * int(rng.integers(3, 13))
        H = int(rng.integers(max(2, 1100 // W), 4096 // W + 1))  # planes above the 2 KiB class, up to 8 KiB
        Ho, Wo = int(rng.integers(24, 80)), int(rng.integers(24, 80))
        pad, align = int(rng.integers(0, 3)), bool(rng.integers(0, 2))
        interp = 2 if case % 3 == 1 else 0
        _say("gs2d channel pairs", dtype, N, C, H, W, Ho, Wo, interp, pad, align)
        x32 = rng.standard_normal((N, C, H, W)).astype(np.float32)
        x32 += np.arange(C, dtype=np.float32).reshape(1, C, 1, 1)
        x = I.cast_np(x32, dtype)
        if case % 3 == 0:
            g32 = rng.uniform(-1.4, 1.4, (N, Ho, Wo, 2)).astype(np.float32)
        else:
            g32 = I.affine_grid(rng, N, Ho, Wo, max_deg=40.0, scale=(0.6, 1.4), shift=0.4)
        if case % 2 == 1:
            g32 = _sprinkle(rng, g32, H, W, align)
        g = I.cast_np(g32, dtype)
        tx, tg = I.to_torch(x, dtype, device), I.to_torch(g, dtype, device)
        ty = torch.empty((N, C, Ho, Wo), dtype=tx.dtype, device=device)
        with aclnn.option("gs_variant", 2):  # the ring kernel also where a pair-layout variant would take the shape
            hs = [aclnn.tensor_handle(t) for t in (tx, tg, ty)]
            st, _, ex = aclnn.get_workspace_size_grid_sampler2d(hs[0], hs[1], interp, pad, align, hs[2])
            assert st == 0
            variant = aclnn.executor_variant(ex)
            key = ("pairs" if variant.startswith("lds_ring_pairs") else "other") + ("_bicubic" if interp == 2 else "")
            seen[key] = seen.get(key, 0) + 1
            aclnn.destroy_executor(ex)
            for h in hs:
                aclnn.destroy_tensor(h)
            y = aclnn.grid_sampler2d(tx, tg, interp, pad, align, out=ty)
            torch.cuda.synchronize()
        ref = oracle.grid_sampler2d(x, g, interp, pad, align, dtype=I.oracle_code(dtype))
        _same(I.from_torch(y, dtype), ref, dtype, (case, dtype, N, C, H, W, Ho, Wo, interp, pad, align, variant))
    assert seen.get("pairs", 0) >= 6 and seen.get("pairs_bicubic", 0) >= 3, seen


def test_random_grid_sampler2d_large_planes(oracle, device, aclnn):
    """input planes from a few KB to beyond the largest LDS class (the direct kernel), few channels"""
    import torch
    rng = np.random.default_rng(9004 + SEED_SHIFT)
    for case in range(45):
        dtype = I.DTYPES[case % 3]
        N, C = int(rng.integers(1, 3)), int(rng.integers(1, 7))
        H, W = _dims(rng, 40, 420, 2)
        Ho, Wo = _dims(rng, 8, 300, 2)
        interp, pad, align = int(rng.integers(0, 3)), int(rng.integers(0, 3)), bool(rng.integers(0, 2))
        _say("gs2d large", dtype, N, C, H, W, Ho, Wo, interp, pad, align)
        x = I.cast_np(rng.standard_normal((N, C, H, W)).astype(np.float32), dtype)
        g32 = rng.uniform(-1.2, 1.2, (N, Ho, Wo, 2)).astype(np.float32)
        if case % 2 == 1:
            g32 = _sprinkle(rng, g32, H, W, align)
        g = I.cast_np(g32, dtype)
        ref = oracle.grid_sampler2d(x, g, interp, pad, align, dtype=I.oracle_code(dtype))
        y = aclnn.grid_sampler2d(I.to_torch(x, dtype, device), I.to_torch(g, dtype, device), interp, pad, align)
        torch.cuda.synchronize()
        _same(I.from_torch(y, dtype), ref, dtype, (case, dtype, N, C, H, W, Ho, Wo, interp, pad, align))


def test_random_grid_sampler2d_box_variant(oracle, device, aclnn):
    """planes beyond the LDS variants under smooth warps of random angle and scale, 16-bit elements: tiles whose box of
    input pixels goes through LDS, next to tiles that fall back to loads from global memory (strong minification,
    sprinkled special values), tiles cut by the edges of the output, channel counts of every remainder"""
    import torch
    rng = np.random.default_rng(9005 + SEED_SHIFT)
    for case in range(30):
        dtype = ("fp16", "bf16")[case % 2]
        N, C = int(rng.integers(1, 3)), int(rng.integers(1, 10))
        H = int(rng.integers(120, 400))
        W = 8 * int(rng.integers((41000 // H) // 8 + 1, 60))  # rows of whole 16-byte units, planes above 80 KB
        Ho = int(rng.integers(32, 200))
        Wo = 2 * int(rng.integers(32, 120))
        interp, pad, align = int(rng.integers(0, 3)), int(rng.integers(0, 3)), bool(rng.integers(0, 2))
        deg = float(rng.choice([5.0, 30.0, 90.0]))
        lo = float(rng.choice([0.3, 0.8, 1.0]))
        _say("gs2d box", dtype, N, C, H, W, Ho, Wo, interp, pad, align, deg, lo)
        x = I.cast_np(rng.standard_normal((N, C, H, W)).astype(np.float32), dtype)
        g32 = I.affine_grid(rng, N, Ho, Wo, max_deg=deg, scale=(lo, lo * 1.5), shift=0.3)
        if case % 3 == 1:
            g32 = _sprinkle(rng, g32, H, W, align)
        g = I.cast_np(g32, dtype)
        tx, tg = I.to_torch(x, dtype, device), I.to_torch(g, dtype, device)
        ty = torch.empty((N, C, Ho, Wo), dtype=tx.dtype, device=device)
        hs = [aclnn.tensor_handle(t) for t in (tx, tg, ty)]
        st, _, ex = aclnn.get_workspace_size_grid_sampler2d(hs[0], hs[1], interp, pad, align, hs[2])
        assert st == 0 and aclnn.executor_variant(ex) == "box_lds", (H, W, Ho, Wo)
        aclnn.destroy_executor(ex)
        for h in hs:
            aclnn.destroy_tensor(h)
        ref = oracle.grid_sampler2d(x, g, interp, pad, align, dtype=I.oracle_code(dtype))
        y = aclnn.grid_sampler2d(tx, tg, interp, pad, align)
        torch.cuda.synchronize()
        _same(I.from_torch(y, dtype), ref, dtype, (case, dtype, N, C, H, W, Ho, Wo, interp, pad, align, deg, lo))


def test_random_resize_family(oracle, device, aclnn, monkeypatch):
    import torch
    rng = np.random.default_rng(9002 + SEED_SHIFT)
    # the reference picks its NCHW template by output pixels against cores * 1024: four cores put both templates in reach
    aclnn.set_option("reference_cores", 4)
    oracle.set_reference_cores(4)
    try:
        _random_resize_family(oracle, device, aclnn, torch, rng)
    finally:
        oracle.set_reference_cores(0)


def _random_resize_family(oracle, device, aclnn, torch, rng):
    for case in range(240):
        dtype = I.DTYPES[case % 3]
        N, C = _dims(rng, 1, 4, 1)[0], _dims(rng, 1, 70, 1)[0]
        H, W = _dims(rng, 1, 90, 2)
        Ho, Wo = _dims(rng, 1, 200, 2)
        align, cl = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        # a third of the cases hand over scales of their own (they replace the size ratio when align_corners is off)
        sh, sw = (float(rng.uniform(0.3, 3.0)), float(rng.uniform(0.3, 3.0))) if case % 3 == 1 else (0.0, 0.0)
        _say("upsample", dtype, N, C, H, W, Ho, Wo, align, cl, sh, sw)
        x = I.cast_np(rng.standard_normal((N, C, H, W)).astype(np.float32), dtype)
        xin = np.ascontiguousarray(x.transpose(0, 2, 3, 1)) if cl else x
        if cl:
            ref = oracle.upsample_bilinear2d_nhwc(xin, (Ho, Wo), align, sh, sw, dtype=I.oracle_code(dtype))
        else:
            ref = oracle.upsample_bilinear2d(x, (Ho, Wo), align, sh, sw, dtype=I.oracle_code(dtype))
        y = aclnn.upsample_bilinear2d(I.to_torch(xin, dtype, device), (Ho, Wo), align, sh, sw, channels_last=cl)
        torch.cuda.synchronize()
        _same(I.from_torch(y, dtype), ref, dtype, (case, "up", dtype, N, C, H, W, Ho, Wo, align, cl, sh, sw))
        # nearest through aclnnResize on the same tensors
        _say("nearest", dtype, N, C, H, W, Ho, Wo, cl)
        scales = (1.0, Ho / H, Wo / W, 1.0) if cl else (1.0, 1.0, Ho / H, Wo / W)
        shape = (N, Ho, Wo, C) if cl else (N, C, Ho, Wo)
        out = torch.empty(shape, dtype=I.to_torch(xin[:1, :1, :1, :1], dtype, device).dtype, device=device)
        try:
            y = aclnn.resize(I.to_torch(xin, dtype, device), scales, "nearest", out=out, channels_last=cl)
        except aclnn.AclnnError:
            continue  # float scales that do not reproduce the extents exactly are rejected, as in the reference
        torch.cuda.synchronize()
        ref = oracle.resize_nearest(xin, (Ho, Wo), channels_last=cl, dtype=I.oracle_code(dtype))
        _same(I.from_torch(y, dtype), ref, dtype, (case, "nearest", dtype, N, C, H, W, Ho, Wo, cl))
        # bilinear through aclnnResize: align_corners off, the size ratio as scale
        _say("resize bilinear", dtype, N, C, H, W, Ho, Wo, cl)
        y = aclnn.resize(I.to_torch(xin, dtype, device), scales, "bilinear", out=out, channels_last=cl)
        torch.cuda.synchronize()
        if cl:
            ref = oracle.upsample_bilinear2d_nhwc(xin, (Ho, Wo), False, dtype=I.oracle_code(dtype))
        else:
            ref = oracle.upsample_bilinear2d(x, (Ho, Wo), False, dtype=I.oracle_code(dtype))
        _same(I.from_torch(y, dtype), ref, dtype, (case, "resize bilinear", dtype, N, C, H, W, Ho, Wo, cl))
        # gradient of the upsample
        _say("upsample backward", dtype, N, C, H, W, Ho, Wo, align, cl)
        gshape = (N, Ho, Wo, C) if cl else (N, C, Ho, Wo)
        go = I.cast_np(rng.standard_normal(gshape).astype(np.float32), dtype)
        ref = oracle.upsample_bilinear2d_backward(go, (H, W), align, channels_last=cl, dtype=I.oracle_code(dtype),
                                                  scales_h=sh, scales_w=sw)
        isz = (N, H, W, C) if cl else (N, C, H, W)
        y = aclnn.upsample_bilinear2d_backward(I.to_torch(go, dtype, device), isz, align, sh, sw, channels_last=cl)
        torch.cuda.synchronize()
        _same(I.from_torch(y, dtype), ref, dtype, (case, "upbwd", dtype, N, C, H, W, Ho, Wo, align, cl, sh, sw))


def test_random_sampler_backward_and_3d(oracle, device, aclnn):
    import torch
    rng = np.random.default_rng(9003 + SEED_SHIFT)
    for case in range(150):
        dtype = I.DTYPES[case % 3]
        N, C = _dims(rng, 1, 3, 1)[0], _dims(rng, 1, 12, 1)[0]
        H, W = _dims(rng, 1, 90, 2)
        Ho, Wo = _dims(rng, 1, 60, 2)
        interp, pad, align = int(rng.integers(0, 3)), int(rng.integers(0, 3)), bool(rng.integers(0, 2))
        _say("gs2d backward", dtype, N, C, H, W, Ho, Wo, interp, pad, align)
        x = I.cast_np(rng.standard_normal((N, C, H, W)).astype(np.float32), dtype)
        g32 = rng.uniform(-1.3, 1.3, (N, Ho, Wo, 2)).astype(np.float32)
        if case % 2 == 1:
            g32 = _sprinkle(rng, g32, H, W, align)
        g = I.cast_np(g32, dtype)
        go = I.cast_np(rng.standard_normal((N, C, Ho, Wo)).astype(np.float32), dtype)
        rdx, rdg = oracle.grid_sampler2d_backward(go, x, g, interp, pad, align, dtype=I.oracle_code(dtype))
        dx, dg = aclnn.grid_sampler2d_backward(I.to_torch(go, dtype, device), I.to_torch(x, dtype, device),
                                               I.to_torch(g, dtype, device), interp, pad, align)
        torch.cuda.synchronize()
        _same(I.from_torch(dx, dtype), rdx, dtype, (case, "dx", dtype, N, C, H, W, Ho, Wo, interp, pad, align))
        _same(I.from_torch(dg, dtype), rdg, dtype, (case, "dgrid", dtype, N, C, H, W, Ho, Wo, interp, pad, align))
    # shapes that the list variant of the input gradient takes (8 channels or more, gradOutput planes of whole
    # 16-byte units) and, every other case, the LDS-ring variant of the grid gradient too (planes of whole 4 KiB, 128
    # workgroups of 256 points or more)
    for case in range(36):
        dtype = I.DTYPES[case % 3]
        esz = 4 if dtype == "fp32" else 2
        C = int(rng.integers(8, 41))
        if case % 2 == 0:
            N = int(rng.integers(4, 10))
            H, W = int(rng.choice([16, 32, 64])), int(rng.choice([32, 64])) * (2 if esz == 2 else 1)
            Ho = Wo = 64
            while N * ((Ho * Wo + 255) // 256) < 128:
                N += 1
        else:
            N = int(rng.integers(1, 4))
            H, W = _dims(rng, 2, 70, 2)
            Ho, Wo = int(rng.integers(1, 80)), 8 * int(rng.integers(1, 12))
        interp, pad, align = 0, int(rng.integers(0, 3)), bool(rng.integers(0, 2))
        _say("gs2d backward lists", dtype, N, C, H, W, Ho, Wo, interp, pad, align)
        x = I.cast_np(rng.standard_normal((N, C, H, W)).astype(np.float32), dtype)
        g32 = rng.uniform(-1.3, 1.3, (N, Ho, Wo, 2)).astype(np.float32)
        if case % 3 == 1:
            g32 = _sprinkle(rng, g32, H, W, align)
        if case % 4 == 3:
            g32 = np.round(g32 * 4) / 4  # points pile up on few elements
        g = I.cast_np(g32, dtype)
        go = I.cast_np(rng.standard_normal((N, C, Ho, Wo)).astype(np.float32), dtype)
        rdx, rdg = oracle.grid_sampler2d_backward(go, x, g, interp, pad, align, dtype=I.oracle_code(dtype))
        dx, dg = aclnn.grid_sampler2d_backward(I.to_torch(go, dtype, device), I.to_torch(x, dtype, device),
                                               I.to_torch(g, dtype, device), interp, pad, align)
        torch.cuda.synchronize()
        _same(I.from_torch(dx, dtype), rdx, dtype, (case, "dx lists", dtype, N, C, H, W, Ho, Wo, pad, align))
        _same(I.from_torch(dg, dtype), rdg, dtype, (case, "dgrid lists", dtype, N, C, H, W, Ho, Wo, pad, align))
    for case in range(150):
        dtype = I.DTYPES[case % 3]
        N, C = _dims(rng, 1, 3, 1)[0], _dims(rng, 1, 20, 1)[0]
        D, H, W = _dims(rng, 1, 20, 3)
        Do, Ho, Wo = _dims(rng, 1, 16, 3)
        interp, pad, align, cl = int(rng.integers(0, 2)), int(rng.integers(0, 3)), bool(rng.integers(0, 2)), bool(
            rng.integers(0, 2))
        _say("gs3d", dtype, N, C, D, H, W, Do, Ho, Wo, interp, pad, align, cl)
        x = I.cast_np(rng.standard_normal((N, C, D, H, W)).astype(np.float32), dtype)
        g32 = rng.uniform(-1.4, 1.4, (N, Do, Ho, Wo, 3)).astype(np.float32)
        if case % 2 == 1:
            flat = g32.reshape(-1)
            k = max(1, flat.size // 25)
            flat[rng.integers(0, flat.size, k)] = SPECIAL_COORDS[rng.integers(0, len(SPECIAL_COORDS), k)]
        g = I.cast_np(g32, dtype)
        ref = oracle.grid_sampler3d(x, g, interp, pad, align, dtype=I.oracle_code(dtype))
        xin = np.ascontiguousarray(x.transpose(0, 2, 3, 4, 1)) if cl else x
        y = aclnn.grid_sampler3d(I.to_torch(xin, dtype, device), I.to_torch(g, dtype, device), interp, pad, align,
                                 channels_last=cl)
        torch.cuda.synchronize()
        got = I.from_torch(y, dtype)
        got = got.transpose(0, 4, 1, 2, 3) if cl else got
        _same(got, ref, dtype, (case, "gs3d", dtype, N, C, D, H, W, Do, Ho, Wo, interp, pad, align, cl))
        if case % 3 == 0:
            # the backward of the same call; volumes above 8192 voxels span several LDS bands
            if case % 6 == 0:
                D, H, W = D + 12, H + 14, W + 16
                x = I.cast_np(rng.standard_normal((N, C, D, H, W)).astype(np.float32), dtype)
            _say("gs3d backward", dtype, N, C, D, H, W, Do, Ho, Wo, interp, pad, align, cl)
            go = I.cast_np(rng.standard_normal((N, C, Do, Ho, Wo)).astype(np.float32), dtype)
            rdx, rdg = oracle.grid_sampler3d_backward(go, x, g, interp, pad, align, dtype=I.oracle_code(dtype))
            xin = np.ascontiguousarray(x.transpose(0, 2, 3, 4, 1)) if cl else x
            gin = np.ascontiguousarray(go.transpose(0, 2, 3, 4, 1)) if cl else go
            dx, dg = aclnn.grid_sampler3d_backward(I.to_torch(gin, dtype, device), I.to_torch(xin, dtype, device),
                                                   I.to_torch(g, dtype, device), interp, pad, align, channels_last=cl)
            torch.cuda.synchronize()
            gdx = I.from_torch(dx, dtype)
            gdx = gdx.transpose(0, 4, 1, 2, 3) if cl else gdx
            what = (case, dtype, N, C, D, H, W, Do, Ho, Wo, interp, pad, align, cl)
            _same(gdx, rdx, dtype, ("gs3d dx",) + what)
            _same(I.from_torch(dg, dtype), rdg, dtype, ("gs3d dgrid",) + what)


def _as_view(torch, rng, t, kind):
    """a tensor with the values and shape of `t` and another memory layout: 1 = a strided window of a larger
    buffer (offset, steps, padding), 2 = dimensions stored in another order; returns (view, backing buffer)"""
    if kind == 1:
        steps = [int(rng.integers(1, 3)) for _ in t.shape]
        offs = [int(rng.integers(0, 3)) for _ in t.shape]
        big = torch.full([o + s * n + int(rng.integers(0, 2)) for o, s, n in zip(offs, steps, t.shape)], 77.0,
                         dtype=t.dtype, device=t.device)
        view = big[tuple(slice(o, o + s * n, s) for o, s, n in zip(offs, steps, t.shape))]
        view.copy_(t)
        return view, big
    if kind == 2:
        perm = [int(i) for i in rng.permutation(t.dim())]
        inv = [perm.index(i) for i in range(t.dim())]
        back = t.permute(perm).contiguous()
        return back.permute(inv), back
    return t, t


def test_random_views(oracle, device, aclnn):
    """every operand of every entry point as a non-contiguous view: strided windows with offsets, permuted storage;
    results land in the view and nowhere else"""
    import torch
    rng = np.random.default_rng(9005 + SEED_SHIFT)

    def views(*arrays_and_dtype):
        *arrays, dtype = arrays_and_dtype
        return [_as_view(torch, rng, I.to_torch(a, dtype, device), int(rng.integers(0, 3)))[0] for a in arrays]

    def out_view(shape, like):
        kind = int(rng.integers(0, 3))
        view, big = _as_view(torch, rng, torch.full(shape, 55.0, dtype=like.dtype, device=device), kind)
        return view, big, kind

    def check_untouched(big, view, kind, what):
        if kind == 1:   # everything outside the window still holds the fill value
            probe = big.clone()
            view_in_probe = probe.as_strided(view.shape, view.stride(), view.storage_offset())
            view_in_probe.fill_(77.0)
            assert bool((probe == 77.0).all()), what

    for case in range(90):
        dtype = I.DTYPES[case % 3]
        op = case % 6
        N, C = int(rng.integers(1, 3)), int(rng.integers(1, 10))
        H, W = _dims(rng, 1, 40, 2)
        Ho, Wo = _dims(rng, 1, 40, 2)
        interp, pad, align = int(rng.integers(0, 3)), int(rng.integers(0, 3)), bool(rng.integers(0, 2))
        _say("views", op, dtype, N, C, H, W, Ho, Wo, interp, pad, align)
        x = I.cast_np(rng.standard_normal((N, C, H, W)).astype(np.float32), dtype)
        g = I.cast_np(rng.uniform(-1.3, 1.3, (N, Ho, Wo, 2)).astype(np.float32), dtype)
        what = (case, op, dtype, N, C, H, W, Ho, Wo, interp, pad, align)
        if op == 0:
            ref = oracle.grid_sampler2d(x, g, interp, pad, align, dtype=I.oracle_code(dtype))
            xt, gt = views(x, g, dtype)
            out, big, kind = out_view((N, C, Ho, Wo), xt)
            aclnn.grid_sampler2d(xt, gt, interp, pad, align, out=out)
            torch.cuda.synchronize()
            _same(I.from_torch(out.contiguous(), dtype), ref, dtype, what)
            check_untouched(big, out, kind, what)
        elif op == 1:
            ref = oracle.upsample_bilinear2d(x, (Ho, Wo), align, dtype=I.oracle_code(dtype))
            (xt,) = views(x, dtype)
            out, big, kind = out_view((N, C, Ho, Wo), xt)
            aclnn.upsample_bilinear2d(xt, (Ho, Wo), align, out=out)
            torch.cuda.synchronize()
            _same(I.from_torch(out.contiguous(), dtype), ref, dtype, what)
            check_untouched(big, out, kind, what)
        elif op == 2:
            ref = oracle.resize_nearest(x, (Ho, Wo), dtype=I.oracle_code(dtype))
            (xt,) = views(x, dtype)
            out, big, kind = out_view((N, C, Ho, Wo), xt)
            try:
                aclnn.resize(xt, (1.0, 1.0, Ho / H, Wo / W), "nearest", out=out)
            except aclnn.AclnnError:
                continue
            torch.cuda.synchronize()
            _same(I.from_torch(out.contiguous(), dtype), ref, dtype, what)
            check_untouched(big, out, kind, what)
        elif op == 3:
            go = I.cast_np(rng.standard_normal((N, C, Ho, Wo)).astype(np.float32), dtype)
            rdx, rdg = oracle.grid_sampler2d_backward(go, x, g, interp, pad, align, dtype=I.oracle_code(dtype))
            got, xt, gt = views(go, x, g, dtype)
            dx, bigx, kx = out_view((N, C, H, W), xt)
            dg, bigg, kg = out_view((N, Ho, Wo, 2), xt)
            aclnn.grid_sampler2d_backward(got, xt, gt, interp, pad, align, input_grad=dx, grid_grad=dg)
            torch.cuda.synchronize()
            _same(I.from_torch(dx.contiguous(), dtype), rdx, dtype, what + ("dx",))
            _same(I.from_torch(dg.contiguous(), dtype), rdg, dtype, what + ("dgrid",))
            check_untouched(bigx, dx, kx, what)
            check_untouched(bigg, dg, kg, what)
        elif op == 4:
            go = I.cast_np(rng.standard_normal((N, C, Ho, Wo)).astype(np.float32), dtype)
            ref = oracle.upsample_bilinear2d_backward(go, (H, W), align, dtype=I.oracle_code(dtype))
            (got,) = views(go, dtype)
            out, big, kind = out_view((N, C, H, W), got)
            aclnn.upsample_bilinear2d_backward(got, (N, C, H, W), align, out=out)
            torch.cuda.synchronize()
            _same(I.from_torch(out.contiguous(), dtype), ref, dtype, what)
            check_untouched(big, out, kind, what)
        else:
            D, Do = int(rng.integers(1, 7)), int(rng.integers(1, 7))
            i3 = interp % 2
            x5 = I.cast_np(rng.standard_normal((N, C, D, H, W)).astype(np.float32), dtype)
            g5 = I.cast_np(rng.uniform(-1.3, 1.3, (N, Do, Ho, Wo, 3)).astype(np.float32), dtype)
            ref = oracle.grid_sampler3d(x5, g5, i3, pad, align, dtype=I.oracle_code(dtype))
            xt, gt = views(x5, g5, dtype)
            out, big, kind = out_view((N, C, Do, Ho, Wo), xt)
            aclnn.grid_sampler3d(xt, gt, i3, pad, align, out=out)
            torch.cuda.synchronize()
            _same(I.from_torch(out.contiguous(), dtype), ref, dtype, what + (D, Do))
            check_untouched(big, out, kind, what)
