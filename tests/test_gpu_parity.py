"""GPU parity: the HIP path, called through the C-ABI, against the CPU oracle on the same seeded inputs.

Bars: nearest mode and every integer tap index bit-exact; bilinear max-abs <= 1e-5 (fp32) and <= 1e-3 relative
(fp16/bf16) as stated for this path.  The kernels keep the oracle's operation order with contraction disabled,
so the tests additionally report (and for fp32 require) bit equality where it holds.
"""
import numpy as np
import pytest

import inputs as I

pytestmark = pytest.mark.gpu

INTERP = {0: "bilinear", 1: "nearest", 2: "bicubic"}
PAD = {0: "zeros", 1: "border", 2: "reflection"}


def _check(y_gpu, y_ref, dtype, interp, what):
    a = I.as_f32(y_gpu, dtype)
    b = I.as_f32(y_ref, dtype)
    nan_a, nan_b = np.isnan(a), np.isnan(b)
    assert np.array_equal(nan_a, nan_b), "%s: NaN positions differ" % what
    a = np.where(nan_a, 0, a)
    b = np.where(nan_b, 0, b)
    if interp == 1:
        assert np.array_equal(a, b), "%s: nearest must be bit-exact, %d mismatches" % (what, (a != b).sum())
        return
    inf = np.isinf(b)
    assert np.array_equal(np.isinf(a), inf) and np.array_equal(a[inf], b[inf]), "%s: inf positions differ" % what
    a = np.where(inf, 0, a)
    b = np.where(inf, 0, b)
    if dtype == "fp32":
        err = np.abs(a - b).max() if a.size else 0.0
        assert err <= 1e-5, "%s: max-abs %g > 1e-5" % (what, err)
    else:
        # 1e-3 relative; values that round to (sub)normal-small outputs are compared against a small absolute floor
        tol = 1e-3 * np.maximum(np.abs(b), 1e-2)
        bad = np.abs(a - b) > tol
        assert not bad.any(), "%s: %d samples beyond 1e-3 relative, worst %g" % (
            what, bad.sum(), (np.abs(a - b) / np.maximum(np.abs(b), 1e-2)).max())


def _assert_same_bits(y_gpu, y_ref, what):
    """The kernels keep the oracle's operation order and rounding, so outside NaN (whose sign and payload are not
    part of the contract) every output has to carry the same bits."""
    nan = np.isnan(I.as_f32(y_ref, "fp16" if y_ref.dtype == np.float16 else ("fp32" if y_ref.dtype == np.float32
                                                                             else "bf16")))
    view = np.uint32 if y_ref.dtype == np.float32 else np.uint16
    a = np.where(nan, 0, y_gpu.view(view))
    b = np.where(nan, 0, y_ref.view(view))
    assert np.array_equal(a, b), "%s: %d outputs differ in their bits" % (what, (a != b).sum())


def _run_gs(oracle, device, x32, g32, dtype, interp, pad, align):
    from ops_cv_amd import aclnn
    x = I.cast_np(x32, dtype)
    g = I.cast_np(g32, dtype)
    y_ref = oracle.grid_sampler2d(x, g, interp, pad, align, dtype=I.oracle_code(dtype))
    y = aclnn.grid_sampler2d(I.to_torch(x, dtype, device), I.to_torch(g, dtype, device), interp, pad, align)
    import torch
    torch.cuda.synchronize()
    return I.from_torch(y, dtype), y_ref


@pytest.mark.parametrize("dtype", I.DTYPES)
@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("pad", [0, 1, 2])
@pytest.mark.parametrize("align", [False, True])
def test_grid_sampler_random(oracle, device, dtype, interp, pad, align):
    rng = np.random.default_rng(1000 + interp * 100 + pad * 10 + int(align))
    for (N, C, H, W, Ho, Wo) in [(2, 5, 13, 17, 19, 23), (1, 3, 64, 64, 32, 32), (3, 8, 1, 1, 7, 5),
                                 (2, 16, 7, 64, 33, 65)]:
        x32 = rng.standard_normal((N, C, H, W)).astype(np.float32)
        g32 = rng.uniform(-1.3, 1.3, (N, Ho, Wo, 2)).astype(np.float32)
        y, y_ref = _run_gs(oracle, device, x32, g32, dtype, interp, pad, align)
        _check(y, y_ref, dtype, interp, "gs %s %s %s align=%s %s" % (dtype, INTERP[interp], PAD[pad], align,
                                                                      (N, C, H, W, Ho, Wo)))
        _assert_same_bits(y, y_ref, "gs %s %s %s align=%s" % (dtype, INTERP[interp], PAD[pad], align))


@pytest.mark.parametrize("dtype", I.DTYPES)
@pytest.mark.parametrize("interp", [0, 1, 2])
def test_grid_sampler_large_planes(oracle, device, dtype, interp):
    """input planes of 20-160 KB and output planes of several tiles with a ragged last one: the staged variants
    that keep eight pixels per lane, and the largest plane class"""
    rng = np.random.default_rng(1500 + interp)
    for (N, C, H, W, Ho, Wo, pad, align) in [(1, 3, 100, 100, 130, 131, 1, True), (2, 2, 120, 96, 129, 129, 0, False),
                                             (1, 2, 200, 100, 150, 150, 2, False)]:
        x32 = rng.standard_normal((N, C, H, W)).astype(np.float32)
        g32 = rng.uniform(-1.1, 1.1, (N, Ho, Wo, 2)).astype(np.float32)
        y, y_ref = _run_gs(oracle, device, x32, g32, dtype, interp, pad, align)
        _check(y, y_ref, dtype, interp, "gs-large %s %s %s" % (dtype, INTERP[interp], (N, C, H, W, Ho, Wo)))
        _assert_same_bits(y, y_ref, "gs-large %s %s" % (dtype, INTERP[interp]))


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("pad", [0, 1, 2])
@pytest.mark.parametrize("align", [False, True])
def test_grid_sampler_pair_layout_variant(oracle, device, dtype, pad, align, monkeypatch):
    """the pair-layout kernel (bilinear, 16-bit elements, several output pixels per input pixel): every staged row
    length class, row counts off the loader's blocks of sixteen, a ragged last pixel tile, coordinates outside the
    image on every side and non-finite ones; bit for bit against the oracle and against the ring kernel"""
    import torch
    from ops_cv_amd import aclnn
    rng = np.random.default_rng(1700 + pad * 10 + int(align))
    for (N, C, H, W, Ho, Wo) in [(2, 9, 40, 32, 97, 98), (1, 16, 64, 64, 150, 152), (2, 8, 21, 96, 90, 91 * 2),
                                 (1, 12, 128, 128, 250, 254), (1, 3, 5, 128, 64, 66)]:
        x32 = rng.standard_normal((N, C, H, W)).astype(np.float32)
        x32[0, 0, 0, :] = 3.0e4  # large values on the image border: a tap wrongly taken from outside would show
        g32 = rng.uniform(-1.4, 1.4, (N, Ho, Wo, 2)).astype(np.float32)
        sv = I.special_grid_values()
        k = min(sv.size, Wo)
        g32[0, 0, :k, 0] = sv[:k]
        g32[0, 1, :k, 1] = sv[:k]
        x, g = I.cast_np(x32, dtype), I.cast_np(g32, dtype)
        xt, gt = I.to_torch(x, dtype, device), I.to_torch(g, dtype, device)
        out = torch.empty((N, C, Ho, Wo), dtype=xt.dtype, device=device)
        hs = [aclnn.tensor_handle(t) for t in (xt, gt, out)]
        st, _, ex = aclnn.get_workspace_size_grid_sampler2d(hs[0], hs[1], 0, pad, align, hs[2])
        assert st == 0
        assert aclnn.executor_variant(ex).startswith("lds_pair_w"), aclnn.executor_variant(ex)
        aclnn.destroy_executor(ex)
        for h in hs:
            aclnn.destroy_tensor(h)
        y_ref = oracle.grid_sampler2d(x, g, 0, pad, align, dtype=I.oracle_code(dtype))
        y = I.from_torch(aclnn.grid_sampler2d(xt, gt, 0, pad, align, out=out), dtype)
        what = "gs-pair %s %s align=%s %s" % (dtype, PAD[pad], align, (N, C, H, W, Ho, Wo))
        _check(y, y_ref, dtype, 0, what)
        _assert_same_bits(y, y_ref, what)
        with aclnn.option("gs_variant", 2):  # the pair-layout variant kept out
            y_ring = I.from_torch(aclnn.grid_sampler2d(xt, gt, 0, pad, align), dtype)
        _assert_same_bits(y_ring, y_ref, what + " (ring kernel)")


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("pad", [0, 1])
@pytest.mark.parametrize("align", [False, True])
def test_grid_sampler_bicubic_pair_layout_variant(oracle, device, dtype, pad, align):
    """the bicubic pair-layout kernel (16-bit elements, zeros and border padding): every staged row length class and
    every loader class (one, two, five runs per lane), row counts off the loader's blocks of sixteen, a ragged last
    pixel tile, one and many channels per workgroup, coordinates outside the image on every side (where the padding
    entries at the row ends and the row of zeros are read), huge and non-finite ones; bit for bit against the oracle
    and against the ring kernel"""
    import torch
    from ops_cv_amd import aclnn
    rng = np.random.default_rng(1900 + pad * 10 + int(align))
    for (N, C, H, W, Ho, Wo) in [(2, 9, 40, 32, 47, 48), (16, 3, 64, 64, 64, 64), (2, 8, 21, 96, 60, 62),
                                 (1, 5, 100, 64, 90, 92), (1, 12, 128, 128, 130, 134), (1, 1, 5, 128, 32, 34)]:
        x32 = rng.standard_normal((N, C, H, W)).astype(np.float32)
        x32[0, 0, 0, :] = 3.0e4  # large values on the image border: a tap wrongly taken from outside would show
        x32[0, 0, :, 0] = -2.0e4
        x32[0, 0, :, W - 1] = 1.0e4
        g32 = rng.uniform(-1.5, 1.5, (N, Ho, Wo, 2)).astype(np.float32)
        sv = I.special_grid_values()
        k = min(sv.size, Wo)
        g32[0, 0, :k, 0] = sv[:k]
        g32[0, 1, :k, 1] = sv[:k]
        g32[0, 2, :k, 0] = sv[:k]
        g32[0, 2, :k, 1] = sv[:k][::-1]
        x, g = I.cast_np(x32, dtype), I.cast_np(g32, dtype)
        xt, gt = I.to_torch(x, dtype, device), I.to_torch(g, dtype, device)
        out = torch.empty((N, C, Ho, Wo), dtype=xt.dtype, device=device)
        hs = [aclnn.tensor_handle(t) for t in (xt, gt, out)]
        st, _, ex = aclnn.get_workspace_size_grid_sampler2d(hs[0], hs[1], 2, pad, align, hs[2])
        assert st == 0
        assert aclnn.executor_variant(ex).startswith("lds_pair_bicubic_w"), aclnn.executor_variant(ex)
        aclnn.destroy_executor(ex)
        for h in hs:
            aclnn.destroy_tensor(h)
        y_ref = oracle.grid_sampler2d(x, g, 2, pad, align, dtype=I.oracle_code(dtype))
        y = I.from_torch(aclnn.grid_sampler2d(xt, gt, 2, pad, align, out=out), dtype)
        what = "gs-bicubic-pair %s %s align=%s %s" % (dtype, PAD[pad], align, (N, C, H, W, Ho, Wo))
        _check(y, y_ref, dtype, 2, what)
        _assert_same_bits(y, y_ref, what)
        with aclnn.option("gs_variant", 2):  # the pair-layout variants kept out
            y_ring = I.from_torch(aclnn.grid_sampler2d(xt, gt, 2, pad, align), dtype)
        _assert_same_bits(y, y_ring, what + " (against the ring kernel)")


@pytest.mark.parametrize("dtype", I.DTYPES)
@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("pad", [0, 1, 2])
def test_grid_sampler_rows_padded_in_lds(oracle, device, dtype, interp, pad):
    """input rows of whole 16-byte units that are not a multiple of 128 bytes (40, 48, 56, 24, 72 ... elements), which
    the ring kernel stages with every row padded to one: enough channels for the loaders' literal-count loop, a
    channel count that leaves a short last block, too few channels for that loop (rows as they are), planes whose
    padded size moves them to the next size class, border padding (the rotated layout on padded rows of 128 bytes),
    smooth and scattered grids with special values; bit for bit against the oracle"""
    import torch
    from ops_cv_amd import aclnn
    rng = np.random.default_rng(2100 + interp * 10 + pad)
    d = 2 if dtype == "fp32" else 1  # the same row bytes for every element type
    # the launch plan pads rows only when every workgroup gets at least as many channels as the ring runs ahead, so
    # the shapes have channels to spare: 10 per block with the uneven split of two workgroups per CU, 12 per block,
    # 11 with a short last block of 5, 2 per block (rows stay as they are), and planes that move up a size class
    shapes = [(16, 160, 56, 56 // d, 56, 56), (32, 180, 40, 40 // d, 40, 40), (16, 170, 48, 48 // d, 64, 64),
              (16, 32, 56, 56 // d, 40, 40), (16, 160, 66, 56 // d, 64, 64)]
    for (N, C, H, W, Ho, Wo) in shapes:
        x32 = rng.standard_normal((N, C, H, W)).astype(np.float32)
        x32[:, :, :, W - 1] += 100.0  # the last column of every row: a tap taken from the padding would show
        x32[:, :, H - 1, :] -= 50.0
        g32 = I.affine_grid(rng, N, Ho, Wo)
        g32[N // 2] = rng.uniform(-1.3, 1.3, (Ho, Wo, 2)).astype(np.float32)
        sv = I.special_grid_values()
        k = min(sv.size, Wo)
        g32[0, 0, :k, 0] = sv[:k]
        g32[0, 1, :k, 1] = sv[:k]
        x, g = I.cast_np(x32, dtype), I.cast_np(g32, dtype)
        xt, gt = I.to_torch(x, dtype, device), I.to_torch(g, dtype, device)
        y_ref = oracle.grid_sampler2d(x, g, interp, pad, False, dtype=I.oracle_code(dtype))
        with aclnn.option("gs_variant", 2):  # the ring kernel also where a pair-layout variant would take the shape
            y = I.from_torch(aclnn.grid_sampler2d(xt, gt, interp, pad, False), dtype)
        what = "gs-padded-rows %s %s %s %s" % (dtype, interp, PAD[pad], (N, C, H, W, Ho, Wo))
        _check(y, y_ref, dtype, interp, what)
        _assert_same_bits(y, y_ref, what)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("pad", [0, 1, 2])
@pytest.mark.parametrize("align", [False, True])
def test_grid_sampler_channel_pairs_in_lds(oracle, device, dtype, pad, align):
    """bilinear samples of 16-bit planes of up to 8 KiB with an even channel count, which the ring kernel stages two
    channels at a time, interleaved: planes that are not whole loads for every loader lane, a last channel block
    shorter than the others, the uneven split of two workgroups per CU, fewer stages than the loaders keep on their
    way, border padding on rows of 128 bytes (the rotated layout) and on other rows, both coordinate rules; bit for bit against the oracle and against the same kernel with
    single-channel stages"""
    import torch
    from ops_cv_amd import aclnn
    rng = np.random.default_rng(2300 + pad * 10 + int(align))
    # (the launch plan takes channel pairs where every channel block gets an even number of channels: 4 per block,
    # 2 with a last block of 2, 6 on planes of 200 16-byte units, 4 with 25 blocks, 2 = a single stage per block,
    # and the headline's 22 + 10)
    # then rows of 112, 80 and 96 bytes, which are staged padded to 128: 56 x 56, 40 x 40 and 48 x 44 planes; last,
    # planes of the 16 KiB class with two output pixels or more per input pixel)
    shapes = [(16, 64, 64, 64, 64, 64), (16, 26, 64, 64, 64, 64), (32, 48, 25, 64, 64, 64), (8, 100, 62, 64, 33, 70),
              (64, 12, 48, 64, 40, 40), (16, 256, 64, 64, 64, 64), (16, 64, 56, 56, 56, 56), (32, 48, 40, 40, 64, 64),
              (16, 96, 44, 48, 50, 60), (16, 64, 96, 64, 192, 128), (8, 96, 64, 128, 100, 180),
              (8, 32, 64, 128, 128, 256)]  # the last: 64 (item, tile) pairs, one workgroup per CU with 8 channels each
    for (N, C, H, W, Ho, Wo) in shapes:
        x32 = rng.standard_normal((N, C, H, W)).astype(np.float32)
        x32 += np.arange(C, dtype=np.float32).reshape(1, C, 1, 1)  # a channel taken for its neighbour shows
        g32 = I.affine_grid(rng, N, Ho, Wo)
        g32[N // 2] = rng.uniform(-1.3, 1.3, (Ho, Wo, 2)).astype(np.float32)
        sv = I.special_grid_values()
        k = min(sv.size, Wo)
        g32[0, 0, :k, 0] = sv[:k]
        g32[0, 1, :k, 1] = sv[:k]
        x, g = I.cast_np(x32, dtype), I.cast_np(g32, dtype)
        xt, gt = I.to_torch(x, dtype, device), I.to_torch(g, dtype, device)
        what = "gs-channel-pairs %s %s align=%s %s" % (dtype, PAD[pad], align, (N, C, H, W, Ho, Wo))
        with aclnn.option("gs_variant", 2):  # the ring kernel also where a pair-layout variant would take the shape
            out = torch.empty((N, C, Ho, Wo), dtype=xt.dtype, device=device)
            hs = [aclnn.tensor_handle(t) for t in (xt, gt, out)]
            st, _, ex = aclnn.get_workspace_size_grid_sampler2d(hs[0], hs[1], 0, pad, align, hs[2])
            assert st == 0
            assert aclnn.executor_variant(ex).startswith("lds_ring_pairs"), (what, aclnn.executor_variant(ex))
            aclnn.destroy_executor(ex)
            for h in hs:
                aclnn.destroy_tensor(h)
            y = I.from_torch(aclnn.grid_sampler2d(xt, gt, 0, pad, align), dtype)
        y_ref = oracle.grid_sampler2d(x, g, 0, pad, align, dtype=I.oracle_code(dtype))
        _check(y, y_ref, dtype, 0, what)
        _assert_same_bits(y, y_ref, what)
        with aclnn.option("gs_variant", 3):  # single-channel stages
            y_single = I.from_torch(aclnn.grid_sampler2d(xt, gt, 0, pad, align), dtype)
        _assert_same_bits(y, y_single, what + " (against single-channel stages)")
        if not align:
            with aclnn.option("gs_variant", 2), aclnn.option("grid_sampler2d_rule", 1):
                y2 = I.from_torch(aclnn.grid_sampler2d(xt, gt, 0, pad, align), dtype)
            y2_ref = oracle.grid_sampler2d_arch35(x, g, pad, align, dtype=I.oracle_code(dtype))
            _assert_same_bits(y2, y2_ref, what + " (second rule)")


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("pad", [0, 1, 2])
@pytest.mark.parametrize("align", [False, True])
def test_grid_sampler_bicubic_channel_pairs_in_lds(oracle, device, dtype, pad, align):
    """bicubic samples (grid_sampler2_d_simt.h:362-458) of 16-bit planes of up to 16 KiB with an even channel count
    through the ring kernel's interleaved stages (sixteen 4-byte reads per pixel serve two channels): one and two
    pixels per lane, rows of 128 bytes and padded rows, a short last channel block, the uneven split of two workgroups
    per CU; bit for bit against the oracle and against the same kernel with single-channel stages.  Reflection is the
    padding that no pair-layout kernel takes, so there the automatic choice is checked as well."""
    import torch
    from ops_cv_amd import aclnn
    rng = np.random.default_rng(2400 + pad * 10 + int(align))
    shapes = [(16, 64, 64, 64, 64, 64), (16, 26, 64, 64, 20, 24), (32, 48, 25, 64, 64, 64), (8, 100, 62, 64, 33, 70),
              (16, 256, 64, 64, 64, 64), (16, 64, 56, 56, 56, 56), (16, 96, 44, 48, 50, 60), (16, 128, 32, 128, 32, 128),
              (16, 64, 48, 80, 40, 40), (16, 128, 50, 72, 60, 64),  # rows of 160 and 144 bytes: interleaved as they are
              (16, 64, 96, 64, 48, 64), (8, 32, 64, 128, 40, 50), (8, 64, 80, 96, 50, 70)]  # planes of the 16 KiB class
    pairs_seen = 0
    for (N, C, H, W, Ho, Wo) in shapes:
        x32 = rng.standard_normal((N, C, H, W)).astype(np.float32)
        x32 += np.arange(C, dtype=np.float32).reshape(1, C, 1, 1)  # a channel taken for its neighbour shows
        g32 = I.affine_grid(rng, N, Ho, Wo)
        g32[N // 2] = rng.uniform(-1.3, 1.3, (Ho, Wo, 2)).astype(np.float32)
        sv = I.special_grid_values()
        k = min(sv.size, Wo)
        g32[0, 0, :k, 0] = sv[:k]
        g32[0, 1, :k, 1] = sv[:k]
        x, g = I.cast_np(x32, dtype), I.cast_np(g32, dtype)
        xt, gt = I.to_torch(x, dtype, device), I.to_torch(g, dtype, device)
        what = "gs-bicubic-channel-pairs %s %s align=%s %s" % (dtype, PAD[pad], align, (N, C, H, W, Ho, Wo))
        y_ref = oracle.grid_sampler2d(x, g, 2, pad, align, dtype=I.oracle_code(dtype))
        for variant_option in ((2, 0) if pad == 2 else (2,)):
            with aclnn.option("gs_variant", variant_option):
                out = torch.empty((N, C, Ho, Wo), dtype=xt.dtype, device=device)
                hs = [aclnn.tensor_handle(t) for t in (xt, gt, out)]
                st, _, ex = aclnn.get_workspace_size_grid_sampler2d(hs[0], hs[1], 2, pad, align, hs[2])
                assert st == 0
                variant = aclnn.executor_variant(ex)
                aclnn.destroy_executor(ex)
                for h in hs:
                    aclnn.destroy_tensor(h)
                pairs_seen += int(variant.startswith("lds_ring_pairs"))
                y = I.from_torch(aclnn.grid_sampler2d(xt, gt, 2, pad, align), dtype)
            _check(y, y_ref, dtype, 2, what + " " + variant)
            _assert_same_bits(y, y_ref, what + " " + variant)
        with aclnn.option("gs_variant", 3):  # single-channel stages
            y_single = I.from_torch(aclnn.grid_sampler2d(xt, gt, 2, pad, align), dtype)
        _assert_same_bits(y, y_single, what + " (against single-channel stages)")
    assert pairs_seen >= 9, pairs_seen


@pytest.mark.parametrize("dtype", I.DTYPES)
@pytest.mark.parametrize("interp", [0, 1])
@pytest.mark.parametrize("pad", [0, 1, 2])
def test_grid_sampler_large_output_planes(oracle, device, dtype, interp, pad):
    """output planes of 8192 pixels and more over planes of the large size classes (eight pixels per lane in the ring
    kernel), with batch sizes and channel counts for which the launch plan takes one channel block fewer than would
    fill the CUs: an uneven last block, a single block, blocks of one channel; bit for bit against the oracle"""
    import torch
    from ops_cv_amd import aclnn
    rng = np.random.default_rng(2200 + interp * 10 + pad)
    d = 2 if dtype == "fp32" else 1
    shapes = [(16, 24, 96, 96 // d, 96, 96), (8, 7, 96, 96 // d, 112, 112), (3, 40, 80, 96 // d, 96, 100),
              (16, 3, 96, 96 // d, 128, 65)]
    for (N, C, H, W, Ho, Wo) in shapes:
        x32 = rng.standard_normal((N, C, H, W)).astype(np.float32)
        g32 = I.affine_grid(rng, N, Ho, Wo)
        g32[N // 2] = rng.uniform(-1.3, 1.3, (Ho, Wo, 2)).astype(np.float32)
        sv = I.special_grid_values()
        k = min(sv.size, Wo)
        g32[0, 0, :k, 0] = sv[:k]
        g32[0, 1, :k, 1] = sv[:k]
        x, g = I.cast_np(x32, dtype), I.cast_np(g32, dtype)
        xt, gt = I.to_torch(x, dtype, device), I.to_torch(g, dtype, device)
        y_ref = oracle.grid_sampler2d(x, g, interp, pad, False, dtype=I.oracle_code(dtype))
        with aclnn.option("gs_variant", 2):  # the ring kernel also where a pair-layout variant would take the shape
            y = I.from_torch(aclnn.grid_sampler2d(xt, gt, interp, pad, False), dtype)
        what = "gs-large-planes %s %s %s %s" % (dtype, interp, PAD[pad], (N, C, H, W, Ho, Wo))
        _check(y, y_ref, dtype, interp, what)
        _assert_same_bits(y, y_ref, what)


@pytest.mark.parametrize("dtype", I.DTYPES)
@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("pad", [0, 1, 2])
@pytest.mark.parametrize("align", [False, True])
def test_grid_sampler_special_coordinates(oracle, device, dtype, interp, pad, align):
    """ties, borders, 1e10, inf and NaN grid values (what the reference handles at grid_sampler2_d_simt.h:136-247)"""
    rng = np.random.default_rng(7)
    g32 = I.special_grid()
    for (H, W) in [(5, 8), (10, 10), (1, 7), (64, 64)]:
        x32 = rng.standard_normal((1, 3, H, W)).astype(np.float32)
        y, y_ref = _run_gs(oracle, device, x32, g32, dtype, interp, pad, align)
        _check(y, y_ref, dtype, interp, "gs-special %s %s %s align=%s %s" % (dtype, INTERP[interp], PAD[pad], align,
                                                                              (H, W)))


@pytest.mark.parametrize("dtype", I.DTYPES)
@pytest.mark.parametrize("pad", [0, 1, 2])
@pytest.mark.parametrize("align", [False, True])
def test_grid_sampler_second_coordinate_rule(oracle, device, dtype, pad, align):
    """option grid_sampler2d_rule = 1: bilinear sampling as the reference's aclnnGridSampler2D computes it on its arch35
    part (grid_sampler_2d_bilinear_smit.h:109-153, grid_sampler_bilinear_smit_common.h:36-90), against the oracle's
    restatement of that kernel: the special coordinates (ties, borders, 1e10, inf, NaN -- zeros here, where the
    default rule writes NaN), random and affine grids, shapes served by the LDS ring, by the direct kernel (planes
    beyond LDS, the ring switched off), channels-last and strided views; bit for bit.  The first phase fixes the rule:
    an executor planned under one rule runs under it whatever the option says at the second phase."""
    import torch
    from ops_cv_amd import aclnn
    rng = np.random.default_rng(3500 + pad * 10 + int(align))
    code = I.oracle_code(dtype)
    variants = set()

    def run(x32, g32, forced=0, channels_last=False):
        x, g = I.cast_np(x32, dtype), I.cast_np(g32, dtype)
        ref = oracle.grid_sampler2d_arch35(x, g, pad, align, dtype=code)
        xt, gt = I.to_torch(x, dtype, device), I.to_torch(g, dtype, device)
        out = None
        if channels_last:
            xt = xt.contiguous(memory_format=torch.channels_last)
            out = torch.empty((x.shape[0], x.shape[1], g.shape[1], g.shape[2]), dtype=xt.dtype,
                              device=device).contiguous(memory_format=torch.channels_last)
        if out is None:
            out = torch.empty((x.shape[0], x.shape[1], g.shape[1], g.shape[2]), dtype=xt.dtype, device=device)
        with aclnn.option("grid_sampler2d_rule", 1), aclnn.option("gs_variant", forced):
            hs = [aclnn.tensor_handle(t) for t in (xt, gt, out)]
            st, _, ex = aclnn.get_workspace_size_grid_sampler2d(hs[0], hs[1], 0, pad, align, hs[2])
            assert st == 0
            variants.add(aclnn.executor_variant(ex))
            aclnn.destroy_executor(ex)
            for h in hs:
                aclnn.destroy_tensor(h)
            y = aclnn.grid_sampler2d(xt, gt, 0, pad, align, out=out)
        torch.cuda.synchronize()
        what = "gs second rule %s %s align=%s %s forced=%d cl=%s" % (dtype, PAD[pad], align, x.shape, forced,
                                                                     channels_last)
        got = I.from_torch(y, dtype)
        assert not np.isnan(I.as_f32(got, dtype)).any() or np.isnan(I.as_f32(x, dtype)).any(), what
        _check(got, ref, dtype, 0, what)
        _assert_same_bits(got, ref, what)
        return got

    special = I.special_grid()
    for (H, W) in [(5, 8), (10, 10), (1, 7), (64, 64)]:
        x32 = rng.standard_normal((1, 3, H, W)).astype(np.float32)
        run(x32, special)
        run(x32, special, forced=1)
    for (N, C, H, W, Ho, Wo) in [(2, 5, 13, 17, 19, 23), (1, 16, 64, 64, 32, 32), (2, 8, 1, 1, 7, 5),
                                 (1, 3, 40, 70, 64, 96)]:
        x32 = rng.standard_normal((N, C, H, W)).astype(np.float32)
        g32 = rng.uniform(-1.4, 1.4, (N, Ho, Wo, 2)).astype(np.float32)
        run(x32, g32)
        run(x32, g32, forced=1)
        run(x32, g32, channels_last=True)
    x32 = rng.standard_normal((2, 32, 64, 64)).astype(np.float32)
    run(x32, I.affine_grid(rng, 2, 64, 64))
    # planes beyond LDS: the rule's own direct kernel
    x32 = rng.standard_normal((1, 2, 300, 310)).astype(np.float32)
    run(x32, I.affine_grid(rng, 1, 120, 130))
    assert any(v.startswith("lds_ring") for v in variants) and "direct_arch35" in variants, variants
    # the default rule on a non-finite coordinate differs (NaN in every channel), so the switch is not vacuous ...
    x32 = rng.standard_normal((1, 2, 6, 6)).astype(np.float32)
    g32 = np.zeros((1, 1, 2, 2), np.float32)
    g32[0, 0, 1, 0] = np.nan
    y_default, _ = _run_gs(oracle, device, x32, g32, dtype, 0, pad, align)
    y_second = run(x32, g32)
    if pad == 0:
        assert np.isnan(I.as_f32(y_default, dtype)[0, :, 0, 1]).all()
    assert (I.as_f32(y_second, dtype)[0, :, 0, 1] == (0.0 if pad == 0 else I.as_f32(y_second, dtype)[0, :, 0, 1])).all()
    # ... and an executor keeps the rule of its first phase
    x, g = I.cast_np(x32, dtype), I.cast_np(g32, dtype)
    xt, gt = I.to_torch(x, dtype, device), I.to_torch(g, dtype, device)
    out = torch.empty((1, 2, 1, 2), dtype=xt.dtype, device=device)
    hs = [aclnn.tensor_handle(t) for t in (xt, gt, out)]
    with aclnn.option("grid_sampler2d_rule", 1):
        st, ws, ex = aclnn.get_workspace_size_grid_sampler2d(hs[0], hs[1], 0, pad, align, hs[2])
        assert st == 0 and ws == 0
    assert aclnn.get_option("grid_sampler2d_rule") == 0
    assert aclnn.load_library().aclnnGridSampler2D(None, 0, ex, aclnn._stream_handle(None)) == 0
    torch.cuda.synchronize()
    for h in hs:
        aclnn.destroy_tensor(h)
    assert np.array_equal(I.from_torch(out, dtype).view(np.uint8), y_second.view(np.uint8))


@pytest.mark.parametrize("dtype", I.DTYPES)
@pytest.mark.parametrize("interp", [0, 1])
@pytest.mark.parametrize("pad", [0, 1, 2])
@pytest.mark.parametrize("align", [False, True])
def test_grid_sampler_taps_bit_exact(oracle, device, dtype, interp, pad, align):
    """every integer corner index, weight and NaN flag equals the oracle's, bit for bit"""
    from ops_cv_amd import aclnn
    rng = np.random.default_rng(11)
    grids = [I.special_grid(), rng.uniform(-1.5, 1.5, (2, 37, 41, 2)).astype(np.float32),
             I.affine_grid(rng, 3, 64, 64)]
    for g32 in grids:
        for (H, W) in [(5, 8), (10, 10), (64, 64), (1080, 1920), (3, 1)]:
            g = I.cast_np(g32, dtype)
            ref = oracle.grid_sampler2d_taps(g, H, W, interp, pad, align, dtype=I.oracle_code(dtype))
            got = aclnn.grid_sampler2d_taps(I.to_torch(g, dtype, device), H, W, interp, pad, align)
            assert np.array_equal(got["flag"], ref["flag"])
            live = ref["flag"] == 0
            assert np.array_equal(got["ix0"][live], ref["ix0"][live])
            assert np.array_equal(got["iy0"][live], ref["iy0"][live])
            assert np.array_equal(got["w"][live].view(np.uint32), ref["w"][live].view(np.uint32))


@pytest.mark.parametrize("dtype", I.DTYPES)
@pytest.mark.parametrize("pad", [0, 1, 2])
@pytest.mark.parametrize("align", [False, True])
def test_grid_sampler_bicubic_taps_bit_exact(oracle, device, dtype, pad, align):
    """bicubic: the four tap columns and rows after padding, the eight coefficients and the NaN flag equal the
    oracle's, bit for bit"""
    from ops_cv_amd import aclnn
    rng = np.random.default_rng(12)
    grids = [I.special_grid(), rng.uniform(-1.5, 1.5, (2, 37, 41, 2)).astype(np.float32),
             I.affine_grid(rng, 3, 64, 64)]
    for g32 in grids:
        for (H, W) in [(5, 8), (10, 10), (64, 64), (1080, 1920), (3, 1)]:
            g = I.cast_np(g32, dtype)
            ref = oracle.grid_sampler2d_bicubic_taps(g, H, W, pad, align, dtype=I.oracle_code(dtype))
            got = aclnn.grid_sampler2d_bicubic_taps(I.to_torch(g, dtype, device), H, W, pad, align)
            assert np.array_equal(got["flag"], ref["flag"])
            live = ref["flag"] == 0
            for f in ("bx", "by"):
                assert np.array_equal(got[f][live], ref[f][live]), f
            for f in ("cx", "cy"):
                assert np.array_equal(got[f][live].view(np.uint32), ref[f][live].view(np.uint32)), f


def _run_up(oracle, device, x32, out_hw, dtype, align, sh=0.0, sw=0.0):
    from ops_cv_amd import aclnn
    import torch
    x = I.cast_np(x32, dtype)
    y_ref = oracle.upsample_bilinear2d(x, out_hw, align, sh, sw, dtype=I.oracle_code(dtype))
    y = aclnn.upsample_bilinear2d(I.to_torch(x, dtype, device), out_hw, align, sh, sw)
    torch.cuda.synchronize()
    return I.from_torch(y, dtype), y_ref


@pytest.mark.parametrize("dtype", I.DTYPES)
@pytest.mark.parametrize("align", [False, True])
def test_upsample_random(oracle, device, dtype, align):
    rng = np.random.default_rng(50 + int(align))
    cases = [((2, 3, 7, 9), (14, 18)), ((1, 2, 5, 5), (13, 7)), ((2, 2, 16, 16), (5, 3)), ((1, 1, 1, 4), (2, 16)),
             ((1, 1, 1, 4), (3, 16)), ((2, 3, 1, 1), (4, 4)), ((2, 3, 1, 1), (16, 16)), ((2, 3, 6, 6), (1, 1)),
             ((1, 4, 9, 11), (9, 11)), ((1, 2, 56, 56), (112, 112)), ((1, 1, 33, 65), (67, 200)),
             ((1, 2, 4, 2), (8, 4)), ((3, 5, 20, 24), (40, 48)), ((2, 2, 30, 16), (11, 8)),
             ((1, 3, 64, 32), (200, 64)), ((600, 1, 8, 8), (16, 16)), ((1, 1, 700, 8), (1400, 16))]
    for shape, out_hw in cases:
        x32 = rng.standard_normal(shape).astype(np.float32)
        y, y_ref = _run_up(oracle, device, x32, out_hw, dtype, align)
        _check(y, y_ref, dtype, 0, "up %s align=%s %s->%s" % (dtype, align, shape, out_hw))
        if dtype == "fp32":
            assert np.array_equal(y.view(np.uint32), y_ref.view(np.uint32)), "fp32 upsample should be bit-exact"


@pytest.mark.parametrize("dtype", I.DTYPES)
def test_upsample_user_scales(oracle, device, dtype):
    rng = np.random.default_rng(60)
    x32 = rng.standard_normal((2, 3, 10, 12)).astype(np.float32)
    for out_hw, sh, sw in [((20, 24), 2.0, 2.0), ((25, 18), 2.5, 1.5), ((15, 30), 1.7, 2.4)]:
        y, y_ref = _run_up(oracle, device, x32, out_hw, dtype, False, sh, sw)
        _check(y, y_ref, dtype, 0, "up-scales %s %s" % (dtype, out_hw))


@pytest.mark.parametrize("dtype", I.DTYPES)
def test_upsample_hw_split_template(oracle, device, dtype, monkeypatch):
    """the reference's NCHW template for large outputs (fraction from the unclamped coordinate), reached at small
    sizes by telling library and oracle that the reference device has one vector core; every NCHW kernel variant"""
    from ops_cv_amd import aclnn
    rng = np.random.default_rng(70)
    cases = [((1, 2, 56, 56), (112, 112), 0, 0), ((1, 1, 33, 65), (67, 200), 0, 0), ((1, 3, 64, 32), (200, 64), 0, 0),
             ((1, 1, 700, 8), (1400, 16), 0, 0), ((2, 2, 20, 300), (47, 1031), 0, 0), ((1, 2, 16, 600), (40, 1536), 0, 0),
             ((2, 3, 30, 36), (75, 54), 2.5, 1.5), ((1, 2, 40, 40), (24, 48), 0, 0)]
    aclnn.set_option("reference_cores", 1)
    differs = 0
    try:
        for forced in ("", "b", "r", "g"):
            aclnn.set_option("resize_variant", {"": 0, "g": 1, "r": 2, "b": 3}[forced])
            for shape, out_hw, sh, sw in cases:
                x32 = rng.standard_normal(shape).astype(np.float32)
                oracle.set_reference_cores(1)
                assert oracle.resize_uses_hw_split(*shape, *out_hw)
                y, y_ref = _run_up(oracle, device, x32, out_hw, dtype, False, sh, sw)
                bits = np.uint32 if dtype == "fp32" else np.uint16
                assert np.array_equal(y.view(bits), y_ref.view(bits)), (dtype, forced, shape, out_hw)
                oracle.set_reference_cores(64)
                plain = oracle.upsample_bilinear2d(I.cast_np(x32, dtype), out_hw, False, sh, sw, dtype=I.oracle_code(dtype))
                differs += int(not np.array_equal(plain.view(bits), y_ref.view(bits)))
        # align_corners never has a negative coordinate: both templates agree
        oracle.set_reference_cores(1)
        x32 = rng.standard_normal((1, 2, 56, 56)).astype(np.float32)
        y, y_ref = _run_up(oracle, device, x32, (112, 112), dtype, True)
        assert np.array_equal(y, y_ref)
    finally:
        oracle.set_reference_cores(0)
    # the test would be vacuous if the two templates agreed on these inputs (16-bit results mostly round back)
    assert differs > 0 or dtype != "fp32"
