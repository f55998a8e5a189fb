"""opscvGridSampler2DNoAlloc (the entry point that allocates nothing) against aclnnGridSampler2D, through the C-ABI.

The static scratch array takes the place of the caller's workspace whenever a view has to be packed; every call on
the device shares it and it keeps the previous call's contents, so the checks run two calls in a row, the second
with smaller tensors, and compare each bit for bit with the two-phase entry point on the same views.
"""
import numpy as np
import pytest

import inputs as I

pytestmark = pytest.mark.gpu


def _views(torch, device, dtype, rng, N, C, H, W, Ho, Wo):
    """Strided views of all three tensors (none contiguous, none channels-last dense): what makes both entry points
    pack through scratch memory."""
    x = I.cast_np(rng.standard_normal((N, C, H, W)).astype(np.float32), dtype)
    g = I.cast_np(rng.uniform(-1.15, 1.15, (N, Ho, Wo, 2)).astype(np.float32), dtype)
    # input: transposed view of an (N,C,W,H) buffer; grid: every second column of a wider buffer
    xt = I.to_torch(np.ascontiguousarray(x.transpose(0, 1, 3, 2)), dtype, device).transpose(2, 3)
    gbig = torch.zeros((N, Ho, 2 * Wo, 2), dtype=xt.dtype, device=device)
    gbig[:, :, ::2, :] = I.to_torch(g, dtype, device)
    gv = gbig[:, :, ::2, :]
    assert not xt.is_contiguous() and not gv.is_contiguous()
    return xt, gv


def _run_pair(torch, aclnn, device, dtype, rng, shape, interp, pad, align):
    N, C, H, W, Ho, Wo = shape
    xt, gv = _views(torch, device, dtype, rng, *shape)
    fill = 3.0
    # outputs: windows of wider buffers, so that writes outside the view would show
    big_a = torch.full((N, C, Ho, Wo + 4), fill, dtype=xt.dtype, device=device)
    big_b = torch.full((N, C, Ho, Wo + 4), fill, dtype=xt.dtype, device=device)
    want = aclnn.grid_sampler2d(xt, gv, interp, pad, align, out=big_a[:, :, :, 2:2 + Wo])
    st = aclnn.grid_sampler2d_noalloc(xt, gv, big_b[:, :, :, 2:2 + Wo], interp, pad, align)
    assert st == 0, aclnn.load_library().aclGetRecentErrMsg()
    torch.cuda.synchronize()
    a = I.from_torch(big_a, dtype).view(np.uint8)
    b = I.from_torch(big_b, dtype).view(np.uint8)
    assert np.array_equal(a, b), "no-alloc result differs from aclnnGridSampler2D for %s %s" % (dtype, shape)
    edge = I.as_f32(I.from_torch(big_b, dtype), dtype)
    assert (edge[..., :2] == fill).all() and (edge[..., 2 + Wo:] == fill).all()
    assert want.shape == (N, C, Ho, Wo)


@pytest.mark.parametrize("dtype", I.DTYPES)
def test_no_alloc_matches_two_phase_on_strided_views(device, aclnn, dtype):
    import torch
    rng = np.random.default_rng(77)
    # two calls in a row on the shared scratch array, the second smaller; then other modes on the small one
    _run_pair(torch, aclnn, device, dtype, rng, (3, 37, 45, 52, 40, 46), 0, 0, False)
    _run_pair(torch, aclnn, device, dtype, rng, (2, 5, 9, 12, 7, 5), 0, 0, False)
    _run_pair(torch, aclnn, device, dtype, rng, (2, 6, 11, 10, 8, 8), 1, 1, True)
    _run_pair(torch, aclnn, device, dtype, rng, (1, 4, 8, 8, 6, 6), 2, 2, False)


def test_no_alloc_contiguous_and_channels_last_use_no_scratch(device, aclnn, oracle):
    import torch
    rng = np.random.default_rng(78)
    x = rng.standard_normal((2, 8, 16, 16)).astype(np.float32)
    g = rng.uniform(-1.1, 1.1, (2, 12, 12, 2)).astype(np.float32)
    ref = oracle.grid_sampler2d(x, g, 0, 0, False)
    xt, gt = torch.from_numpy(x).to(device), torch.from_numpy(g).to(device)
    out = torch.empty((2, 8, 12, 12), device=device)
    assert aclnn.grid_sampler2d_noalloc(xt, gt, out, 0, 0, False) == 0
    xcl = xt.contiguous(memory_format=torch.channels_last)
    ocl = torch.empty((2, 8, 12, 12), device=device).contiguous(memory_format=torch.channels_last)
    assert aclnn.grid_sampler2d_noalloc(xcl, gt, ocl, 0, 0, False) == 0
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), ref)
    assert np.array_equal(ocl.cpu().numpy(), ref)


def test_no_alloc_rejects_what_does_not_fit_and_bad_arguments(device, aclnn):
    import torch
    # the packed input view alone exceeds the static array: refused with 161002, nothing launched
    C = aclnn.NOALLOC_SCRATCH_BYTES // (64 * 64 * 4) + 1
    big = torch.zeros((1, C, 64, 64), device=device).transpose(2, 3)
    g = torch.zeros((1, 4, 4, 2), device=device)
    out = torch.full((1, C, 4, 4), 5.0, device=device)
    assert aclnn.grid_sampler2d_noalloc(big, g, out, 0, 0, False) == aclnn.ACLNN_ERR_PARAM_INVALID
    assert b"static" in aclnn.load_library().aclGetRecentErrMsg()
    torch.cuda.synchronize()
    assert (out == 5.0).all().item()
    # the same validation as the two-phase entry point
    x = torch.zeros((1, 2, 4, 4), device=device)
    assert aclnn.grid_sampler2d_noalloc(x, g, torch.zeros((1, 2, 4, 4), device=device), 3, 0, False) == \
        aclnn.ACLNN_ERR_PARAM_INVALID
    L = aclnn.load_library()
    h = aclnn.tensor_handle(x)
    assert L.opscvGridSampler2DNoAlloc(h, None, 0, 0, False, h, None) == aclnn.ACLNN_ERR_PARAM_NULLPTR
    aclnn.destroy_tensor(h)


def test_no_alloc_in_a_graph_on_strided_views(device, aclnn):
    """The entry point under stream capture, after one warm call on the device (which looks up the static array and
    sets kernel attributes): the recorded graph packs the strided views into the static array, samples and scatters
    the result into a window; every replay on new data equals the two-phase call on the same views."""
    import torch
    rng = np.random.default_rng(79)
    shape = (2, 19, 23, 30, 17, 21)
    N, C, H, W, Ho, Wo = shape
    for dtype in ("fp16", "fp32"):
        xt, gv = _views(torch, device, dtype, rng, *shape)
        x_store, g_store = xt.transpose(2, 3), gv  # x_store is the dense buffer behind the transposed view
        big = torch.full((N, C, Ho, Wo + 4), 3.0, dtype=xt.dtype, device=device)
        win = big[:, :, :, 2:2 + Wo]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            assert aclnn.grid_sampler2d_noalloc(xt, gv, win, 0, 0, False) == 0  # the warm call
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            st = aclnn.grid_sampler2d_noalloc(xt, gv, win, 0, 0, False)
        assert st == 0, aclnn.load_library().aclGetRecentErrMsg()
        for r in range(3):
            x_new, g_new = _views(torch, device, dtype, rng, *shape)
            x_store.copy_(x_new.transpose(2, 3))
            g_store.copy_(g_new)
            big.fill_(3.0)
            graph.replay()
            torch.cuda.synchronize()
            want = aclnn.grid_sampler2d(x_new, g_new, 0, 0, False)
            torch.cuda.synchronize()
            got = I.from_torch(win.contiguous(), dtype).view(np.uint8)
            assert np.array_equal(got, I.from_torch(want, dtype).view(np.uint8)), (dtype, r)
            edge = I.as_f32(I.from_torch(big, dtype), dtype)
            assert (edge[..., :2] == 3.0).all() and (edge[..., 2 + Wo:] == 3.0).all()
