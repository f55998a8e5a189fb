"""The entry points under HIP graph capture: phase 2 of every operator only launches kernels on the caller's stream
(no allocation, no memset, no synchronisation), so a caller may record it into a graph and replay it.  Each graph is
replayed several times on new data, with eager work and synchronisations in between, and every replay is compared
with the eager result of the same call, which the parity tests compare with the oracle."""
import numpy as np
import pytest

import inputs as I

pytestmark = pytest.mark.gpu


def _replays(torch, device, make_inputs, call, outputs_of, rounds=3):
    """Records `call` on static tensors, then: new inputs -> replay -> compare with an eager call on the same inputs."""
    static_in = [t.clone() for t in make_inputs(0)]
    ws = torch.empty(96 << 20, dtype=torch.uint8, device=device)
    static_out = outputs_of(static_in)
    call(static_in, static_out, ws)  # first calls set function attributes: keep them out of the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(static_in, static_out, ws)
    torch.cuda.synchronize()
    for r in range(1, rounds + 1):
        fresh = make_inputs(r)
        for s, f in zip(static_in, fresh):
            s.copy_(f)
        for o in static_out:
            o.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        eager_out = outputs_of(fresh)
        eager_ws = torch.empty_like(ws)
        call(fresh, eager_out, eager_ws)
        torch.cuda.synchronize()
        for got, want in zip(static_out, eager_out):
            g, w = got.view(torch.uint8).cpu().numpy(), want.view(torch.uint8).cpu().numpy()
            assert np.array_equal(g, w), r


def test_forward_sampler_and_resize_in_a_graph(device, aclnn):
    import torch
    rng = np.random.default_rng(900)

    def sampler_inputs(r):
        x = I.to_torch(I.cast_np(rng.standard_normal((2, 16, 64, 64)).astype(np.float32), "fp16"), "fp16", device)
        g = I.to_torch(I.cast_np(rng.uniform(-1.1, 1.1, (2, 64, 64, 2)).astype(np.float32), "fp16"), "fp16", device)
        return [x, g]

    _replays(torch, device, sampler_inputs,
             lambda i, o, ws: aclnn.grid_sampler2d(i[0], i[1], 0, 0, False, out=o[0], workspace=ws),
             lambda i: [torch.empty((2, 16, 64, 64), dtype=i[0].dtype, device=device)])

    def resize_inputs(r):
        return [torch.from_numpy(rng.standard_normal((2, 8, 56, 56)).astype(np.float32)).to(device)]

    _replays(torch, device, resize_inputs,
             lambda i, o, ws: aclnn.upsample_bilinear2d(i[0], (112, 112), False, out=o[0], workspace=ws),
             lambda i: [torch.empty((2, 8, 112, 112), dtype=i[0].dtype, device=device)])


def test_sampler_backwards_in_a_graph(device, aclnn):
    """The backward operators launch several kernels that hand scratch memory to each other (cell counts cleared by a
    kernel, not a memset): list variant and LDS-ring variant in two dimensions, gather variant in three."""
    import torch
    rng = np.random.default_rng(901)

    def inputs2(r):
        N, C, H, W = 8, 16, 64, 64
        go = I.to_torch(I.cast_np(rng.standard_normal((N, C, 64, 64)).astype(np.float32), "fp16"), "fp16", device)
        x = I.to_torch(I.cast_np(rng.standard_normal((N, C, H, W)).astype(np.float32), "fp16"), "fp16", device)
        g32 = rng.uniform(-1.1, 1.1, (N, 64, 64, 2)).astype(np.float32)
        if r % 2 == 1:
            g32[r % N] = 0.25  # a piled-up item: the sorted path of the list variant
        return [go, x, I.to_torch(I.cast_np(g32, "fp16"), "fp16", device)]

    def call2(i, o, ws):
        h = [aclnn.tensor_handle(t) for t in i + o]
        m = aclnn.create_bool_array([True, True])
        st, _, ex = aclnn.get_workspace_size_grid_sampler2d_backward(h[0], h[1], h[2], 0, 0, False, m, h[3], h[4])
        assert st == 0 and aclnn.executor_variant(ex) == "gs2d_grad_lists_lds"
        aclnn.destroy_executor(ex)
        aclnn.destroy_bool_array(m)
        for t in h:
            aclnn.destroy_tensor(t)
        aclnn.grid_sampler2d_backward(i[0], i[1], i[2], 0, 0, False, input_grad=o[0], grid_grad=o[1], workspace=ws)

    _replays(torch, device, inputs2, call2, lambda i: [torch.empty_like(i[1]), torch.empty_like(i[2])])

    def inputs3(r):
        N, C, D, H, W = 3, 4, 6, 12, 10
        ax = [np.linspace(-1 + 1 / n, 1 - 1 / n, n) for n in (D, H, W)]
        gz, gy, gx = np.meshgrid(*ax, indexing="ij")
        g32 = (np.stack([gx, gy, gz], -1)[None] * rng.uniform(0.9, 1.1, (N, 1, 1, 1, 3)) +
               rng.normal(0, 0.03, (N, D, H, W, 3))).astype(np.float32)
        if r % 2 == 0:
            g32[1] = 0.1  # a piled-up item: left to the ordered kernel
        go = I.to_torch(I.cast_np(rng.standard_normal((N, C, D, H, W)).astype(np.float32), "fp16"), "fp16", device)
        x = I.to_torch(I.cast_np(rng.standard_normal((N, C, D, H, W)).astype(np.float32), "fp16"), "fp16", device)
        return [go, x, I.to_torch(I.cast_np(g32, "fp16"), "fp16", device)]

    _replays(torch, device, inputs3,
             lambda i, o, ws: aclnn.grid_sampler3d_backward(i[0], i[1], i[2], 0, 0, False, input_grad=o[0],
                                                            grid_grad=o[1], workspace=ws),
             lambda i: [torch.empty_like(i[1]), torch.empty_like(i[2])])
