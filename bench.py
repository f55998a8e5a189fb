#!/usr/bin/env python3
"""Benchmark of the bilinear gather/interpolate path on one MI355X.

A "step" is one full two-phase call (GetWorkspaceSize + launch) of the hot path over one synthetic batch whose
tensors already live in HBM.  The headline workload is the grid_sampler2d fp16 N=16 C=256 configuration; the
other configurations are reported beside it in "other_workloads".  Steps rotate over several independent
tensor sets so that a step does not find its operands in the last-level cache left by the previous one.

Prints ONE JSON line (see the keys below).  `roofline.achieved` = algorithmic bytes (every tensor touched
once) / average launch duration measured with HIP events on the launch stream.  `cpu_baseline` = the CPU
oracle (a port of the reference arithmetic) timed on this machine's host cores on the same workload.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "tests")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0

# HBM bytes per launch measured with rocprofv3 FETCH_SIZE / WRITE_SIZE counter runs (scaled by a plain copy of known
# size), keyed by (workload, kernel variant the figure was measured on) and holding the data-movement revision of that
# variant at the time (opscvVariantRevision; the profile records the kernel's symbol beside it).  The figure is
# reported only when the run picks that same variant at that same revision, together with the summary file it comes
# from; anything else reports null -- a kernel change that moves bytes differently bumps the revision in the library
# and thereby retires the figure until the counters are read again.
MEASURED_TRAFFIC = {
    ("C3", "lds_ring_p8208_1x6"): (67.58e6, 4, "profiles/gs2d_lds_ring_C3_fp16_n16_c256.md"),
    ("C3", "lds_ring_pairs_p16400_2x2"): (67.59e6, 1, "profiles/gs2d_lds_ring_pairs_C3_fp16_n16_c256.md"),
    ("C4", "nchw_band_lds"): (1415.4e6, 1, "profiles/resize_band_lds_C4_fp16_4k_upscale.md"),
    ("C2", "nchw_flat_lds"): (32.43e6, 1, "profiles/resize_flat_lds_C2_fp32_56_to_112.md"),
    ("C5", "lds_pair_w128"): (170.05e6, 2, "profiles/gs2d_lds_pair_C5_bf16_random_gather.md"),
    ("L1", "box_lds"): (742.5e6, 1, "profiles/gs2d_box_L1_fp16_1080p.md"),
    ("V1", "gs3d_bilinear"): (38.72e6, 1, "profiles/gs3d_V1_fp16_22x4x16x64x64.md"),
    ("G3", "gs2d_grad_lists_lds"): (151.8e6, 4, "profiles/gs2d_grad_G3_fp16_n16_c256.md"),
    ("W1", "gs3d_grad_lists"): (200.1e6, 1, "profiles/gs3d_grad_W1_fp16_22x4x16x64x64.md"),
    ("B4", "resize_grad_lds"): (1340.0e6, 1, "profiles/resize_grad_lds_B4_fp16_4k.md"),
    ("R4", "nearest_nchw_lds"): (1327.3e6, 1, "profiles/resize_nearest_lds_R4_fp16_4k.md"),
}

# the type the arithmetic runs in, per workload: every kernel of this path converts its 16-bit elements to fp32,
# computes in fp32 (products and sums rounded separately, as the reference does) and rounds once on the way out
ARITHMETIC = {"C1": "f32", "C2": "f32", "C3": "f32", "C4": "f32", "C5": "f32", "L1": "f32", "V1": "f32", "V1cl": "f32",
              "G3": "f32", "W1": "f32", "W1s": "f32", "B4": "f32", "R4": "f32"}

# few grid points in a large volume (128 voxels a point): the input gradient of the 3-D sampler keeps its ordered kernel
# here (the gather variant walks every voxel's cells and is 4 to 25 times slower on such shapes)
W1_SPARSE = dict(shape=(4, 4, 64, 128, 128), points=(8, 32, 32), label="W1s")

MIN_TIMED_LAUNCHES = 50  # floor for the secondary workloads, whatever --steps says for the headline

# name -> description of the workloads (shapes as in the baseline configuration list)
GS_WORKLOADS = {
    "C1": dict(dtype="fp32", x=(1, 3, 64, 64), grid=(1, 32, 32), kind="uniform", interp=0, pad=0, align=False,
               sets=4),
    "C3": dict(dtype="fp16", x=(16, 256, 64, 64), grid=(16, 64, 64), kind="affine", interp=0, pad=0, align=False,
               sets=8),
    "C5": dict(dtype="bf16", x=(8, 128, 128, 128), grid=(8, 256, 256), kind="random", interp=0, pad=1, align=True,
               sets=3),
    # not a BASELINE configuration: input planes of 4 MB, far beyond the LDS variants (image warps)
    "L1": dict(dtype="fp16", x=(2, 32, 1080, 1920), grid=(2, 1080, 1920), kind="affine", interp=0, pad=0, align=False,
               sets=2),
}
UP_WORKLOADS = {
    "C2": dict(dtype="fp32", x=(8, 64, 56, 56), out=(112, 112), align=False, scales=(2.0, 2.0), dist="normal",
               sets=8),
    "C4": dict(dtype="fp16", x=(4, 16, 1080, 1920), out=(2160, 3840), align=True, scales=(2.0, 2.0),
               dist="uniform", sets=2),
}
INTERP_NAMES = {0: "bilinear", 1: "nearest", 2: "bicubic"}
PAD_NAMES = {0: "zeros", 1: "border", 2: "reflection"}


def esize(dtype):
    return 4 if dtype == "fp32" else 2


def make_gs_inputs(name, seed_base):
    import numpy as np
    import inputs as I
    w = GS_WORKLOADS[name]
    N, C, H, W = w["x"]
    _, Ho, Wo = w["grid"]
    rng = np.random.default_rng(seed_base)
    if name == "C1":
        x32 = rng.uniform(0, 1, w["x"]).astype(np.float32)
    else:
        x32 = rng.standard_normal(w["x"], dtype=np.float32)
    if w["kind"] == "uniform":
        g32 = rng.uniform(-1, 1, (N, Ho, Wo, 2)).astype(np.float32)
    elif w["kind"] == "affine":
        g32 = I.affine_grid(rng, N, Ho, Wo)
    else:
        g32 = rng.uniform(-1.1, 1.1, (N, Ho, Wo, 2)).astype(np.float32)
    return I.cast_np(x32, w["dtype"]), I.cast_np(g32, w["dtype"])


def make_up_input(name, seed_base):
    import numpy as np
    import inputs as I
    w = UP_WORKLOADS[name]
    rng = np.random.default_rng(seed_base)
    if w["dist"] == "normal":
        x32 = rng.standard_normal(w["x"], dtype=np.float32)
    else:
        x32 = rng.random(w["x"], dtype=np.float32)
    return I.cast_np(x32, w["dtype"])


_BENCH_LIB = None


def load_bench_lib():
    global _BENCH_LIB
    if _BENCH_LIB is not None:
        return _BENCH_LIB
    path = os.path.join(ROOT, "ops_cv_amd", "libopscv_bench.so")
    if not os.path.exists(path):
        raise RuntimeError("libopscv_bench.so is not built: run `python -m ops_cv_amd.build`")
    L = ctypes.CDLL(path)
    vp, i64, u64 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_uint64
    pd = ctypes.POINTER(ctypes.c_double)
    L.opscv_bench_grid_sampler2d.restype = ctypes.c_int
    L.opscv_bench_grid_sampler2d.argtypes = [ctypes.POINTER(vp), ctypes.POINTER(vp), ctypes.POINTER(vp), ctypes.c_int,
                                            i64, i64, ctypes.c_bool, vp, u64, ctypes.c_int, ctypes.c_int, vp, pd, pd]
    L.opscv_bench_upsample_bilinear2d.restype = ctypes.c_int
    L.opscv_bench_upsample_bilinear2d.argtypes = [ctypes.POINTER(vp), ctypes.POINTER(vp), ctypes.c_int, vp,
                                                 ctypes.c_bool, ctypes.c_double, ctypes.c_double, vp, u64,
                                                 ctypes.c_int, ctypes.c_int, vp, pd, pd]
    L.opscv_bench_grid_sampler2d_backward.restype = ctypes.c_int
    L.opscv_bench_grid_sampler2d_backward.argtypes = [ctypes.POINTER(vp)] * 5 + [ctypes.c_int, i64, i64, ctypes.c_bool,
                                                                                 vp, vp, u64, ctypes.c_int, ctypes.c_int, vp, pd, pd]
    L.opscv_bench_grid_sampler3d_backward.restype = ctypes.c_int
    L.opscv_bench_grid_sampler3d_backward.argtypes = L.opscv_bench_grid_sampler2d_backward.argtypes
    L.opscv_bench_grid_sampler3d.restype = ctypes.c_int
    L.opscv_bench_grid_sampler3d.argtypes = L.opscv_bench_grid_sampler2d.argtypes
    L.opscv_bench_upsample_bilinear2d_backward.restype = ctypes.c_int
    L.opscv_bench_upsample_bilinear2d_backward.argtypes = [ctypes.POINTER(vp), ctypes.POINTER(vp), ctypes.c_int, vp,
                                                          vp, ctypes.c_bool, ctypes.c_double, ctypes.c_double, vp,
                                                          u64, ctypes.c_int, ctypes.c_int, vp, pd, pd]
    L.opscv_bench_resize.restype = ctypes.c_int
    L.opscv_bench_resize.argtypes = [ctypes.POINTER(vp), ctypes.POINTER(vp), ctypes.c_int, vp, ctypes.c_char_p, vp,
                                     u64, ctypes.c_int, ctypes.c_int, vp, pd, pd]
    L.opscv_bench_host_us.restype = None
    L.opscv_bench_host_us.argtypes = [pd, pd]
    L.opscv_bench_stream.restype = ctypes.c_int
    L.opscv_bench_stream.argtypes = [ctypes.POINTER(vp), ctypes.POINTER(vp), ctypes.c_int, u64, u64, ctypes.c_int, vp,
                                     ctypes.c_int, ctypes.c_int, pd]
    _BENCH_LIB = L
    return L


def stream_reference_us(L, xs, ys, steps, stream):
    """A kernel that only reads the operator's input bytes once and writes its output bytes once (16-byte vector
    accesses, non-temporal stores, same buffer rotation, events on the same stream), the fastest of a small sweep over
    loads in flight per lane and grid size: what the memory system gives a well-tuned launch of this size.  The
    roofline fraction is quoted against the 8 TB/s peak; this figure says how much of the gap to that peak a
    do-nothing kernel of the same size leaves open as well."""
    n = len(xs)
    src = (ctypes.c_void_p * n)(*[t.data_ptr() for t in xs])
    dst = (ctypes.c_void_p * n)(*[t.data_ptr() for t in ys])
    in_b = xs[0].numel() * xs[0].element_size() // 16 * 16
    out_b = ys[0].numel() * ys[0].element_size() // 16 * 16
    if in_b == 0 or out_b == 0:
        return None
    ev = ctypes.c_double(0)
    saved = [y.clone() for y in ys[:1]]
    best = None
    # (loads in flight per lane, workgroups per CU; 0 = one lane per 16-byte unit of work)
    for unroll, groups in ((4, 8), (1, 8), (4, 4), (2, 16), (1, 32), (4, 0)):
        for k in (max(steps, 200), steps):
            if L.opscv_bench_stream(src, dst, n, in_b, out_b, k, stream, unroll, groups, ctypes.byref(ev)) != 0:
                return None
        us = ev.value * 1e3 / steps
        best = us if best is None else min(best, us)
    ys[0].copy_(saved[0])
    return best


PREHEAT_MS = 300.0


def preheat(run, warmup):
    """`warmup` untimed steps, then more untimed steps until PREHEAT_MS of GPU work have run: the clocks of an
    idle MI355X take tens of milliseconds of load to settle, far longer than a few 20-microsecond launches."""
    done_ms = 0.0
    if warmup > 0:
        done_ms += run(warmup).step_ms * warmup
    chunk = max(warmup, 10)
    while done_ms < PREHEAT_MS:
        t = run(chunk)
        done_ms += t.step_ms * chunk
        chunk = min(chunk * 2, 4096)


class Timed:
    def __init__(self, event_ms, wall_ms, steps):
        self.kernel_us = event_ms * 1e3 / steps
        self.step_ms = wall_ms / steps
        self.stream_us = None
        # host time per call inside GetWorkspaceSize (validation + plan) and inside the second phase (launches only:
        # the kernels run asynchronously), measured in the same loop
        p1, p2 = ctypes.c_double(0), ctypes.c_double(0)
        load_bench_lib().opscv_bench_host_us(ctypes.byref(p1), ctypes.byref(p2))
        self.host_phase1_us, self.host_phase2_us = p1.value, p2.value


def bench_gs(name, steps, warmup, interp=None, pad=None, align=None, sets=None, check=True, channels_last=False):
    import numpy as np
    import torch
    import inputs as I
    import oracle_lib
    from ops_cv_amd import aclnn
    w = dict(GS_WORKLOADS[name])
    if interp is not None:
        w["interp"] = interp
    if pad is not None:
        w["pad"] = pad
    if align is not None:
        w["align"] = align
    nsets = w["sets"] if sets is None else sets
    dev = torch.device("cuda:0")
    L = load_bench_lib()
    N, C, H, W = w["x"]
    _, Ho, Wo = w["grid"]
    xs, gs, ys, hx, hg, hy = [], [], [], [], [], []
    x0 = g0 = None
    for s in range(nsets):
        x, g = make_gs_inputs(name, 1000 + s)
        if s == 0:
            x0, g0 = x, g
        xs.append(I.to_torch(x, w["dtype"], dev))
        gs.append(I.to_torch(g, w["dtype"], dev))
        ys.append(torch.empty((N, C, Ho, Wo), dtype=xs[-1].dtype, device=dev))
        if channels_last:
            # (N,C,H,W) views over NHWC memory, as a framework's channels_last tensors are handed over
            xs[-1] = xs[-1].contiguous(memory_format=torch.channels_last)
            ys[-1] = ys[-1].contiguous(memory_format=torch.channels_last)
        hx.append(aclnn.tensor_handle(xs[-1]))
        hg.append(aclnn.tensor_handle(gs[-1]))
        hy.append(aclnn.tensor_handle(ys[-1]))
    arr = lambda hs: (ctypes.c_void_p * len(hs))(*hs)
    ax, ag, ay = arr(hx), arr(hg), arr(hy)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ev, wall = ctypes.c_double(0), ctypes.c_double(0)

    def run(k, warm=0):
        rc = L.opscv_bench_grid_sampler2d(ax, ag, ay, nsets, w["interp"], w["pad"], w["align"], None, 0, warm, k, stream,
                                          ctypes.byref(ev), ctypes.byref(wall))
        if rc != 0:
            raise RuntimeError("bench loop failed rc=%d: %s" % (rc, aclnn.load_library().aclGetRecentErrMsg()))
        return Timed(ev.value, wall.value, k)

    st, _, ex = aclnn.get_workspace_size_grid_sampler2d(hx[0], hg[0], w["interp"], w["pad"], w["align"], hy[0])
    variant = aclnn.executor_variant(ex)
    aclnn.destroy_executor(ex)
    preheat(run, warmup)
    torch.cuda.synchronize()
    t = run(steps, warmup)
    torch.cuda.synchronize()
    t.stream_us = stream_reference_us(L, xs, ys, steps, stream) if check else None
    torch.cuda.synchronize()
    parity = None
    if check:
        ref = oracle_lib.grid_sampler2d(x0, g0, w["interp"], w["pad"], w["align"], dtype=I.oracle_code(w["dtype"]))
        got = I.from_torch(ys[0], w["dtype"])
        a, b = I.as_f32(got, w["dtype"]), I.as_f32(ref, w["dtype"])
        nan = np.isnan(b)
        assert np.array_equal(np.isnan(a), nan)
        d = np.abs(np.where(nan, 0, a) - np.where(nan, 0, b))
        parity = {"max_abs_err": float(d.max()), "bit_exact": bool(np.array_equal(got.view(np.uint8),
                                                                                    ref.view(np.uint8)))}
    for h in hx + hg + hy:
        aclnn.destroy_tensor(h)
    samples = N * C * Ho * Wo
    e = esize(w["dtype"])
    alg_bytes = (N * C * H * W + N * Ho * Wo * 2 + samples) * e
    desc = "%s grid_sampler2d %s x%s grid%s %s %s align_corners=%s%s" % (
        name, w["dtype"], tuple(w["x"]), (N, Ho, Wo, 2), INTERP_NAMES[w["interp"]], PAD_NAMES[w["pad"]], w["align"],
        " channels_last views" if channels_last else "")
    return dict(steps=steps, workload=desc, samples=samples, alg_bytes=alg_bytes, timed=t, variant=variant, parity=parity,
                sets=nsets, cpu=(x0, g0, w), default_modes=(interp is None and pad is None and align is None and not channels_last))


def bench_up(name, steps, warmup, sets=None, check=True):
    import numpy as np
    import torch
    import inputs as I
    import oracle_lib
    from ops_cv_amd import aclnn
    w = UP_WORKLOADS[name]
    nsets = w["sets"] if sets is None else sets
    dev = torch.device("cuda:0")
    L = load_bench_lib()
    N, C, Hs, Ws = w["x"]
    Hd, Wd = w["out"]
    xs, ys, hx, hy = [], [], [], []
    x0 = None
    for s in range(nsets):
        x = make_up_input(name, 2000 + s)
        if s == 0:
            x0 = x
        xs.append(I.to_torch(x, w["dtype"], dev))
        ys.append(torch.empty((N, C, Hd, Wd), dtype=xs[-1].dtype, device=dev))
        hx.append(aclnn.tensor_handle(xs[-1], aclnn.ACL_FORMAT_NCHW))
        hy.append(aclnn.tensor_handle(ys[-1], aclnn.ACL_FORMAT_NCHW))
    arr = lambda hs: (ctypes.c_void_p * len(hs))(*hs)
    ax, ay = arr(hx), arr(hy)
    size = aclnn.create_int_array([Hd, Wd])
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ev, wall = ctypes.c_double(0), ctypes.c_double(0)

    def run(k, warm=0):
        rc = L.opscv_bench_upsample_bilinear2d(ax, ay, nsets, size, w["align"], w["scales"][0], w["scales"][1], None,
                                               0, warm, k, stream, ctypes.byref(ev), ctypes.byref(wall))
        if rc != 0:
            raise RuntimeError("bench loop failed rc=%d: %s" % (rc, aclnn.load_library().aclGetRecentErrMsg()))
        return Timed(ev.value, wall.value, k)

    st, _, ex = aclnn.get_workspace_size_upsample_bilinear2d(hx[0], size, w["align"], w["scales"][0], w["scales"][1],
                                                             hy[0])
    variant = aclnn.executor_variant(ex)
    aclnn.destroy_executor(ex)
    preheat(run, warmup)
    torch.cuda.synchronize()
    t = run(steps, warmup)
    torch.cuda.synchronize()
    t.stream_us = stream_reference_us(L, xs, ys, steps, stream) if check else None
    torch.cuda.synchronize()
    parity = None
    if check:
        # the oracle on the first plane block only (the full 4K case would take minutes on one core)
        planes = min(N * C, 4)
        xsub = x0.reshape(N * C, 1, Hs, Ws)[:planes]
        ref = oracle_lib.upsample_bilinear2d(xsub, (Hd, Wd), w["align"], w["scales"][0], w["scales"][1],
                                             dtype=I.oracle_code(w["dtype"]))
        got = I.from_torch(ys[0], w["dtype"]).reshape(N * C, 1, Hd, Wd)[:planes]
        d = np.abs(I.as_f32(got, w["dtype"]) - I.as_f32(ref, w["dtype"]))
        parity = {"max_abs_err": float(d.max()), "bit_exact": bool(np.array_equal(got.view(np.uint8),
                                                                                    ref.view(np.uint8))),
                  "planes_checked": planes}
    for h in hx + hy:
        aclnn.destroy_tensor(h)
    aclnn.destroy_int_array(size)
    samples = N * C * Hd * Wd
    e = esize(w["dtype"])
    alg_bytes = (N * C * Hs * Ws + samples) * e
    desc = "%s upsample_bilinear2d %s %s->%s align_corners=%s" % (name, w["dtype"], tuple(w["x"]),
                                                                  (N, C, Hd, Wd), w["align"])
    return dict(steps=steps, workload=desc, samples=samples, alg_bytes=alg_bytes, timed=t, variant=variant, parity=parity,
                sets=nsets, cpu=(x0, w))


def _finish(L, run, xs, ys, steps, warmup, stream):
    import torch
    preheat(run, warmup)
    torch.cuda.synchronize()
    t = run(steps, warmup)
    torch.cuda.synchronize()
    t.stream_us = stream_reference_us(L, xs, ys, steps, stream)
    torch.cuda.synchronize()
    return t


def _parity(got, ref, dtype, **extra):
    import numpy as np
    import inputs as I
    d = np.abs(I.as_f32(got, dtype) - I.as_f32(ref, dtype))
    out = {"max_abs_err": float(d.max()), "bit_exact": bool(np.array_equal(got.view(np.uint8), ref.view(np.uint8)))}
    out.update(extra)
    return out


def bench_gs3d(steps, warmup, sets=4, channels_last=False):
    """Volumetric sampler on the shape the reference singles out (22 x 4 x 16 x 64 x 64, fp16, an affine warp);
    with channels_last the same data as dense NDHWC tensors."""
    import numpy as np
    import torch
    import inputs as I
    import oracle_lib
    from ops_cv_amd import aclnn
    dev = torch.device("cuda:0")
    L = load_bench_lib()
    N, C, D, H, W = 22, 4, 16, 64, 64
    dtype = "fp16"
    xs, gs, ys, hs = [], [], [], [[], [], []]
    x0 = g0 = None
    for s in range(sets):
        rng = np.random.default_rng(3000 + s)
        x = I.cast_np(rng.standard_normal((N, C, D, H, W)).astype(np.float32), dtype)
        # identity lattice, mildly scaled and shifted per batch item, with jitter: a registration-style warp
        ax = [np.linspace(-1, 1, n, dtype=np.float32) for n in (D, H, W)]
        gz, gy, gx = np.meshgrid(*ax, indexing="ij")
        base = np.stack([gx, gy, gz], -1)[None]
        g = base * rng.uniform(0.9, 1.1, (N, 1, 1, 1, 3)) + rng.uniform(-0.1, 0.1, (N, 1, 1, 1, 3))
        g = I.cast_np((g + rng.normal(0, 0.01, g.shape)).astype(np.float32), dtype)
        if s == 0:
            x0, g0 = x, g
        if channels_last:
            xs.append(I.to_torch(np.ascontiguousarray(x.transpose(0, 2, 3, 4, 1)), dtype, dev))
            ys.append(torch.empty((N, D, H, W, C), dtype=xs[-1].dtype, device=dev))
        else:
            xs.append(I.to_torch(x, dtype, dev))
            ys.append(torch.empty((N, C, D, H, W), dtype=xs[-1].dtype, device=dev))
        gs.append(I.to_torch(g, dtype, dev))
        fmt = aclnn.ACL_FORMAT_NDHWC if channels_last else aclnn.ACL_FORMAT_NCDHW
        for lst, t, f in zip(hs, (xs[-1], gs[-1], ys[-1]), (fmt, aclnn.ACL_FORMAT_NCDHW, fmt)):
            lst.append(aclnn.tensor_handle(t, f))
    arr = lambda h: (ctypes.c_void_p * len(h))(*h)
    ax_, ag, ay = arr(hs[0]), arr(hs[1]), arr(hs[2])
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ev, wall = ctypes.c_double(0), ctypes.c_double(0)

    def run(k, warm=0):
        rc = L.opscv_bench_grid_sampler3d(ax_, ag, ay, sets, 0, 0, False, None, 0, warm, k, stream, ctypes.byref(ev),
                                          ctypes.byref(wall))
        if rc != 0:
            raise RuntimeError("bench loop failed rc=%d: %s" % (rc, aclnn.load_library().aclGetRecentErrMsg()))
        return Timed(ev.value, wall.value, k)

    st, _, ex = aclnn.get_workspace_size_grid_sampler3d(hs[0][0], hs[1][0], 0, 0, False, hs[2][0])
    variant = aclnn.executor_variant(ex)
    aclnn.destroy_executor(ex)
    t = _finish(L, run, xs, ys, steps, warmup, stream)
    ref = oracle_lib.grid_sampler3d(x0, g0, 0, 0, False, dtype=I.oracle_code(dtype))
    got = I.from_torch(ys[0], dtype)
    if channels_last:
        got = np.ascontiguousarray(got.transpose(0, 4, 1, 2, 3))
    parity = _parity(got, ref, dtype)
    for lst in hs:
        for h in lst:
            aclnn.destroy_tensor(h)
    samples = N * C * D * H * W
    alg = (N * C * D * H * W * 2 + N * D * H * W * 3) * esize(dtype)
    return dict(steps=steps, workload="V1 grid_sampler3d fp16 x(22,4,16,64,64) grid(22,16,64,64,3) bilinear zeros "
                         "align_corners=False" + (" NDHWC tensors" if channels_last else ""), samples=samples, alg_bytes=alg, timed=t, variant=variant,
                parity=parity, sets=sets, default_modes=True)


def bench_gs3d_backward(steps, warmup, sets=2, mask=(True, True), shape=(22, 4, 16, 64, 64), points=None, label="W1"):
    """Backward of the volumetric workload (fp16 22 x 4 x 16 x 64 x 64, the same registration-style warp): both
    gradients.  `points` (Do, Ho, Wo): a grid coarser than the volume (W1s: few points in a large volume, where the
    library keeps its ordered kernel for the input gradient)."""
    import numpy as np
    import torch
    import inputs as I
    import oracle_lib
    from ops_cv_amd import aclnn
    dev = torch.device("cuda:0")
    L = load_bench_lib()
    N, C, D, H, W = shape
    Do, Ho, Wo = points if points is not None else (D, H, W)
    dtype = "fp16"
    ts, hs = [[] for _ in range(5)], [[] for _ in range(5)]
    first = None
    for s in range(sets):
        rng = np.random.default_rng(3100 + s)
        x = I.cast_np(rng.standard_normal((N, C, D, H, W)).astype(np.float32), dtype)
        ax = [np.linspace(-1, 1, n, dtype=np.float32) for n in (Do, Ho, Wo)]
        gz, gy, gx = np.meshgrid(*ax, indexing="ij")
        base = np.stack([gx, gy, gz], -1)[None]
        g = base * rng.uniform(0.9, 1.1, (N, 1, 1, 1, 3)) + rng.uniform(-0.1, 0.1, (N, 1, 1, 1, 3))
        g = I.cast_np((g + rng.normal(0, 0.01, g.shape)).astype(np.float32), dtype)
        go = I.cast_np(rng.standard_normal((N, C, Do, Ho, Wo)).astype(np.float32), dtype)
        if s == 0:
            first = (go, x, g)
        tens = [I.to_torch(go, dtype, dev), I.to_torch(x, dtype, dev), I.to_torch(g, dtype, dev)]
        tens += [torch.empty_like(tens[1]), torch.empty_like(tens[2])]
        for lst, hl, t in zip(ts, hs, tens):
            lst.append(t)
            hl.append(aclnn.tensor_handle(t, aclnn.ACL_FORMAT_NCDHW))
    arr = lambda h: (ctypes.c_void_p * len(h))(*h)
    arrs = [arr(h) for h in hs]
    m = aclnn.create_bool_array(list(mask))
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ev, wall = ctypes.c_double(0), ctypes.c_double(0)
    st, ws_bytes, ex = aclnn.get_workspace_size_grid_sampler3d_backward(hs[0][0], hs[1][0], hs[2][0], 0, 0, False, m,
                                                                        hs[3][0], hs[4][0])
    assert st == 0
    variant = aclnn.executor_variant(ex)
    aclnn.destroy_executor(ex)
    work = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)  # the spans of the chunks of grid points
    wptr = ctypes.c_void_p(work.data_ptr())

    def run(k, warm=0):
        rc = L.opscv_bench_grid_sampler3d_backward(*arrs, sets, 0, 0, False, m, wptr, ws_bytes, warm, k, stream,
                                                   ctypes.byref(ev), ctypes.byref(wall))
        if rc != 0:
            raise RuntimeError("bench loop failed rc=%d: %s" % (rc, aclnn.load_library().aclGetRecentErrMsg()))
        return Timed(ev.value, wall.value, k)

    t = _finish(L, run, ts[0], ts[3], steps, warmup, stream)
    rdx, rdg = oracle_lib.grid_sampler3d_backward(*first, 0, 0, False, dtype=I.oracle_code(dtype))
    parity = _parity(I.from_torch(ts[3][0], dtype), rdx, dtype)
    parity["grid_grad_bit_exact"] = bool(np.array_equal(I.from_torch(ts[4][0], dtype).view(np.uint8),
                                                        rdg.view(np.uint8)))
    for hl in hs:
        for h in hl:
            aclnn.destroy_tensor(h)
    aclnn.destroy_bool_array(m)
    e = esize(dtype)
    # gradOutput read by both gradients' kernels, input read once, grid read twice, both gradients written
    alg = (2 * N * C * Do * Ho * Wo + 2 * N * C * D * H * W + 3 * N * Do * Ho * Wo * 3) * e
    return dict(steps=steps, workload="%s grid_sampler3d_backward fp16 x(%d,%d,%d,%d,%d) grid(%d,%d,%d,%d,3) bilinear zeros "
                         "align_corners=False both gradients" % (label, N, C, D, H, W, N, Do, Ho, Wo),
                samples=N * C * Do * Ho * Wo, alg_bytes=alg, timed=t, variant=variant, parity=parity, sets=sets,
                default_modes=True)


def bench_gs_backward(steps, warmup, sets=4, mask=(True, True)):
    """Backward of the headline sampler workload (fp16 N16 C256 64x64, affine grid): both gradients."""
    import numpy as np
    import torch
    import inputs as I
    import oracle_lib
    from ops_cv_amd import aclnn
    dev = torch.device("cuda:0")
    L = load_bench_lib()
    w = GS_WORKLOADS["C3"]
    dtype = w["dtype"]
    N, C, H, W = w["x"]
    _, Ho, Wo = w["grid"]
    ts, hs = [[] for _ in range(5)], [[] for _ in range(5)]
    first = None
    for s in range(sets):
        x, g = make_gs_inputs("C3", 5000 + s)
        go = I.cast_np(np.random.default_rng(5100 + s).standard_normal((N, C, Ho, Wo)).astype(np.float32), dtype)
        if s == 0:
            first = (go, x, g)
        tens = [I.to_torch(go, dtype, dev), I.to_torch(x, dtype, dev), I.to_torch(g, dtype, dev)]
        tens += [torch.empty_like(tens[1]), torch.empty_like(tens[2])]
        for lst, hl, t in zip(ts, hs, tens):
            lst.append(t)
            hl.append(aclnn.tensor_handle(t))
    arr = lambda h: (ctypes.c_void_p * len(h))(*h)
    arrs = [arr(h) for h in hs]
    m = aclnn.create_bool_array(list(mask))
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ev, wall = ctypes.c_double(0), ctypes.c_double(0)

    st, ws_bytes, ex = aclnn.get_workspace_size_grid_sampler2d_backward(hs[0][0], hs[1][0], hs[2][0], 0, 0, False, m,
                                                                        hs[3][0], hs[4][0])
    assert st == 0
    variant = aclnn.executor_variant(ex)
    aclnn.destroy_executor(ex)
    work = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)  # the input gradient's contribution lists
    wptr = ctypes.c_void_p(work.data_ptr()) if ws_bytes else None

    def run(k, warm=0):
        rc = L.opscv_bench_grid_sampler2d_backward(*arrs, sets, 0, 0, False, m, wptr, ws_bytes, warm, k, stream,
                                                   ctypes.byref(ev), ctypes.byref(wall))
        if rc != 0:
            raise RuntimeError("bench loop failed rc=%d: %s" % (rc, aclnn.load_library().aclGetRecentErrMsg()))
        return Timed(ev.value, wall.value, k)

    t = _finish(L, run, ts[0], ts[3], steps, warmup, stream)
    rdx, rdg = oracle_lib.grid_sampler2d_backward(*first, 0, 0, False, dtype=I.oracle_code(dtype))
    parity = _parity(I.from_torch(ts[3][0], dtype), rdx, dtype)
    parity["grid_grad_bit_exact"] = bool(np.array_equal(I.from_torch(ts[4][0], dtype).view(np.uint8),
                                                        rdg.view(np.uint8)))
    for hl in hs:
        for h in hl:
            aclnn.destroy_tensor(h)
    aclnn.destroy_bool_array(m)
    e = esize(dtype)
    # gradOutput read for both gradients' kernels, input read once, grid read, both gradients written
    alg = (N * C * Ho * Wo + 2 * N * C * H * W + 2 * N * Ho * Wo * 2) * e
    return dict(steps=steps, workload="G3 grid_sampler2d_backward fp16 x(16,256,64,64) grid(16,64,64,2) bilinear zeros "
                         "align_corners=False both gradients", samples=N * C * Ho * Wo, alg_bytes=alg, timed=t,
                variant=variant, parity=parity, sets=sets, default_modes=True)


def bench_resize_like(kind, steps, warmup, sets=2):
    """The 4K workload through the neighbouring entry points: kind "backward" (aclnnUpsampleBilinear2dBackward, the
    gradient of the 2x upscale) or "nearest" (aclnnResize, mode nearest)."""
    import numpy as np
    import torch
    import inputs as I
    import oracle_lib
    from ops_cv_amd import aclnn
    dev = torch.device("cuda:0")
    L = load_bench_lib()
    dtype = "fp16"
    N, C, Hs, Ws, Hd, Wd = 4, 16, 1080, 1920, 2160, 3840
    in_shape = (N, C, Hd, Wd) if kind == "backward" else (N, C, Hs, Ws)
    out_shape = (N, C, Hs, Ws) if kind == "backward" else (N, C, Hd, Wd)
    xs, ys, hx, hy = [], [], [], []
    x0 = None
    for s in range(sets):
        rng = np.random.default_rng(4000 + s)
        x = I.cast_np(rng.uniform(-1, 1, in_shape).astype(np.float32), dtype)
        if s == 0:
            x0 = x
        xs.append(I.to_torch(x, dtype, dev))
        ys.append(torch.empty(out_shape, dtype=xs[-1].dtype, device=dev))
        hx.append(aclnn.tensor_handle(xs[-1], aclnn.ACL_FORMAT_NCHW))
        hy.append(aclnn.tensor_handle(ys[-1], aclnn.ACL_FORMAT_NCHW))
    arr = lambda h: (ctypes.c_void_p * len(h))(*h)
    ax, ay = arr(hx), arr(hy)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ev, wall = ctypes.c_double(0), ctypes.c_double(0)
    planes = 2
    if kind == "backward":
        osz, isz = aclnn.create_int_array([Hd, Wd]), aclnn.create_int_array([N, C, Hs, Ws])

        def run(k, warm=0):
            rc = L.opscv_bench_upsample_bilinear2d_backward(ax, ay, sets, osz, isz, True, 2.0, 2.0, None, 0, warm, k, stream,
                                                            ctypes.byref(ev), ctypes.byref(wall))
            if rc != 0:
                raise RuntimeError("bench loop failed rc=%d: %s" % (rc, aclnn.load_library().aclGetRecentErrMsg()))
            return Timed(ev.value, wall.value, k)

        st, _, ex = aclnn.get_workspace_size_upsample_bilinear2d_backward(hx[0], osz, isz, True, 2.0, 2.0, hy[0])
        ref = oracle_lib.upsample_bilinear2d_backward(x0.reshape(N * C, 1, Hd, Wd)[:planes], (Hs, Ws), True,
                                                      dtype=I.oracle_code(dtype))
        desc = "B4 upsample_bilinear2d_backward fp16 grad(4,16,2160,3840)->(4,16,1080,1920) align_corners=True"
    else:
        sc = aclnn.create_float_array([1.0, 1.0, 2.0, 2.0])

        def run(k, warm=0):
            rc = L.opscv_bench_resize(ax, ay, sets, sc, b"nearest", None, 0, warm, k, stream, ctypes.byref(ev),
                                      ctypes.byref(wall))
            if rc != 0:
                raise RuntimeError("bench loop failed rc=%d: %s" % (rc, aclnn.load_library().aclGetRecentErrMsg()))
            return Timed(ev.value, wall.value, k)

        st, _, ex = aclnn.get_workspace_size_resize(hx[0], sc, b"nearest", hy[0])
        ref = oracle_lib.resize_nearest(x0.reshape(N * C, 1, Hs, Ws)[:planes], (Hd, Wd), dtype=I.oracle_code(dtype))
        desc = "R4 resize nearest fp16 (4,16,1080,1920)->(4,16,2160,3840)"
    assert st == 0, aclnn.load_library().aclGetRecentErrMsg()
    variant = aclnn.executor_variant(ex)
    aclnn.destroy_executor(ex)
    t = _finish(L, run, xs, ys, steps, warmup, stream)
    got = I.from_torch(ys[0], dtype).reshape((N * C, 1) + out_shape[2:])[:planes]
    parity = _parity(got, ref, dtype, planes_checked=planes)
    for h in hx + hy:
        aclnn.destroy_tensor(h)
    samples = int(np.prod(out_shape))
    alg = (int(np.prod(in_shape)) + samples) * esize(dtype)
    return dict(steps=steps, workload=desc, samples=samples, alg_bytes=alg, timed=t, variant=variant, parity=parity, sets=sets,
                default_modes=True)


def roofline_of(r):
    gbs = r["alg_bytes"] / (r["timed"].kernel_us * 1e-6) / 1e9
    name = r["workload"].split(" ")[0]
    from ops_cv_amd import aclnn
    traffic, source = None, None
    revision = aclnn.variant_revision(r["variant"])
    if r.get("default_modes", True):
        traffic, measured_revision, source = MEASURED_TRAFFIC.get((name, r["variant"]), (None, None, None))
        if measured_revision != revision:
            traffic, source = None, None  # measured on another revision of the kernel: not this run's traffic
    out = {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
           "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": traffic, "traffic_source": source if traffic else None,
           "kernel_us": round(r["timed"].kernel_us, 3), "algorithmic_bytes": r["alg_bytes"],
           "kernel": r["variant"], "kernel_revision": revision}
    su = r["timed"].stream_us
    if su:
        # a kernel that only moves the same input and output bytes, measured the same way in the same run
        out["streaming_reference_us"] = round(su, 3)
        out["frac_of_streaming_reference"] = round(su / r["timed"].kernel_us, 4)
    return out


def host_of(r):
    t = r["timed"]
    return {"phase1_get_workspace_size": round(t.host_phase1_us, 3), "phase2_launch": round(t.host_phase2_us, 3)}


def summary_of(r):
    t = r["timed"]
    return {"workload": r["workload"], "samples_per_s": r["samples"] / (t.step_ms * 1e-3),
            "ms_per_step": round(t.step_ms, 6), "roofline": roofline_of(r), "host_us_per_call": host_of(r),
            "parity_vs_oracle": r["parity"], "tensor_sets": r["sets"], "timed_launches": r.get("steps")}


def cpu_baseline_gs(x0, g0, w, budget_s=12.0):
    """The CPU oracle on the full headline workload, all host threads, repeated for about `budget_s` seconds."""
    import inputs as I
    import oracle_lib
    threads = oracle_lib.lib().oracle_max_threads()
    N, C = w["x"][0], w["x"][1]
    Ho, Wo = w["grid"][1], w["grid"][2]
    samples = N * C * Ho * Wo
    reps, t0 = 0, time.perf_counter()
    while True:
        oracle_lib.grid_sampler2d(x0, g0, w["interp"], w["pad"], w["align"], dtype=I.oracle_code(w["dtype"]),
                                  threads=threads)
        reps += 1
        el = time.perf_counter() - t0
        if el > budget_s or reps >= 200:
            break
    t1 = time.perf_counter()
    oracle_lib.grid_sampler2d(x0, g0, w["interp"], w["pad"], w["align"], dtype=I.oracle_code(w["dtype"]), threads=1)
    one = time.perf_counter() - t1
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            for ln in f:
                if ln.startswith("model name"):
                    model = ln.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {"value": samples * reps / el, "unit": "samples/s", "cores": threads, "kind": "port", "cpu_model": model,
            "sample": "full workload (%d output samples) x %d repetitions, OpenMP static over output pixels" % (
                samples, reps),
            "single_thread_samples_per_s": samples / one}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="C3", help="headline workload: C1..C5, L1 (sampler on 1080p planes), or one of the neighbouring entry points V1 (3-D sampler), G3 "
                         "(sampler backward), W1 (3-D sampler backward; W1s: few points in a large volume), B4 (resize backward), R4 (nearest resize)")
    ap.add_argument("--only", action="store_true", help="skip the other workloads and the CPU baseline")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy (torch copy_) so that a counter run of this command "
                         "holds a kernel of known traffic to scale FETCH_SIZE / WRITE_SIZE by")
    ap.add_argument("--sets", type=int, default=None,
                    help="tensor sets rotated through by the headline workload (default: enough to exceed the last-level "
                         "cache; 1 = the same buffers every step, operands warm)")
    ap.add_argument("--interp", type=int, default=None, help="sampler workloads: interpolation mode instead of the workload's own")
    ap.add_argument("--pad", type=int, default=None, help="sampler workloads: padding mode instead of the workload's own")
    ap.add_argument("--preheat-ms", type=float, default=300.0,
                    help="untimed GPU work before each timed region, on top of --warmup steps")
    args = ap.parse_args()
    global PREHEAT_MS
    PREHEAT_MS = args.preheat_ms
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path shards over the batch axis with no "
              "communication); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(3)
    torch.cuda.set_device(0)

    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda:0").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    head = args.workload
    if head in GS_WORKLOADS:
        r = bench_gs(head, args.steps, args.warmup, sets=args.sets, interp=args.interp, pad=args.pad)
    elif head in UP_WORKLOADS:
        r = bench_up(head, args.steps, args.warmup, sets=args.sets)
    elif head == "V1":
        r = bench_gs3d(args.steps, args.warmup)
    elif head == "V1cl":
        r = bench_gs3d(args.steps, args.warmup, channels_last=True)
    elif head == "G3":
        r = bench_gs_backward(args.steps, args.warmup)
    elif head == "W1":
        r = bench_gs3d_backward(args.steps, args.warmup)
    elif head == "W1s":
        r = bench_gs3d_backward(args.steps, args.warmup, **W1_SPARSE)
    elif head == "B4":
        r = bench_resize_like("backward", args.steps, args.warmup)
    elif head == "R4":
        r = bench_resize_like("nearest", args.steps, args.warmup)
    else:
        print("bench.py: unknown workload %s" % head, file=sys.stderr)
        sys.exit(2)
    t = r["timed"]
    line = {
        "metric": "output samples/s, grid_sampler2d fp16 N16 C256 (achieved HBM GB/s in roofline)" if head == "C3"
        else "output samples/s",
        "value": r["samples"] / (t.step_ms * 1e-3),
        "unit": "samples/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "preheat_ms": args.preheat_ms,
        "ms_per_step": t.step_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": ARITHMETIC[head],
        "data": "synthetic",
        "config": {"workload": r["workload"], "tensor_sets_rotated": r["sets"], "kernel": r["variant"],
                   "parity_vs_oracle": r["parity"]},
        "roofline": roofline_of(r),
        "host_us_per_call": host_of(r),
    }
    try:
        props = torch.cuda.get_device_properties(0)
        line["device"] = {"name": props.name, "compute_units": props.multi_processor_count,
                          "memory_GiB": round(props.total_memory / 2**30, 1),
                          "memory_clock_kHz": getattr(props, "memory_clock_rate", None),
                          "memory_bus_bits": getattr(props, "memory_bus_width", None)}
    except Exception:  # informational only
        line["device"] = None
    if not args.only and not args.no_cpu and head in GS_WORKLOADS:
        line["cpu_baseline"] = cpu_baseline_gs(*r["cpu"])
    else:
        line["cpu_baseline"] = None
    if not args.only:
        others = {}
        # the secondary workloads are timed over at least MIN_TIMED_LAUNCHES launches each, so that their figures
        # are reproducible whatever --steps asks for the headline
        ko = max(MIN_TIMED_LAUNCHES, args.steps)
        if head == "C3":
            for interp in (0, 1):
                for pad in (0, 1, 2):
                    if interp == 0 and pad == 0:
                        continue
                    rr = bench_gs("C3", ko, args.warmup, interp=interp, pad=pad)
                    others["C3_%s_%s" % (INTERP_NAMES[interp], PAD_NAMES[pad])] = summary_of(rr)
            rr = bench_gs("C3", ko, args.warmup, sets=1)
            others["C3_bilinear_zeros_same_buffers_every_step"] = summary_of(rr)
            # warm operands beside the cold headline: the closer the two, the less the kernel is bound by HBM
            line["roofline"]["kernel_us_same_buffers_every_step"] = round(rr["timed"].kernel_us, 3)
            others["C3_bilinear_zeros_align_corners"] = summary_of(bench_gs("C3", ko, args.warmup, align=True))
            others["C3_bilinear_zeros_channels_last"] = summary_of(bench_gs("C3", ko, args.warmup,
                                                                             channels_last=True))
            # the third interpolation mode on the same tensors (not part of the headline set)
            others["C3_bicubic_zeros"] = summary_of(bench_gs("C3", ko, args.warmup, interp=2))
        for name in ("C1", "C5"):
            if name != head:
                others[name] = summary_of(bench_gs(name, ko, args.warmup))
        for name in ("C2", "C4"):
            if name != head:
                others[name] = summary_of(bench_up(name, ko, args.warmup))
        if head != "L1":
            # not a BASELINE configuration: planes beyond LDS (1080p), the shape image warps come in
            others["L1_sampler_1080p_planes"] = summary_of(bench_gs("L1", min(ko, 50), min(args.warmup, 5)))
        # the entry points either side of the path, on shapes of the same scale
        others["V1_grid_sampler3d"] = summary_of(bench_gs3d(ko, args.warmup))
        others["V1_grid_sampler3d_ndhwc"] = summary_of(bench_gs3d(ko, args.warmup, channels_last=True))
        others["G3_grid_sampler2d_backward"] = summary_of(bench_gs_backward(ko, args.warmup))
        others["W1_grid_sampler3d_backward"] = summary_of(bench_gs3d_backward(ko, args.warmup))
        others["W1s_grid_sampler3d_backward_sparse_volume"] = summary_of(bench_gs3d_backward(min(ko, 50), min(args.warmup, 5),
                                                                                           **W1_SPARSE))
        others["B4_upsample_backward"] = summary_of(bench_resize_like("backward", ko, args.warmup))
        others["R4_resize_nearest"] = summary_of(bench_resize_like("nearest", ko, args.warmup))
        line["other_workloads"] = others
        if head == "C3" and "C4" in others:
            # the second configuration with a bandwidth target (the 4K upscale), in the headline's own roofline object
            c4 = others["C4"]
            line["roofline"]["second_target"] = {
                "workload": c4["workload"], "kernel": c4["roofline"]["kernel"], "ms_per_step": c4["ms_per_step"],
                "kernel_us": c4["roofline"]["kernel_us"], "achieved": c4["roofline"]["achieved"], "unit": "GB/s",
                "frac": c4["roofline"]["frac"], "algorithmic_bytes": c4["roofline"]["algorithmic_bytes"],
                "streaming_reference_us": c4["roofline"].get("streaming_reference_us"),
                "parity_vs_oracle": c4["parity_vs_oracle"], "timed_launches": c4["timed_launches"]}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
