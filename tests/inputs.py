"""Seeded synthetic inputs shared by the parity tests, the smoke entry and the benchmark.

Everything is generated on the host with numpy so that the CPU oracle and the GPU kernels see the same bits.
bf16 tensors travel as uint16 bit patterns on the numpy side.
"""
import numpy as np

from oracle_lib import f32_to_bf16_bits

DTYPES = ("fp32", "fp16", "bf16")


def cast_np(a32, dtype):
    """float32 numpy array -> the numpy carrier of `dtype` (float32, float16, or uint16 bf16 bits)."""
    if dtype == "fp32":
        return np.ascontiguousarray(a32, dtype=np.float32)
    if dtype == "fp16":
        with np.errstate(over="ignore"):  # special-value grids hold 1e10 and 3e38 on purpose (they become inf)
            return np.ascontiguousarray(a32).astype(np.float16)
    if dtype == "bf16":
        return f32_to_bf16_bits(a32)
    raise ValueError(dtype)


def oracle_code(dtype):
    return {"fp32": 0, "fp16": 1, "bf16": 2}[dtype]


def to_torch(a, dtype, device):
    import torch
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype == "bf16":
        t = t.view(torch.bfloat16)
    return t.to(device)


def from_torch(t, dtype):
    import torch
    t = t.detach().cpu().contiguous()
    if dtype == "bf16":
        return t.view(torch.uint16).numpy() if hasattr(torch, "uint16") else t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def as_f32(a, dtype):
    """numpy carrier -> float32 values (for error metrics)."""
    if dtype == "bf16":
        return (a.astype(np.uint32) << 16).view(np.float32)
    return a.astype(np.float32)


def affine_grid(rng, N, Ho, Wo, max_deg=30.0, scale=(0.8, 1.2), shift=0.2):
    """Per-batch affine warps of the align_corners=False pixel-centre lattice (float32, (N,Ho,Wo,2))."""
    theta = np.deg2rad(rng.uniform(-max_deg, max_deg, N))
    s = rng.uniform(scale[0], scale[1], N)
    t = rng.uniform(-shift, shift, (N, 2))
    xs = (2.0 * np.arange(Wo) + 1.0) / Wo - 1.0
    ys = (2.0 * np.arange(Ho) + 1.0) / Ho - 1.0
    px, py = np.meshgrid(xs, ys)  # (Ho,Wo)
    g = np.empty((N, Ho, Wo, 2), dtype=np.float32)
    for n in range(N):
        c, sn = np.cos(theta[n]) * s[n], np.sin(theta[n]) * s[n]
        g[n, ..., 0] = c * px - sn * py + t[n, 0]
        g[n, ..., 1] = sn * px + c * py + t[n, 1]
    return g


def special_grid_values():
    """Coordinates that exercise ties, borders, huge magnitudes and non-finite values."""
    vals = [-1.0, 1.0, 0.0, -0.0, 0.5, -0.5, 0.25, 0.75, -0.999, 0.999, 1.0001, -1.0001, 1.5, -1.5, 2.0, -2.0, 3.0,
            -3.0, 7.3, -7.3, 100.0, -100.0, 1e10, -1e10, 3e38, -3e38, np.inf, -np.inf, np.nan, 1e-30, -1e-30,
            0.6999999, 0.7, 0.33333334, 0.125, -0.125, 0.875, -0.875]
    return np.array(vals, dtype=np.float32)


def special_grid(W_out_hint=None):
    """(1, K, K, 2) grid holding every ordered pair of the special values."""
    v = special_grid_values()
    gx, gy = np.meshgrid(v, v)
    g = np.stack([gx, gy], axis=-1)[None].astype(np.float32)
    return g
