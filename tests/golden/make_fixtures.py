"""Writes the golden fixtures of this directory with the PyTorch that is installed in the build container.

PyTorch's CPU grid_sample / interpolate are the library routines the whole path reduces to (the reference's own
golden scripts delegate to them: image/grid_sampler2_d/tests/assets/golden.py:71-77,
image/upsample_bilinear2d/tests/ut/op_kernel/upsample_bilinear2d_data/gen_data.py:39).  No reference file is
imported or executed here.  16-bit cases follow the reference's convention of computing in fp32 and casting back
(image/grid_sample/tests/st/aclnnGridSampler2D/executor_aclnnGridSampler2D.py:48-52).

Run:  python tests/golden/make_fixtures.py      (deterministic; rewrites the .npz files)
"""
import os

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
MODES = ["bilinear", "nearest"]
PADS = ["zeros", "border", "reflection"]


def special_values():
    return np.array([-1.0, 1.0, 0.0, -0.0, 0.5, -0.5, 0.25, 0.75, -0.999, 0.999, 1.0001, -1.0001, 1.5, -1.5, 2.0,
                     -2.0, 3.0, -3.0, 7.3, -7.3, 100.0, -100.0, 1e10, -1e10, np.inf, -np.inf, np.nan, 0.6999999,
                     0.7, 0.33333334, 0.125, -0.875], dtype=np.float32)


def main():
    rng = np.random.default_rng(20240607)
    out = {}
    # ---- grid sampler: random coordinates, every mode combination ----
    shapes = [(2, 3, 5, 8, 4, 6), (1, 2, 10, 10, 7, 9), (1, 1, 1, 7, 3, 5), (2, 2, 13, 17, 11, 5)]
    for si, (N, C, H, W, Ho, Wo) in enumerate(shapes):
        x = rng.standard_normal((N, C, H, W)).astype(np.float32)
        g = rng.uniform(-1.4, 1.4, (N, Ho, Wo, 2)).astype(np.float32)
        out["gs%d_x" % si] = x
        out["gs%d_grid" % si] = g
        for m in range(2):
            for p in range(3):
                for a in (0, 1):
                    y = F.grid_sample(torch.from_numpy(x), torch.from_numpy(g), mode=MODES[m], padding_mode=PADS[p],
                                      align_corners=bool(a)).numpy()
                    out["gs%d_y_m%d_p%d_a%d" % (si, m, p, a)] = y
    # ---- grid sampler: special coordinates (ties, borders, huge, non-finite) ----
    v = special_values()
    gx, gy = np.meshgrid(v, v)
    g = np.stack([gx, gy], axis=-1)[None].astype(np.float32)
    for si, (H, W) in enumerate([(5, 8), (10, 10), (4, 1)]):
        x = rng.standard_normal((1, 2, H, W)).astype(np.float32)
        out["sp%d_x" % si] = x
        out["sp%d_grid" % si] = g
        for m in range(2):
            for p in range(3):
                for a in (0, 1):
                    y = F.grid_sample(torch.from_numpy(x), torch.from_numpy(g), mode=MODES[m], padding_mode=PADS[p],
                                      align_corners=bool(a)).numpy()
                    out["sp%d_y_m%d_p%d_a%d" % (si, m, p, a)] = y
    # ---- the fma-vs-mul tap: W=10, gx=0.6999999 lands a hair below 8.0 only with the fused unnormalize ----
    x = np.zeros((1, 1, 1, 10), dtype=np.float32)
    x[..., 8] = 1e6
    g = np.array([[[[0.6999999, 0.0]]]], dtype=np.float32)
    out["fma_x"] = x
    out["fma_grid"] = g
    out["fma_y"] = F.grid_sample(torch.from_numpy(x), torch.from_numpy(g), mode="bilinear", padding_mode="zeros",
                                 align_corners=False).numpy()
    # ---- 16-bit grid sampler: fp32 compute on the 16-bit values, cast back ----
    x = rng.standard_normal((1, 3, 9, 12)).astype(np.float32)
    g = rng.uniform(-1.2, 1.2, (1, 6, 7, 2)).astype(np.float32)
    for name, dt in (("f16", torch.float16), ("bf16", torch.bfloat16)):
        xt = torch.from_numpy(x).to(dt)
        gt = torch.from_numpy(g).to(dt)
        out["h_%s_x" % name] = xt.view(torch.int16).numpy().view(np.uint16)
        out["h_%s_grid" % name] = gt.view(torch.int16).numpy().view(np.uint16)
        for m in range(2):
            for p in range(3):
                for a in (0, 1):
                    y = F.grid_sample(xt.float(), gt.float(), mode=MODES[m], padding_mode=PADS[p],
                                      align_corners=bool(a)).to(dt)
                    out["h_%s_y_m%d_p%d_a%d" % (name, m, p, a)] = y.view(torch.int16).numpy().view(np.uint16)
    np.savez_compressed(os.path.join(HERE, "grid_sampler2d.npz"), **out)

    # ---- bicubic mode on the same inputs (outputs only; inputs are read from grid_sampler2d.npz) ----
    bic = {}
    for key in sorted(out):
        if not key.endswith("_x") or key == "fma_x":
            continue
        stem = key[:-2]
        x, g = out[key], out[stem + "_grid"]
        if stem.startswith("h_"):
            dt = torch.float16 if stem == "h_f16" else torch.bfloat16
            xt = torch.from_numpy(x.view(np.int16)).view(dt)
            gt = torch.from_numpy(g.view(np.int16)).view(dt)
        for p in range(3):
            for a in (0, 1):
                if stem.startswith("h_"):
                    y = F.grid_sample(xt.float(), gt.float(), mode="bicubic", padding_mode=PADS[p],
                                      align_corners=bool(a)).to(dt).view(torch.int16).numpy().view(np.uint16)
                else:
                    y = F.grid_sample(torch.from_numpy(x), torch.from_numpy(g), mode="bicubic", padding_mode=PADS[p],
                                      align_corners=bool(a)).numpy()
                bic["%s_y_m2_p%d_a%d" % (stem, p, a)] = y
    np.savez_compressed(os.path.join(HERE, "grid_sampler2d_bicubic.npz"), **bic)

    # ---- upsample ----
    up = {}
    cases = [((1, 1, 4, 2), (8, 4)), ((2, 3, 7, 9), (14, 18)), ((1, 2, 5, 5), (13, 7)), ((2, 2, 16, 16), (5, 3)),
             ((1, 1, 1, 4), (2, 16)), ((1, 1, 1, 4), (3, 16)), ((2, 3, 1, 1), (4, 4)), ((1, 2, 6, 6), (1, 1)),
             ((1, 2, 9, 11), (9, 11)), ((1, 1, 33, 65), (67, 200))]
    for ci, (shape, size) in enumerate(cases):
        x = rng.standard_normal(shape).astype(np.float32)
        if ci == 0:
            x = np.arange(8, dtype=np.float32).reshape(shape)  # the reference example's input
        up["up%d_x" % ci] = x
        up["up%d_size" % ci] = np.array(size, dtype=np.int64)
        for a in (0, 1):
            y = F.interpolate(torch.from_numpy(x), size=size, mode="bilinear", align_corners=bool(a)).numpy()
            up["up%d_y_a%d" % (ci, a)] = y
    # user scale factors (recompute_scale_factor=False keeps the given scale)
    x = rng.standard_normal((1, 2, 10, 12)).astype(np.float32)
    up["ups_x"] = x
    for si, (sh, sw) in enumerate([(2.0, 2.0), (2.5, 1.5), (1.7, 2.4)]):
        y = F.interpolate(torch.from_numpy(x), scale_factor=(sh, sw), mode="bilinear", align_corners=False,
                          recompute_scale_factor=False).numpy()
        up["ups_y_%d" % si] = y
        up["ups_scale_%d" % si] = np.array([sh, sw], dtype=np.float64)
    np.savez_compressed(os.path.join(HERE, "upsample_bilinear2d.npz"), **up)
    print("wrote", sorted(os.listdir(HERE)))


if __name__ == "__main__":
    main()
