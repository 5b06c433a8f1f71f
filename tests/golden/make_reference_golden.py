"""Writes tests/golden/reference_conventions.npz from the reference's own Python, run on the CPU.

What it pins are the drop-in conventions that no closed form fixes and that were otherwise only
checked against a restatement of the same source text: the module's initialisation (RNG call
order, std, bias edits; src/igs/gs2d.py:480-501), the `gs_feature` split order and activations
of `forward` (:635-644, :673-675), `xy_grid` (:503-522), `pos_map_offset` (:654-667), and
`naive_gaussian_2d` (:24-44) through `render(fused=False)` (:548-609).

Run in the build container only (the reference checkout does not travel):

    python tests/golden/make_reference_golden.py [/root/reference]

Dynamo is switched off (the reference decorates `render` with torch.compile) and only CPU code of
the reference runs: `fused=False`, the plain-torch debug path.  The fixture holds inputs and
outputs only.
"""
import os
import sys

os.environ["TORCHDYNAMO_DISABLE"] = "1"

import numpy as np  # noqa: E402
import torch  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def main(ref_root: str) -> int:
    sys.path.insert(0, os.path.join(ref_root, "src"))
    from igs import gs2d as R  # the reference

    torch.set_num_threads(1)
    out = {}

    # 1. module initialisation under a fixed seed
    torch.manual_seed(20240607)
    m = R.GaussianSplatting2D(4, 32)
    sd = m.state_dict()
    assert sorted(sd) == ["proj.bias", "proj.weight"]
    out["init_seed"] = np.int64(20240607)
    out["init_weight"] = sd["proj.weight"].numpy().copy()
    out["init_bias"] = sd["proj.bias"].numpy().copy()

    # 2. a tiny forward through the plain-torch path
    g = torch.Generator().manual_seed(7)
    x = torch.randn(2, 5, 32, generator=g)
    with torch.no_grad():
        # make the head's output non-trivial and well conditioned: spread positions, scales around
        # exp(-1) of the image extent (every pixel then has a weight sum far above eps, so the
        # fp32 reference output is accurate to a few 1e-6)
        m.proj.weight.mul_(10.0)
        m.proj.bias.view(4, 9)[:, 2:4] = -1.0
        image, feat = m(x, size=(6, 10), fused=False)
    out["fwd_weight"] = m.proj.weight.detach().numpy().copy()
    out["fwd_bias"] = m.proj.bias.detach().numpy().copy()
    out["fwd_x"] = x.numpy()
    out["fwd_image"] = image.numpy()
    out["fwd_gs_feature"] = feat.numpy()

    # 3. the same with pos_map_offset (positions relative to one grid point per feature)
    torch.manual_seed(11)
    mo = R.GaussianSplatting2D(3, 16, output_dim=2, pos_map_offset=True)
    xo = torch.randn(1, 6, 16, generator=g)      # 6 features = a 2 x 3 grid
    yy, xx = torch.meshgrid(torch.linspace(-1, 1, 2), torch.linspace(-1.5, 1.5, 3), indexing="ij")
    grid = torch.stack([yy, xx])[None]            # [1, 2, 2, 3]: h positions first, as the reference expects
    with torch.no_grad():
        mo.proj.weight.mul_(10.0)
        mo.proj.bias.view(3, 8)[:, 2:4] = -1.0
        image_o, feat_o = mo(xo, grid=grid, fused=False)
    out["off_weight"] = mo.proj.weight.detach().numpy().copy()
    out["off_bias"] = mo.proj.bias.detach().numpy().copy()
    out["off_x"] = xo.numpy()
    out["off_grid"] = grid.numpy()
    out["off_image"] = image_o.numpy()
    out["off_gs_feature"] = feat_o.numpy()

    # 4. xy_grid on a non-square size
    xg, yg = R.GaussianSplatting2D.xy_grid((6, 10))
    out["xy_size"] = np.array([6, 10])
    out["xy_x"] = xg.contiguous().numpy()
    out["xy_y"] = yg.contiguous().numpy()

    # 5. naive_gaussian_2d on two tiny cases (operator-level arguments)
    for tag, (B, N, H, W, C) in (("naive_a", (2, 5, 3, 4, 3)), ("naive_b", (1, 7, 4, 2, 1))):
        gx = torch.rand(B, 1, H, W, generator=g) * 2 - 1
        gy = torch.rand(B, 1, H, W, generator=g) * 2 - 1
        pos = torch.rand(B, N, 2, generator=g) * 2 - 1
        s = torch.rand(B, N, 2, generator=g) * 0.5 + 0.2
        th = torch.rand(B, N, generator=g) * 6.28
        c, sn = torch.cos(th), torch.sin(th)
        i0, i1 = 1 / s[..., 0] ** 2, 1 / s[..., 1] ** 2
        a = (c * c * i0 + sn * sn * i1)[..., None, None]
        b = (c * sn * (i0 - i1))[..., None, None]
        d = (sn * sn * i0 + c * c * i1)[..., None, None]
        al = torch.rand(B, N, generator=g)
        col = torch.rand(B, N, C, generator=g)
        res = R.naive_gaussian_2d(gx, gy, pos, a, b, d, al, col, 1e-6)
        for k, v in dict(x=gx, y=gy, position=pos, a=a, b=b, d=d, alphas=al, colors=col, out=res).items():
            out[f"{tag}_{k}"] = v.numpy()

    # 6. render(fused=False): the covariance preamble + naive expression from scales / rotations
    B, N, H, W, C = 2, 6, 5, 7, 3
    pos = torch.rand(B, N, 2, generator=g) * 2 - 1
    col = torch.rand(B, N, C, generator=g)
    sc = torch.rand(B, N, 2, generator=g) * 0.4 + 0.2
    rot = torch.rand(B, N, generator=g) * 6.28
    al = torch.rand(B, N, generator=g)
    xg, yg = R.GaussianSplatting2D.xy_grid((H, W))
    xg, yg = xg[None].repeat(B, 1, 1, 1), yg[None].repeat(B, 1, 1, 1)
    res = R.gaussian_splatting_2d(pos, col, sc, rot, al, xg, yg, 1e-6, False)
    for k, v in dict(positions=pos, colors=col, scales=sc, rotations=rot, alphas=al, x=xg, y=yg, out=res).items():
        out[f"render_{k}"] = v.numpy()

    path = os.path.join(HERE, "reference_conventions.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, {k: v.shape for k, v in out.items() if hasattr(v, "shape")})
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference"))
