"""The benchmark configurations at their FULL sizes, where the CPU oracle would take minutes:
checked through properties that do not depend on size.

* integers: rem0 are multiples of pd+1 that sum to zero, ranks are permutations, barycentric
  weights are non-negative and sum to one, and the vertex count equals the number of distinct
  per-point keys counted independently (sort + unique of all N*(pd+1) keys on the GPU);
* a constant input comes back as that constant (the normalisation cancels the weights);
* the bare operator (no normalisation) is linear, and the reverse pass is its adjoint:
  <A_forward x, y> = <x, A_reverse y>, because every axis blur is a symmetric matrix and slice is
  the transpose of splat (the forward order on both sides is off by about 1 %: the check
  discriminates);
* build + apply equals filter.
"""
import numpy as np
import pytest
import torch

from permutohedral_lattice_amd import synth

import permutohedral_lattice_amd as pla

pytestmark = pytest.mark.gpu


def _positions(name):
    if name == "cfg1_512_rgb":
        img = synth.blob_image(512, 512, seed=0xC0FFEE + 1)
        return 5, 4, (512, 512), synth.bilateral_positions(img, 8.0, 0.125)
    if name == "north_star_1024_rgb":
        img = synth.blob_image(1024, 1024, seed=0xC0FFEE)
        return 5, 4, (1024, 1024), synth.bilateral_positions(img, 8.0, 0.125)
    if name == "cfg2_1024_spatial":
        return 2, 2, (1024, 1024), synth.spatial_positions((1024, 1024), 8.0)
    if name == "cfg3_1024_guided":
        img = synth.blob_image(1024, 1024, seed=0xC0FFEE + 3)
        return 5, 2, (1024, 1024), synth.bilateral_positions(img, 8.0, 0.125)
    if name == "cfg4_volume_128x256x256":
        vol = synth.ellipsoid_volume(128, 256, 256, seed=0xC0FFEE + 4)
        return 4, 2, (128, 256, 256), synth.bilateral_positions(vol, 5.0, 0.1)
    if name == "cfg5_512_crf_bilateral":
        img = synth.blob_image(512, 512, seed=0xC0FFEE + 5) * 255.0
        return 5, 22, (512, 512), synth.bilateral_positions(img, 80.0, 13.0)
    if name == "cfg5_512_crf_spatial":
        return 2, 22, (512, 512), synth.spatial_positions((512, 512), 3.0)
    raise KeyError(name)


CONFIGS = ["cfg1_512_rgb", "north_star_1024_rgb", "cfg2_1024_spatial", "cfg3_1024_guided",
           "cfg4_volume_128x256x256", "cfg5_512_crf_bilateral", "cfg5_512_crf_spatial"]


def _dot(a, b):
    return float((a.double() * b.double()).sum())


@pytest.mark.parametrize("name", CONFIGS)
def test_full_size_properties(name):
    pd, vd, shape, pos = _positions(name)
    n = pos.shape[0]
    gen = torch.Generator(device="cuda").manual_seed(1234)
    d_pos = torch.from_numpy(pos).cuda()
    lat = pla.PermutohedralLattice(pd, vd, n)
    lat.set_point_grid(shape)

    # --- integers -------------------------------------------------------------------------
    d = lat.debug_simplex(d_pos)
    rem0, rank, keys, bary = d["rem0"].int(), d["rank"].int(), d["keys"], d["barycentric"]
    assert int((rem0 % (pd + 1)).abs().max()) == 0
    assert int(rem0.sum(dim=1).abs().max()) == 0
    assert int((rank.sum(dim=1) - pd * (pd + 1) // 2).abs().max()) == 0
    assert int(((rank * rank).sum(dim=1) - pd * (pd + 1) * (2 * pd + 1) // 6).abs().max()) == 0
    assert float(bary.min()) >= -1e-6
    assert float((bary.double().sum(dim=1) - 1.0).abs().max()) <= 1e-5
    distinct = torch.unique(keys.reshape(-1, pd), dim=0).shape[0]
    del d, rem0, rank, keys, bary

    # --- constant in, constant out; build + apply == filter -------------------------------
    const = torch.full((n, vd - 1), 0.625, dtype=torch.float32, device="cuda")
    out = torch.empty_like(const)
    lat.filter(out, const, d_pos, False)
    torch.cuda.synchronize()
    assert lat.num_vertices == distinct
    assert float((out - 0.625).abs().max()) <= 1e-5
    x = torch.rand((n, vd - 1), generator=gen, device="cuda")
    lat.filter(out, x, d_pos, True)
    out2 = torch.empty_like(out)
    lat.build(d_pos)
    lat.apply(out2, x, True)
    torch.cuda.synchronize()
    assert float((out - out2).abs().max()) <= 1e-5
    assert float(out.min()) >= -1e-6 and float(out.max()) <= 1.0 + 1e-5   # a weighted mean of [0,1]

    # --- the bare operator: linear, and reverse is the adjoint of forward -------------------
    lat.set_option(pla.PL_OPT_NORMALIZE, 0)
    lat.build(d_pos)
    xa = torch.randn((n, vd), generator=gen, device="cuda")
    xb = torch.randn((n, vd), generator=gen, device="cuda")
    ya, yb, yc = (torch.empty_like(xa) for _ in range(3))
    lat.apply(ya, xa, False)
    lat.apply(yb, xb, False)
    lat.apply(yc, 2.0 * xa - 3.0 * xb, False)
    torch.cuda.synchronize()
    lin = 2.0 * ya - 3.0 * yb
    assert float((yc - lin).double().norm() / lin.double().norm()) <= 1e-5
    rev_b = torch.empty_like(xb)
    lat.apply(rev_b, xb, True)
    torch.cuda.synchronize()
    lhs, rhs = _dot(ya, xb), _dot(xa, rev_b)
    assert abs(lhs - rhs) <= 1e-5 * max(abs(lhs), abs(rhs))
    if pd >= 2:
        # the control: forward order on both sides is a different number
        wrong = _dot(xa, yb)
        assert abs(lhs - wrong) > 1e-4 * abs(lhs)


def test_full_size_properties_in_double():
    """The headline configuration on a lattice of doubles: the same size-independent properties,
    at double precision."""
    pd, vd, shape, pos = _positions("north_star_1024_rgb")
    n = pos.shape[0]
    gen = torch.Generator(device="cuda").manual_seed(4321)
    d_pos = torch.from_numpy(pos).cuda().double()
    lat = pla.PermutohedralLattice(pd, vd, n, dtype=torch.float64)
    lat.set_point_grid(shape)
    d = lat.debug_simplex(d_pos)
    rem0, rank, keys, bary = d["rem0"].int(), d["rank"].int(), d["keys"], d["barycentric"]
    assert int((rem0 % (pd + 1)).abs().max()) == 0
    assert int(rem0.sum(dim=1).abs().max()) == 0
    assert int((rank.sum(dim=1) - pd * (pd + 1) // 2).abs().max()) == 0
    assert float(bary.min()) >= -1e-14
    assert float((bary.sum(dim=1) - 1.0).abs().max()) <= 1e-14
    distinct = torch.unique(keys.reshape(-1, pd), dim=0).shape[0]
    del d, rem0, rank, keys, bary

    const = torch.full((n, vd - 1), 0.625, dtype=torch.float64, device="cuda")
    out = torch.empty_like(const)
    lat.filter(out, const, d_pos, False)
    torch.cuda.synchronize()
    assert lat.num_vertices == distinct
    assert float((out - 0.625).abs().max()) <= 1e-13

    lat.set_option(pla.PL_OPT_NORMALIZE, 0)
    lat.build(d_pos)
    xa = torch.randn((n, vd), generator=gen, device="cuda", dtype=torch.float64)
    xb = torch.randn((n, vd), generator=gen, device="cuda", dtype=torch.float64)
    ya, rev_b, yb = (torch.empty_like(xa) for _ in range(3))
    lat.apply(ya, xa, False)
    lat.apply(rev_b, xb, True)
    lat.apply(yb, xb, False)
    torch.cuda.synchronize()
    lhs, rhs, wrong = _dot(ya, xb), _dot(xa, rev_b), _dot(xa, yb)
    assert abs(lhs - rhs) <= 1e-11 * max(abs(lhs), abs(rhs))      # reverse is the adjoint of forward
    assert abs(lhs - wrong) > 1e-4 * abs(lhs)                     # and forward is not
