"""A seeded sweep over shapes the fixed cases do not name: every pd, a spread of channel counts and
point counts (ragged last workgroups, single points, tiles that do not divide the grid), with and
without a 2-D or 3-D grid hint, both value types, both blur orders.  Each case is checked against
the CPU oracle like the fixed ones: lattice integers and vertex count exactly, outputs within the
float or the double tolerance."""
import numpy as np
import pytest
import torch

from conftest import MAX_ABS_TOL, REL_L2_TOL, bits, rel_l2, sorted_keys

import oracle
import permutohedral_lattice_amd as pla

pytestmark = pytest.mark.gpu

VDS = (2, 3, 4, 5, 8, 13, 22)
# largest |position| that keeps the lattice coordinates inside the packed key for each pd
SPAN = {1: 40.0, 2: 40.0, 3: 40.0, 4: 40.0, 5: 30.0, 6: 12.0, 7: 6.0, 8: 3.0}


def _case(seed):
    rng = np.random.default_rng(1000 + seed)
    pd = 1 + seed % 8
    vd = VDS[int(rng.integers(len(VDS)))]
    grid = None
    kind = seed % 3
    if kind == 1:
        grid = (int(rng.integers(3, 70)), int(rng.integers(3, 90)))
    elif kind == 2:
        grid = (int(rng.integers(2, 9)), int(rng.integers(3, 20)), int(rng.integers(3, 24)))
    n = int(np.prod(grid)) if grid else int(rng.integers(1, 6000))
    f64 = seed % 4 >= 2
    reverse = bool(rng.integers(2))
    if grid:
        # smooth features over the grid, so that neighbouring points share vertices as pixels do
        axes = np.meshgrid(*[np.arange(g) for g in grid], indexing="ij")
        base = np.stack([a.reshape(-1) for a in axes], axis=1).astype(np.float64)
        mix = rng.uniform(-0.4, 0.4, (base.shape[1], pd))
        pos = base @ mix + rng.uniform(-0.3, 0.3, (n, pd))
        pos *= SPAN[pd] / max(1.0, np.abs(pos).max())
    else:
        pos = rng.uniform(-SPAN[pd], SPAN[pd], (n, pd)) * rng.uniform(0.1, 1.0, pd)
    val = rng.uniform(0, 1, (n, vd - 1))
    dtype = np.float64 if f64 else np.float32
    return pd, vd, n, grid, reverse, pos.astype(dtype), val.astype(dtype)


@pytest.mark.parametrize("seed", range(48))
def test_random_case_matches_the_oracle(seed):
    pd, vd, n, grid, reverse, pos, val = _case(seed)
    f64 = pos.dtype == np.float64
    tdtype = torch.float64 if f64 else torch.float32
    lat = pla.PermutohedralLattice(pd, vd, n, dtype=tdtype)
    if grid:
        lat.set_point_grid(grid)
    d_pos, d_val = torch.from_numpy(pos).cuda(), torch.from_numpy(val).cuda()

    d = {k: v.cpu().numpy() for k, v in lat.debug_simplex(d_pos).items()}
    o = oracle.dump_simplex(pos, dtype=pos.dtype)
    for k in ("rem0", "rank", "keys"):
        assert (d[k] == o[k]).all(), k
    assert (bits(d["barycentric"]) == bits(o["barycentric"])).all()

    ora = oracle.Lattice(pd, vd, n, dtype=pos.dtype)
    want = ora.filter(val, pos, reverse)
    out = torch.empty((n, vd - 1), dtype=tdtype, device="cuda")
    lat.filter(out, d_val, d_pos, reverse)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert lat.num_vertices == ora.num_vertices
    assert (sorted_keys(lat.debug_keys().cpu().numpy())[0] == sorted_keys(ora.keys())[0]).all()
    assert np.isfinite(got).all()
    if f64:
        assert np.abs(got - want).max() <= 1e-12
    else:
        assert np.abs(got - want).max() <= MAX_ABS_TOL and rel_l2(got, want) <= REL_L2_TOL
    # the same handle again, the other way round: build + apply
    lat.build(d_pos)
    lat.apply(out, d_val, not reverse)
    torch.cuda.synchronize()
    want2 = oracle.Lattice(pd, vd, n, dtype=pos.dtype).filter(val, pos, not reverse)
    assert np.abs(out.cpu().numpy() - want2).max() <= (1e-12 if f64 else MAX_ABS_TOL)
