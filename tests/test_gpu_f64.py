"""T = double: the lattices of pl_create_f64 against the golden vectors the reference's CPU header
gives for T = double and against the CPU oracle compiled for double.

Integers (rem0, rank, keys, vertex count, key set) and the barycentric weights are bit-equal.
Values agree to rounding: the splat adds a vertex's contributions in another order than the
sequential CPU loop, every addition is off by at most half an ulp of a sum of order 1..100, and
blur and slice are the same double expressions as on the CPU.  Tolerance: 1e-12 absolute on data
in [0, 1], seven orders below the float path's 1e-5 differences, so a result computed in float
anywhere on the way fails it.
"""
import ctypes as C

import numpy as np
import pytest
import torch

from conftest import bits, golden_lattice_cases, load_golden, sorted_keys
from permutohedral_lattice_amd import synth

import oracle
import permutohedral_lattice_amd as pla

pytestmark = pytest.mark.gpu

F64_TOL = 1e-12


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def gpu_filter(pd, vd, positions, values, reverse=False, lattice=None):
    n = positions.shape[0]
    lat = lattice or pla.PermutohedralLattice(pd, vd, n, dtype=torch.float64)
    out = torch.empty((n, vd - 1), dtype=torch.float64, device="cuda")
    lat.filter(out, dev(values), dev(positions), reverse)
    torch.cuda.synchronize()
    return host(out), lat


@pytest.mark.parametrize("name", golden_lattice_cases(f64=True))
def test_simplex_is_bit_equal_to_the_reference(name):
    g = load_golden("lattice_" + name)
    pos = g["positions"]
    assert pos.dtype == np.float64
    pd = int(g["pd"])
    lat = pla.PermutohedralLattice(pd, 2, pos.shape[0], dtype=torch.float64)
    d = {k: host(v) for k, v in lat.debug_simplex(dev(pos)).items()}
    assert (d["rem0"] == g["rem0"]).all()
    assert (d["rank"] == g["rank"]).all()
    assert (d["keys"] == g["keys"]).all()
    assert d["barycentric"].dtype == np.float64
    assert (bits(d["barycentric"]) == bits(g["barycentric"])).all()


@pytest.mark.parametrize("name", golden_lattice_cases(f64=True))
def test_filter_matches_the_reference(name):
    g = load_golden("lattice_" + name)
    pd, vd = int(g["pd"]), int(g["vd"])
    distinct = np.unique(g["keys"].reshape(-1, pd), axis=0)
    for reverse, key in ((False, "output_forward"), (True, "output_reverse")):
        out, lat = gpu_filter(pd, vd, g["positions"], g["values"], reverse)
        assert out.dtype == np.float64 and np.isfinite(out).all()
        assert np.abs(out - g[key]).max() <= F64_TOL
        assert lat.num_vertices == len(distinct) == int(g["num_vertices"])
        assert (sorted_keys(host(lat.debug_keys()))[0] == sorted_keys(distinct)[0]).all()
    # the double result is not the float result: the two paths are really different computations
    f32 = load_golden("lattice_" + name[:-len("_f64")])
    assert np.abs(g["output_forward"] - f32["output_forward"]).max() > 1e-9


@pytest.mark.parametrize("name", ["2d_rgb", "3d_grey", "2d_spatial", "2d_crf"])
def test_positions_are_bit_equal_to_the_reference(name):
    g = load_golden("positions")
    sdims, rc = [int(s) for s in g[name + "_sdims"]], int(g[name + "_rc"])
    s_std, f_std = [float(x) for x in g[name + "_stds"]]
    ref = dev(g[name + "_reference"].astype(np.float64).reshape(*sdims, -1)) if rc else None
    pos = pla.compute_positions(ref, sdims, s_std, f_std, dtype=torch.float64)
    assert pos.dtype == torch.float64
    assert (bits(host(pos)) == bits(g[name + "_positions_f64"])).all()


@pytest.mark.parametrize("pd,vd,n,seed", [(5, 4, 30000, 1), (2, 2, 50000, 2), (4, 2, 20000, 3),
                                          (3, 6, 9000, 4), (5, 22, 3000, 5), (8, 3, 4000, 6)])
def test_random_points_match_the_oracle(pd, vd, n, seed):
    rng = np.random.default_rng(seed)
    pos = rng.uniform(0, 30, (n, pd)) * rng.uniform(0.05, 1.0, pd)
    if pd == 8:
        pos *= 0.5           # keep the lattice coordinates inside the 7-bit key fields of pd = 8
    val = rng.uniform(0, 1, (n, vd - 1))
    lat = pla.PermutohedralLattice(pd, vd, n, dtype=torch.float64)
    d = {k: host(v) for k, v in lat.debug_simplex(dev(pos)).items()}
    o = oracle.dump_simplex(pos, dtype=np.float64)
    for k in ("rem0", "rank", "keys"):
        assert (d[k] == o[k]).all()
    assert (bits(d["barycentric"]) == bits(o["barycentric"])).all()
    for reverse in (False, True):
        ora = oracle.Lattice(pd, vd, n, dtype=np.float64)
        want = ora.filter(val, pos, reverse)
        got, _ = gpu_filter(pd, vd, pos, val, reverse, lattice=lat)
        assert lat.num_vertices == ora.num_vertices
        assert np.abs(got - want).max() <= F64_TOL


def test_build_then_apply_equals_filter_and_handles_are_reusable():
    img = synth.blob_image(96, 80, seed=31).astype(np.float64)
    pos = synth.bilateral_positions(img.astype(np.float32), 8.0, 0.125).astype(np.float64)
    n = pos.shape[0]
    val = img.reshape(-1, 3)
    lat = pla.PermutohedralLattice(5, 4, n, dtype=torch.float64)
    lat.set_point_grid((96, 80))
    want = {r: oracle.Lattice(5, 4, n, dtype=np.float64).filter(val, pos, r) for r in (False, True)}
    d_val, d_pos = dev(val), dev(pos)
    out = torch.empty((n, 3), dtype=torch.float64, device="cuda")
    for reverse in (False, True, False):
        lat.filter(out, d_val, d_pos, reverse)
        torch.cuda.synchronize()
        assert np.abs(host(out) - want[reverse]).max() <= F64_TOL
    lat.build(d_pos)
    for reverse in (True, False):
        out.zero_()
        lat.apply(out, d_val, reverse)
        torch.cuda.synchronize()
        assert np.abs(host(out) - want[reverse]).max() <= F64_TOL
    # the unnormalised operator: all vd channels in and out
    lat.set_option(pla.PL_OPT_NORMALIZE, 0)
    rng = np.random.default_rng(32)
    raw = rng.standard_normal((n, 4))
    out4 = torch.empty((n, 4), dtype=torch.float64, device="cuda")
    lat.filter(out4, dev(raw), d_pos, False)
    torch.cuda.synchronize()
    want_raw = oracle.Lattice(5, 4, n, dtype=np.float64).filter_raw(raw, pos, False)
    assert np.abs(host(out4) - want_raw).max() <= 1e-11


@pytest.mark.parametrize("n", [0, 1, 65, 257])
def test_small_and_empty_inputs(n):
    rng = np.random.default_rng(40 + n)
    pos = rng.uniform(0, 5, (n, 3))
    val = rng.uniform(0, 1, (n, 2))
    lat = pla.PermutohedralLattice(3, 3, n, dtype=torch.float64)
    out = torch.empty((n, 2), dtype=torch.float64, device="cuda")
    lat.filter(out, dev(val), dev(pos), False)
    torch.cuda.synchronize()
    if n:
        want = oracle.Lattice(3, 3, n, dtype=np.float64).filter(val, pos, False)
        assert np.abs(host(out) - want).max() <= F64_TOL


def test_op_on_doubles_with_gradient():
    b, h, w = 2, 40, 48
    guide = np.stack([synth.blob_image(h, w, seed=50 + i) for i in range(b)]).astype(np.float64)
    inp = synth.uniform_image((b, h, w, 2), 52).astype(np.float64)
    up = np.random.default_rng(53).standard_normal((b, h, w, 2))
    want = oracle.lattice_filter(inp, guide, True, 8.0, 0.125, 1.0, False)
    want_grad = oracle.lattice_filter(up, guide, True, 8.0, 0.125, 1.0, True)
    assert want.dtype == np.float64
    x = dev(inp).requires_grad_(True)
    y = pla.lattice_filter(x, dev(guide), bilateral=True, theta_alpha=8.0, theta_beta=0.125)
    assert y.dtype == torch.float64
    y.backward(dev(up))
    torch.cuda.synchronize()
    assert np.abs(host(y) - want).max() <= F64_TOL
    assert np.abs(host(x.grad) - want_grad).max() <= 1e-11      # gradients are not in [0, 1]
    # spatial only: theta_gamma, reference ignored
    want_sp = oracle.lattice_filter(inp, guide, False, 1.0, 1.0, 3.0, False)
    y_sp = pla.lattice_filter(dev(inp), dev(guide), bilateral=False, theta_gamma=3.0)
    torch.cuda.synchronize()
    assert np.abs(host(y_sp) - want_sp).max() <= F64_TOL


def test_each_entry_point_refuses_the_other_kind_of_lattice():
    n = 64
    f32 = pla.PermutohedralLattice(2, 2, n)
    f64 = pla.PermutohedralLattice(2, 2, n, dtype=torch.float64)
    buf = torch.zeros(n * 4, dtype=torch.float64, device="cuda")
    p = C.c_void_p(buf.data_ptr())
    lib = pla._lib
    assert lib.pl_filter(f64._h, p, p, p, 0) == pla.PL_EINVAL
    assert lib.pl_build(f64._h, p) == pla.PL_EINVAL
    assert lib.pl_apply(f64._h, p, p, 0) == pla.PL_EINVAL
    assert lib.pl_filter_begin(f64._h, p, p, p, 0) == pla.PL_EINVAL
    assert lib.pl_debug_simplex(f64._h, p, None, None, None, None) == pla.PL_EINVAL
    assert lib.pl_filter_f64(f32._h, p, p, p, 0) == pla.PL_EINVAL
    assert lib.pl_build_f64(f32._h, p) == pla.PL_EINVAL
    assert lib.pl_apply_f64(f32._h, p, p, 0) == pla.PL_EINVAL
    assert lib.pl_debug_simplex_f64(f32._h, p, None, None, None, None) == pla.PL_EINVAL
    with pytest.raises(TypeError):
        f64.filter(buf[:n].float(), buf[:n].float(), buf[:2 * n].float())
    with pytest.raises(TypeError):
        pla.PermutohedralLattice(2, 2, n, dtype=torch.float16)


def test_key_range_overflow_is_reported():
    n = 300
    pos = np.random.default_rng(60).uniform(0, 1, (n, 5))
    pos[17] = 1e7          # lattice coordinates far outside the 12-bit key fields of pd = 5
    lat = pla.PermutohedralLattice(5, 2, n, dtype=torch.float64)
    out = torch.empty((n, 1), dtype=torch.float64, device="cuda")
    with pytest.raises(pla.PermutohedralError) as e:
        lat.filter(out, dev(np.ones((n, 1))), dev(pos), False)
    assert e.value.status == pla.PL_EOVERFLOW
    # and the handle still works
    pos[17] = 0.5
    lat.filter(out, dev(np.ones((n, 1))), dev(pos), False)
    torch.cuda.synchronize()
    assert np.abs(host(out) - 1.0).max() <= F64_TOL


def test_coordinates_within_the_reference_short_keys_are_filtered_in_double():
    """Lattice coordinates beyond the packed key's 12 bits (pd = 5) but within the reference's
    short keys (src/PermutohedralLatticeCPU.h:297-304): keys of two words, same lattice and
    outputs as the CPU path for T = double."""
    rng = np.random.default_rng(205)
    n, pd = 2500, 5
    pos = rng.uniform(0.0, 1.0, (n, pd))
    pos[:, 0] = rng.uniform(0.0, 7500.0, n)
    pos[: n // 2, 1:] = pos[n // 2 : 2 * (n // 2), 1:]
    pos[: n // 2, 0] = pos[n // 2 : 2 * (n // 2), 0] + rng.uniform(0.0, 0.3, n // 2)
    val = rng.uniform(0, 1, (n, 2))
    cpu = oracle.Lattice(pd, 3, n, dtype=np.float64)
    want = cpu.filter(val, pos)
    got, lat = gpu_filter(pd, 3, pos, val)
    assert lat.num_vertices == cpu.num_vertices
    assert (sorted_keys(host(lat.debug_keys()))[0] == sorted_keys(cpu.keys())[0]).all()
    assert np.abs(got - want).max() <= F64_TOL
