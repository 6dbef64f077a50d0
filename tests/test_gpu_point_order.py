"""A plain list of points (no grid given, none to be found in the positions) is worked on in an
order in which neighbours in space are neighbours in the list (PL_OPT_ORDER_POINTS), so that the
workgroups of the build can merge their keys as they do for an image.  The order only orders the
work: integers, vertex set and replay rows are those of the oracle bit for bit, outputs within the
tolerances of conftest, with the option on and off."""
import numpy as np
import pytest
import torch

from conftest import MAX_ABS_TOL, REL_L2_TOL, bits, rel_l2, sorted_keys
from permutohedral_lattice_amd import synth

import oracle
import permutohedral_lattice_amd as pla

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def point_lists():
    """name -> (pd, vd, positions, values): lists with no grid in them"""
    cases = {}
    h, w = 96, 112
    img = synth.blob_image(h, w, seed=5)
    rng = np.random.default_rng(6)
    shuffle = rng.permutation(h * w)
    cases["image_with_its_pixels_shuffled"] = (5, 4, synth.bilateral_positions(img, 8.0, 0.125)[shuffle],
                                               img.reshape(-1, 3)[shuffle])
    n = 30000
    cases["cloud_in_a_box"] = (3, 2, rng.uniform(0, 1, (n, 3)).astype(np.float32) * [25.0, 40.0, 6.0],
                               rng.uniform(0, 1, (n, 1)))
    cases["cloud_in_clumps"] = (4, 3, (rng.normal(0, 1, (n, 4)) + rng.integers(0, 3, (n, 1)) * 30.0),
                                rng.uniform(0, 1, (n, 2)))
    vol = synth.ellipsoid_volume(24, 40, 48, seed=7)
    vpos = synth.bilateral_positions(vol, 5.0, 0.1)
    shuffle3 = rng.permutation(vpos.shape[0])
    cases["volume_as_a_list"] = (4, 2, vpos, vol.reshape(-1, 1))
    cases["volume_with_its_voxels_shuffled"] = (4, 2, vpos[shuffle3], vol.reshape(-1, 1)[shuffle3])
    cases["points_on_a_line"] = (1, 2, rng.uniform(-50, 50, (5000, 1)), rng.uniform(0, 1, (5000, 1)))
    flat = rng.uniform(0, 30, (9000, 2))
    flat[:, 1] = 7.25                      # (no extent along the second feature)
    cases["second_feature_constant"] = (2, 2, flat, rng.uniform(0, 1, (9000, 1)))
    cases["first_feature_constant"] = (2, 2, flat[:, ::-1], rng.uniform(0, 1, (9000, 1)))
    cases["one_place"] = (3, 2, np.full((8192, 3), 1.375), rng.uniform(0, 1, (8192, 1)))
    far = rng.uniform(0, 20, (6000, 2))
    far[17] = [9000.0, -7000.0]            # (one point far away stretches the box: few bins hold all)
    cases["one_point_far_away"] = (2, 3, far, rng.uniform(0, 1, (6000, 2)))
    return {k: (pd, vd, np.ascontiguousarray(p, dtype=np.float32), np.ascontiguousarray(v, dtype=np.float32))
            for k, (pd, vd, p, v) in cases.items()}


LISTS = point_lists()


def check_against_oracle(lat, cpu, pos, out, want):
    assert lat.num_vertices == cpu.num_vertices
    keys = host(lat.debug_keys())
    assert (sorted_keys(keys)[0] == sorted_keys(cpu.keys())[0]).all()
    # every point has its row of vertices and weights: the order is a permutation of the list
    vertex, weight = (host(t) for t in lat.debug_replay())
    o = oracle.dump_simplex(pos)
    assert (keys[vertex.T] == o["keys"]).all()
    assert (bits(weight.T) == bits(o["barycentric"])).all()
    got = host(out)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= MAX_ABS_TOL
    assert rel_l2(got, want) <= REL_L2_TOL


@pytest.mark.parametrize("name", sorted(LISTS))
def test_plain_list_in_the_order_of_space(name):
    pd, vd, pos, val = LISTS[name]
    n = pos.shape[0]
    cpu = oracle.Lattice(pd, vd, n)
    want = cpu.filter(val, pos)
    want_reverse = oracle.Lattice(pd, vd, n).filter(val, pos, True)
    d_pos, d_val = dev(pos), dev(val)
    outs = {}
    for ordered in (1, 0):
        lat = pla.PermutohedralLattice(pd, vd, n)
        lat.set_option(pla.PL_OPT_GUESS_GRID, 0)
        lat.set_option(pla.PL_OPT_ORDER_POINTS, ordered)
        out = torch.empty((n, vd - 1), dtype=torch.float32, device="cuda")
        for _ in range(2):      # (the second call runs on what the first left in the scratch arrays)
            out.fill_(float("nan"))
            lat.filter(out, d_val, d_pos, False)
            torch.cuda.synchronize()
            check_against_oracle(lat, cpu, pos, out, want)
        assert lat.point_grid == ()
        outs[ordered] = host(out).copy()
        lat.filter(out, d_val, d_pos, True)
        torch.cuda.synchronize()
        check_against_oracle(lat, cpu, pos, out, want_reverse)
        lat.close()
    assert np.abs(outs[1] - outs[0]).max() <= 2e-5


def test_ordered_list_merges_its_keys_like_an_image():
    """The point of the order: the build of a shuffled image runs in the merging kernel."""
    pd, vd, pos, val = LISTS["image_with_its_pixels_shuffled"]
    n = pos.shape[0]
    out = torch.empty((n, vd - 1), dtype=torch.float32, device="cuda")
    for ordered in (1, 0):
        lat = pla.PermutohedralLattice(pd, vd, n)
        lat.set_option(pla.PL_OPT_GUESS_GRID, 0)
        lat.set_option(pla.PL_OPT_ORDER_POINTS, ordered)
        lat.filter(out, dev(val), dev(pos), False)
        torch.cuda.synchronize()
        assert lat.info(pla.PL_INFO_BUILD_MERGED) == ordered
        lat.close()


def test_one_handle_many_lists():
    """The ordering pass keeps its bounding box and its counts in the handle and leaves them zero
    for the next call: lists with other extents, one after the other, and a lattice that is built
    once and applied twice."""
    pd, vd, n = 3, 2, 30000
    rng = np.random.default_rng(31)
    lat = pla.PermutohedralLattice(pd, vd, n)
    lat.set_option(pla.PL_OPT_GUESS_GRID, 0)
    out = torch.empty((n, vd - 1), dtype=torch.float32, device="cuda")
    val = rng.uniform(0, 1, (n, 1)).astype(np.float32)
    for extent, shift in ((30.0, 0.0), (3.0, -400.0), (200.0, 55.0), (30.0, 0.0)):
        pos = (rng.uniform(0, 1, (n, pd)) * extent + shift).astype(np.float32)
        cpu = oracle.Lattice(pd, vd, n)
        want = cpu.filter(val, pos)
        lat.filter(out, dev(val), dev(pos), False)
        torch.cuda.synchronize()
        check_against_oracle(lat, cpu, pos, out, want)
    lat.build(dev(pos))
    for reverse in (False, True, False):
        other = rng.uniform(0, 1, (n, 1)).astype(np.float32)
        lat.apply(out, dev(other), reverse)
        torch.cuda.synchronize()
        want = oracle.Lattice(pd, vd, n).filter(other, pos, reverse)
        assert np.abs(host(out) - want).max() <= MAX_ABS_TOL
        assert rel_l2(host(out), want) <= REL_L2_TOL
    lat.close()


def test_list_of_doubles():
    pd, vd, pos, val = LISTS["image_with_its_pixels_shuffled"]
    n = pos.shape[0]
    pos64, val64 = pos.astype(np.float64) * 1.0000001, val.astype(np.float64)
    cpu = oracle.Lattice(pd, vd, n, dtype=np.float64)
    want = cpu.filter(val64, pos64)
    for ordered in (1, 0):
        lat = pla.PermutohedralLattice(pd, vd, n, dtype=torch.float64)
        lat.set_option(pla.PL_OPT_ORDER_POINTS, ordered)
        out = torch.empty((n, vd - 1), dtype=torch.float64, device="cuda")
        for _ in range(2):
            lat.filter(out, dev(val64), dev(pos64), False)
            torch.cuda.synchronize()
            assert lat.num_vertices == cpu.num_vertices
            assert np.abs(host(out) - want).max() <= 1e-12
        assert (sorted_keys(host(lat.debug_keys()))[0] == sorted_keys(cpu.keys())[0]).all()
        assert lat.info(pla.PL_INFO_BUILD_MERGED) == ordered
        # built once and applied (the splat and the slice of doubles read the order as well)
        lat.build(dev(pos64))
        lat.apply(out, dev(val64), True)
        torch.cuda.synchronize()
        want_reverse = oracle.Lattice(pd, vd, n, dtype=np.float64).filter(val64, pos64, True)
        assert np.abs(host(out) - want_reverse).max() <= 1e-12
        lat.close()


def test_list_of_doubles_with_many_channels():
    pd, vd, n = 3, 7, 6000
    rng = np.random.default_rng(77)
    pos = rng.uniform(0, 9, (n, pd))
    val = rng.uniform(0, 1, (n, vd - 1))
    cpu = oracle.Lattice(pd, vd, n, dtype=np.float64)
    want = cpu.filter(val, pos)
    lat = pla.PermutohedralLattice(pd, vd, n, dtype=torch.float64)
    out = torch.empty((n, vd - 1), dtype=torch.float64, device="cuda")
    lat.filter(out, dev(val), dev(pos), False)
    torch.cuda.synchronize()
    assert lat.num_vertices == cpu.num_vertices
    assert lat.info(pla.PL_INFO_BUILD_MERGED) == 1
    assert np.abs(host(out) - want).max() <= 1e-12
    lat.close()


def test_large_lists_against_the_grid():
    """More points than one workgroup scans the bins of (the scan then runs in three launches): a
    volume of 2.6 million voxels as a grid, as a list in its own order and as a shuffled list must
    give the same lattice and, point by point, the same outputs."""
    dims, pd, vd = (128, 160, 128), 4, 2
    n = int(np.prod(dims))
    vol = synth.ellipsoid_volume(*dims, seed=11)
    pos = synth.bilateral_positions(vol, 5.0, 0.1)
    val = vol.reshape(-1, 1).astype(np.float32)
    d_pos, d_val = dev(pos), dev(val)
    out = torch.empty((n, vd - 1), dtype=torch.float32, device="cuda")
    grid = pla.PermutohedralLattice(pd, vd, n)
    grid.set_point_grid(dims)
    grid.filter(out, d_val, d_pos, False)
    torch.cuda.synchronize()
    want, m = out.clone(), grid.num_vertices
    want_keys = sorted_keys(host(grid.debug_keys()))[0]
    grid.close()
    shuffle = torch.randperm(n, device="cuda", generator=torch.Generator("cuda").manual_seed(3))
    for l_pos, l_val, l_want in ((d_pos, d_val, want),
                                 (d_pos[shuffle].contiguous(), d_val[shuffle].contiguous(), want[shuffle])):
        lat = pla.PermutohedralLattice(pd, vd, n)
        lat.set_option(pla.PL_OPT_GUESS_GRID, 0)
        for _ in range(2):
            out.fill_(float("nan"))
            lat.filter(out, l_val, l_pos, False)
            torch.cuda.synchronize()
            assert lat.info(pla.PL_INFO_BUILD_MERGED) == 1
            assert lat.num_vertices == m
            assert float((out - l_want).abs().max()) <= 2e-5
        assert (sorted_keys(host(lat.debug_keys()))[0] == want_keys).all()
        lat.close()


@pytest.mark.parametrize("pd,vd,n", [(1, 2, 4096), (2, 3, 4097), (3, 4, 5000), (4, 2, 4100), (5, 3, 6000),
                                     (6, 2, 4500), (7, 2, 4200), (8, 3, 4300), (5, 9, 5200), (3, 22, 4800)])
def test_lists_just_long_enough_to_be_ordered(pd, vd, n):
    """Every pd, few and many channels, lengths around the 4096 points from which a list is
    ordered (ragged last workgroups, bins with a handful of points)."""
    rng = np.random.default_rng(100 * pd + vd)
    pos = (rng.uniform(0, 1, (n, pd)) * rng.uniform(2, 12, pd)).astype(np.float32)
    val = rng.uniform(0, 1, (n, vd - 1)).astype(np.float32)
    cpu = oracle.Lattice(pd, vd, n)
    want = cpu.filter(val, pos)
    lat = pla.PermutohedralLattice(pd, vd, n)
    lat.set_option(pla.PL_OPT_GUESS_GRID, 0)
    out = torch.empty((n, vd - 1), dtype=torch.float32, device="cuda")
    for _ in range(2):
        lat.filter(out, dev(val), dev(pos), False)
        torch.cuda.synchronize()
        check_against_oracle(lat, cpu, pos, out, want)
    lat.build(dev(pos))
    lat.apply(out, dev(val), True)
    torch.cuda.synchronize()
    want_reverse = oracle.Lattice(pd, vd, n).filter(val, pos, True)
    assert np.abs(host(out) - want_reverse).max() <= MAX_ABS_TOL
    assert rel_l2(host(out), want_reverse) <= REL_L2_TOL
    lat.close()
