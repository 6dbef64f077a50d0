"""Parity of the HIP library (through its C ABI) with the CPU oracle and the golden fixtures.

Integers (rem0, rank, per-point keys, vertex count, key set) must be bit-equal; filter outputs
within max|d| <= 1e-3 (data in [0,1]) and relative L2 <= 1e-4 -- the tolerances are in conftest.
"""
import numpy as np
import pytest
import torch

from conftest import (MAX_ABS_TOL, REL_L2_TOL, bits, golden_lattice_cases, load_golden, rel_l2,
                      sorted_keys)
from permutohedral_lattice_amd import synth

import oracle
import permutohedral_lattice_amd as pla

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def gpu_filter(pd, vd, positions, values, reverse=False, lattice=None):
    n = positions.shape[0]
    lat = lattice or pla.PermutohedralLattice(pd, vd, n)
    out = torch.empty((n, vd - 1), dtype=torch.float32, device="cuda")
    lat.filter(out, dev(values), dev(positions), reverse)
    torch.cuda.synchronize()
    return host(out), lat


def assert_float_parity(got, want, scale=1.0):
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= MAX_ABS_TOL * scale
    assert rel_l2(got, want) <= REL_L2_TOL


def check_integers(pd, positions, lat=None):
    n = positions.shape[0]
    lat = lat or pla.PermutohedralLattice(pd, 2, n)
    d = {k: host(v) for k, v in lat.debug_simplex(dev(positions)).items()}
    o = oracle.dump_simplex(positions)
    assert (d["rem0"] == o["rem0"]).all()
    assert (d["rank"] == o["rank"]).all()
    assert (d["keys"] == o["keys"]).all()
    # the weights follow the same operations in the same order: bit-equal as well
    assert (bits(d["barycentric"]) == bits(o["barycentric"])).all()
    return o


# ---------------------------------------------------------------------------------------------
# golden fixtures (outputs of the reference's own CPU header)
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("name", golden_lattice_cases())
def test_golden_integers(name):
    g = load_golden("lattice_" + name)
    pd = int(g["pd"])
    n = g["positions"].shape[0]
    lat = pla.PermutohedralLattice(pd, int(g["vd"]), n)
    d = {k: host(v) for k, v in lat.debug_simplex(dev(g["positions"])).items()}
    assert (d["rem0"] == g["rem0"]).all()
    assert (d["rank"] == g["rank"]).all()
    assert (d["keys"] == g["keys"]).all()
    if g["barycentric"].size:
        assert (bits(d["barycentric"]) == bits(g["barycentric"])).all()


@pytest.mark.parametrize("name", golden_lattice_cases())
def test_golden_filter(name):
    g = load_golden("lattice_" + name)
    pd, vd = int(g["pd"]), int(g["vd"])
    out_f, lat = gpu_filter(pd, vd, g["positions"], g["values"], False)
    # vertex count and key set: one vertex per distinct key (the reference's list may repeat a
    # key once per doubling of its index; the fixture keeps that list as the reference made it)
    distinct = np.unique(g["vertex_keys"], axis=0)
    assert lat.num_vertices == len(distinct)
    assert (sorted_keys(host(lat.debug_keys()))[0] == sorted_keys(distinct)[0]).all()
    assert_float_parity(out_f, g["output_forward"])
    out_r, _ = gpu_filter(pd, vd, g["positions"], g["values"], True, lattice=lat)
    assert_float_parity(out_r, g["output_reverse"])


# ---------------------------------------------------------------------------------------------
# the benchmark configurations at sizes the oracle finishes in seconds
# ---------------------------------------------------------------------------------------------

def _config_case(name):
    if name == "cfg1_bilateral_rgb":
        img = synth.blob_image(256, 256, seed=1)
        return 5, 4, synth.bilateral_positions(img, 8.0, 0.125), img.reshape(-1, 3)
    if name == "cfg2_spatial":
        return 2, 2, synth.spatial_positions((512, 512), 8.0), synth.uniform_image((512 * 512, 1), 2)
    if name == "cfg3_guided_grey":
        guide = synth.blob_image(256, 256, seed=3)
        return 5, 2, synth.bilateral_positions(guide, 8.0, 0.125), synth.uniform_image((256 * 256, 1), 4)
    if name == "cfg4_volume":
        vol = synth.ellipsoid_volume(32, 64, 64, seed=5)
        return 4, 2, synth.bilateral_positions(vol, 5.0, 0.1), vol.reshape(-1, 1)
    if name == "cfg5_crf_bilateral":
        guide = synth.blob_image(128, 128, seed=6) * 255.0
        return 5, 22, synth.bilateral_positions(guide, 80.0, 13.0), synth.softmax_logits((128 * 128, 21), 7)
    if name == "cfg5_crf_spatial":
        return 2, 22, synth.spatial_positions((128, 128), 3.0), synth.softmax_logits((128 * 128, 21), 7)
    if name == "odd_size_pd3_vd5":
        rng = np.random.default_rng(8)
        return 3, 5, rng.uniform(0, 9, (1000 * 3 + 37, 3)).astype(np.float32), \
            rng.uniform(0, 1, (3037, 4)).astype(np.float32)
    if name == "wide_pd6_vd9":
        rng = np.random.default_rng(9)
        return 6, 9, rng.uniform(0, 3, (5000, 6)).astype(np.float32), \
            rng.uniform(0, 1, (5000, 8)).astype(np.float32)
    raise KeyError(name)


CONFIG_CASES = ["cfg1_bilateral_rgb", "cfg2_spatial", "cfg3_guided_grey", "cfg4_volume",
                "cfg5_crf_bilateral", "cfg5_crf_spatial", "odd_size_pd3_vd5", "wide_pd6_vd9"]


@pytest.mark.parametrize("name", CONFIG_CASES)
def test_config_parity_with_oracle(name):
    pd, vd, pos, val = _config_case(name)
    n = pos.shape[0]
    lat = pla.PermutohedralLattice(pd, vd, n)
    o = check_integers(pd, pos, lat)
    cpu = oracle.Lattice(pd, vd, n)
    want_f = cpu.filter(val, pos, False)
    got_f, _ = gpu_filter(pd, vd, pos, val, False, lattice=lat)
    assert lat.num_vertices == cpu.num_vertices == len(np.unique(o["keys"].reshape(-1, pd), axis=0))
    assert (sorted_keys(host(lat.debug_keys()))[0] == sorted_keys(cpu.keys())[0]).all()
    assert_float_parity(got_f, want_f)
    want_r = oracle.Lattice(pd, vd, n).filter(val, pos, True)
    got_r, _ = gpu_filter(pd, vd, pos, val, True, lattice=lat)
    assert_float_parity(got_r, want_r)
    assert np.abs(want_f - want_r).max() > 0  # the two orders are different computations


def test_replay_matrix_matches_oracle():
    """Vertex numbering differs (first touch on the CPU, arbitrary on the GPU), so replay rows are
    compared through the vertex keys they point at."""
    pd, vd, pos, val = _config_case("cfg1_bilateral_rgb")
    n = pos.shape[0]
    got, lat = gpu_filter(pd, vd, pos, val)
    vertex, weight = (host(t) for t in lat.debug_replay())
    keys = host(lat.debug_keys())
    o = oracle.dump_simplex(pos)
    assert vertex.min() >= 0 and vertex.max() < lat.num_vertices
    assert (keys[vertex.T] == o["keys"]).all()          # [N, pd+1, pd]
    assert (bits(weight.T) == bits(o["barycentric"])).all()


def test_gradient_pass_on_normal_upstream_gradient():
    """cfg3: the backward pass filters an N(0,1) upstream gradient with reverse=True."""
    guide = synth.blob_image(192, 192, seed=11)
    pos = synth.bilateral_positions(guide, 8.0, 0.125)
    grad = synth.normal_image((192 * 192, 1), 12)
    want = oracle.Lattice(5, 2, 192 * 192).filter(grad, pos, True)
    got, _ = gpu_filter(5, 2, pos, grad, True)
    assert_float_parity(got, want, scale=float(np.abs(want).max()))


# ---------------------------------------------------------------------------------------------
# lattice reuse, object semantics, edge cases
# ---------------------------------------------------------------------------------------------

def test_build_once_apply_many_equals_filter():
    pd, vd, pos, val = _config_case("cfg3_guided_grey")
    n = pos.shape[0]
    lat = pla.PermutohedralLattice(pd, vd, n)
    lat.build(dev(pos))
    out = torch.empty((n, 1), dtype=torch.float32, device="cuda")
    grad = synth.normal_image((n, 1), 13)
    for values, reverse in ((val, False), (grad, True), (val, True), (val, False)):
        lat.apply(out, dev(values), reverse)
        torch.cuda.synchronize()
        want = oracle.Lattice(pd, vd, n).filter(values, pos, reverse)
        assert_float_parity(host(out), want, scale=max(1.0, float(np.abs(want).max())))


@pytest.mark.parametrize("dims,pd,vd", [((64, 64), 5, 4), ((37, 53), 5, 4), ((5, 300), 2, 2),
                                         ((20, 24, 28), 4, 2), ((3, 9, 17, 21), 4, 3),
                                         ((2, 50, 40), 5, 22), ((1, 1, 700), 3, 2)])
def test_point_grid_hint_changes_nothing_but_the_order_of_work(dims, pd, vd):
    """With the grid hint workgroups take 2-D / 3-D tiles (ragged at the edges here); integers,
    vertex set, replay rows and outputs are those of the plain order and of the oracle."""
    n = int(np.prod(dims))
    rng = np.random.default_rng(sum(dims))
    grids = np.meshgrid(*[np.arange(d, dtype=np.float32) for d in dims], indexing="ij")
    spatial = np.stack([g.reshape(-1) for g in grids[-2:]], axis=1) / 4.0
    extra = rng.uniform(0, 6, (n, pd - 2)).astype(np.float32)
    pos = np.concatenate([spatial, extra], axis=1).astype(np.float32)
    val = rng.uniform(0, 1, (n, vd - 1)).astype(np.float32)
    cpu = oracle.Lattice(pd, vd, n)
    want = cpu.filter(val, pos)
    lat = pla.PermutohedralLattice(pd, vd, n)
    plain, _ = gpu_filter(pd, vd, pos, val, lattice=lat)
    lat.set_point_grid(dims)
    tiled, _ = gpu_filter(pd, vd, pos, val, lattice=lat)
    assert lat.num_vertices == cpu.num_vertices
    assert (sorted_keys(host(lat.debug_keys()))[0] == sorted_keys(cpu.keys())[0]).all()
    vertex, weight = (host(t) for t in lat.debug_replay())
    o = oracle.dump_simplex(pos)
    assert (host(lat.debug_keys())[vertex.T] == o["keys"]).all()
    assert (bits(weight.T) == bits(o["barycentric"])).all()
    assert_float_parity(tiled, want)
    assert_float_parity(plain, want)
    tiled_rev, _ = gpu_filter(pd, vd, pos, val, True, lattice=lat)
    assert_float_parity(tiled_rev, oracle.Lattice(pd, vd, n).filter(val, pos, True))
    lat.set_point_grid(None)
    again, _ = gpu_filter(pd, vd, pos, val, lattice=lat)
    assert_float_parity(again, want)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_points_crowded_into_one_band_of_the_first_feature(dtype):
    """With a grid hint the hash table is divided by bands of feature 0 between the first and the
    last point.  Here those two points are far apart and every other point sits in a narrow range
    between them, so that all vertices fall into one band, more of them than that band's part of
    the table holds: the keys must spill over the whole table, the result must not change, and the
    call must not take longer than a few probe steps per key (a chain through a full part of the
    table would take minutes)."""
    import time
    dims, pd, vd = (256, 256), 3, 2
    n = dims[0] * dims[1]
    rng = np.random.default_rng(77)
    pos = rng.uniform(0, 1, (n, pd)) * np.array([10.0, 60.0, 60.0]) + np.array([245.0, 0.0, 0.0])
    pos[0, 0], pos[-1, 0] = 0.0, 500.0
    pos = pos.astype(dtype)
    val = rng.uniform(0, 1, (n, vd - 1)).astype(dtype)
    torch_dtype = torch.float32 if dtype == np.float32 else torch.float64
    cpu = oracle.Lattice(pd, vd, n, dtype=dtype)
    want = cpu.filter(val, pos)
    lat = pla.PermutohedralLattice(pd, vd, n, dtype=torch_dtype)
    lat.set_point_grid(dims)
    out = torch.empty((n, vd - 1), dtype=torch_dtype, device="cuda")
    d_val, d_pos = dev(val), dev(pos)
    for _ in range(3):          # the table has its final size from the second call on
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        lat.filter(out, d_val, d_pos, False)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        assert elapsed < 2.0
        assert lat.num_vertices == cpu.num_vertices
        if dtype == np.float32:
            assert_float_parity(host(out), want)
        else:
            assert np.abs(host(out) - want).max() <= 1e-12
    assert (sorted_keys(host(lat.debug_keys()))[0] == sorted_keys(cpu.keys())[0]).all()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_merging_build_equals_the_plain_build(dtype):
    """With a grid hint the build merges each tile's keys and sums in LDS before they go to the
    hash table (PL_OPT_MERGE_TILES); without the option every wavefront goes to the table itself.
    Same vertices, same replay rows, same outputs to rounding, for a smooth image (tiles share
    most vertices) and for one with noise in every feature (a tile then has more distinct keys
    than its LDS table holds, and the lattice must fall back by itself, for this and later calls;
    after 32 builds it tries merging again, which must again give the right answer)."""
    h, w, pd, vd = 96, 112, 5, 4
    n = h * w
    torch_dtype = torch.float32 if dtype == np.float32 else torch.float64
    img = synth.blob_image(h, w, seed=91)
    smooth = synth.bilateral_positions(img, 8.0, 0.125)
    rng = np.random.default_rng(92)
    noisy = np.concatenate([smooth[:, :2], rng.uniform(0, 40, (n, 3)).astype(np.float32)], axis=1)
    val = img.reshape(-1, 3).astype(dtype)
    noisy_pos = noisy.astype(dtype)
    for pos in (smooth.astype(dtype), noisy_pos):
        cpu = oracle.Lattice(pd, vd, n, dtype=dtype)
        want = cpu.filter(val, pos)
        outs = {}
        for merge in (1, 0):
            lat = pla.PermutohedralLattice(pd, vd, n, dtype=torch_dtype)
            lat.set_point_grid((h, w))
            lat.set_option(pla.PL_OPT_MERGE_TILES, merge)
            out = torch.empty((n, vd - 1), dtype=torch_dtype, device="cuda")
            for _ in range(36 if pos is noisy_pos and merge else 2):   # later calls run on what the first learnt
                lat.filter(out, dev(val), dev(pos), False)
                torch.cuda.synchronize()
                assert lat.num_vertices == cpu.num_vertices
            assert (sorted_keys(host(lat.debug_keys()))[0] == sorted_keys(cpu.keys())[0]).all()
            outs[merge] = host(out).copy()
            if dtype == np.float32:
                assert_float_parity(outs[merge], want)
            else:
                assert np.abs(outs[merge] - want).max() <= 1e-12
        assert np.abs(outs[1] - outs[0]).max() <= (2e-6 if dtype == np.float32 else 1e-13)


def test_point_grid_must_match_the_number_of_points():
    lat = pla.PermutohedralLattice(2, 2, 100)
    with pytest.raises(pla.PermutohedralError) as e:
        lat.set_point_grid((10, 11))
    assert e.value.status == pla.PL_EINVAL


def test_handle_is_reusable_and_each_filter_is_fresh():
    """The reference object is single-shot; here every filter() behaves as on a new lattice, also
    when the positions change between calls."""
    rng = np.random.default_rng(14)
    n = 5000
    lat = pla.PermutohedralLattice(3, 3, n)
    for trial in range(3):
        pos = rng.uniform(0, 5 + 10 * trial, (n, 3)).astype(np.float32)
        val = rng.uniform(0, 1, (n, 2)).astype(np.float32)
        got, _ = gpu_filter(3, 3, pos, val, lattice=lat)
        cpu = oracle.Lattice(3, 3, n)
        want = cpu.filter(val, pos)
        assert lat.num_vertices == cpu.num_vertices
        assert_float_parity(got, want)


@pytest.mark.parametrize("pd,vd", [(5, 4), (4, 2), (2, 2), (3, 7), (5, 22)])
def test_two_axes_per_launch_is_bit_identical_to_one(pd, vd):
    """Blurring two axes in one kernel must give exactly the values of two separate passes."""
    rng = np.random.default_rng(pd * 100 + vd)
    n = 20000
    pos = rng.uniform(0, 12, (n, pd)).astype(np.float32) * np.linspace(1.0, 0.3, pd, dtype=np.float32)
    val = rng.uniform(0, 1, (n, vd - 1)).astype(np.float32)
    lat = pla.PermutohedralLattice(pd, vd, n)
    lat.build(dev(pos))
    out = torch.empty((n, vd - 1), dtype=torch.float32, device="cuda")
    results = {}
    for pair in (1, 0):
        lat.set_option(pla.PL_OPT_PAIR_BLUR, pair)
        for reverse in (False, True):
            lat.apply(out, dev(val), reverse)
            torch.cuda.synchronize()
            results[(pair, reverse)] = host(out).copy()
    # splat sums differ in the last bits between runs (atomics), the blur itself must not add to that
    for reverse in (False, True):
        assert np.abs(results[(1, reverse)] - results[(0, reverse)]).max() <= 2e-6
        assert_float_parity(results[(1, reverse)], oracle.Lattice(pd, vd, n).filter(val, pos, reverse))


@pytest.mark.parametrize("pd,vd,shape", [(2, 6, (96, 70)), (3, 13, (40, 30, 20)), (2, 17, (70, 90)),
                                         (5, 33, (64, 48)), (2, 40, (50, 60)), (3, 70, (3000,)),
                                         (8, 5, (2500,))])
def test_many_channels(pd, vd, shape):
    """The kernels for more than four channels: 16, 32 and 64 lanes per member in the splat,
    input rows beyond 64 channels, odd and even row lengths in the slice; filter and apply, with
    and without a grid hint, normalised and as the bare linear operator."""
    n = int(np.prod(shape))
    rng = np.random.default_rng(pd * 1000 + vd)
    # smooth positions over the grid plus noise, so that wavefronts see groups of several sizes
    grid = np.stack(np.meshgrid(*[np.arange(s, dtype=np.float32) for s in shape], indexing="ij"), -1)
    pos = np.concatenate([grid.reshape(n, -1) / (np.asarray(shape, np.float32) / 12.0),
                          rng.uniform(0, 2.5, (n, pd)).astype(np.float32)], axis=1)[:, :pd]
    pos = np.ascontiguousarray(pos, np.float32)
    val = rng.uniform(0, 1, (n, vd - 1)).astype(np.float32)
    want = {rev: oracle.Lattice(pd, vd, n).filter(val, pos, rev) for rev in (False, True)}
    for hint in (None, shape if len(shape) > 1 else None):
        lat = pla.PermutohedralLattice(pd, vd, n)
        if hint:
            lat.set_point_grid(hint)
        got, _ = gpu_filter(pd, vd, pos, val, False, lattice=lat)
        assert_float_parity(got, want[False])
        out = torch.empty((n, vd - 1), dtype=torch.float32, device="cuda")
        lat.apply(out, dev(val), True)
        torch.cuda.synchronize()
        assert_float_parity(host(out), want[True])
    # bare operator: vd channels in and out, nothing divided; equals the oracle's raw filter
    lat = pla.PermutohedralLattice(pd, vd, n)
    lat.set_option(pla.PL_OPT_NORMALIZE, 0)
    raw_in = rng.uniform(0, 1, (n, vd)).astype(np.float32)
    out = torch.empty((n, vd), dtype=torch.float32, device="cuda")
    lat.filter(out, dev(raw_in), dev(pos), False)
    torch.cuda.synchronize()
    want_raw = oracle.Lattice(pd, vd, n).filter_raw(raw_in, pos, False)
    assert np.abs(host(out) - want_raw).max() <= MAX_ABS_TOL * max(1.0, float(np.abs(want_raw).max()))
    assert rel_l2(host(out), want_raw) <= REL_L2_TOL


def test_apply_before_build_is_an_error():
    lat = pla.PermutohedralLattice(2, 2, 16)
    x = torch.zeros((16, 1), device="cuda")
    with pytest.raises(pla.PermutohedralError) as e:
        lat.apply(x, x)
    assert e.value.status == pla.PL_ESTATE


@pytest.mark.parametrize("n", [0, 1, 63, 64, 65, 257])
def test_tiny_and_ragged_sizes(n):
    rng = np.random.default_rng(n)
    pos = rng.uniform(0, 3, (n, 4)).astype(np.float32)
    val = rng.uniform(0, 1, (n, 2)).astype(np.float32)
    got, lat = gpu_filter(4, 3, pos, val)
    if n == 0:
        assert got.shape == (0, 2)
        return
    check_integers(4, pos)
    want = oracle.Lattice(4, 3, n).filter(val, pos)
    assert_float_parity(got, want)


def test_isolated_points_pass_through():
    """Features so far apart that no two points share a vertex and no vertex has a neighbour:
    blur only halves every value, and normalisation restores it: out == in."""
    n = 200
    pos = (np.arange(n, dtype=np.float32)[:, None] * 50.0 + np.array([[0.3, 0.1]], np.float32))
    val = np.random.default_rng(15).uniform(0, 1, (n, 3)).astype(np.float32)
    got, lat = gpu_filter(2, 4, pos, val)
    assert lat.num_vertices == 3 * n
    assert np.abs(got - val).max() <= 1e-5


def test_hash_table_growth_is_transparent():
    """Force a table far too small: the build detects the overflow, regrows and reruns."""
    pd, vd, pos, val = _config_case("cfg1_bilateral_rgb")
    n = pos.shape[0]
    lat = pla.PermutohedralLattice(pd, vd, n)
    lat.set_option(pla.PL_OPT_TABLE_CELLS, 4096)
    got, _ = gpu_filter(pd, vd, pos, val, lattice=lat)
    cpu = oracle.Lattice(pd, vd, n)
    want = cpu.filter(val, pos)
    assert cpu.num_vertices > 4096 // 2
    assert lat.num_vertices == cpu.num_vertices
    assert_float_parity(got, want)


def test_all_points_in_one_simplex_collide_on_every_vertex():
    n = 4096
    pos = np.tile(np.array([[0.31, 0.12, 0.55, 0.2, 0.4]], np.float32), (n, 1))
    val = np.random.default_rng(16).uniform(0, 1, (n, 3)).astype(np.float32)
    got, lat = gpu_filter(5, 4, pos, val)
    assert lat.num_vertices == 6
    want = oracle.Lattice(5, 4, n).filter(val, pos)
    assert_float_parity(got, want)
    assert np.abs(got - val.mean(axis=0)).max() <= 1e-4


def test_coordinates_beyond_the_packed_key_range_are_reported():
    """Lattice coordinates beyond a short, where the reference's own keys wrap, must fail loudly
    (pd=5 packs 12 bits per coordinate and goes to keys of two words first)."""
    n = 256
    pos = np.full((n, 5), 1.0, np.float32)
    pos[7, 0] = 30000.0
    lat = pla.PermutohedralLattice(5, 2, n)
    out = torch.empty((n, 1), dtype=torch.float32, device="cuda")
    with pytest.raises(pla.PermutohedralError) as e:
        lat.filter(out, dev(np.ones((n, 1), np.float32)), dev(pos))
    assert e.value.status == pla.PL_EOVERFLOW
    # pd <= 4 holds the full short range of the reference's keys
    pos4 = np.full((n, 4), 1.0, np.float32)
    pos4[7, 0] = 5000.0
    val = np.random.default_rng(17).uniform(0, 1, (n, 1)).astype(np.float32)
    got, _ = gpu_filter(4, 2, pos4, val)
    check_integers(4, pos4)
    assert_float_parity(got, oracle.Lattice(4, 2, n).filter(val, pos4))


@pytest.mark.parametrize("pd,reach", [(5, 7500.0), (6, 6400.0), (8, 5000.0)])
def test_coordinates_within_the_reference_short_keys_are_filtered(pd, reach):
    """The reference's keys are shorts at every pd (src/PermutohedralLatticeCPU.h:297-304); the
    packed 64-bit key has 12, 10 and 7 bits per coordinate at pd = 5, 6, 8.  Lattice coordinates
    beyond those but within a short are filtered with keys of two words: same vertex count, same
    keys, same outputs as the CPU path; and the handle goes on working for positions near zero."""
    rng = np.random.default_rng(100 + pd)
    n = 3000
    pos = rng.uniform(0.0, 1.0, (n, pd)).astype(np.float32)
    pos[:, 0] = rng.uniform(0.0, reach, n).astype(np.float32)      # far out along one feature
    pos[: n // 2, 1:] = pos[n // 2 : 2 * (n // 2), 1:]              # and vertices that are shared
    pos[: n // 2, 0] = pos[n // 2 : 2 * (n // 2), 0] + rng.uniform(0.0, 0.3, n // 2).astype(np.float32)
    o = oracle.dump_simplex(pos)
    coords = o["keys"].astype(np.int64)
    beyond_packed = (1 << (min(16, 60 // pd) - 1)) * (pd + 1)
    assert np.abs(coords).max() > beyond_packed and np.abs(o["rem0"].astype(np.int64)).max() < 32000
    val = rng.uniform(0, 1, (n, 2)).astype(np.float32)
    cpu = oracle.Lattice(pd, 3, n)
    want = cpu.filter(val, pos)
    got, lat = gpu_filter(pd, 3, pos, val)
    assert lat.num_vertices == cpu.num_vertices
    assert (sorted_keys(host(lat.debug_keys()))[0] == sorted_keys(cpu.keys())[0]).all()
    assert_float_parity(got, want)
    got_r, _ = gpu_filter(pd, 3, pos, val, reverse=True, lattice=lat)
    assert_float_parity(got_r, oracle.Lattice(pd, 3, n).filter(val, pos, reverse=True))
    near = rng.uniform(0.0, 4.0, (n, pd)).astype(np.float32)
    got_n, _ = gpu_filter(pd, 3, near, val, lattice=lat)
    cpu_n = oracle.Lattice(pd, 3, n)
    assert_float_parity(got_n, cpu_n.filter(val, near))
    assert lat.num_vertices == cpu_n.num_vertices


def test_handle_filters_correctly_after_a_refused_call_that_also_overflowed_its_table():
    """A call refused for a coordinate out of range, whose build had overflowed a small table as
    well, must not leave sums behind that the next call on the handle adds its own to."""
    rng = np.random.default_rng(41)
    n = 64 * 64
    img = rng.uniform(0, 1, (64, 64, 3)).astype(np.float32)      # noise: many vertices
    pos = synth.bilateral_positions(img, 2.0, 0.05)
    bad = pos.copy()
    bad[n // 2, 0] = 3.0e6                                        # beyond the reference's short keys
    val = rng.uniform(0, 1, (n, 3)).astype(np.float32)
    lat = pla.PermutohedralLattice(5, 4, n)
    lat.set_point_grid((64, 64))
    lat.set_option(pla.PL_OPT_TABLE_CELLS, 4096)
    out = torch.empty((n, 3), dtype=torch.float32, device="cuda")
    with pytest.raises(pla.PermutohedralError) as e:
        lat.filter(out, dev(val), dev(bad))
    assert e.value.status == pla.PL_EOVERFLOW
    cpu = oracle.Lattice(5, 4, n)
    want = cpu.filter(val, pos)
    for _ in range(2):
        got, _ = gpu_filter(5, 4, pos, val, lattice=lat)
        assert lat.num_vertices == cpu.num_vertices
        assert_float_parity(got, want)


def test_large_lattice_coordinates_pd5_within_range():
    rng = np.random.default_rng(18)
    n = 20000
    pos = rng.uniform(0, 1, (n, 5)).astype(np.float32) * np.array([[1900, 1400, 8, 8, 8]], np.float32)
    val = rng.uniform(0, 1, (n, 3)).astype(np.float32)
    o = check_integers(5, pos)
    assert np.abs(o["keys"]).max() > 4000
    got, lat = gpu_filter(5, 4, pos, val)
    cpu = oracle.Lattice(5, 4, n)
    want = cpu.filter(val, pos)
    assert lat.num_vertices == cpu.num_vertices
    assert_float_parity(got, want)


# ---------------------------------------------------------------------------------------------
# feature builder and the op
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("name", ["2d_rgb", "3d_grey", "2d_spatial", "2d_crf"])
def test_compute_positions_bit_exact(name):
    g = load_golden("positions")
    sdims, rc = [int(s) for s in g[name + "_sdims"]], int(g[name + "_rc"])
    s_std, f_std = [float(x) for x in g[name + "_stds"]]
    ref = dev(g[name + "_reference"]) if rc else None
    pos = host(pla.compute_positions(ref, sdims, s_std, f_std))
    assert (bits(pos) == bits(g[name + "_positions"])).all()


def test_compute_positions_bit_exact_at_size_with_awkward_stds():
    sdims, rc = (96, 80, 70), 2
    n = int(np.prod(sdims))
    ref = synth.uniform_image((n, rc), 19)
    for s_std, f_std in ((5.0, 0.1), (3.0, 13.0), (7.3, 0.017)):
        want = oracle.compute_positions(ref, sdims, s_std, f_std, rc)
        got = host(pla.compute_positions(dev(ref), sdims, s_std, f_std))
        assert (bits(got) == bits(want)).all()


def test_op_bilateral_batch_and_gradient():
    b, h, w = 2, 96, 80
    guide = np.stack([synth.blob_image(h, w, seed=20 + i) for i in range(b)])
    inp = synth.uniform_image((b, h, w, 2), 22)
    want = oracle.lattice_filter(inp, guide, True, 8.0, 0.125, 1.0, False)
    x = dev(inp).requires_grad_(True)
    y = pla.lattice_filter(x, dev(guide), bilateral=True, theta_alpha=8.0, theta_beta=0.125)
    assert y.shape == x.shape
    assert_float_parity(host(y), want)
    up = synth.normal_image(inp.shape, 23)
    y.backward(dev(up))
    want_grad = oracle.lattice_filter(up, guide, True, 8.0, 0.125, 1.0, True)
    assert_float_parity(host(x.grad), want_grad, scale=float(np.abs(want_grad).max()))


def test_op_spatial_only_uses_theta_gamma_and_ignores_the_reference():
    inp = synth.uniform_image((1, 64, 48, 3), 24)
    want = oracle.lattice_filter(inp, None, False, 77.0, 77.0, 3.0, False)
    got = pla.lattice_filter(dev(inp), dev(synth.uniform_image((1, 64, 48, 5), 25)), bilateral=False,
                             theta_alpha=77.0, theta_beta=77.0, theta_gamma=3.0)
    assert_float_parity(host(got), want)
    got2 = pla.lattice_filter(dev(inp), None, bilateral=False, theta_gamma=3.0)
    assert_float_parity(host(got2), want)


def test_op_3d_volume():
    vol = synth.ellipsoid_volume(24, 40, 32, seed=26)[None]
    want = oracle.lattice_filter(vol, vol, True, 5.0, 0.1, 1.0, False)
    got = pla.lattice_filter(dev(vol), dev(vol), theta_alpha=5.0, theta_beta=0.1)
    assert_float_parity(host(got), want, scale=max(1.0, float(np.abs(want).max())))


@pytest.mark.parametrize("sdims,rc,vd,stds", [((96, 80), 3, 4, (8.0, 0.125)),
                                               ((37, 53), 3, 4, (7.3, 0.017)),
                                               ((20, 24, 28), 1, 2, (5.0, 0.1)),
                                               ((64, 48), 0, 3, (3.0, 1.0)),
                                               ((300,), 2, 3, (3.0, 13.0)),
                                               ((6, 5, 4, 7), 1, 2, (1.5, 0.3))])
def test_features_built_on_the_fly_give_the_lattice_of_the_positions_array(sdims, rc, vd, stds):
    """pl_filter_image / pl_build_image against compute_positions + filter: same vertex count and
    key set as the oracle gets from the oracle's positions (so every division rounded alike),
    outputs within tolerance, forward and reverse."""
    n, pd = int(np.prod(sdims)), len(sdims) + rc
    ref = synth.uniform_image((n, rc), 41) if rc else None
    val = synth.uniform_image((n, vd - 1), 42)
    pos = oracle.compute_positions(ref, sdims, stds[0], stds[1], rc)
    d_ref = dev(ref) if rc else None
    lat = pla.PermutohedralLattice(pd, vd, n)
    out = torch.empty((n, vd - 1), dtype=torch.float32, device="cuda")
    for reverse in (False, True):
        cpu = oracle.Lattice(pd, vd, n)
        want = cpu.filter(val, pos, reverse)
        lat.filter_image(out, dev(val), d_ref, sdims, stds[0], stds[1], reverse)
        torch.cuda.synchronize()
        assert lat.num_vertices == cpu.num_vertices
        assert (sorted_keys(host(lat.debug_keys()))[0] == sorted_keys(cpu.keys())[0]).all()
        assert_float_parity(host(out), want)
    # build once from the image, apply many
    lat2 = pla.PermutohedralLattice(pd, vd, n)
    lat2.build_image(d_ref, sdims, stds[0], stds[1])
    assert lat2.num_vertices == lat.num_vertices
    out2 = torch.empty_like(out)
    lat2.apply(out2, dev(val), True)
    torch.cuda.synchronize()
    assert_float_parity(host(out2), host(out))


def test_image_entry_points_check_their_shapes():
    lat = pla.PermutohedralLattice(5, 4, 64 * 64)
    x = torch.zeros((64 * 64, 3), device="cuda")
    ref = torch.zeros((64 * 64, 3), device="cuda")
    with pytest.raises(pla.PermutohedralError) as e:       # extents do not multiply to N
        lat.filter_image(torch.empty_like(x), x, ref, (64, 63), 8.0, 0.125)
    assert e.value.status == pla.PL_EINVAL
    lat3 = pla.PermutohedralLattice(4, 4, 64 * 64)          # pd != spatial dims + channels
    status = pla._lib.pl_filter_image(lat3._h, x.data_ptr(), x.data_ptr(), ref.data_ptr(), 3, 2,
                                      (pla.C.c_int * 2)(64, 64), 8.0, 0.125, 0)
    assert status == pla.PL_EINVAL


def test_op_rejects_unsupported_dimensions():
    x = torch.zeros((1, 8, 8, 2), device="cuda")
    ref = torch.zeros((1, 8, 8, 7), device="cuda")   # pd = 9
    with pytest.raises(pla.PermutohedralError) as e:
        pla.lattice_filter(x, ref)
    assert e.value.status == pla.PL_EUNSUPPORTED


# ---------------------------------------------------------------------------------------------
# the reference's image fixtures
# ---------------------------------------------------------------------------------------------

def test_reference_image_fixtures():
    """input.bmp -> bilateral_out_1.bmp (batch of two, as Tests/bilateral_filter.py) and
    gray_original.bmp -> filtered_grey.bmp under the RGB guide (Tests/greyscale_test.py), theta
    8 / 0.125, rounded to 8 bits: no value off by more than one level, almost none off at all."""
    im = load_golden("reference_images")
    rgb = (im["input"] / 255.0).astype(np.float32)
    batch = dev(np.stack([rgb, rgb]))
    out = host(pla.lattice_filter(batch, batch, theta_alpha=8.0, theta_beta=0.125))
    for item in out:
        q = np.round(item.astype(np.float64) * 255).astype(np.int64)
        diff = np.abs(q - im["bilateral_out_1"].astype(np.int64))
        assert diff.max() <= 1
        assert (diff != 0).mean() <= 2e-4
    grey = (im["gray_original"] / 255.0).astype(np.float32)[None, :, :, None]
    out = host(pla.lattice_filter(dev(grey), dev(rgb[None]), theta_alpha=8.0, theta_beta=0.125))
    q = np.round(out[0, :, :, 0].astype(np.float64) * 255).astype(np.int64)
    diff = np.abs(q - im["filtered_grey"].astype(np.int64))
    assert diff.max() <= 1
    assert (diff != 0).mean() <= 1e-3


# ---------------------------------------------------------------------------------------------
# grid found in the positions
# ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("case", ["image", "image_ragged", "volume", "spatial_only", "scattered",
                                  "image_with_repeated_row", "guessing_off"])
def test_grid_is_found_in_positions_of_images_and_volumes(case):
    """A handle that was given no grid recognises positions made by the feature builder (feature
    0 changes exactly every row, feature 1 every point or every line of a volume) and orders its
    work by tiles; anything else stays a plain list.  Results never depend on it."""
    rng = np.random.default_rng(5)
    if case in ("image", "guessing_off"):
        img = synth.blob_image(96, 128, seed=81)
        pd, vd, pos, val, want_grid = 5, 4, synth.bilateral_positions(img, 8.0, 0.125), img.reshape(-1, 3), (96, 128)
    elif case == "image_ragged":
        img = synth.blob_image(71, 103, seed=82)
        pd, vd, pos, val, want_grid = 5, 4, synth.bilateral_positions(img, 5.0, 0.2), img.reshape(-1, 3), (71, 103)
    elif case == "volume":
        vol = synth.ellipsoid_volume(12, 24, 36, seed=83)
        pd, vd, pos, val, want_grid = 4, 2, synth.bilateral_positions(vol, 5.0, 0.1), vol.reshape(-1, 1), (12, 24, 36)
    elif case == "spatial_only":
        pd, vd, pos, want_grid = 2, 3, synth.spatial_positions((80, 64), 3.0), (80, 64)
        val = synth.uniform_image((80 * 64, 2), 84)
    elif case == "scattered":
        pd, vd, want_grid = 3, 3, ()
        pos = rng.uniform(0, 9, (6000, 3)).astype(np.float32)
        val = rng.uniform(0, 1, (6000, 2)).astype(np.float32)
    else:   # two rows share their first feature: not the positions of an image
        img = synth.blob_image(64, 96, seed=85)
        pd, vd, val, want_grid = 5, 4, img.reshape(-1, 3), ()
        pos = synth.bilateral_positions(img, 8.0, 0.125).copy()
        pos.reshape(64, 96, 5)[17, :, 0] = pos.reshape(64, 96, 5)[16, 0, 0]
    n = pos.shape[0]
    lat = pla.PermutohedralLattice(pd, vd, n)
    if case == "guessing_off":
        lat.set_option(pla.PL_OPT_GUESS_GRID, 0)
        want_grid = ()
    assert lat.point_grid == ()
    got, _ = gpu_filter(pd, vd, pos, val, False, lattice=lat)
    assert lat.point_grid == want_grid
    cpu = oracle.Lattice(pd, vd, n)
    want = cpu.filter(val, pos, False)
    assert_float_parity(got, want)
    assert lat.num_vertices == cpu.num_vertices
    got_r, _ = gpu_filter(pd, vd, pos, val, True, lattice=lat)
    assert_float_parity(got_r, oracle.Lattice(pd, vd, n).filter(val, pos, True))
    # an explicit hint replaces what was found, its removal leaves a plain list
    if len(want_grid) == 2:
        lat.set_point_grid(want_grid)
        assert lat.point_grid == want_grid
        lat.set_point_grid(None)
        assert lat.point_grid == ()
        got, _ = gpu_filter(pd, vd, pos, val, False, lattice=lat)
        assert lat.point_grid == ()
        assert_float_parity(got, want)


def test_vertex_count_far_from_the_previous_one():
    """The kernels over the vertices are launched for an estimate taken from the handle's previous
    build; a lattice with twenty times as many vertices (or a twentieth) must come out the same."""
    n = 40000
    rng = np.random.default_rng(91)
    val = rng.uniform(0, 1, (n, 3)).astype(np.float32)
    few = rng.uniform(0, 1.5, (n, 5)).astype(np.float32)       # everything in a handful of simplices
    many = rng.uniform(0, 14, (n, 5)).astype(np.float32)       # nearly every point alone
    lat = pla.PermutohedralLattice(5, 4, n)
    counts = []
    for pos in (few, many, few, many):
        cpu = oracle.Lattice(5, 4, n)
        want = cpu.filter(val, pos, False)
        got, _ = gpu_filter(5, 4, pos, val, False, lattice=lat)
        assert lat.num_vertices == cpu.num_vertices
        counts.append(lat.num_vertices)
        assert_float_parity(got, want)
        out = torch.empty((n, 3), dtype=torch.float32, device="cuda")
        lat.apply(out, dev(val), True)
        torch.cuda.synchronize()
        assert_float_parity(host(out), oracle.Lattice(5, 4, n).filter(val, pos, True))
    assert counts[1] > 20 * counts[0]


@pytest.mark.parametrize("segments", [8, 64])
def test_vertex_numbers_drawn_from_eight_or_sixty_four_counters(segments):
    """A build that numbers its vertices itself, with the numbers of every eighth of the image in
    one run or in eight (what a build of more than 8192 workgroups uses): same lattice, same
    outputs; the exports close the gaps between the runs."""
    side = 384
    img = synth.blob_image(side, side, seed=31)
    pos = synth.bilateral_positions(img, 4.0, 0.08)
    val = np.ascontiguousarray(img.reshape(-1, 3))
    n = side * side
    lat = pla.PermutohedralLattice(5, 4, n)
    lat.set_point_grid((side, side))
    lat.set_option(pla.PL_OPT_NUMBER_SEGMENTS, segments)
    lat.set_option(pla.PL_OPT_TABLE_CELLS, 1 << 21)     # (room for 64 runs of 2048 numbers or more)
    cpu = oracle.Lattice(5, 4, n)
    for reverse in (False, True):
        got, _ = gpu_filter(5, 4, pos, val, reverse, lattice=lat)
        want = oracle.Lattice(5, 4, n).filter(val, pos, reverse) if reverse else cpu.filter(val, pos, False)
        assert lat.num_vertices == cpu.num_vertices
        assert_float_parity(got, want)
    got_keys, _ = sorted_keys(host(lat.debug_keys()))
    want_keys, _ = sorted_keys(cpu.keys())
    assert (got_keys == want_keys).all()
    # replay rows through the keys they point to
    vertex, weight = lat.debug_replay()
    keys = host(lat.debug_keys())
    point_keys = oracle.dump_simplex(pos)["keys"]
    v = host(vertex)
    for r in (0, 3, 5):
        assert (keys[v[r]] == point_keys[:, r, :]).all()
