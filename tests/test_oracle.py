"""Pins the CPU oracle (oracle/pl_oracle.c) before anything is compared with it:
golden vectors produced by the reference's own CPU header, the image fixtures the reference's
tests hold, and what the mathematics fixes (closed forms, invariants, a dense brute force)."""
import itertools
import math

import numpy as np
import pytest

from conftest import bits, golden_lattice_cases, load_golden, rel_l2, sorted_keys
from permutohedral_lattice_amd import synth

import oracle


# ---------------------------------------------------------------------------------------------
# golden vectors from the reference header
# ---------------------------------------------------------------------------------------------

ALL_GOLDEN = golden_lattice_cases() + golden_lattice_cases(f64=True)


@pytest.mark.parametrize("dtype,suffix,rtol", [(np.float32, "", 3e-7), (np.float64, "_f64", 1e-15)])
def test_scale_factor_golden_and_closed_form(dtype, suffix, rtol):
    g = load_golden("scale_factor")
    for pd in range(1, 9):
        sf = oracle.scale_factor(pd, dtype)
        assert sf.dtype == dtype
        assert (bits(sf) == bits(g["pd%d%s" % (pd, suffix)])).all()
        closed = [(pd + 1) * math.sqrt(2.0 / 3.0) / math.sqrt((i + 1) * (i + 2)) for i in range(pd)]
        assert np.allclose(sf, closed, rtol=rtol, atol=0)


@pytest.mark.parametrize("dtype,suffix", [(np.float32, ""), (np.float64, "_f64")])
@pytest.mark.parametrize("name", ["2d_rgb", "3d_grey", "2d_spatial", "2d_crf"])
def test_compute_positions_golden_and_closed_form(name, dtype, suffix):
    g = load_golden("positions")
    sdims, rc = g[name + "_sdims"], int(g[name + "_rc"])
    s_std, f_std = [float(x) for x in g[name + "_stds"]]
    ref = g[name + "_reference"]
    pos = oracle.compute_positions(ref, sdims, s_std, f_std, rc, dtype=dtype)
    assert pos.dtype == dtype
    assert (bits(pos) == bits(g[name + "_positions" + suffix])).all()
    # closed form: coordinate / std in tensor order (last spatial dimension fastest)
    grids = np.meshgrid(*[np.arange(s, dtype=dtype) for s in sdims], indexing="ij")
    for k, gk in enumerate(grids):
        assert (bits(pos[:, k]) == bits(gk.reshape(-1) / dtype(s_std))).all()
    for c in range(rc):
        assert (bits(pos[:, len(sdims) + c]) == bits(ref[:, c].astype(dtype) / dtype(f_std))).all()


@pytest.mark.parametrize("name", ALL_GOLDEN)
def test_simplex_matches_reference_bit_exact(name):
    g = load_golden("lattice_" + name)
    dtype = g["positions"].dtype
    assert dtype == (np.float64 if name.endswith("_f64") else np.float32)
    d = oracle.dump_simplex(g["positions"], want_elevated=True, dtype=dtype)
    assert d["elevated"].dtype == dtype and d["barycentric"].dtype == dtype
    if g["elevated"].size:
        assert (bits(d["elevated"]) == bits(g["elevated"])).all()
        assert (bits(d["barycentric"]) == bits(g["barycentric"])).all()
    assert (d["rem0"] == g["rem0"]).all()
    assert (d["rank"] == g["rank"]).all()
    assert (d["keys"] == g["keys"]).all()


@pytest.mark.parametrize("name", ALL_GOLDEN)
def test_filter_matches_reference_bit_exact(name):
    """With the reference's index-growth quirk reproduced, every stage is bit-identical."""
    g = load_golden("lattice_" + name)
    pd, vd = int(g["pd"]), int(g["vd"])
    n = g["positions"].shape[0]
    dtype = g["positions"].dtype
    for reverse, blur_key, out_key in ((False, "after_blur_forward", "output_forward"),
                                       (True, "after_blur_reverse", "output_reverse")):
        lat = oracle.Lattice(pd, vd, n, reference_growth_quirk=True, dtype=dtype)
        lat.splat(g["values"], g["positions"])
        assert lat.num_vertices == int(g["num_vertices"])
        assert (lat.keys() == g["vertex_keys"]).all()
        assert (bits(lat.values()) == bits(g["after_splat"])).all()
        lat.blur(reverse)
        assert (bits(lat.values()) == bits(g[blur_key])).all()
        out = lat.slice()
        assert out.dtype == dtype
        assert (bits(out) == bits(g[out_key])).all()
        # and through the one-call entry point
        out2 = oracle.Lattice(pd, vd, n, reference_growth_quirk=True, dtype=dtype).filter(
            g["values"], g["positions"], reverse)
        assert (bits(out2) == bits(g[out_key])).all()


@pytest.mark.parametrize("name", ALL_GOLDEN)
def test_vertex_count_is_number_of_distinct_keys(name):
    """Without the quirk the lattice has exactly one vertex per distinct key; the reference has
    at most one more per doubling of its index, and the outputs barely move."""
    g = load_golden("lattice_" + name)
    pd, vd = int(g["pd"]), int(g["vd"])
    n = g["positions"].shape[0]
    lat = oracle.Lattice(pd, vd, n, dtype=g["positions"].dtype)
    out = lat.filter(g["values"], g["positions"])
    distinct = np.unique(g["keys"].reshape(-1, pd), axis=0)
    assert lat.num_vertices == len(distinct)
    assert (sorted_keys(lat.keys())[0] == sorted_keys(distinct)[0]).all()
    extra = int(g["num_vertices"]) - lat.num_vertices
    assert 0 <= extra <= lat.num_growths
    assert np.abs(out - g["output_forward"]).max() <= 1e-4
    # first-touch order: the reference's key list with its duplicates dropped
    _, first = np.unique(g["vertex_keys"], axis=0, return_index=True)
    assert (lat.keys() == g["vertex_keys"][np.sort(first)]).all()


def test_growth_quirk_case_really_has_a_duplicate():
    g = load_golden("lattice_growth_duplicate_pd5_vd4")
    assert len(np.unique(g["vertex_keys"], axis=0)) == int(g["num_vertices"]) - 1


@pytest.mark.skipif(not oracle.have_reference(), reason="reference build absent (oracle/_ref)")
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("pd,vd,n,seed", [(5, 4, 30000, 1), (2, 2, 50000, 2), (4, 2, 20000, 3),
                                          (3, 6, 9000, 4), (5, 22, 3000, 5)])
def test_against_live_reference_build(pd, vd, n, seed, dtype):
    ref = oracle.reference()
    rng = np.random.default_rng(seed)
    pos = (rng.uniform(0, 30, (n, pd)) * rng.uniform(0.05, 1.0, pd)).astype(dtype)
    val = rng.uniform(0, 1, (n, vd - 1)).astype(dtype)
    d = oracle.dump_simplex(pos, want_elevated=True, dtype=dtype)
    r = ref.dump_simplex(pos, dtype=dtype)
    for k in ("rem0", "rank", "keys"):
        assert (d[k] == r[k]).all()
    for k in ("elevated", "barycentric"):
        assert (bits(d[k]) == bits(r[k])).all()
    for reverse in (False, True):
        lat = oracle.Lattice(pd, vd, n, reference_growth_quirk=True, dtype=dtype)
        out = lat.filter(val, pos, reverse)
        rout, m, keys, _ = ref.filter(pd, vd, val, pos, reverse, dtype=dtype)
        assert lat.num_vertices == m
        assert (lat.keys() == keys).all()
        assert (bits(out) == bits(rout)).all()


# ---------------------------------------------------------------------------------------------
# what the mathematics fixes
# ---------------------------------------------------------------------------------------------

def _elevation_matrix(pd):
    """E of the permutohedral paper: columns are the basis of the hyperplane sum(x)=0."""
    e = np.zeros((pd + 1, pd))
    for i in range(pd):          # column i: ones in rows 0..i, -(i+1) in row i+1
        e[: i + 1, i] = 1.0
        e[i + 1, i] = -(i + 1)
    return e


@pytest.mark.parametrize("pd", [1, 2, 3, 4, 5, 8])
def test_embedding_is_the_rotation_onto_the_hyperplane(pd):
    rng = np.random.default_rng(pd)
    pos = rng.uniform(-50, 50, (500, pd)).astype(np.float32)
    el = oracle.dump_simplex(pos, want_elevated=True)["elevated"].astype(np.float64)
    sf = oracle.scale_factor(pd).astype(np.float64)
    expect = (pos.astype(np.float64) * sf) @ _elevation_matrix(pd).T
    assert np.abs(el - expect).max() <= 1e-4 * max(1.0, np.abs(expect).max()) * 1e-1
    assert np.abs(el.sum(axis=1)).max() <= 1e-3


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("pd", [1, 2, 3, 4, 5, 6, 8])
def test_simplex_invariants(pd, dtype):
    rng = np.random.default_rng(100 + pd)
    pos = rng.uniform(-40, 40, (4000, pd)).astype(dtype)
    # include exact ties: integer positions
    pos[:500] = np.round(pos[:500])
    d = oracle.dump_simplex(pos, want_elevated=True, dtype=dtype)
    d1 = pd + 1
    rem0, rank, el = d["rem0"].astype(np.int64), d["rank"].astype(np.int64), d["elevated"].astype(np.float64)
    assert (rem0 % d1 == 0).all()
    assert (rem0.sum(axis=1) == 0).all()
    assert (np.sort(rank, axis=1) == np.arange(d1)).all()
    # residuals are ordered by rank (rank 0 = largest) and spread less than pd+1
    resid = el - rem0
    by_rank = np.take_along_axis(resid, np.argsort(rank, axis=1), axis=1)
    assert (np.diff(by_rank, axis=1) <= 1e-4).all()
    assert ((by_rank[:, 0] - by_rank[:, -1]) <= d1 + 1e-4).all()
    # weights: non-negative, sum to one, and reconstruct the elevated point from the vertices
    w = d["barycentric"].astype(np.float64)
    assert (w >= -1e-5).all()
    assert np.abs(w.sum(axis=1) - 1.0).max() <= 1e-5
    keys = d["keys"].astype(np.int64)                       # [N, d1 vertices, pd]
    last = -keys.sum(axis=2, keepdims=True)                 # implicit coordinate
    full = np.concatenate([keys, last], axis=2)             # [N, d1, d1]
    for r in range(d1):
        assert ((full[:, r, :] - r) % d1 == 0).all()        # all coords congruent to r
    recon = (w[:, :, None] * full).sum(axis=1)
    assert np.abs(recon - el).max() <= 2e-3


def test_simplex_by_brute_force_nearest_vertices():
    """The enclosing simplex's vertices are lattice points (coords congruent mod pd+1, sum 0)
    and the remainder-0 one is the nearest remainder-0 point to the elevated position."""
    pd, d1 = 2, 3
    rng = np.random.default_rng(7)
    pos = rng.uniform(-3, 3, (300, pd)).astype(np.float32)
    d = oracle.dump_simplex(pos, want_elevated=True)
    cand = [np.array(c) * d1 for c in itertools.product(range(-12, 13), repeat=d1) if sum(c) == 0]
    cand = np.array(cand, np.float64)
    for n in range(pos.shape[0]):
        el = d["elevated"][n].astype(np.float64)
        dist = ((cand - el) ** 2).sum(axis=1)
        best = dist.min()
        mine = ((d["rem0"][n].astype(np.float64) - el) ** 2).sum()
        # the reference's greedy rounding + rank fix-up reaches a remainder-0 vertex of the
        # enclosing simplex; it is within the simplex diameter of the nearest one
        assert mine <= best + 2.0 * d1 * d1 + 1e-6
        # containment: barycentric weights non-negative means el is inside the simplex
        assert (d["barycentric"][n] >= -1e-5).all()


class _DenseLattice:
    """Dense linear-algebra restatement on tiny inputs: W (N x M) from per-point keys/weights,
    one M x M blur matrix per axis built from key arithmetic, out = W B W^T v."""

    def __init__(self, positions):
        self.pd = positions.shape[1]
        d = oracle.dump_simplex(positions, dtype=positions.dtype)
        self.index = {}
        n, d1 = d["rank"].shape
        rows = []
        for i in range(n):
            for r in range(d1):
                k = tuple(int(x) for x in d["keys"][i, r])
                v = self.index.setdefault(k, len(self.index))
                rows.append((i, v, float(d["barycentric"][i, r])))
        m = len(self.index)
        self.W = np.zeros((n, m))
        for i, v, w in rows:
            self.W[i, v] += w
        self.B = []
        pd = self.pd
        for axis in range(pd + 1):
            b = np.zeros((m, m))
            for k, v in self.index.items():
                b[v, v] += 0.5
                for sign in (1, -1):
                    nk = [x + sign for x in k]
                    if axis < pd:
                        nk[axis] = k[axis] - sign * pd
                    u = self.index.get(tuple(nk))
                    if u is not None:
                        b[v, u] += 0.25
            self.B.append(b)

    def apply(self, values_vd, reverse):
        x = self.W.T @ values_vd
        order = range(self.pd, -1, -1) if reverse else range(self.pd + 1)
        for axis in order:
            x = self.B[axis] @ x
        return self.W @ x


@pytest.mark.parametrize("dtype,tol", [(np.float32, 2e-5), (np.float64, 1e-13)])
@pytest.mark.parametrize("pd,vd,n", [(2, 3, 64), (3, 2, 80), (5, 4, 60)])
def test_filter_equals_dense_brute_force(pd, vd, n, dtype, tol):
    """In double the oracle and the dense product agree to rounding: any difference in structure
    (a wrong neighbour, a missing tap, the wrong axis order) would show at 1e-3."""
    rng = np.random.default_rng(pd * 10 + vd)
    pos = rng.uniform(0, 4, (n, pd)).astype(dtype)
    val = rng.uniform(0, 1, (n, vd - 1)).astype(dtype)
    dense = _DenseLattice(pos)
    hom = np.concatenate([val.astype(np.float64), np.ones((n, 1))], axis=1)
    for reverse in (False, True):
        raw = dense.apply(hom, reverse)
        expect = raw[:, :-1] / raw[:, -1:]
        lat = oracle.Lattice(pd, vd, n, dtype=dtype)
        out = lat.filter(val, pos, reverse)
        assert lat.num_vertices == len(dense.index)
        assert np.abs(out - expect).max() <= tol
        raw_out = oracle.Lattice(pd, vd, n, dtype=dtype).filter_raw(hom.astype(dtype), pos, reverse)
        assert np.abs(raw_out - raw).max() <= tol
    # blur matrices are symmetric: the + neighbour of u is v iff the - neighbour of v is u
    for b in dense.B:
        assert np.abs(b - b.T).max() == 0.0


def test_constant_input_gives_constant_output():
    img = synth.blob_image(48, 48, seed=3)
    pos = synth.bilateral_positions(img, 8.0, 0.125)
    val = np.full((48 * 48, 3), 0.37, np.float32)
    out = oracle.Lattice(5, 4, 48 * 48).filter(val, pos)
    assert np.abs(out - 0.37).max() <= 1e-6


def test_channels_are_filtered_independently():
    img = synth.blob_image(40, 40, seed=4)
    pos = synth.bilateral_positions(img, 8.0, 0.125)
    val = img.reshape(-1, 3)
    together = oracle.Lattice(5, 4, 1600).filter(val, pos)
    for c in range(3):
        alone = oracle.Lattice(5, 2, 1600).filter(val[:, c:c + 1].copy(), pos)
        assert np.abs(alone[:, 0] - together[:, c]).max() <= 1e-6


def test_reverse_is_the_adjoint_of_forward():
    """<A_fwd x, y> == <x, A_rev y> for the unnormalised operator; with the forward order on
    both sides the identity fails, so the test tells the two orders apart."""
    img = synth.blob_image(64, 64, seed=5)
    pos = synth.bilateral_positions(img, 8.0, 0.125)
    n, vd = 64 * 64, 3
    rng = np.random.default_rng(6)
    x = rng.standard_normal((n, vd)).astype(np.float32)
    y = rng.standard_normal((n, vd)).astype(np.float32)
    ax = oracle.Lattice(5, vd, n).filter_raw(x, pos, False).astype(np.float64)
    ay_rev = oracle.Lattice(5, vd, n).filter_raw(y, pos, True).astype(np.float64)
    ay_fwd = oracle.Lattice(5, vd, n).filter_raw(y, pos, False).astype(np.float64)
    lhs = (ax * y).sum()
    good = abs(lhs - (x * ay_rev).sum()) / abs(lhs)
    bad = abs(lhs - (x * ay_fwd).sum()) / abs(lhs)
    assert good <= 1e-5
    assert bad >= 1e-3
    # and forward differs from reverse on ordinary data
    val = synth.uniform_image((n, 3), 8)
    f = oracle.Lattice(5, 4, n).filter(val, pos, False)
    r = oracle.Lattice(5, 4, n).filter(val, pos, True)
    assert np.abs(f - r).max() >= 1e-4


def test_spatial_impulse_response_is_gaussian_of_the_requested_std():
    """The lattice filter at features x/sigma approximates a Gaussian of std sigma."""
    size, sigma = 129, 6.0
    pos = synth.spatial_positions((size, size), sigma)
    val = np.zeros((size * size, 1), np.float32)
    c = size // 2
    val[c * size + c] = 1.0
    ones = np.ones((size * size, 1), np.float32)
    # unnormalised response to an impulse, normalised by the response to all-ones
    lat = oracle.Lattice(2, 2, size * size)
    raw = lat.filter_raw(np.concatenate([val, np.zeros_like(val)], axis=1), pos, False)[:, 0]
    resp = raw.reshape(size, size).astype(np.float64)
    assert resp.min() >= -1e-7
    resp /= resp.sum()
    yy, xx = np.meshgrid(np.arange(size) - c, np.arange(size) - c, indexing="ij")
    var_y, var_x = (resp * yy * yy).sum(), (resp * xx * xx).sum()
    assert abs(math.sqrt(var_y) - sigma) / sigma <= 0.15
    assert abs(math.sqrt(var_x) - sigma) / sigma <= 0.15
    del ones


# ---------------------------------------------------------------------------------------------
# the reference's image fixtures, through the op
# ---------------------------------------------------------------------------------------------

@pytest.fixture(scope="module")
def reference_images():
    return load_golden("reference_images")


def test_op_reproduces_bilateral_out_1(reference_images):
    """Tests/bilateral_filter.py of the reference: theta_alpha=8, theta_beta=0.125 on input.bmp,
    rounded to 8 bits.  All but a handful of values agree, none by more than one level."""
    rgb = reference_images["input"].astype(np.float64) / 255.0
    img = rgb.astype(np.float32)[None]
    out = oracle.lattice_filter(img, img, bilateral=True, theta_alpha=8.0, theta_beta=0.125)
    q = np.round(out[0].astype(np.float64) * 255).astype(np.int64)
    diff = np.abs(q - reference_images["bilateral_out_1"].astype(np.int64))
    assert diff.max() <= 1
    assert (diff != 0).mean() <= 1e-4


def test_op_reproduces_filtered_grey(reference_images):
    """Tests/greyscale_test.py of the reference: grey image filtered under the RGB guide."""
    rgb8 = reference_images["input"]
    grey8 = np.array(0.2989 * rgb8[:, :, 0] + 0.5870 * rgb8[:, :, 1] + 0.1140 * rgb8[:, :, 2]).astype(np.uint8)
    assert (grey8 == reference_images["gray_original"]).all()
    grey = (grey8 / 255.0).astype(np.float32)[None, :, :, None]
    guide = (rgb8 / 255.0).astype(np.float32)[None]
    out = oracle.lattice_filter(grey, guide, bilateral=True, theta_alpha=8.0, theta_beta=0.125)
    q = np.round(out[0, :, :, 0].astype(np.float64) * 255).astype(np.int64)
    diff = np.abs(q - reference_images["filtered_grey"].astype(np.int64))
    assert diff.max() <= 1
    assert (diff != 0).mean() <= 5e-4


def test_op_uses_theta_gamma_when_not_bilateral():
    img = synth.uniform_image((1, 32, 32, 2), 9)
    out = oracle.lattice_filter(img, None, bilateral=False, theta_alpha=99.0, theta_beta=99.0,
                                theta_gamma=4.0)
    pos = synth.spatial_positions((32, 32), 4.0)
    direct = oracle.Lattice(2, 3, 1024).filter(img.reshape(-1, 2), pos)
    assert (bits(out.reshape(-1, 2)) == bits(direct)).all()
    assert rel_l2(out, img) > 1e-3


# ---------------------------------------------------------------------------------------------
# three doublings of the reference's index: where its outputs differ from one vertex per key
# ---------------------------------------------------------------------------------------------

def _growth_fixture():
    import hashlib
    from permutohedral_lattice_amd import synth
    g = load_golden("growth_three_doublings_pd5_vd4")
    img = g["image"]
    pos = synth.bilateral_positions(img, float(g["thetas"][0]), float(g["thetas"][1]))
    assert hashlib.sha256(pos.tobytes()).digest() == g["positions_sha256"].tobytes()
    return g, pos, np.ascontiguousarray(img.reshape(-1, 3))


def test_three_doublings_quirk_mode_is_the_reference_bit_for_bit():
    g, pos, val = _growth_fixture()
    n = pos.shape[0]
    lat = oracle.Lattice(5, 4, n, reference_growth_quirk=True)
    out = lat.filter(val, pos, False)
    assert lat.num_growths == 3 and len(g["growth_keys"]) == 3
    assert lat.num_vertices == int(g["num_vertices"])
    assert np.array_equal(lat.keys(), g["vertex_keys"])
    assert np.array_equal(lat.replay()[0].reshape(n, 6), g["replay_vertex"])
    assert np.array_equal(bits(out), bits(g["output_forward"]))
    assert np.array_equal(lat.growth_keys, g["growth_keys"])
    rev = oracle.Lattice(5, 4, n, reference_growth_quirk=True).filter(val, pos, True)
    assert np.array_equal(bits(rev), bits(g["output_reverse"]))


def test_three_doublings_difference_is_confined_to_the_keys_looked_up_at_the_doublings():
    """One vertex per distinct key (the oracle's default, what the HIP library builds) against the
    reference's own outputs: bit-equal at every point that has no simplex vertex within one blur
    step per axis of a key that was being looked up when the index doubled; the duplicated key is
    one of those; the deviation inside is the documented one (above the 1e-3 tolerance here)."""
    from growth_quirk import blur_neighbourhood, duplicated_keys, points_touching
    g, pos, val = _growth_fixture()
    n = pos.shape[0]
    dup_keys, n_dup = duplicated_keys(g["vertex_keys"])
    assert n_dup == 1
    growth = {k.tobytes() for k in g["growth_keys"]}
    assert all(k.tobytes() in growth for k in dup_keys)
    lat = oracle.Lattice(5, 4, n)
    out = lat.filter(val, pos, False)
    rev = oracle.Lattice(5, 4, n).filter(val, pos, True)
    assert lat.num_vertices == int(g["num_vertices"]) - n_dup
    near = points_touching(oracle.dump_simplex(pos)["keys"], blur_neighbourhood(g["growth_keys"], 5))
    assert 0 < near.sum() <= 256 * len(g["growth_keys"])          # 543 of 65 536 points
    # the points whose replay rows name a duplicated vertex are among them
    dup_vertices = [v for v in range(len(g["vertex_keys"]))
                    if any((g["vertex_keys"][v] == k).all() for k in dup_keys)]
    named = np.isin(g["replay_vertex"], dup_vertices).any(axis=1)
    assert named.any() and not (named & ~near).any()
    for got, want in ((out, g["output_forward"]), (rev, g["output_reverse"])):
        assert np.array_equal(bits(got[~near]), bits(want[~near]))
        d = np.abs(got - want).max(axis=1)
        assert 1e-3 < d.max() < 5e-3                                # 1.43e-3 both ways
        assert (d > 1e-4).sum() <= 64 * len(g["growth_keys"])       # 110 forward, 85 reverse
