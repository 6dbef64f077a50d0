"""pl_apply on a lattice built by pl_build splats by gathering along per-vertex lists (the
transpose of the replay matrix).  Against the oracle, and against the same lattice with the lists
switched off (the splat of pl_filter: sums per wavefront, atomics)."""
import zlib

import numpy as np
import pytest
import torch

from conftest import MAX_ABS_TOL, REL_L2_TOL, rel_l2
from permutohedral_lattice_amd import synth

import oracle
import permutohedral_lattice_amd as pla

pytestmark = pytest.mark.gpu


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _apply(pd, vd, pos, val, reverse, lists, grid=None, stop_after=0):
    n = pos.shape[0]
    lat = pla.PermutohedralLattice(pd, vd, n)
    lat.set_option(pla.PL_OPT_VERTEX_LISTS, 1 if lists else 0)
    if grid:
        lat.set_point_grid(grid)
    lat.build(_dev(pos))
    out = torch.full((n, vd - 1), float("nan"), dtype=torch.float32, device="cuda")
    d_val = _dev(val)
    if stop_after:
        lat.set_option(pla.PL_OPT_STOP_AFTER, stop_after)
    lat.apply(out, d_val, reverse)
    lat.apply(out, d_val, reverse)      # a second apply on the same lattice: nothing left over
    torch.cuda.synchronize()
    return out.cpu().numpy(), lat


CASES = [
    ("image_pd5_vd4", 5, 4, (96, 112)),
    ("image_pd5_vd2", 5, 2, (64, 80)),
    ("image_pd5_vd3", 5, 3, (40, 40)),
    ("crf_pd5_vd22", 5, 22, (64, 64)),
    ("spatial_pd2_vd22", 2, 22, (64, 64)),
    ("spatial_pd2_vd2", 2, 2, (128, 128)),
    ("crf_pd5_vd70", 5, 70, (24, 24)),
    ("crf_pd5_vd9", 5, 9, (32, 40)),
    # every width of the four-channels-per-lane kernels and their edges: 4 lanes (5..16 channels),
    # 8 (17..32), 16 (33..64), more than 64; input rows of a multiple of four floats and not
    ("crf_pd5_vd5", 5, 5, (32, 32)),
    ("crf_pd3_vd13", 3, 13, (40, 24)),
    ("crf_pd5_vd16", 5, 16, (24, 24)),
    ("crf_pd5_vd17", 5, 17, (24, 24)),
    ("spatial_pd2_vd32", 2, 32, (32, 32)),
    ("spatial_pd2_vd33", 2, 33, (32, 32)),
    ("crf_pd5_vd48", 5, 48, (24, 24)),
    ("spatial_pd2_vd64", 2, 64, (24, 24)),
    ("spatial_pd2_vd65", 2, 65, (24, 24)),
]


def _inputs(name, pd, vd, shape):
    h, w = shape
    rng = np.random.default_rng(zlib.crc32(name.encode()) % 1000)
    if pd == 2:
        pos = synth.spatial_positions(shape, 3.0)
    elif pd == 3:
        pos = synth.bilateral_positions(synth.blob_image(h, w, seed=7)[..., :1] * 255.0, 20.0, 13.0)
    elif vd > 4:
        pos = synth.bilateral_positions(synth.blob_image(h, w, seed=7) * 255.0, 80.0, 13.0)
    else:
        pos = synth.bilateral_positions(synth.blob_image(h, w, seed=8), 8.0, 0.125)
    val = rng.uniform(0, 1, (h * w, vd - 1)).astype(np.float32)
    return pos, val


@pytest.mark.parametrize("name,pd,vd,shape", CASES)
@pytest.mark.parametrize("reverse", [False, True])
def test_apply_from_vertex_lists_matches_oracle_and_atomic_splat(name, pd, vd, shape, reverse):
    pos, val = _inputs(name, pd, vd, shape)
    n = pos.shape[0]
    got, lat = _apply(pd, vd, pos, val, reverse, True, grid=shape)
    plain, lat0 = _apply(pd, vd, pos, val, reverse, False, grid=shape)
    cpu = oracle.Lattice(pd, vd, n)
    want = cpu.filter(val, pos, reverse)
    assert lat.num_vertices == cpu.num_vertices == lat0.num_vertices
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= MAX_ABS_TOL and rel_l2(got, want) <= REL_L2_TOL
    assert np.abs(got - plain).max() <= 1e-5


@pytest.mark.parametrize("pd,vd,shape", [(5, 22, (48, 48)), (2, 13, (40, 40)), (5, 4, (64, 48)),
                                         (2, 36, (24, 24)), (5, 8, (32, 32))])
def test_apply_without_normalisation_takes_input_rows_of_vd_channels(pd, vd, shape):
    """PL_OPT_NORMALIZE = 0: the input carries all vd channels and the output is the bare sum
    (the gathers and the slice then read and write rows of vd floats, not vd - 1)."""
    h, w = shape
    n = h * w
    rng = np.random.default_rng(vd)
    pos = (synth.spatial_positions(shape, 3.0) if pd == 2 else
           synth.bilateral_positions(synth.blob_image(h, w, seed=3) * 255.0, 60.0, 13.0))
    val = rng.uniform(0, 1, (n, vd)).astype(np.float32)
    outs = []
    for lists in (1, 0):
        lat = pla.PermutohedralLattice(pd, vd, n)
        lat.set_option(pla.PL_OPT_VERTEX_LISTS, lists)
        lat.set_option(pla.PL_OPT_NORMALIZE, 0)
        lat.set_point_grid(shape)
        lat.build(_dev(pos))
        out = torch.full((n, vd), float("nan"), dtype=torch.float32, device="cuda")
        lat.apply(out, _dev(val), False)
        torch.cuda.synchronize()
        outs.append(out.cpu().numpy())
    want = oracle.Lattice(pd, vd, n).filter_raw(val, pos, False)
    scale = max(1.0, np.abs(want).max())
    assert np.isfinite(outs[0]).all()
    assert np.abs(outs[0] - want).max() <= MAX_ABS_TOL * scale and rel_l2(outs[0], want) <= REL_L2_TOL
    assert np.abs(outs[0] - outs[1]).max() <= 1e-5 * scale


def test_vertex_values_after_the_gathering_splat():
    """The splat alone (PL_OPT_STOP_AFTER = 1): vertex values by key against the oracle's."""
    pos, val = _inputs("image_pd5_vd4", 5, 4, (96, 112))
    n = pos.shape[0]
    _, lat = _apply(5, 4, pos, val, False, True, grid=(96, 112), stop_after=1)
    keys = lat.debug_keys().cpu().numpy()
    values = lat.debug_values().cpu().numpy()
    cpu = oracle.Lattice(5, 4, n)
    cpu.splat(val, pos)
    want = {k.tobytes(): v for k, v in zip(cpu.keys(), cpu.values())}
    assert len(want) == len(keys)
    ref = np.stack([want[k.tobytes()] for k in keys])
    assert np.abs(values - ref).max() <= 1e-4 * max(1.0, np.abs(ref).max())


def test_lists_of_a_plain_list_and_of_a_crowded_vertex():
    # a plain list of points (no grid): the ordering pass maps threads to points
    rng = np.random.default_rng(5)
    n = 20000
    pos = rng.uniform(0, 6, (n, 3)).astype(np.float32)
    val = rng.uniform(0, 1, (n, 2)).astype(np.float32)
    got, lat = _apply(3, 3, pos, val, False, True)
    want = oracle.Lattice(3, 3, n).filter(val, pos, False)
    assert np.abs(got - want).max() <= MAX_ABS_TOL and rel_l2(got, want) <= REL_L2_TOL
    # all points in one simplex: six lists of n entries each
    n = 5000
    pos = np.tile(np.array([[0.31, 0.12, 0.55, 0.2, 0.4]], np.float32), (n, 1))
    val = rng.uniform(0, 1, (n, 3)).astype(np.float32)
    got, lat = _apply(5, 4, pos, val, True, True)
    assert lat.num_vertices == 6
    want = oracle.Lattice(5, 4, n).filter(val, pos, True)
    assert np.abs(got - want).max() <= MAX_ABS_TOL and rel_l2(got, want) <= REL_L2_TOL
    # fewer points than a workgroup, and a single point
    for n in (1, 37):
        pos = rng.uniform(0, 3, (n, 4)).astype(np.float32)
        val = rng.uniform(0, 1, (n, 1)).astype(np.float32)
        got, _ = _apply(4, 2, pos, val, False, True)
        want = oracle.Lattice(4, 2, n).filter(val, pos, False)
        assert np.abs(got - want).max() <= MAX_ABS_TOL


def test_rebuilding_a_lattice_renews_its_lists():
    pos1, val1 = _inputs("image_pd5_vd4", 5, 4, (64, 64))
    img2 = synth.blob_image(64, 64, seed=99)
    pos2 = synth.bilateral_positions(img2, 4.0, 0.1)
    n = pos1.shape[0]
    lat = pla.PermutohedralLattice(5, 4, n)
    lat.set_point_grid((64, 64))
    out = torch.empty((n, 3), dtype=torch.float32, device="cuda")
    for pos in (pos1, pos2, pos1):
        lat.build(_dev(pos))
        lat.apply(out, _dev(val1), False)
        torch.cuda.synchronize()
        want = oracle.Lattice(5, 4, n).filter(val1, pos, False)
        assert np.abs(out.cpu().numpy() - want).max() <= MAX_ABS_TOL
    # a filter() on the same handle in between drops the lists (they described another build)
    lat.filter(out, _dev(val1), _dev(pos2), False)
    lat.apply(out, _dev(val1), True)
    torch.cuda.synchronize()
    want = oracle.Lattice(5, 4, n).filter(val1, pos2, True)
    assert np.abs(out.cpu().numpy() - want).max() <= MAX_ABS_TOL
