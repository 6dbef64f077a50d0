"""pl_filter_static: the entry point that allocates nothing (its lattice lives in a static device
array inside the library) against pl_filter on a handle, through the C ABI."""
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


def _case(h, w, seed):
    img = synth.blob_image(h, w, seed=seed)
    return synth.bilateral_positions(img, 8.0, 0.125), img.reshape(-1, 3)


def _check_against_handle_and_oracle(pos, val, pd, vd, reverse):
    n = pos.shape[0]
    d_pos, d_val = _dev(pos), _dev(val)
    got = torch.full((n, vd - 1), float("nan"), dtype=torch.float32, device="cuda")
    pla.filter_static(got, d_val, d_pos, pd, vd, reverse)
    # (the call returns when its work is complete: no synchronisation here on purpose)
    got = got.cpu().numpy()
    lat = pla.PermutohedralLattice(pd, vd, n)
    lat.set_option(pla.PL_OPT_GUESS_GRID, 0)
    want = torch.empty((n, vd - 1), dtype=torch.float32, device="cuda")
    lat.filter(want, d_val, d_pos, reverse)
    torch.cuda.synchronize()
    want = want.cpu().numpy()
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= MAX_ABS_TOL and rel_l2(got, want) <= REL_L2_TOL
    cpu = oracle.Lattice(pd, vd, n).filter(val, pos, reverse)
    assert np.abs(got - cpu).max() <= MAX_ABS_TOL and rel_l2(got, cpu) <= REL_L2_TOL


def test_static_filter_twice_in_a_row_the_second_smaller():
    pos, val = _case(96, 80, 101)
    _check_against_handle_and_oracle(pos, val, 5, 4, False)
    pos, val = _case(40, 50, 102)            # smaller: what the first call left must not show
    _check_against_handle_and_oracle(pos, val, 5, 4, False)
    _check_against_handle_and_oracle(pos, val, 5, 4, True)
    # other dimensions in the same array: many channels (no splat inside the build), pd = 2
    rng = np.random.default_rng(103)
    pos = synth.spatial_positions((60, 70), 3.0)
    val = rng.uniform(0, 1, (60 * 70, 7)).astype(np.float32)
    _check_against_handle_and_oracle(pos, val, 2, 8, False)


def test_static_filter_at_its_size_limit_and_beyond():
    rng = np.random.default_rng(104)
    n = 131072 // 6
    pos = rng.uniform(0, 12, (n, 5)).astype(np.float32)     # scattered: nearly every vertex distinct
    val = rng.uniform(0, 1, (n, 3)).astype(np.float32)
    _check_against_handle_and_oracle(pos, val, 5, 4, False)
    n = 131072 // 9
    pos = rng.uniform(0, 4, (n, 8)).astype(np.float32)
    val = rng.uniform(0, 1, (n, 7)).astype(np.float32)
    _check_against_handle_and_oracle(pos, val, 8, 8, True)
    n = 131072 // 6 + 1
    out = torch.empty((n, 3), dtype=torch.float32, device="cuda")
    with pytest.raises(pla.PermutohedralError) as e:
        pla.filter_static(out, out, torch.empty((n, 5), dtype=torch.float32, device="cuda"), 5, 4)
    assert e.value.status == pla.PL_ETOOLARGE
    with pytest.raises(pla.PermutohedralError) as e:
        pla.filter_static(torch.empty((64, 8), dtype=torch.float32, device="cuda"),
                          torch.empty((64, 8), dtype=torch.float32, device="cuda"),
                          torch.empty((64, 2), dtype=torch.float32, device="cuda"), 2, 9)
    assert e.value.status == pla.PL_ETOOLARGE


def test_static_filter_leaves_the_free_device_memory_as_it_was():
    """hipMemGetInfo before and after: an allocation that crept into the path (and was not given
    back) would show, and so would one that is given back only later (the figures are read while
    nothing else runs in this process)."""
    pos, val = _case(64, 64, 105)
    n = pos.shape[0]
    d_pos, d_val = _dev(pos), _dev(val)
    out = torch.empty((n, 3), dtype=torch.float32, device="cuda")
    pla.filter_static(out, d_val, d_pos, 5, 4, False)      # (the first call on a device looks the array up)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    lowest = free_before
    for reverse in (False, True, False):
        pla.filter_static(out, d_val, d_pos, 5, 4, reverse)
        lowest = min(lowest, torch.cuda.mem_get_info()[0])
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before and lowest == free_before


def test_static_filter_refuses_a_stream_of_another_kind_of_argument():
    # (one GPU here: a stream of another device cannot be made; the current device's own stream passes)
    pos, val = _case(32, 32, 106)
    d_pos, d_val = _dev(pos), _dev(val)
    out = torch.empty((pos.shape[0], 3), dtype=torch.float32, device="cuda")
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        pla.filter_static(out, d_val, d_pos, 5, 4, False, stream=s)
    want = oracle.Lattice(5, 4, pos.shape[0]).filter(val, pos, False)
    assert np.abs(out.cpu().numpy() - want).max() <= MAX_ABS_TOL
