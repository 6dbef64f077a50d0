"""Stage by stage: the vertex values behind the splat and behind the blur (forward and reverse
order), read through pl_debug_values and matched to the reference's vertices by key, for every
golden lattice case.  A splat or blur error that a later stage happened to hide would show here."""
import numpy as np
import pytest
import torch

from conftest import golden_lattice_cases, load_golden

import oracle
import permutohedral_lattice_amd as pla

pytestmark = pytest.mark.gpu


def _by_key(keys, values):
    """Rows of `values` summed per distinct key, in lexicographic key order (the reference's
    vertex list may hold a key twice: once per doubling of its index)."""
    keys = np.asarray(keys)
    uniq, inverse = np.unique(keys, axis=0, return_inverse=True)
    out = np.zeros((len(uniq), values.shape[1]), np.float64)
    np.add.at(out, inverse.reshape(-1), values.astype(np.float64))
    return uniq, out


def _stage(lat, d_val, d_pos, out, stop, reverse):
    lat.set_option(pla.PL_OPT_STOP_AFTER, stop)
    lat.filter(out, d_val, d_pos, reverse)
    torch.cuda.synchronize()
    keys = lat.debug_keys().cpu().numpy()
    vals = lat.debug_values().cpu().numpy()
    lat.set_option(pla.PL_OPT_STOP_AFTER, 0)
    return _by_key(keys, vals)


@pytest.mark.parametrize("name", golden_lattice_cases() + golden_lattice_cases(f64=True))
@pytest.mark.parametrize("entry", ["filter", "build_apply"])
def test_vertex_values_after_splat_and_after_blur(name, entry):
    g = load_golden("lattice_" + name)
    pd, vd = int(g["pd"]), int(g["vd"])
    pos, val = g["positions"], g["values"]
    n = pos.shape[0]
    f64 = pos.dtype == np.float64
    tdt = torch.float64 if f64 else torch.float32
    rtol, atol = (1e-12, 1e-12) if f64 else (1e-5, 1e-5)
    d_pos, d_val = torch.from_numpy(pos).cuda(), torch.from_numpy(val).cuda()
    out = torch.empty((n, vd - 1), dtype=tdt, device="cuda")
    lat = pla.PermutohedralLattice(pd, vd, n, dtype=tdt)
    has_duplicates = len(np.unique(g["vertex_keys"], axis=0)) != len(g["vertex_keys"])

    def stage(stop, reverse):
        if entry == "filter":
            return _stage(lat, d_val, d_pos, out, stop, reverse)
        lat.set_option(pla.PL_OPT_STOP_AFTER, stop)
        lat.build(d_pos)
        lat.apply(out, d_val, reverse)
        torch.cuda.synchronize()
        res = _by_key(lat.debug_keys().cpu().numpy(), lat.debug_values().cpu().numpy())
        lat.set_option(pla.PL_OPT_STOP_AFTER, 0)
        return res

    # the oracle's stages (bit-equal to the golden ones when it reproduces the reference's
    # duplicate vertices, tests/test_oracle.py); here one vertex per key, like the library
    for reverse, blur_key in ((False, "after_blur_forward"), (True, "after_blur_reverse")):
        cpu = oracle.Lattice(pd, vd, n, dtype=pos.dtype)
        cpu.splat(val, pos)
        want_keys, want_splat = _by_key(cpu.keys(), cpu.values())
        got_keys, got_splat = stage(1, reverse)
        assert (got_keys == want_keys).all()
        assert np.allclose(got_splat, want_splat, rtol=rtol, atol=atol)
        # against the reference's own numbers: its splat sums per key whatever its duplicates
        ref_keys, ref_splat = _by_key(g["vertex_keys"], g["after_splat"])
        assert (ref_keys == got_keys).all()
        assert np.allclose(got_splat, ref_splat, rtol=rtol, atol=atol)
        cpu.blur(reverse)
        _, want_blur = _by_key(cpu.keys(), cpu.values())
        got_keys, got_blur = stage(2, reverse)
        assert (got_keys == want_keys).all()
        assert np.allclose(got_blur, want_blur, rtol=rtol, atol=atol)
        if not has_duplicates:
            _, ref_blur = _by_key(g["vertex_keys"], g[blur_key])
            assert np.allclose(got_blur, ref_blur, rtol=rtol, atol=atol)
    # and a full call afterwards is untouched by the stops
    lat.filter(out, d_val, d_pos, False)
    torch.cuda.synchronize()
    assert np.abs(out.cpu().numpy() - g["output_forward"]).max() <= (1e-10 if f64 else 1e-3)
