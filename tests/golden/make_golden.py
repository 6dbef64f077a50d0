"""Writes the golden fixtures of this directory.  Run once, in the build container:

    make -C oracle ref && python tests/golden/make_golden.py

Vectors come from the reference's own CPU header compiled as oracle/_ref/libplref.so (the
harness around it is oracle/ref_harness.cpp); images are the data files the reference's tests
hold (Images/*.bmp), re-encoded losslessly as compressed arrays.  The fixtures are data only:
inputs and the reference's outputs.  Nothing here runs on the GPU box.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from permutohedral_lattice_amd import synth  # noqa: E402

REFERENCE_IMAGES = "/root/reference/Images"


def lattice_case(ref, name, pd, vd, positions, values, per_point=True, dtype=np.float32):
    """dtype: the reference's template parameter T.  float64 cases start from the same float32
    inputs, widened, and are stored as lattice_<name>_f64.npz."""
    positions = np.ascontiguousarray(positions, dtype)
    values = np.ascontiguousarray(values, dtype)
    dump = ref.dump_simplex(positions, dtype=dtype)
    if not per_point:  # large case: keep the per-point integers, drop the per-point floats
        dump["elevated"] = dump["elevated"][:0]
        dump["barycentric"] = dump["barycentric"][:0]
    fwd = ref.filter_stages(pd, vd, values, positions, reverse=False, dtype=dtype)
    rev = ref.filter_stages(pd, vd, values, positions, reverse=True, dtype=dtype)
    _, m, keys, _ = ref.filter(pd, vd, values, positions, False, dtype=dtype)
    assert m == fwd["M"] == rev["M"]
    out = dict(pd=np.int32(pd), vd=np.int32(vd), positions=positions, values=values,
               elevated=dump["elevated"], rem0=dump["rem0"], rank=dump["rank"], keys=dump["keys"],
               barycentric=dump["barycentric"], num_vertices=np.int32(m), vertex_keys=keys,
               after_splat=fwd["after_splat"], after_blur_forward=fwd["after_blur"],
               after_blur_reverse=rev["after_blur"], output_forward=fwd["output"],
               output_reverse=rev["output"])
    if np.dtype(dtype) == np.float64:
        name += "_f64"
    path = os.path.join(HERE, "lattice_%s.npz" % name)
    np.savez_compressed(path, **out)
    print("%-28s N=%6d pd=%d vd=%2d M=%6d  %7.1f KB" % (name, positions.shape[0], pd, vd, m,
                                                       os.path.getsize(path) / 1024))


def growth_case(ref, name, side, theta_alpha, theta_beta, seed, noise):
    """A case whose vertex count makes the reference's hash index double three times.  The lookup
    that triggers a doubling probes from a stale cell (src/PermutohedralLatticeCPU.h:163-165, :62):
    it can enter a key a second time or miss a neighbour.  Stored: the image (positions are
    synth.bilateral_positions of it, values its colours), and from the reference's own build the
    outputs of both blur orders, the vertex keys in first-touch order (a duplicated key appears
    twice) and the vertex each replay row names; from the oracle with the quirk reproduced, the
    key that was being looked up at each doubling."""
    import hashlib
    img = synth.blob_image(side, side, seed=seed, noise=noise)
    positions = synth.bilateral_positions(img, theta_alpha, theta_beta)
    values = np.ascontiguousarray(img.reshape(-1, 3))
    fwd = ref.filter_replay(5, 4, values, positions, False)
    rev = ref.filter_replay(5, 4, values, positions, True)
    assert fwd["M"] == rev["M"] and np.array_equal(fwd["keys"], rev["keys"])
    quirk = oracle.Lattice(5, 4, side * side, reference_growth_quirk=True)
    assert np.array_equal(quirk.filter(values, positions, False), fwd["output"])
    growth_keys = quirk.growth_keys
    path = os.path.join(HERE, "%s.npz" % name)
    np.savez_compressed(
        path, pd=np.int32(5), vd=np.int32(4), side=np.int32(side),
        thetas=np.array([theta_alpha, theta_beta], np.float32), image=img.astype(np.float32),
        positions_sha256=np.frombuffer(hashlib.sha256(positions.tobytes()).digest(), np.uint8),
        num_vertices=np.int32(fwd["M"]), vertex_keys=fwd["keys"],
        replay_vertex=fwd["replay_vertex"].astype(np.int32),
        output_forward=fwd["output"], output_reverse=rev["output"],
        growth_keys=growth_keys)
    distinct = len(np.unique(fwd["keys"], axis=0))
    print("%-28s N=%6d M=%6d distinct=%6d doublings=%d  %7.1f KB" % (
        name, side * side, fwd["M"], distinct, len(growth_keys), os.path.getsize(path) / 1024))


def main():
    ref = oracle.reference()
    if ref is None:
        raise SystemExit("oracle/_ref/libplref.so is missing: run `make -C oracle ref` first")

    # `make_golden.py growth` writes only the case of three doublings (the other fixtures are
    # reproduced bit for bit by a full run, but their archives would change with the date)
    growth_only = len(sys.argv) > 1 and sys.argv[1] == "growth"
    growth_case(ref, "growth_three_doublings_pd5_vd4", 256, 3.0, 0.04, 141, 0.03)
    if growth_only:
        return

    # scale factors, bit patterns
    factors = {"pd%d" % pd: ref.scale_factor(pd) for pd in range(1, 9)}
    factors.update({"pd%d_f64" % pd: ref.scale_factor(pd, np.float64) for pd in range(1, 9)})
    np.savez(os.path.join(HERE, "scale_factor.npz"), **factors)

    # feature builder: 2-D and 3-D, stds that are not powers of two
    rng = np.random.default_rng(11)
    pos_cases = {}
    for name, sdims, rc, s_std, f_std in (("2d_rgb", (9, 13), 3, 8.0, 0.125),
                                          ("3d_grey", (5, 7, 6), 1, 5.0, 0.1),
                                          ("2d_spatial", (12, 10), 0, 3.0, -1.0),
                                          ("2d_crf", (8, 8), 3, 80.0, 13.0)):
        n = int(np.prod(sdims))
        # the op's attributes are floats for every T: the stds are float values also in double
        s_std, f_std = float(np.float32(s_std)), float(np.float32(f_std))
        refimg = rng.uniform(0, 255 if f_std > 1 else 1, (n, max(rc, 1))).astype(np.float32)
        pos_cases[name + "_sdims"] = np.array(sdims, np.int32)
        pos_cases[name + "_rc"] = np.int32(rc)
        pos_cases[name + "_stds"] = np.array([s_std, f_std], np.float32)
        pos_cases[name + "_reference"] = refimg
        pos_cases[name + "_positions"] = ref.compute_positions(refimg, sdims, s_std, f_std, rc)
        pos_cases[name + "_positions_f64"] = ref.compute_positions(refimg, sdims, s_std, f_std, rc,
                                                                   dtype=np.float64)
    np.savez_compressed(os.path.join(HERE, "positions.npz"), **pos_cases)

    # lattice cases, one per (pd, vd) of the benchmark configurations, at small sizes
    img = synth.blob_image(40, 48, seed=101)
    lattice_case(ref, "bilateral_pd5_vd4", 5, 4, synth.bilateral_positions(img, 8.0, 0.125),
                 img.reshape(-1, 3))
    lattice_case(ref, "spatial_pd2_vd2", 2, 2, synth.spatial_positions((64, 64), 8.0),
                 synth.uniform_image((64 * 64, 1), 102))
    guide = synth.blob_image(40, 40, seed=103)
    lattice_case(ref, "guided_pd5_vd2", 5, 2, synth.bilateral_positions(guide, 8.0, 0.125),
                 synth.uniform_image((1600, 1), 104))
    vol = synth.ellipsoid_volume(12, 16, 16, seed=105)
    lattice_case(ref, "volume_pd4_vd2", 4, 2, synth.bilateral_positions(vol, 5.0, 0.1),
                 vol.reshape(-1, 1))
    crf_guide = synth.blob_image(24, 24, seed=106) * 255.0
    q = synth.softmax_logits((576, 21), 107)
    lattice_case(ref, "crf_bilateral_pd5_vd22", 5, 22, synth.bilateral_positions(crf_guide, 80.0, 13.0), q)
    lattice_case(ref, "crf_spatial_pd2_vd22", 2, 22, synth.spatial_positions((24, 24), 3.0), q)
    # a fine lattice over a noisy image: M passes 16383, so the reference's hash index doubles, and
    # with this seed the lookup that triggers the doubling misses a key that is present and enters
    # it a second time (the vertex list has one duplicate)
    noisy = synth.blob_image(144, 144, seed=122, noise=0.08)
    lattice_case(ref, "growth_duplicate_pd5_vd4", 5, 4, synth.bilateral_positions(noisy, 2.0, 0.05),
                 noisy.reshape(-1, 3), per_point=False)
    # exact ties: integer grid positions with unit std put many points on simplex faces
    gx, gy, gz = np.meshgrid(np.arange(12), np.arange(12), np.arange(6), indexing="ij")
    tie_pos = np.stack([gx, gy, gz], -1).reshape(-1, 3).astype(np.float32)
    lattice_case(ref, "ties_pd3_vd2", 3, 2, tie_pos, synth.uniform_image((tie_pos.shape[0], 1), 109))
    # pd = 1, 6, 7, 8 to cover every instantiated dimension
    for pd in (1, 6, 7, 8):
        rng = np.random.default_rng(110 + pd)
        lattice_case(ref, "random_pd%d_vd3" % pd, pd, 3,
                     rng.uniform(-6, 6, (700, pd)).astype(np.float32),
                     rng.uniform(0, 1, (700, 2)).astype(np.float32))

    # T = double: the colour case, exact ties, the guided case and the highest dimension
    lattice_case(ref, "bilateral_pd5_vd4", 5, 4, synth.bilateral_positions(img, 8.0, 0.125),
                 img.reshape(-1, 3), dtype=np.float64)
    lattice_case(ref, "ties_pd3_vd2", 3, 2, tie_pos, synth.uniform_image((tie_pos.shape[0], 1), 109),
                 dtype=np.float64)
    lattice_case(ref, "guided_pd5_vd2", 5, 2, synth.bilateral_positions(guide, 8.0, 0.125),
                 synth.uniform_image((1600, 1), 104), dtype=np.float64)
    rng = np.random.default_rng(118)
    lattice_case(ref, "random_pd8_vd3", 8, 3, rng.uniform(-6, 6, (700, 8)).astype(np.float32),
                 rng.uniform(0, 1, (700, 2)).astype(np.float32), dtype=np.float64)

    # the reference's image fixtures (Tests/bilateral_filter.py, Tests/greyscale_test.py)
    from PIL import Image
    images = {}
    for key, fname in (("input", "input.bmp"), ("bilateral_out_1", "bilateral_out_1.bmp"),
                       ("gray_original", "gray_original.bmp"), ("filtered_grey", "filtered_grey.bmp"),
                       ("cli_output", "output.bmp")):
        images[key] = np.array(Image.open(os.path.join(REFERENCE_IMAGES, fname)))
    path = os.path.join(HERE, "reference_images.npz")
    np.savez_compressed(path, **images)
    print("reference_images.npz %.1f MB" % (os.path.getsize(path) / 1e6))


if __name__ == "__main__":
    main()
