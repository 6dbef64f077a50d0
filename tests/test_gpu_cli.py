"""The command-line bilateral filter (permutohedral_lattice_amd/csrc/bilateral_filter_cli.cpp)
against the image the reference keeps as the output of its own command line
(Images/output.bmp, made by `test_bilateral_gpu Images/input.bmp Images/output.bmp 8 0.125`,
README.md:51-59 of the reference), and its BMP reader/writer against PIL."""
import os
import subprocess

import numpy as np
import pytest

from conftest import ROOT, load_golden

BIN = os.path.join(ROOT, "permutohedral_lattice_amd", "bilateral_filter_hip.bin")


def run_cli(*args):
    if not os.path.exists(BIN):
        pytest.fail("%s is missing: run __graft_entry__.build() first" % BIN)
    res = subprocess.run([BIN] + [str(a) for a in args], stdout=subprocess.PIPE,
                         stderr=subprocess.STDOUT, text=True, timeout=100)
    print(res.stdout)
    return res


@pytest.mark.gpu
def test_cli_reproduces_the_reference_output_image(tmp_path):
    from PIL import Image
    im = load_golden("reference_images")
    src, dst = tmp_path / "input.bmp", tmp_path / "output.bmp"
    Image.fromarray(im["input"]).save(src)
    res = run_cli(src, dst, 8, 0.125)
    assert res.returncode == 0, res.stdout
    # the float run, then the double run as in the reference's program, close to each other
    assert res.stdout.count("Measured from function call") == 2
    assert "Testing for double precision" in res.stdout
    double_vs_float = float(res.stdout.split("max |double - float|")[1].split(")")[0])
    # (points on simplex faces -- 8-bit colours make many -- may fall to either side in float)
    assert 0.0 < double_vs_float <= 1e-2
    got = np.array(Image.open(dst)).astype(np.int64)
    want = im["cli_output"].astype(np.int64)
    assert got.shape == want.shape
    diff = np.abs(got - want)
    # the fixture came from the reference's CUDA path, whose splat order and scale factor differ in
    # the last bits; after truncation to 8 bits that moves a fraction of a percent by one level
    assert diff.max() <= 1
    assert (diff != 0).mean() <= 5e-3


@pytest.mark.gpu
def test_cli_filters_a_grey_palette_image_under_a_colour_guide(tmp_path):
    from PIL import Image
    import torch
    import permutohedral_lattice_amd as pla
    im = load_golden("reference_images")
    guide = im["input"][:200, :300]
    grey = im["gray_original"][:200, :300]
    g_path, s_path, dst = tmp_path / "guide.bmp", tmp_path / "grey.bmp", tmp_path / "out.bmp"
    Image.fromarray(np.ascontiguousarray(guide)).save(g_path)
    Image.fromarray(np.ascontiguousarray(grey)).save(s_path)     # 8-bit BMP with a grey palette
    res = run_cli(g_path, dst, 8, 0.125, s_path)
    assert res.returncode == 0, res.stdout
    got = np.array(Image.open(dst)).astype(np.int64)
    # the same through the op, truncated the same way
    x = np.repeat((grey / np.float32(255.0)).astype(np.float32)[None, :, :, None], 3, axis=3)
    r = (guide / np.float32(255.0)).astype(np.float32)[None]
    out = pla.lattice_filter(torch.from_numpy(x).cuda(), torch.from_numpy(r).cuda(),
                             theta_alpha=8.0, theta_beta=0.125).cpu().numpy()[0]
    levels = out * np.float32(255.0)
    want = np.clip(levels.astype(np.int64), 0, 255)
    diff = np.abs(got - want)
    assert diff.max() <= 1
    # truncation: a flat grey area filters to k/255 up to the order of the float sums, which
    # lands on either side of level k; anything else must agree
    near_a_level = np.abs(levels - np.round(levels)) < 0.05
    assert (near_a_level | (diff == 0)).all()


def test_cli_usage_and_errors(tmp_path):
    res = run_cli()
    assert res.returncode == 1 and "Usage" in res.stdout
    bad = tmp_path / "not_a.bmp"
    bad.write_bytes(b"hello")
    res = run_cli(bad, tmp_path / "o.bmp", 8, 0.125)
    assert res.returncode == 2 and "not a BMP" in res.stdout
