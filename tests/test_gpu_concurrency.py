"""Several lattices in flight: the two halves of filter (pl_filter_begin / pl_filter_end) on
lattices with streams of their own, and the op spreading a batch over concurrent lattices.
Results must not depend on how many items run at a time; parity is against the CPU oracle."""
import numpy as np
import pytest
import torch

from conftest import MAX_ABS_TOL, REL_L2_TOL, rel_l2
from permutohedral_lattice_amd import synth

import oracle
import permutohedral_lattice_amd as pla

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def close(got, want, scale=1.0):
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= MAX_ABS_TOL * scale
    assert rel_l2(got, want) <= REL_L2_TOL


def test_two_lattices_in_flight_on_two_streams():
    h = w = 160
    cases = []
    for seed, reverse in ((31, False), (32, True), (33, False)):
        img = synth.blob_image(h, w, seed=seed)
        pos = synth.bilateral_positions(img, 8.0, 0.125)
        val = synth.uniform_image((h * w, 3), seed + 100)
        cases.append((pos, val, reverse, oracle.Lattice(5, 4, h * w).filter(val, pos, reverse)))
    streams = [torch.cuda.Stream() for _ in cases]
    lattices, outs = [], []
    torch.cuda.synchronize()
    for (pos, val, reverse, _), s in zip(cases, streams):
        d_pos, d_val = dev(pos), dev(val)
        out = torch.empty((h * w, 3), dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()          # the uploads ran on the current stream
        lat = pla.PermutohedralLattice(5, 4, h * w, stream=s)
        lat.filter_begin(out, d_val, d_pos, reverse)
        lattices.append(lat)
        outs.append(out)
    for lat in lattices:
        lat.filter_end()
    for lat, out, (_, _, _, want) in zip(lattices, outs, cases):
        close(out.cpu().numpy(), want)
        assert lat.num_vertices > 0
    lattices[0].filter_end()               # nothing in flight: fine


def test_only_end_may_follow_begin():
    n = 64 * 64
    img = synth.blob_image(64, 64, seed=35)
    d_pos = dev(synth.bilateral_positions(img, 8.0, 0.125))
    d_val = dev(img.reshape(-1, 3))
    out = torch.empty_like(d_val)
    lat = pla.PermutohedralLattice(5, 4, n)
    lat.filter_begin(out, d_val, d_pos)
    for call in (lambda: lat.apply(out, d_val), lambda: lat.build(d_pos),
                 lambda: lat.filter(out, d_val, d_pos), lambda: lat.set_point_grid((64, 64)),
                 lambda: lat.filter_begin(out, d_val, d_pos), lambda: lat.num_vertices):
        with pytest.raises(pla.PermutohedralError) as e:
            call()
        assert e.value.status == pla.PL_ESTATE
    lat.filter_end()
    want = oracle.Lattice(5, 4, n).filter(img.reshape(-1, 3), synth.bilateral_positions(img, 8.0, 0.125))
    close(out.cpu().numpy(), want)
    lat.apply(out, d_val)                  # usable again


def test_end_repeats_the_call_when_the_table_was_too_small():
    rng = np.random.default_rng(36)
    n = 20000
    pos = rng.uniform(0, 40, (n, 3)).astype(np.float32)    # scattered: about 4 vertices per point
    val = rng.uniform(0, 1, (n, 2)).astype(np.float32)
    cpu = oracle.Lattice(3, 3, n)
    want = cpu.filter(val, pos, False)
    lat = pla.PermutohedralLattice(3, 3, n)
    lat.set_option(pla.PL_OPT_TABLE_CELLS, 4096)
    out = torch.empty((n, 2), dtype=torch.float32, device="cuda")
    lat.filter_begin(out, dev(val), dev(pos))
    lat.filter_end()
    assert lat.num_vertices == cpu.num_vertices > 4096
    close(out.cpu().numpy(), want)


def test_several_lattices_built_side_by_side_then_applied():
    """pl_build_begin / pl_build_image_begin on lattices with streams of their own, then
    pl_build_end on each: applies give what filter gives (the oracle), also for a table that had to
    grow in between, and with or without the per-vertex lists."""
    h = w = 96
    n = h * w
    cases = []
    for seed, reverse, image, lists in ((51, False, False, 1), (52, True, True, 1), (53, False, True, 0),
                                        (54, True, False, 0)):
        img = synth.blob_image(h, w, seed=seed)
        pos = synth.bilateral_positions(img, 6.0, 0.1)
        val = synth.uniform_image((n, 3), seed + 100)
        cases.append((img, pos, val, reverse, image, lists,
                      oracle.Lattice(5, 4, n).filter(val, pos, reverse)))
    streams = [torch.cuda.Stream() for _ in cases]
    lattices, keep = [], []
    torch.cuda.synchronize()
    for k, ((img, pos, val, reverse, image, lists, _), s) in enumerate(zip(cases, streams)):
        lat = pla.PermutohedralLattice(5, 4, n, stream=s)
        lat.set_option(pla.PL_OPT_VERTEX_LISTS, lists)
        if k == 1:
            lat.set_option(pla.PL_OPT_TABLE_CELLS, 2048)       # too small: build_end repeats the build
        d_val = dev(val)
        d_img, d_pos = dev(img.reshape(n, 3)), dev(pos)
        torch.cuda.synchronize()          # the uploads ran on the current stream
        if image:
            lat.build_image_begin(d_img, (h, w), 6.0, 0.1)
        else:
            lat.set_point_grid((h, w))
            lat.build_begin(d_pos)
        lattices.append(lat)
        keep.append((d_val, d_img, d_pos))
    with pytest.raises(pla.PermutohedralError) as e:
        lattices[0].filter_end()           # a build is in flight, not a filter
    assert e.value.status == pla.PL_ESTATE
    with pytest.raises(pla.PermutohedralError) as e:
        lattices[0].apply(torch.empty((n, 3), device="cuda"), keep[0][0])
    assert e.value.status == pla.PL_ESTATE
    for lat in lattices:
        lat.build_end()
    lattices[0].build_end()                # nothing in flight: fine
    for lat, (d_val, _, _), (_, _, _, reverse, _, _, want) in zip(lattices, keep, cases):
        out = torch.empty((n, 3), dtype=torch.float32, device="cuda")
        lat.apply(out, d_val, reverse)
        torch.cuda.synchronize()
        close(out.cpu().numpy(), want)
        lat.apply(out, d_val, reverse)     # and again
        torch.cuda.synchronize()
        close(out.cpu().numpy(), want)


@pytest.mark.parametrize("batch", [1, 3, 6])
def test_op_results_do_not_depend_on_the_number_of_items_in_flight(batch):
    h, w = 72, 88
    guide = np.stack([synth.blob_image(h, w, seed=40 + i) for i in range(batch)])
    inp = synth.uniform_image((batch, h, w, 2), 47)
    want = oracle.lattice_filter(inp, guide, True, 8.0, 0.125, 1.0, False)
    try:
        for lanes in (1, 2, 4):
            pla.set_op_concurrency(lanes)
            got = pla.lattice_filter(dev(inp), dev(guide), theta_alpha=8.0, theta_beta=0.125)
            torch.cuda.synchronize()
            close(got.cpu().numpy(), want)
    finally:
        pla.set_op_concurrency(4)
    with pytest.raises(pla.PermutohedralError):
        pla.set_op_concurrency(0)


def test_op_on_a_side_stream_is_ordered_with_that_stream():
    h, w = 64, 64
    guide = np.stack([synth.blob_image(h, w, seed=50 + i) for i in range(3)])
    inp = synth.uniform_image((3, h, w, 1), 53)
    want = oracle.lattice_filter(inp, guide, True, 8.0, 0.125, 1.0, True)
    s = torch.cuda.Stream()
    d_inp, d_guide = dev(inp), dev(guide)
    torch.cuda.synchronize()
    with torch.cuda.stream(s):
        x = d_inp * 2.0                     # producer on the side stream
        y = pla._lattice_filter_raw(x, d_guide, True, 8.0, 0.125, 1.0, True)
        z = y * 0.5                         # consumer on the side stream
    s.synchronize()
    close(z.cpu().numpy(), want)


@pytest.mark.parametrize("points", ["grid", "list"])
def test_apply_can_be_captured_in_a_graph_and_replayed(points):
    """pl_apply only launches kernels on the lattice's stream (no allocation, no wait, no memset),
    so a caller may capture it in a HIP graph: the mean-field loop of a dense CRF replays the same
    splat/blur/slice sequence many times.  Every replay is checked against the eager result, with
    eager work and synchronisations in between.  (list: the points as a plain list, which the
    build puts in the order of space; the kernels of the apply then read that order.)"""
    h = w = 96
    n, vd = h * w, 6
    guide = synth.blob_image(h, w, seed=60) * 255.0
    pos = synth.bilateral_positions(guide, 40.0, 13.0)
    s = torch.cuda.Stream()
    lat = pla.PermutohedralLattice(5, vd, n, stream=s)
    d_pos = dev(pos)
    torch.cuda.synchronize()
    with torch.cuda.stream(s):
        if points == "grid":
            lat.set_point_grid((h, w))
        else:
            lat.set_option(pla.PL_OPT_GUESS_GRID, 0)
        lat.build(d_pos)
        assert lat.info(pla.PL_INFO_BUILD_MERGED) == 1
        static_in = torch.zeros((n, vd - 1), dtype=torch.float32, device="cuda")
        static_out = torch.zeros_like(static_in)
        lat.apply(static_out, static_in, False)      # warm-up outside the capture
    s.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=s):
        lat.apply(static_out, static_in, False)
    for seed in (61, 62, 63):
        val = synth.uniform_image((n, vd - 1), seed)
        want = oracle.Lattice(5, vd, n).filter(val, pos, False)
        static_in.copy_(dev(val))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        close(static_out.cpu().numpy(), want)
        eager = torch.empty_like(static_out)          # eager work between the replays
        with torch.cuda.stream(s):
            lat.apply(eager, static_in, True)
        s.synchronize()
        close(eager.cpu().numpy(), oracle.Lattice(5, vd, n).filter(val, pos, True))


def test_backward_reuses_the_lattices_of_forward():
    """With an input that needs a gradient the op keeps the lattices it built: backward is then a
    reversed apply under the same positions.  Same numbers as the op called twice; the lattices go
    back to the pool when the graph is freed, and past the pool's limit the op rebuilds."""
    import gc
    b, h, w = 3, 80, 72
    guide = np.stack([synth.blob_image(h, w, seed=70 + i) for i in range(b)])
    inp = synth.uniform_image((b, h, w, 2), 73)
    up = synth.normal_image(inp.shape, 74)
    want = oracle.lattice_filter(inp, guide, True, 8.0, 0.125, 1.0, False)
    want_grad = oracle.lattice_filter(up, guide, True, 8.0, 0.125, 1.0, True)
    d_guide = dev(guide)
    pool = pla._pool
    gc.collect()
    assert pool.lent == 0
    x = dev(inp).requires_grad_(True)
    y = pla.lattice_filter(x, d_guide, theta_alpha=8.0, theta_beta=0.125)
    assert pool.lent == b
    close(y.detach().cpu().numpy(), want)
    y.backward(dev(up), retain_graph=True)
    first = x.grad.clone()
    close(first.cpu().numpy(), want_grad, scale=float(np.abs(want_grad).max()))
    x.grad = None
    y.backward(dev(up))                      # a second backward over the retained graph
    close(x.grad.cpu().numpy(), want_grad, scale=float(np.abs(want_grad).max()))
    del y
    gc.collect()
    assert pool.lent == 0
    # more outputs alive than the pool lends lattices for: the rest are computed by the plain op
    alive = [pla.lattice_filter(dev(inp).requires_grad_(True), d_guide, theta_alpha=8.0, theta_beta=0.125)
             for _ in range(pool.max_lent // b + 2)]
    assert pool.lent <= pool.max_lent
    for y in alive:
        close(y.detach().cpu().numpy(), want)
    alive[-1].backward(dev(up))
    del alive, y
    gc.collect()
    assert pool.lent == 0
