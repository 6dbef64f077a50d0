"""Benchmark of the permutohedral-lattice filter on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--size 1024] [--no-cpu]

One step = the hot path over one synthetic image: a bilateral filter (pd=5, vd=4) of a
1024 x 1024 RGB image under itself as guide, forward then reverse (two filter() calls, each
building its lattice from the positions, as the reference's op does).  Inputs are resident in
HBM before the timed region.  Prints one JSON line.
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, vendor figure


def algorithmic_bytes(n, m, pd, vd):
    """Compulsory bytes of one filter() call, per kernel: positions, input and output streams once;
    vertex keys once; the vertex value table written by splat, read and written once per blur axis,
    read by slice.  Replay matrix, hash cells, neighbour table and clears are not counted."""
    return {
        "build": 4 * n * pd + 2 * pd * m,
        "splat": 4 * n * (vd - 1) + 4 * vd * m,
        "blur_axis": 2 * 4 * vd * m,
        "slice": 4 * vd * m + 4 * n * (vd - 1),
        "filter": 4 * n * (pd + 2 * (vd - 1)) + m * (2 * pd + 4 * vd * (2 * (pd + 1) + 2)),
    }


SETTLE_STEPS = 60   # untimed steps of the headline workload before its warm-up (see main)


def kernel_source_hash():
    """Short hash of the sources the HIP library is built from: what a counter measurement is
    stamped with, so that a figure taken from an older build shows as stale."""
    from permutohedral_lattice_amd.build import source_hash
    return source_hash()


def measured_traffic(kernel_name, grid_threads, stem="bench_bilateral_1024_pd5_vd4"):
    """HBM bytes per launch of a kernel (read + written) as rocprofv3's FETCH_SIZE / WRITE_SIZE gave
    them for this workload, scaled by the copy calibration; the summary under profiles/ holds the
    commands.  -> (bytes or None, stamp) where stamp says which build of the kernels the counters
    were taken on and whether that is the build running now."""
    path = os.path.join(ROOT, "profiles", stem + "_hbm_traffic.json")
    try:
        record = json.load(open(path))
        table = record["per_kernel_bytes"]
    except (OSError, ValueError, KeyError):
        return None, None
    now = kernel_source_hash()
    stamp = {"measured_on_sources": record.get("kernel_source_hash"), "running_sources": now,
             "stale": record.get("kernel_source_hash") != now}
    key = "%s@%d" % (kernel_name, grid_threads)
    if key not in table:
        return None, stamp
    return int(sum(table[key])), stamp


def kernel_names(pd, vd, in_channels=None, gathered=False):
    """The kernels a filter() call of a grid of points runs for these dimensions, by stage
    (gathered: an apply of a lattice that pl_build gave per-vertex lists)."""
    fused = vd <= 4
    d1 = pd + 1
    lanes = 4 if vd <= 16 else (8 if vd <= 32 else 16)
    if fused:
        blur = "k_blur3_row<%d, float>" % vd if pd == 2 else "k_blur2_row<%d, float>" % vd
        slice_k = "k_slice_point<%d, %d>" % (vd, d1)
    else:
        blur = "k_blur2_element<float>"
        if vd <= 8:
            slice_k = "k_slice_point<%d, 0>" % vd
        elif vd <= 64:
            slice_k = "k_slice_quads<%d, %d>" % (d1, lanes)
        else:
            slice_k = "k_slice_channels<%d>" % d1
    width = 16 if vd <= 16 else (32 if vd <= 32 else 64)
    if gathered:
        splat = ("k_splat_gather<%d, %d>" % (vd, in_channels if in_channels else vd - 1) if fused
                 else "k_splat_gather_channels<%d>" % lanes)
    else:
        splat = "k_splat_dpp<%d, %d>" % (vd, d1) if fused else "k_splat_channels<%d>" % width
    return {"build": "k_build_tile<%d, %d, float>" % (pd, vd if fused else 0),
            "splat": splat, "blur_axis": blur, "slice": slice_k}


def stage_report(lat, call, n, pd, vd, samples=5, fused_splat=True, gathered=False):
    """Per-stage milliseconds of `call()` (one filter or apply on `lat`) from HIP events on the
    lattice's stream, and the stage that takes longest with its share of the HBM roofline."""
    import permutohedral_lattice_amd as pla
    lat.set_option(pla.PL_OPT_PROFILE, 1)
    rows = []
    for _ in range(samples):
        call()
        rows.append(lat.stage_ms())
    lat.set_option(pla.PL_OPT_PROFILE, 0)
    stages = {k: statistics.mean(r[k] for r in rows) for k in rows[0]}
    stages["blur_axis"] = stages["blur"] / (pd + 1)
    m = lat.num_vertices
    alg = algorithmic_bytes(n, m, pd, vd)
    if vd <= 4 and fused_splat:
        alg["build"] += alg["splat"]      # filter() splats inside the build kernel
    names = kernel_names(pd, vd, gathered=gathered)
    candidates = [k for k in ("build", "splat", "slice") if stages[k] > 0.0]
    dominant = max(candidates, key=lambda k: stages[k])
    if stages["blur"] > stages[dominant]:
        dominant = "blur_axis"
    gbs = alg[dominant] / (stages[dominant] * 1e-3) / 1e9
    return stages, {"kernel": names[dominant], "launch_ms": round(stages[dominant], 5),
                    "algorithmic_bytes_per_launch": alg[dominant], "achieved_GBs": round(gbs, 1),
                    "frac": round(gbs / HBM_PEAK_GBS, 5)}


def parity(got, want):
    import numpy as np
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return {"max_abs": float(np.abs(got - want).max()),
            "rel_l2": float(np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-30))}


def timed(fn, warmup, reps):
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / reps


def run_configs(args, pla, synth, with_cpu):
    """Every BASELINE configuration at its full size: time per filter() call (what one call moves
    against the HBM roofline), the kernel that takes longest with its own roofline share, and the
    outputs against the CPU reference on the same arrays."""
    import numpy as np
    import torch
    from permutohedral_lattice_amd.crf import MeanField
    cpu = None
    if with_cpu:
        import oracle
        cpu = oracle.reference()
    out = {}

    def dev(a):
        return torch.from_numpy(np.ascontiguousarray(a)).cuda()

    # Parity is taken against the oracle with one vertex per distinct key, which is what the library
    # builds.  The reference's own header enters a key a second time at some doublings of its hash
    # index (its lookup starts from a cell computed before the growth); those few vertices split
    # their values, and under a normalisation by small weights the outputs around them move by more
    # than the tolerance.  The figures against the reference's build are printed beside, as they are.
    def both(got, port, ref_out):
        rec = {"parity_vs_cpu": port(got)}
        if ref_out is not None:
            rec["against_reference_build_with_its_duplicate_vertices"] = ref_out(got)
        return rec

    # cfg5: dense-CRF mean field, 512 x 512, batch 2, 21 classes, five iterations + reverse pass
    # (timed before any CPU leg of this function: its step is a chain of some 250 short launches
    # that the host barely keeps ahead of, and the host side of this process is slower once the
    # CPU reference has run in it -- 2.0 against 2.2 ms per step)
    batch5, side5, classes = 2, 512, 21
    guide5 = np.stack([synth.blob_image(side5, side5, seed=0xC0FFEE + 50 + b) * 255.0
                      for b in range(batch5)]).astype(np.float32)
    logits = synth.normal_image((batch5, side5, side5, classes), 0xC0FFEE + 5)
    upstream = synth.normal_image((batch5, side5, side5, classes), 0xC0FFEE + 6)
    d_guide5, d_logits, d_up = dev(guide5), dev(logits), dev(upstream)
    mf = MeanField(d_guide5, classes)
    res5 = {}

    def cfg5_step():
        mf.rebuild(d_guide5)                       # four builds: two lattices per item
        res5["q"] = mf.infer(d_logits, 5)          # 20 applies
        res5["rev"] = mf.reverse(d_up)             # 4 reversed applies

    seconds5 = timed(cfg5_step, 3, 8)
    n5 = side5 * side5
    calls = batch5 * 2 * 6
    m_bi, m_sp = mf.bilateral[0].num_vertices, mf.spatial[0].num_vertices
    q0 = torch.softmax(d_logits[0].view(n5, classes), dim=-1)
    msg = torch.empty_like(q0)
    torch.cuda.synchronize()      # (the lattices work on streams of their own)
    st_bi, dom_bi = stage_report(mf.bilateral[0], lambda: mf.bilateral[0].apply(msg, q0, False), n5, 5,
                                 classes + 1, fused_splat=False, gathered=True)
    st_sp, dom_sp = stage_report(mf.spatial[0], lambda: mf.spatial[0].apply(msg, q0, False), n5, 2,
                                 classes + 1, fused_splat=False, gathered=True)
    # an apply moves what a filter moves less the positions and the keys (the lattice is there)
    def apply_bytes(m, pd, vd):
        return 4 * n5 * 2 * (vd - 1) + m * 4 * vd * (2 * (pd + 1) + 2)
    alg5 = batch5 * 6 * (apply_bytes(m_bi, 5, classes + 1) + apply_bytes(m_sp, 2, classes + 1))
    rec5 = {"workload": "dense-CRF mean field, 512x512, batch 2, 21 classes (vd=22): five iterations of "
                       "softmax(logits + bilateral(Q; 80, 13) + spatial(Q; 3)) and the reverse pass of both "
                       "filters on an N(0,1) upstream; two lattices per item built once per step (4 builds), "
                       "24 applies",
           "points": n5 * batch5, "num_vertices_item0": {"bilateral_pd5": m_bi, "spatial_pd2": m_sp},
           "ms_per_step": round(seconds5 * 1e3, 4), "filter_calls_per_step": calls,
           "us_per_filter": round(seconds5 * 1e6 / calls, 1),
           "Mpoints_per_s": round(calls * n5 / seconds5 / 1e6, 1),
           "algorithmic_bytes_per_step": alg5,
           "frac_of_hbm_peak": round(alg5 / seconds5 / 1e9 / HBM_PEAK_GBS, 5),
           "dominant_kernel": {"bilateral_apply": dom_bi, "spatial_apply": dom_sp},
           "stage_ms": {"bilateral_apply": {k: round(v, 5) for k, v in st_bi.items()},
                        "spatial_apply": {k: round(v, 5) for k, v in st_sp.items()}}}

    def one_filter(name, what, pd, vd, grid, pos, val, reps):
        n = pos.shape[0]
        lat = pla.PermutohedralLattice(pd, vd, n)
        lat.set_point_grid(grid)
        d_pos, d_val = dev(pos), dev(val)
        d_out = torch.empty_like(d_val)
        seconds = timed(lambda: lat.filter(d_out, d_val, d_pos, False), 3 if n < (1 << 22) else 1, reps)
        m = lat.num_vertices
        stages, dominant = stage_report(lat, lambda: lat.filter(d_out, d_val, d_pos, False), n, pd, vd,
                                        samples=5 if n < (1 << 22) else 3)
        alg = algorithmic_bytes(n, m, pd, vd)["filter"]
        rec = {"workload": what, "points": n, "pd": pd, "vd": vd, "num_vertices": m,
               "us_per_filter": round(seconds * 1e6, 1), "Mpoints_per_s": round(n / seconds / 1e6, 1),
               "algorithmic_bytes_per_filter": alg,
               "frac_of_hbm_peak": round(alg / seconds / 1e9 / HBM_PEAK_GBS, 5),
               "merged_tiles": bool(lat.info(pla.PL_INFO_BUILD_MERGED)),
               "dominant_kernel": dominant,
               "stage_ms": {k: round(v, 5) for k, v in stages.items()}}
        if with_cpu:
            lat.filter(d_out, d_val, d_pos, False)
            torch.cuda.synchronize()
            got = d_out.cpu().numpy()
            t0 = time.perf_counter()
            want = oracle.Lattice(pd, vd, n).filter(val, pos, False)
            rec["cpu_seconds_per_filter"] = round(time.perf_counter() - t0, 4)
            rec.update(both(got, lambda g: parity(g, want),
                            (lambda g: parity(g, cpu.filter(pd, vd, val, pos, False)[0])) if cpu else None))
        lat.close()
        out[name] = rec

    # cfg1: 512 x 512 RGB bilateral
    img = synth.blob_image(512, 512, seed=0xC0FFEE + 1)
    one_filter("cfg1", "bilateral RGB 512x512, pd=5 vd=4, theta 8/0.125, one filter() forward", 5, 4,
               (512, 512), synth.bilateral_positions(img, 8.0, 0.125), img.reshape(-1, 3), 20)
    # cfg2: 1024 x 1024 spatial-only Gaussian
    one_filter("cfg2", "spatial-only 1024x1024 grey, pd=2 vd=2, theta 8, one filter() forward", 2, 2,
               (1024, 1024), synth.spatial_positions((1024, 1024), 8.0),
               synth.uniform_image((1 << 20, 1), 0xC0FFEE + 2), 20)

    # cfg3: batch 4 grey under an RGB guide, forward + reverse, through the op
    batch, side = 4, 1024
    guide = np.stack([synth.blob_image(side, side, seed=0xC0FFEE + 30 + i) for i in range(batch)])
    inp = synth.uniform_image((batch, side, side, 1), 0xC0FFEE + 3)
    grad = synth.normal_image((batch, side, side, 1), 0xC0FFEE + 4)
    d_guide, d_inp, d_grad = dev(guide), dev(inp), dev(grad)
    res = {}

    def cfg3_step():
        res["f"] = pla._lattice_filter_raw(d_inp, d_guide, True, 8.0, 0.125, 1.0, False)
        res["r"] = pla._lattice_filter_raw(d_grad, d_guide, True, 8.0, 0.125, 1.0, True)

    seconds = timed(cfg3_step, 2, 5)
    n = side * side
    lat = pla.PermutohedralLattice(5, 2, n)
    d_out1 = torch.empty((n, 1), dtype=torch.float32, device="cuda")
    call = lambda: lat.filter_image(d_out1, d_inp[0].view(n, 1), d_guide[0].view(n, 3), (side, side), 8.0, 0.125)
    call()
    m = lat.num_vertices
    stages, dominant = stage_report(lat, call, n, 5, 2)
    # the op builds its features inside the first kernel: the reference image is read, not positions
    alg = 4 * n * (3 + 2) + m * (2 * 5 + 4 * 2 * (2 * 6 + 2))
    rec = {"workload": "greyscale under an RGB guide, batch 4, 1024x1024, pd=5 vd=2, theta 8/0.125: the op "
                       "forward on the input, then reverse on an N(0,1) upstream gradient (8 filters per step)",
           "points": n * batch, "pd": 5, "vd": 2, "num_vertices_item0": m,
           "ms_per_step": round(seconds * 1e3, 4), "us_per_filter": round(seconds * 1e6 / (2 * batch), 1),
           "Mpoints_per_s": round(2 * batch * n / seconds / 1e6, 1),
           "algorithmic_bytes_per_filter": alg,
           "frac_of_hbm_peak": round(2 * batch * alg / seconds / 1e9 / HBM_PEAK_GBS, 5),
           "dominant_kernel": dominant, "stage_ms": {k: round(v, 5) for k, v in stages.items()}}
    lat.close()
    if with_cpu:
        cfg3_step()
        torch.cuda.synchronize()
        got_f, got_r = res["f"].cpu().numpy(), res["r"].cpu().numpy()

        def against(op):
            return {"forward": parity(got_f, op(inp, guide, True, 8.0, 0.125, 1.0, False)),
                    "reverse": parity(got_r, op(grad, guide, True, 8.0, 0.125, 1.0, True))}

        t0 = time.perf_counter()
        rec["parity_vs_cpu"] = against(oracle.lattice_filter)
        rec["cpu_seconds_per_step"] = round(time.perf_counter() - t0, 3)
        if cpu is not None:
            rec["against_reference_build_with_its_duplicate_vertices"] = against(cpu.lattice_filter)
    out["cfg3"] = rec
    del d_guide, d_inp, d_grad, res

    # cfg4: 128 x 256 x 256 volume
    vol = synth.ellipsoid_volume(128, 256, 256, seed=0xC0FFEE + 4)
    one_filter("cfg4", "volumetric bilateral 128x256x256, pd=4 vd=2, theta 5/0.1, one filter() forward", 4, 2,
               (128, 256, 256), synth.bilateral_positions(vol, 5.0, 0.1), vol.reshape(-1, 1), 3)
    del vol

    # cfg5 (timed first, see above): its outputs against the CPU
    rec = rec5
    if with_cpu:
        cfg5_step()
        torch.cuda.synchronize()
        got_q, got_rev = res5["q"].cpu().numpy(), res5["rev"].cpu().numpy()

        def against(op):
            want_q, want_rev = oracle.mean_field(logits, guide5, 5, upstream=upstream, op=op)
            return {"Q": parity(got_q, want_q), "reverse": parity(got_rev, want_rev)}

        t0 = time.perf_counter()
        rec["parity_vs_cpu"] = against(None)
        rec["cpu_seconds_per_step"] = round(time.perf_counter() - t0, 3)
        if cpu is not None:
            rec["against_reference_build_with_its_duplicate_vertices"] = against(cpu.lattice_filter)
    mf.close()
    out["cfg5"] = rec
    return out


def run_real_image(args, pla, with_cpu):
    """The reference's own 800 x 1200 photograph (Images/input.bmp of the reference tree, kept as a
    test fixture), theta 8/0.125 as its tests filter it: what an image that is not smooth costs and
    whether the build that merges tiles in LDS holds on it."""
    import numpy as np
    import torch
    path = os.path.join(ROOT, "tests", "golden", "reference_images.npz")
    if not os.path.exists(path):
        return None
    rgb = (np.load(path)["input"].astype(np.float32) / np.float32(255.0))
    h, w = rgb.shape[:2]
    n = h * w
    d_img = torch.from_numpy(np.ascontiguousarray(rgb.reshape(n, 3))).cuda()
    d_out = torch.empty_like(d_img)
    lat = pla.PermutohedralLattice(5, 4, n)
    call = lambda: lat.filter_image(d_out, d_img, d_img, (h, w), 8.0, 0.125, False)
    seconds = timed(call, 3, 20)
    m = lat.num_vertices
    stages, dominant = stage_report(lat, call, n, 5, 4)
    alg = 4 * n * (3 + 2 * 3) + m * (2 * 5 + 4 * 4 * (2 * 6 + 2))
    rec = {"workload": "the reference's 800x1200 photograph under itself, pd=5 vd=4, theta 8/0.125, "
                       "filter_image() forward", "points": n, "num_vertices": m,
           "us_per_filter": round(seconds * 1e6, 1), "Mpoints_per_s": round(n / seconds / 1e6, 1),
           "merged_tiles": bool(lat.info(pla.PL_INFO_BUILD_MERGED)),
           "algorithmic_bytes_per_filter": alg,
           "frac_of_hbm_peak": round(alg / seconds / 1e9 / HBM_PEAK_GBS, 5),
           "dominant_kernel": dominant, "stage_ms": {k: round(v, 5) for k, v in stages.items()}}
    if with_cpu:
        import oracle
        cpu = oracle.reference()
        call()
        torch.cuda.synchronize()
        got = d_out.cpu().numpy().reshape((1,) + rgb.shape)
        rec["parity_vs_cpu"] = parity(got, oracle.lattice_filter(rgb[None], rgb[None], True, 8.0, 0.125, 1.0, False))
        if cpu is not None:
            rec["against_reference_build_with_its_duplicate_vertices"] = parity(
                got, cpu.lattice_filter(rgb[None], rgb[None], True, 8.0, 0.125, 1.0, False))
    lat.close()
    return rec



def run_plain_legs(args, pla, lat, d_pos, d_val, d_grad, out_f, out_r):
    """The headline step on handles that were given no grid -> {leg: ms per step}"""
    import torch

    # the same without the grid hint (a caller of filter() that only has N points): once with the
    # library left to find the image in the positions, once with the points as a plain list
    # (and the plain list with its points in no order at all, and that list taken in the order it
    # comes in instead of the order of space the library puts it in)
    plain = {}
    shuffle = torch.randperm(lat.N, device="cuda", generator=torch.Generator("cuda").manual_seed(5))
    s_pos, s_val, s_grad = (t[shuffle].contiguous() for t in (d_pos, d_val, d_grad))
    for name, guess, ordered, (l_pos, l_val, l_grad) in (
            ("grid_found_by_the_library", 1, 1, (d_pos, d_val, d_grad)),
            ("plain_list", 0, 1, (d_pos, d_val, d_grad)),
            ("plain_list_shuffled", 0, 1, (s_pos, s_val, s_grad)),
            ("plain_list_shuffled_in_list_order", 0, 0, (s_pos, s_val, s_grad))):
        if args.plain_legs and name not in args.plain_legs.split(","):
            continue
        other = pla.PermutohedralLattice(lat.pd, lat.vd, lat.N)
        other.set_option(pla.PL_OPT_GUESS_GRID, guess)
        other.set_option(pla.PL_OPT_ORDER_POINTS, ordered)

        def other_step():
            other.filter(out_f, l_val, l_pos, False)
            other.filter(out_r, l_grad, l_pos, True)

        for _ in range(2):
            other_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            other_step()
        torch.cuda.synchronize()
        plain[name] = 1e3 * (time.perf_counter() - t0) / args.steps
        other.close()
    return plain


def run_reuse_leg(args, pla, lat, d_pos, d_val, d_grad, out_f, out_r):
    """Build once, apply forward and reverse (what a caller that keeps the lattice gets): with the
    per-vertex lists pl_build writes (the applies splat by gathering) and without them (the applies
    splat as filter() does).  -> {mode: {build_ms, ms_per_step}}"""
    import torch
    out = {}
    for name, lists in (("without_vertex_lists", 0), ("with_vertex_lists", 1)):
        lat.set_option(pla.PL_OPT_VERTEX_LISTS, lists)
        for _ in range(2):
            lat.build(d_pos)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(5):
            lat.build(d_pos)
        torch.cuda.synchronize()
        build_ms = 1e3 * (time.perf_counter() - t0) / 5
        for _ in range(2):
            lat.apply(out_f, d_val, False)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            lat.apply(out_f, d_val, False)
            lat.apply(out_r, d_grad, True)
        torch.cuda.synchronize()
        out[name] = {"build_ms": round(build_ms, 4),
                     "ms_per_step": round(1e3 * (time.perf_counter() - t0) / args.steps, 4)}
    return out


def run_side_legs(args, pla, synth, lat, step, img, d_pos, d_val, d_grad, out_f, out_r, side, batch):
    """The legs beside the headline: no grid hint, lattice reuse, the op's boundary, a batch."""
    import numpy as np
    import torch

    plain_ms = run_plain_legs(args, pla, lat, d_pos, d_val, d_grad, out_f, out_r)

    reuse = run_reuse_leg(args, pla, lat, d_pos, d_val, d_grad, out_f, out_r)

    # the op's boundary: the reference image comes in, not a positions array.  First as the
    # reference does it (feature kernel, then filter), then with the features built on the fly.
    d_img = torch.from_numpy(np.ascontiguousarray(img.reshape(-1, 3))).cuda()
    d_pos2 = torch.empty_like(d_pos)

    def op_step_two_kernels():
        for o, v, rev in ((out_f, d_val, False), (out_r, d_grad, True)):
            pla.compute_positions(d_img, (side, side), 8.0, 0.125, out=d_pos2)
            lat.filter(o, v, d_pos2, rev)

    def op_step_fused():
        for o, v, rev in ((out_f, d_val, False), (out_r, d_grad, True)):
            lat.filter_image(o, v, d_img, (side, side), 8.0, 0.125, rev)

    # through the autograd function: backward applies the lattices forward built
    x4 = d_val.view(1, side, side, 3).clone().requires_grad_(True)
    ref4 = d_img.view(1, side, side, 3)
    up4 = d_grad.view(1, side, side, 3)

    def op_step_autograd():
        y = pla.lattice_filter(x4, ref4, theta_alpha=8.0, theta_beta=0.125)
        y.backward(up4)
        x4.grad = None

    op_ms = {}
    for name, fn in (("positions_then_filter", op_step_two_kernels), ("features_on_the_fly", op_step_fused),
                     ("autograd_forward_backward", op_step_autograd)):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        op_ms[name] = 1e3 * (time.perf_counter() - t0) / args.steps

    # a batch through the op: four images, forward then reverse, one item at a time as the
    # reference's loop runs them, and with the items spread over concurrent lattices
    b_img = torch.from_numpy(np.stack([synth.blob_image(side, side, seed=0xC0FFEE + 10 + i)
                                       for i in range(batch)])).cuda()
    b_grad = torch.from_numpy(synth.normal_image((batch, side, side, 3), 0xC0FFEE + 20)).cuda()
    batch_ms = {}
    for lanes in (1, 4):
        pla.set_op_concurrency(lanes)
        for _ in range(2):
            pla._lattice_filter_raw(b_img, b_img, True, 8.0, 0.125, 1.0, False)
        torch.cuda.synchronize()
        reps = max(3, args.steps // 5)
        t0 = time.perf_counter()
        for _ in range(reps):
            pla._lattice_filter_raw(b_img, b_img, True, 8.0, 0.125, 1.0, False)
            pla._lattice_filter_raw(b_grad, b_img, True, 8.0, 0.125, 1.0, True)
        torch.cuda.synchronize()
        batch_ms["%d_at_a_time" % lanes] = 1e3 * (time.perf_counter() - t0) / reps
    pla.set_op_concurrency(4)
    del b_img, b_grad

    # the same step on a lattice of doubles (the reference's T = double), grid hint set
    lat64 = pla.PermutohedralLattice(lat.pd, lat.vd, lat.N, dtype=torch.float64)
    lat64.set_point_grid((side, side))
    pos64, val64, grad64 = d_pos.double(), d_val.double(), d_grad.double()
    out64 = torch.empty_like(val64)

    def step64():
        lat64.filter(out64, val64, pos64, False)
        lat64.filter(out64, grad64, pos64, True)

    for _ in range(2):
        step64()
    torch.cuda.synchronize()
    reps = max(3, args.steps // 5)
    t0 = time.perf_counter()
    for _ in range(reps):
        step64()
    torch.cuda.synchronize()
    double_ms = 1e3 * (time.perf_counter() - t0) / reps
    lat64.close()

    return plain_ms, reuse, op_ms, batch_ms, double_ms


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--size", type=int, default=1024, help="image side (default 1024)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline and parity legs")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the leg that runs every BASELINE configuration at full size")
    ap.add_argument("--headline-only", action="store_true",
                    help="only the timed steps and the per-stage timing (what a rocprofv3 run of "
                         "this file should see): no side legs, no CPU baseline")
    ap.add_argument("--plain-only", action="store_true",
                    help="only the legs without a grid hint (for profiling the ordering of plain lists)")
    ap.add_argument("--plain-legs", default="",
                    help="with --plain-only: the legs to run, comma-separated (default: all)")
    ap.add_argument("--reuse-only", action="store_true",
                    help="only the timed steps and the build-once / apply-many leg (for profiling the "
                         "kernels of pl_build's lists and of pl_apply)")
    ap.add_argument("--configs-only", action="store_true",
                    help="only the leg that runs every BASELINE configuration at full size, without "
                         "the CPU reference (what a rocprofv3 run for the kernels of those "
                         "configurations should see); prints that leg's record")
    ap.add_argument("--calibrate-copy-mib", type=int, default=0,
                    help="only run device-to-device copies of this many MiB (a kernel of known "
                         "traffic, for scaling rocprofv3's FETCH_SIZE / WRITE_SIZE) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (got --gpus %d); there is no "
                 "multi-GPU path to measure" % args.gpus)

    import numpy as np
    import torch

    import permutohedral_lattice_amd as pla
    from permutohedral_lattice_amd import synth

    torch.cuda.set_device(0)
    if args.calibrate_copy_mib:
        nbytes = args.calibrate_copy_mib << 20
        src = torch.arange(nbytes // 4, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "5 x dst.copy_(src), float32", "bytes_read_per_copy": nbytes,
                          "bytes_written_per_copy": nbytes}))
        return
    if args.configs_only:
        print(json.dumps({"configs": run_configs(args, pla, synth, False)}))
        return
    side = args.size
    n, pd, vd = side * side, 5, 4
    img = synth.blob_image(side, side, seed=0xC0FFEE)
    pos = synth.bilateral_positions(img, 8.0, 0.125)
    val = img.reshape(-1, 3)
    grad = synth.normal_image((n, 3), 0xC0FFEE + 1)  # upstream gradient of the reverse pass

    d_pos = torch.from_numpy(pos).cuda()
    d_val = torch.from_numpy(val).cuda()
    d_grad = torch.from_numpy(grad).cuda()
    out_f = torch.empty_like(d_val)
    out_r = torch.empty_like(d_val)
    lat = pla.PermutohedralLattice(pd, vd, n)
    # what the op passes along with its tensors: the points are a side x side row-major grid
    lat.set_point_grid((side, side))

    def step():
        lat.filter(out_f, d_val, d_pos, False)
        lat.filter(out_r, d_grad, d_pos, True)

    # Before the warm-up steps asked for: the lattice's first calls size its hash table, and the GPU
    # takes some milliseconds of work to reach its clocks (steps timed right after three warm-up
    # steps read 3 % slower than steps timed after fifty).  Untimed, like the warm-up.
    for _ in range(SETTLE_STEPS):
        step()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    seconds = time.perf_counter() - t0
    ms_per_step = 1e3 * seconds / args.steps
    m = lat.num_vertices
    pixels_per_step = 2 * n
    value = pixels_per_step / (ms_per_step * 1e-3) / 1e6

    if args.plain_only:
        plain = run_plain_legs(args, pla, lat, d_pos, d_val, d_grad, out_f, out_r)
        print(json.dumps({"no_grid_hint_ms_per_step": {k: round(v, 4) for k, v in plain.items()}}))
        return
    side_legs = not args.headline_only
    # The legs beside the headline drive entry points whose kernels hand arrays to each other in
    # layouts this file's helpers assume; a library built from other sources than the ones in the
    # tree (an experiment left in place) gets the headline only.
    library_sources, tree_sources = pla.library_source_hash(), kernel_source_hash()
    side_legs_refused = side_legs and library_sources != tree_sources
    if side_legs_refused:
        side_legs = False
        print("bench.py: the loaded library was built from sources %s, the tree holds %s: headline "
              "only; rebuild with `python permutohedral_lattice_amd/build.py`"
              % (library_sources, tree_sources), file=sys.stderr)
    plain_ms, reuse, double_ms = {}, {}, 0.0
    op_ms, batch_ms, batch = {}, {}, 4
    if args.reuse_only:
        print(json.dumps({"reuse": run_reuse_leg(args, pla, lat, d_pos, d_val, d_grad, out_f, out_r)}))
        return
    if side_legs:
        plain_ms, reuse, op_ms, batch_ms, double_ms = run_side_legs(args, pla, synth, lat, step, img, d_pos,
                                                            d_val, d_grad, out_f, out_r, side, batch)

    # per-kernel durations from HIP events on the lattice's stream
    lat.set_option(pla.PL_OPT_PROFILE, 1)
    stage_samples = []
    for _ in range(max(5, min(20, args.steps))):
        for o, v, rev in ((out_f, d_val, False), (out_r, d_grad, True)):
            lat.filter(o, v, d_pos, rev)
            stage_samples.append(lat.stage_ms())
    lat.set_option(pla.PL_OPT_PROFILE, 0)
    stages = {k: statistics.mean(s[k] for s in stage_samples) for k in stage_samples[0]}
    stages["blur_axis"] = stages["blur"] / (pd + 1)

    alg = algorithmic_bytes(n, m, pd, vd)
    # for vd <= 4 filter() splats inside the build kernel: that launch then carries both shares
    fused = vd <= 4
    if fused:
        alg["build"] += alg["splat"]
    per_launch_ms = {k: stages[k] for k in ("build", "splat", "blur_axis", "slice")}
    candidates = ("build", "slice") if fused else ("build", "splat", "slice")
    dominant = max(candidates, key=lambda k: stages[k])
    if stages["blur"] > stages[dominant]:
        dominant = "blur_axis"
    achieved = alg[dominant] / (per_launch_ms[dominant] * 1e-3) / 1e9
    kernel_name = {"build": "k_build_tile<5, 4, float>" if fused else "k_build_tile<5, 0, float>", "splat": "k_splat_dpp<4, 6>",
                   "blur_axis": "k_blur2_row<4, float>", "slice": "k_slice_point<4, 6>"}[dominant]
    traffic, traffic_stamp = measured_traffic(kernel_name, n)
    roofline = {"bound": "hbm", "kernel": kernel_name, "achieved": round(achieved, 2),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 5),
                "traffic": traffic, "traffic_from": traffic_stamp,
                "algorithmic_bytes_per_launch": alg[dominant],
                "launch_ms": round(per_launch_ms[dominant], 5)}
    gpu_kernel_ms = sum(stages[k] for k in ("clear", "build", "ids", "neighbours", "fill", "splat",
                                            "blur", "slice"))
    filter_gbs = 2 * alg["filter"] / (ms_per_step * 1e-3) / 1e9

    result = {
        "metric": "Mpixels/sec, bilateral pd=5 vd=4 on 1 MI355X; % of HBM peak; CPU baseline",
        "value": round(value, 3), "unit": "Mpixels/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "settle_steps": SETTLE_STEPS, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "bilateral RGB %dx%d, pd=5 vd=4, theta 8/0.125, filter() forward + "
                               "filter() reverse per step, positions given, grid hint set as the "
                               "op sets it" % (side, side),
                   "pixels_per_step": pixels_per_step, "num_vertices": m},
        "roofline": roofline,
        "filter_roofline": {"algorithmic_bytes_per_step": 2 * alg["filter"],
                            "achieved": round(filter_gbs, 2), "unit": "GB/s",
                            "frac": round(filter_gbs / HBM_PEAK_GBS, 5)},
        "stage_ms": {k: round(v, 5) for k, v in stages.items()},
        "kernel_ms_per_filter": round(gpu_kernel_ms, 4),
        "library_sources": library_sources,
    }
    if side_legs_refused:
        result["side_legs_refused"] = "library built from sources %s, tree holds %s" % (
            library_sources, tree_sources)
    if side_legs:
        result.update({
            "no_grid_hint": {"what": "same step on a handle that was given no grid",
                             "ms_per_step": {k: round(v, 4) for k, v in plain_ms.items()},
                             "value": {k: round(pixels_per_step / (v * 1e-3) / 1e6, 3)
                                       for k, v in plain_ms.items()}},
            "reuse": {"what": "build once (build_ms), apply forward + reverse per step: with the per-vertex "
                              "lists pl_build writes, so that an apply splats by gathering, and without",
                      "ms_per_step": reuse["with_vertex_lists"]["ms_per_step"],
                      "value": round(pixels_per_step / (reuse["with_vertex_lists"]["ms_per_step"] * 1e-3) / 1e6, 3),
                      "modes": reuse},
            "op_level": {"what": "reference image in, forward + reverse per step: feature kernel + "
                                 "filter(), filter_image() (features built inside the first kernel), and "
                                 "lattice_filter(...).backward(...) (backward applies forward's lattice)",
                         "ms_per_step": {k: round(v, 4) for k, v in op_ms.items()},
                         "value": {k: round(pixels_per_step / (v * 1e-3) / 1e6, 3)
                                   for k, v in op_ms.items()}},
            "op_batch": {"what": "the op on a batch of %d such images, forward + reverse per step, "
                                 "items one at a time, and with the op's concurrency set to four (of items this "
                                 "large it then runs two at a time)" % batch,
                         "ms_per_step": {k: round(v, 4) for k, v in batch_ms.items()},
                         "value": {k: round(batch * pixels_per_step / (v * 1e-3) / 1e6, 3)
                                   for k, v in batch_ms.items()}},
            "double": {"what": "same step on a lattice of doubles (the reference's T = double)",
                       "ms_per_step": round(double_ms, 4),
                       "value": round(pixels_per_step / (double_ms * 1e-3) / 1e6, 3)},
        })

    if side_legs and not args.no_configs:
        result["configs"] = run_configs(args, pla, synth, not args.no_cpu)
        result["real_image"] = run_real_image(args, pla, not args.no_cpu)

    if not args.no_cpu and not args.headline_only and not side_legs_refused:
        import oracle
        ref = oracle.reference()
        cores = 1
        times, outs = [], None
        reps = 9 if n >= (1 << 20) else 15
        for rep in range(reps + 1):  # first repetition is the warm-up
            t0 = time.perf_counter()
            if ref is not None:
                o_f = ref.filter(pd, vd, val, pos, False)[0]
                o_r = ref.filter(pd, vd, grad, pos, True)[0]
            else:
                o_f = oracle.Lattice(pd, vd, n, reference_growth_quirk=True).filter(val, pos, False)
                o_r = oracle.Lattice(pd, vd, n, reference_growth_quirk=True).filter(grad, pos, True)
            dt = time.perf_counter() - t0
            if rep:
                times.append(dt)
            outs = (o_f, o_r)
        cpu_s = statistics.median(times)
        result["cpu_baseline"] = {
            "value": round(pixels_per_step / cpu_s / 1e6, 4), "unit": "Mpixels/s", "cores": cores,
            "kind": "reference" if ref is not None else "port",
            "sample": "the whole step (forward + reverse of the same %dx%d arrays), median of %d "
                      "after one warm-up" % (side, side, reps),
            "seconds_per_step": round(cpu_s, 4), "host_cpus": os.cpu_count()}
        lat.filter(out_f, d_val, d_pos, False)
        lat.filter(out_r, d_grad, d_pos, True)
        torch.cuda.synchronize()
        got_f, got_r = out_f.cpu().numpy(), out_r.cpu().numpy()
        result["parity_vs_cpu"] = {
            "forward": parity(got_f, oracle.Lattice(pd, vd, n).filter(val, pos, False)),
            "reverse": parity(got_r, oracle.Lattice(pd, vd, n).filter(grad, pos, True))}
        if ref is not None:
            result["against_reference_build_with_its_duplicate_vertices"] = {
                "forward": parity(got_f, outs[0]), "reverse": parity(got_r, outs[1])}

    print(json.dumps(result))


if __name__ == "__main__":
    main()
