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


def measured_traffic(kernel_name, side):
    """HBM bytes per launch of a kernel (read + written) as rocprofv3's FETCH_SIZE / WRITE_SIZE gave
    them for this workload, scaled by the copy calibration; the summary under profiles/ holds the
    commands.  None when there is no measurement for this kernel and size."""
    path = os.path.join(ROOT, "profiles", "bench_bilateral_%d_pd5_vd4_hbm_traffic.json" % side)
    try:
        table = json.load(open(path))["per_kernel_bytes"]
    except (OSError, ValueError, KeyError):
        return None
    key = "%s@%d" % (kernel_name, side * side)
    if key not in table:
        return None
    return int(sum(table[key]))


def run_side_legs(args, pla, synth, lat, step, img, d_pos, d_val, d_grad, out_f, out_r, side, batch):
    """The legs beside the headline: no grid hint, lattice reuse, the op's boundary, a batch."""
    import numpy as np
    import torch

    # the same without the grid hint (a caller of filter() that only has N points): once with the
    # library left to find the image in the positions, once with the points as a plain list
    plain = {}
    for name, guess in (("grid_found_by_the_library", 1), ("plain_list", 0)):
        other = pla.PermutohedralLattice(lat.pd, lat.vd, lat.N)
        other.set_option(pla.PL_OPT_GUESS_GRID, guess)

        def other_step():
            other.filter(out_f, d_val, d_pos, False)
            other.filter(out_r, d_grad, d_pos, True)

        for _ in range(2):
            other_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            other_step()
        torch.cuda.synchronize()
        plain[name] = 1e3 * (time.perf_counter() - t0) / args.steps
        other.close()
    plain_ms = plain

    # build once, apply forward and reverse (what a caller that keeps the lattice gets)
    lat.build(d_pos)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        lat.apply(out_f, d_val, False)
        lat.apply(out_r, d_grad, True)
    torch.cuda.synchronize()
    reuse_ms = 1e3 * (time.perf_counter() - t0) / args.steps

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

    return plain_ms, reuse_ms, op_ms, batch_ms, double_ms


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--size", type=int, default=1024, help="image side (default 1024)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline and parity legs")
    ap.add_argument("--headline-only", action="store_true",
                    help="only the timed steps and the per-stage timing (what a rocprofv3 run of "
                         "this file should see): no side legs, no CPU baseline")
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

    side_legs = not args.headline_only
    plain_ms, reuse_ms, double_ms = {}, 0.0, 0.0
    op_ms, batch_ms, batch = {}, {}, 4
    if side_legs:
        plain_ms, reuse_ms, op_ms, batch_ms, double_ms = run_side_legs(args, pla, synth, lat, step, img, d_pos,
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
    roofline = {"bound": "hbm", "kernel": kernel_name, "achieved": round(achieved, 2),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 5),
                "traffic": measured_traffic(kernel_name, side),
                "algorithmic_bytes_per_launch": alg[dominant],
                "launch_ms": round(per_launch_ms[dominant], 5)}
    gpu_kernel_ms = sum(stages[k] for k in ("clear", "build", "ids", "neighbours", "fill", "splat",
                                            "blur", "slice"))
    filter_gbs = 2 * alg["filter"] / (ms_per_step * 1e-3) / 1e9

    result = {
        "metric": "Mpixels/sec, bilateral pd=5 vd=4 on 1 MI355X; % of HBM peak; CPU baseline",
        "value": round(value, 3), "unit": "Mpixels/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
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
    }
    if side_legs:
        result.update({
            "no_grid_hint": {"what": "same step on a handle that was given no grid",
                             "ms_per_step": {k: round(v, 4) for k, v in plain_ms.items()},
                             "value": {k: round(pixels_per_step / (v * 1e-3) / 1e6, 3)
                                       for k, v in plain_ms.items()}},
            "reuse": {"what": "build once, apply forward + reverse per step",
                      "ms_per_step": round(reuse_ms, 4),
                      "value": round(pixels_per_step / (reuse_ms * 1e-3) / 1e6, 3)},
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

    if not args.no_cpu and not args.headline_only:
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
        parity = {}
        for name, got, want in (("forward", out_f.cpu().numpy(), outs[0]),
                                ("reverse", out_r.cpu().numpy(), outs[1])):
            parity[name] = {"max_abs": float(np.abs(got - want).max()),
                            "rel_l2": float(np.linalg.norm(got - want) / np.linalg.norm(want))}
        result["parity_vs_cpu"] = parity

    print(json.dumps(result))


if __name__ == "__main__":
    main()
