#!/usr/bin/env python3
"""Benchmark of the rasterizer hot path on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2] [--no-cpu-baseline]

A step is one forward + backward of the public API (GaussianRasterizer(...)(...) followed by
image.backward(v_image)) on a synthetic scene whose inputs are already resident in HBM.
Prints ONE JSON line: ms/iter for the workload, the roofline figure of the dominant kernel
(per-kernel times come from events recorded on the launch stream during a second pass of the
same K steps, because the event packets themselves slow a step by about a tenth)
and the CPU oracle (OpenMP build) timed on the host cores for the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
VALU_PEAK_TFLOPS = 157.3       # MI355X vector FP32 (packed); scalar-FP32 code can reach half

# algorithmic FP32 operations per evaluated (pixel, Gaussian) pair
FWD_PAIR_FLOPS, FWD_REJECT_FLOPS = 25, 15
BWD_PAIR_FLOPS, BWD_REJECT_FLOPS = 72, 15


def measured_traffic(workload, num_keys):
    """HBM bytes per launch of every kernel from the FETCH_SIZE / WRITE_SIZE counters: the figures of
    profiles/<workload>_hbm_traffic_per_kernel.json, which bench_profiles.py writes from two
    rocprofv3 --pmc runs of this script (counters cannot be read from inside the process).  They are
    reported only for the workload and pair count they were taken at; the record carries the
    commit they were measured on.  Returns (dict kernel -> bytes, source description) or ({}, None)."""
    path = os.path.join(ROOT, "profiles", "%s_hbm_traffic_per_kernel.json" % workload)
    if not os.path.exists(path):
        return {}, None
    with open(path) as f:
        rec = json.load(f)
    if int(rec.get("num_keys", -1)) != int(num_keys):
        return {}, None
    return rec.get("kernels", {}), {"file": os.path.relpath(path, ROOT), "commit": rec.get("commit"),
                                    "scale_fetch": rec.get("scale_fetch"), "scale_write": rec.get("scale_write")}


def algorithmic_work(kernel, n, k, pixels, lists, coeffs, counters, marked, carries_rects=True, binned=True):
    """(bound, work per launch, unit): algorithmic HBM bytes or FP32 operations per launch.
    k: pairs of the tile lists as built (per bin of tiles); lists: how many lists they are partitioned into;
    marked: Gaussians whose accumulator record received a term in the blend backward;
    binned: the lists are per bin of tiles (a pair's slot word then has 32 bits, half of them the mask of the
    bin's tiles that its Gaussian covers, and the sorted words are kept for the blend kernels)."""
    slot_bytes = 4 if binned else (2 if lists + 1 <= 65535 else 4)
    if kernel == "project_fwd_kernel":
        # inputs 44 + 12c bytes, outputs radii + splat record + depth key + tile rectangle (the 3-D
        # covariance is not stored on this path: the backward rebuilds it)
        return "hbm", n * (44 + 12 * coeffs + 4 + 48 + 4 + 8), "B"
    if kernel == "gaussian_bwd_kernel":
        # one byte per Gaussian (did its record receive a term?), then for the marked ones only: reads 88 (no
        # stored covariance), writes v_mean3d 12 + v_means2d 12 + v_scale 12 + v_quat 16 + v_shs 12c (v_colors and
        # v_cov3d are not written: the step gives neither colours nor covariances, so nothing takes them).  The
        # zeros of everybody else's outputs are stored by the blend backward's wavefronts (n * (52 + 12c) bytes).
        return "hbm", n + marked * (88 + 52 + 12 * coeffs), "B"
    if kernel == "hist32_kernel":
        return "hbm", 4 * n, "B"
    if kernel == "onesweep32_kernel<sort>":
        # depth sort of the Gaussians: key + id, in and out; images of at most 255 x 255 tiles also carry each
        # Gaussian's packed tile rectangle through the passes (4 bytes in and out) instead of gathering them
        return "hbm", (24 if carries_rects else 16) * n, "B"
    if kernel == "ordered_block_sums_kernel":
        return "hbm", 8 * n, "B"
    if kernel == "emit_ordered_kernel":
        return "hbm", 12 * n + (slot_bytes + 4) * k, "B"
    if kernel == "onesweep32_kernel<tile partition>":
        # tile partition: slot + id in and out, except that the last pass writes no slots (average per launch)
        passes = 1 if lists + 1 <= 256 else (2 if lists + 1 <= 65536 else 3)
        if binned:
            return "hbm", 2 * (slot_bytes + 4) * k, "B"
        return "hbm", (2 * (slot_bytes + 4) * passes - slot_bytes) * k / passes, "B"
    if kernel == "blend_fwd_kernel" and counters is not None:
        rej = counters.pairs_fwd - counters.pairs_fwd_applied
        return "valu", counters.pairs_fwd_applied * FWD_PAIR_FLOPS + rej * FWD_REJECT_FLOPS, "FLOP"
    if kernel == "blend_bwd_kernel" and counters is not None:
        rej = counters.pairs_bwd - counters.pairs_bwd_valid
        return "valu", counters.pairs_bwd_valid * BWD_PAIR_FLOPS + rej * BWD_REJECT_FLOPS, "FLOP"
    return None, 0, ""


def roofline_entry(name, avg, lps, bound, work, traffic):
    if bound == "hbm":
        achieved = work / (avg * 1e-3) / 1e9
        return {"kernel": name, "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic, "avg_launch_ms": round(avg, 4),
                "launches_per_step": lps, "algorithmic_bytes_per_launch": int(work)}
    achieved = work / (avg * 1e-3) / 1e12
    # the published vector figure counts packed FP32; this build issues one FP32 operation per lane
    # and instruction (packed FP32 is compiled out), which tops out at half of it
    return {"kernel": name, "bound": "valu", "achieved": round(achieved, 2), "peak": VALU_PEAK_TFLOPS,
            "unit": "TFLOP/s", "frac": round(achieved / VALU_PEAK_TFLOPS, 4),
            "frac_of_unpacked_fp32_peak": round(achieved / (VALU_PEAK_TFLOPS / 2), 4), "traffic": traffic,
            "avg_launch_ms": round(avg, 4), "launches_per_step": lps, "algorithmic_flop_per_launch": int(work)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # defaults long enough for the clocks to settle (0.15 s of GPU work): with 3 + 20 steps the compute-bound
    # kernels are still getting faster from launch to launch and the step reads 3 % longer
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--workload", default="cfg2")
    ap.add_argument("--n", type=int, default=None, help="override the number of Gaussians (debugging)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--list-bin", type=int, default=0, choices=(0, 1, 2, 4, 8),
                    help="tiles per side of the bins the tile lists are built for (0: the library's choice)")
    ap.add_argument("--verbose", action="store_true", help="per-kernel table on stderr")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one 1 GiB device copy: a kernel of known traffic that scales the HBM byte counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path runs on ONE GPU; --gpus %d is not supported (no collectives, no sharding "
              "in this build)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    from ds_splat import GaussianRasterizationSettings, GaussianRasterizer
    from ds_splat_amd import _native
    from ds_splat_amd.synthetic import WORKLOADS, make_scene

    _native.set_default_list_bin(args.list_bin)
    spec = WORKLOADS[args.workload]
    dev = torch.device("cuda:0")
    sc = make_scene(spec, n=args.n)
    n, W, H = sc["n"], sc["width"], sc["height"]
    coeffs = (sc["sh_degree"] + 1) ** 2
    t = {k: (v.to(dev) if isinstance(v, torch.Tensor) else v) for k, v in sc.items()}
    settings = GaussianRasterizationSettings(
        image_height=H, image_width=W, tanfovx=sc["tanfovx"], tanfovy=sc["tanfovy"], bg=t["bg"],
        scale_modifier=1.0, viewmatrix=t["viewmatrix"], projmatrix=t["projmatrix"], sh_degree=sc["sh_degree"],
        max_sh_degree=3, campos=t["campos"], prefiltered=False, debug=False)
    rasterizer = GaussianRasterizer(settings)
    do_backward = spec.backward
    leaves = [t["means_3d"], torch.zeros_like(t["means_3d"]), t["shs"], t["opacities"], t["scales"], t["rotations"]]
    if do_backward:
        leaves = [x.clone().requires_grad_(True) for x in leaves]
    means, means2d, shs, opac, scales, rots = leaves
    v_image = t["v_image"]

    def step():
        image, radii = rasterizer(means, means2d, shs, None, opac, scales, rots, None)
        if do_backward:
            for p in leaves:
                p.grad = None
            image.backward(v_image)
        return image

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    if args.copy_probe:
        src = torch.ones(1 << 28, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # timed region: K steps, nothing but the public API between the two synchronisations
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps

    # what a step costs the host: the duration of the call with the GPU idle when it starts (kernel
    # enqueues, allocations, and the one blocking wait for the pair count in the middle of the
    # forward, which includes the projection's run time).  Outside the timed region.
    host_steps = min(args.steps, 20)
    host_ms = 0.0
    for _ in range(host_steps):
        torch.cuda.synchronize()
        h0 = time.perf_counter()
        step()
        host_ms += (time.perf_counter() - h0) * 1e3
    torch.cuda.synchronize()
    host_ms_per_step = host_ms / host_steps

    # the same K steps again with an event pair around every kernel launch (on the launch stream):
    # per-kernel averages for the roofline.  The event packets cost about 0.15 ms per step, so this
    # pass is not the one `value` comes from; its own wall time is reported beside it.
    _native.trace_enable(True)
    _native.trace_read()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    trace = _native.trace_read()
    _native.trace_enable(False)
    ms_per_step_traced = (t1 - t0) * 1e3 / args.steps

    per_kernel = {}
    for name, ms in trace:
        tot, cnt = per_kernel.get(name, (0.0, 0))
        per_kernel[name] = (tot + ms, cnt + 1)

    # key count of this workload
    from ds_splat_amd import stages
    cam = stages.camera_from_scene(sc, dev)
    _, st = stages.forward(cam, t["means_3d"], t["scales"], t["rotations"], t["opacities"], t["shs"])
    marked = 0
    if do_backward:
        marked = int(stages.backward(cam, st, 16, t["means_3d"], t["scales"], t["rotations"], v_image)["marks"].sum())
    torch.cuda.synchronize()
    k = st.num_keys
    tiles = cam.num_tiles
    list_bin = stages.list_bin(cam)
    lists = (((W + 15) // 16 + list_bin - 1) // list_bin) * (((H + 15) // 16 + list_bin - 1) // list_bin)
    k_per_tile = int(st.ranges[-1].item())      # pairs of the per-tile lists (the reference's K)

    # ---- CPU baseline: the oracle's OpenMP build on the host cores, same inputs -----------------
    cpu_baseline = None
    counters = None
    if not args.no_cpu_baseline:
        from oracle.binding import Oracle, make_settings
        O = Oracle(omp=True)
        s = make_settings(H, W, sc["tanfovx"], sc["tanfovy"], sc["bg"].numpy(), 1.0,
                          sc["viewmatrix"].t().contiguous().numpy(), sc["projmatrix"].t().contiguous().numpy(),
                          sc["sh_degree"], sc["campos"].numpy())
        A = {kk: v.numpy() for kk, v in sc.items() if isinstance(v, torch.Tensor)}
        # one warm-up iteration (first touch of ~2 GB of vectors), then the median of the timed ones;
        # fewer timed iterations for the workloads whose iteration takes many seconds
        timed = 3 if spec.name in ("cfg0", "cfg1", "cfg2") else 1
        runs = []
        k_cpu = -1
        for it in range(1 + timed):
            c0 = time.perf_counter()
            img_o, radii_o, ost = O.forward(s, A["means_3d"], A["scales"], A["rotations"], A["opacities"], A["shs"])
            c1 = time.perf_counter()
            if do_backward:
                B = O.backward(s, ost, 16, A["means_3d"], A["scales"], A["rotations"], A["opacities"], A["v_image"])
                counters = B["counters"]
                del B
            else:
                counters = O.state(s, ost, n)["counters"]
            c2 = time.perf_counter()
            k_cpu = int(O.lib.dsxo_state_num_keys(ost))
            O.free(ost)
            if it > 0:
                runs.append(((c2 - c0) * 1e3, (c1 - c0) * 1e3, (c2 - c1) * 1e3))
        runs.sort()
        cpu_ms, fwd_ms, bwd_ms = runs[len(runs) // 2]
        cpu_baseline = {
            "value": round(cpu_ms, 1), "unit": "ms/iter", "cores": O.num_threads(), "kind": "port",
            "iterations": timed, "warmup_iterations": 1,
            "sample": "median of %d iteration%s of the full %s workload after 1 warm-up (forward %.0f ms%s), "
                      "C++ oracle built -O3 -fopenmp" % (timed, "" if timed == 1 else "s", spec.name, fwd_ms,
                                                         (", backward %.0f ms" % bwd_ms) if do_backward else ""),
            "all_iterations_ms": [round(r[0], 1) for r in runs],
            "keys_match_gpu": bool(k_cpu == k_per_tile),
        }

    # ---- roofline of the dominant kernel (and of the dominant HBM-bound one, if that is another) ----
    table = []
    for name, (tot, cnt) in per_kernel.items():
        launches_per_step = cnt / args.steps
        avg = tot / cnt
        bound, work, unit = algorithmic_work(name, n, k, W * H, lists, coeffs, counters, marked,
                                             (W + 15) // 16 <= 255 and (H + 15) // 16 <= 255, list_bin > 1)
        table.append((tot / args.steps, name, avg, launches_per_step, bound, work, unit))
    table.sort(reverse=True)
    measured, traffic_source = measured_traffic(spec.name, k) if args.n is None else ({}, None)
    roofline = None
    roofline_hbm = None
    for ms_step, name, avg, lps, bound, work, unit in table:
        if bound is None:
            continue
        traffic = measured.get(name)
        entry = roofline_entry(name, avg, lps, bound, work, int(traffic) if traffic else None)
        # the blend kernels carry stores for their neighbours (the launch time and the traffic include them,
        # the algorithmic work does not): the forward prepares the backward's accumulator, the backward
        # writes the zeros of the per-Gaussian backward's outputs
        if name == "blend_bwd_kernel":
            entry["side_job_bytes"] = int(n * (52 + 12 * coeffs))
        elif name == "blend_fwd_kernel" and do_backward:
            entry["side_job_bytes"] = int(n * (48 + 16 + 1))   # record written, conic read, mark cleared
        if roofline is None:
            roofline = entry
        if roofline_hbm is None and bound == "hbm":
            roofline_hbm = entry
        if roofline is not None and roofline_hbm is not None:
            break
    if args.verbose:
        for ms_step, name, avg, lps, bound, work, unit in table:
            extra = ""
            if bound == "hbm":
                extra = "%8.1f GB/s (%.1f%% of HBM peak)" % (work / (avg * 1e-3) / 1e9,
                                                            100 * work / (avg * 1e-3) / 1e9 / HBM_PEAK_GBS)
            elif bound == "valu":
                extra = "%8.2f TFLOP/s" % (work / (avg * 1e-3) / 1e12)
            print("%-28s %8.3f ms/step  %7.4f ms/launch x %4.1f  %s" % (name, ms_step, avg, lps, extra),
                  file=sys.stderr)
        print("sum of kernels %.3f ms/step; wall %.3f ms/step (%.3f with kernel events); K = %d keys" %
              (sum(r[0] for r in table), ms_per_step, ms_per_step_traced, k), file=sys.stderr)

    out = {
        "metric": "fwd+bwd ms/iter at 3M Gaussians 1080p SH3" if spec.name == "cfg2" else
                  ("%s ms/iter (%s)" % ("fwd+bwd" if do_backward else "fwd", spec.name)),
        "value": round(ms_per_step, 4), "unit": "ms/iter", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "%s: %d Gaussians, %dx%d, SH degree %d, %s" %
                               (spec.name, n, W, H, sc["sh_degree"], "forward+backward" if do_backward else "forward"),
                   "num_keys": int(k), "num_keys_per_tile_lists": k_per_tile, "tiles": int(tiles),
                   "list_bin_tiles": list_bin, "lists": int(lists), "gaussians_with_gradient": marked,
                   # (from the CPU oracle's counters, when it ran: pixel-entry pairs that the blend kernels
                   # walk, and those among them that are blended)
                   "pairs_walked_fwd": int(counters.pairs_fwd) if counters is not None else None,
                   "pairs_blended_fwd": int(counters.pairs_fwd_applied) if counters is not None else None,
                   "pairs_walked_bwd": int(counters.pairs_bwd) if counters is not None else None,
                   "pairs_valid_bwd": int(counters.pairs_bwd_valid) if counters is not None else None},
        "mpix_per_s": round(W * H / (ms_per_step * 1e-3) / 1e6, 1),
        "ms_per_step_with_kernel_events": round(ms_per_step_traced, 4),
        # the host's share of a step (enqueue + the wait for the pair count) and the device's (sum of the
        # kernels' own times): the step is host-bound when the first is not hidden behind the second
        "host_ms_per_step": round(host_ms_per_step, 4),
        "kernels_sum_ms_per_step": round(sum(r[0] for r in table), 4),
        "host_bound": bool(sum(r[0] for r in table) < 0.9 * ms_per_step),
        "traffic_source": traffic_source,
        "kernels_ms_per_step": {name: round(ms_step, 4) for ms_step, name, *_ in table},
        "roofline": roofline,
        "roofline_hbm": roofline_hbm,
        "cpu_baseline": cpu_baseline,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
