#!/usr/bin/env python3
"""Benchmark of the octree rendering hot path on one MI355X.

Workload "sparse512_sh16" (the headline configuration of this benchmark): a seeded sparse octree with a 512^3
finest grid refined only near the surface of a union of spheres, SH16 leaf records (49 floats).
  forward  : one step renders 8 poses of 800x800 pixels with step_size 5e-4 and
             sigma_thresh = stop_thresh = 1e-2 through VolumeRenderer.render_persp, all poses in
             one launch (the same step with one call per pose is reported as fwd_per_call);
  fwd+bwd  : one step renders 1M rays drawn from those 8 poses, back-propagates a random
             grad_output ~ N(0, 1e-2) into d(data) and applies one SGD update to tree.data.
`value` is forward Mrays/s with everything resident in HBM; the fwd+bwd figure, the roofline of the
dominant kernel and a CPU baseline measured on this host ride along in the same JSON line.

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0  # MI355X published HBM3E bandwidth


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def forward_bytes(stats, n_rays, K, ray_io_bytes):
    """Algorithmic bytes of one forward launch: per ray its input/output, per visited leaf one
    child-table entry and sigma, per shaded leaf the K-1 colour coefficients."""
    return n_rays * ray_io_bytes + stats["samples"] * 8 + stats["samples_shaded"] * 4 * (K - 1)


def backward_bytes(stats, n_rays, K, ray_io_bytes, data_bytes):
    """Two marches that read what the forward reads (without thresholds), an atomic read-modify-
    write of the K gradients of every leaf with sigma > 0, and the zero-fill of d(data)."""
    per_march = stats["samples_bwd"] * 8 + stats["samples_bwd_pos"] * 4 * (K - 1)
    return n_rays * ray_io_bytes + 2 * per_march + stats["samples_bwd_pos"] * 8 * K + data_bytes


def kernel_source_stamp():
    """sha256 over the sources the HIP library is built from: what a rocprofv3 summary under profiles/ is stamped with,
    so that counters taken on other kernels are not mixed with this run's timings."""
    import hashlib
    h = hashlib.sha256()
    src = os.path.join(ROOT, "svox_amd", "csrc")
    for name in sorted(os.listdir(src)):
        if name.endswith((".h", ".hip")):
            h.update(name.encode())
            h.update(open(os.path.join(src, name), "rb").read())
    return h.hexdigest()[:16]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--depth", type=int, default=9, help="finest grid is 2^depth per axis")
    ap.add_argument("--size", type=int, default=800, help="image width and height")
    ap.add_argument("--poses", type=int, default=8)
    ap.add_argument("--train-rays", type=int, default=1 << 20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-bwd", action="store_true", help="skip the forward+backward leg")
    ap.add_argument("--no-query", action="store_true", help="skip the point-query leg")
    ap.add_argument("--no-large", action="store_true", help="skip the depth-10 SH25 NDC leg")
    ap.add_argument("--no-generic", action="store_true", help="skip the fp64 / SG / softplus leg (generic kernels)")
    ap.add_argument("--print-stamp", action="store_true", help="print the stamp of the kernel sources and exit")
    args = ap.parse_args()
    if args.print_stamp:
        print(kernel_source_stamp())
        return
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (rays would shard "
              "trivially across GPUs), run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import bench_probes
    import svox_amd as svox
    from svox_amd import csrc as C
    from svox_amd import synth
    from svox_amd.renderer import _make_camera_spec, _rays_spec_from_rays

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    C._abi.load_library()

    # ---------------------------------------------------------------- workload
    t0 = time.time()
    tree = synth.shell_tree(depth=args.depth, n_spheres=24, data_format="SH16", seed=0, device=dev)
    torch.cuda.synchronize()
    K = tree.data_dim
    data_bytes = tree.data.numel() * 4
    log(f"[bench] tree built in {time.time() - t0:.1f}s: {tree.info}, data {data_bytes / 2**30:.2f} GiB")
    W = H = args.size
    fx = 1111.111 * W / 800.0
    poses = [p.to(dev) for p in synth.orbit_poses(args.poses, seed=1, radius=4.0)]
    renderer = svox.VolumeRenderer(tree, step_size=5e-4)
    opt = renderer._get_options(True)  # fast: sigma_thresh = stop_thresh = 1e-2
    n_rays_step = args.poses * W * H

    # visit counts per pose from the library's counter kernel (outside the timed region)
    spec = tree._spec()
    pose_stats = [C.volume_render_stats(spec, _make_camera_spec(p, W, H, fx, fx), opt) for p in poses]
    fwd_bytes = [forward_bytes(s, W * H, K, 12) for s in pose_stats]

    pose_stack = torch.stack(poses).contiguous()          # (poses, 3, 4)

    def forward_step(events=None):
        """All poses of the step in one launch (render_persp with a stack of poses)."""
        with torch.no_grad():
            if events is not None:
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
            imgs = renderer.render_persp(pose_stack, width=W, height=H, fx=fx, fast=True)
            if events is not None:
                b.record()
                events.append((a, b))
        return imgs

    def forward_step_per_call():
        """The reference's calling pattern: one render_persp call (one launch) per pose."""
        with torch.no_grad():
            for p in poses:
                img = renderer.render_persp(p, width=W, height=H, fx=fx, fast=True)
        return img

    step_spread = {}

    def timed(fn, label=None):
        """Mean wall-clock milliseconds per step over args.steps steps (synchronised on both sides); with a label,
        the median and the minimum of the steps' own durations (an event between every two steps) are kept too."""
        for _ in range(args.warmup):
            fn()
        marks_ = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        marks_[0].record()
        for i in range(args.steps):
            fn()
            marks_[i + 1].record()
        torch.cuda.synchronize()
        mean_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        if label:
            per = np.array([marks_[i].elapsed_time(marks_[i + 1]) for i in range(args.steps)])
            step_spread[label] = {"median_ms": round(float(np.median(per)), 4), "min_ms": round(float(per.min()), 4),
                                  "max_ms": round(float(per.max()), 4)}
        return mean_ms

    fwd_ms = timed(forward_step, "forward")
    fwd_mrays = n_rays_step / (fwd_ms * 1e-3) / 1e6
    per_call_ms = timed(forward_step_per_call, "forward_per_call")

    # Launch duration of the dominant kernel with events on the launching stream.  A launch of this
    # size marks the empty leaves first (C._marks_for_this_call: a small kernel of its own, inside
    # `value`'s timed region); the render launch is timed here alone, with such marks already made.
    marked_spec = tree._spec()
    made = C._marks_for_this_call(marked_spec, opt, n_rays_step)
    marks = None
    if made is not None:
        marks, marked_spec.child_marks_thresh = made
        marked_spec.child_marks_softplus = bool(opt.density_softplus)
    marked_spec.child_marks = marks
    cam_all = _make_camera_spec(pose_stack, W, H, fx, fx)
    events = []
    for _ in range(max(3, args.steps)):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        C.volume_render_images(marked_spec, cam_all, opt)
        b.record()
        events.append((a, b))
    torch.cuda.synchronize()
    durs = np.array([a.elapsed_time(b) for (a, b) in events])  # ms
    if marks is not None:
        # the density of a leaf marked empty is not read: 4 bytes are counted for it only where the leaf is shaded
        launch_bytes = np.array([float(sum(W * H * 12 + st["samples"] * 4 + st["samples_shaded"] * 4 * K
                                           for st in pose_stats))])
    else:
        launch_bytes = np.array([float(sum(fwd_bytes))])
    achieved = launch_bytes.mean() / (durs.mean() * 1e-3) / 1e9
    marks_made_in_call = marks is not None
    del marked_spec, marks

    # the launches of the reference's calling pattern (one pose per call, no marks), timed the same way
    single = []
    plain_spec = tree._spec()
    for p in poses:
        cam_p = _make_camera_spec(p.contiguous(), W, H, fx, fx)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        C.volume_render_image(plain_spec, cam_p, opt)
        b.record()
        single.append((a, b))
    torch.cuda.synchronize()
    single_ms = np.array([a.elapsed_time(b) for a, b in single])
    single_bytes = float(sum(fwd_bytes))          # (no marks: the density of every visited leaf is read)

    # copy ceiling of this device (read + write of 1 GiB)
    src = torch.empty(1 << 28, dtype=torch.float32, device=dev)
    dst = torch.empty_like(src)
    dst.copy_(src)
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(5):
        dst.copy_(src)
    b.record()
    torch.cuda.synchronize()
    copy_gbs = 5 * 2 * src.numel() * 4 / (a.elapsed_time(b) * 1e-3) / 1e9
    del src, dst

    # the ceiling this gather-bound launch runs against: random 128-byte lines out of a buffer of the
    # size of tree.data (index_select of 8 Mi rows of 32 floats), in lines per microsecond
    rows = data_bytes // 128
    table = torch.empty(rows, 32, dtype=torch.float32, device=dev)
    idx = torch.randint(0, rows, (1 << 23,), generator=torch.Generator().manual_seed(11)).to(dev)
    torch.index_select(table, 0, idx)
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(3):
        torch.index_select(table, 0, idx)
    b.record()
    torch.cuda.synchronize()
    gather_lines_per_us = 3 * idx.numel() / (a.elapsed_time(b) * 1e3)
    del table, idx

    # what the memory system serves when nothing else is in the way: the library's gather probe (every lane
    # reads 16 bytes of random 64-byte pieces, four reads in flight) on the tree's records, 1.13 GiB (every
    # read misses L2), and on 2 MiB of them (every read hits L2 once warm)
    def probe_rate(buffer, unit_bytes=64, lanes=1):
        bench_probes.gather_probe(buffer, unit_bytes=unit_bytes, iters=16, lanes_per_unit=lanes)
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        units = bench_probes.gather_probe(buffer, unit_bytes=unit_bytes, iters=64 * lanes, lanes_per_unit=lanes)
        b.record()
        torch.cuda.synchronize()
        return units / (a.elapsed_time(b) * 1e3)

    flat_data = tree.data.detach().view(-1)
    probe_miss_per_us = probe_rate(flat_data)
    probe_hit_per_us = probe_rate(flat_data[: (2 << 20) // 4])
    # whole 128-byte lines (8 lanes x 16 bytes): the same lines per microsecond as one 16-byte read per line --
    # the memory system moves lines, so this rate x 128 bytes is the bandwidth scattered reads can have
    probe_lines_per_us = probe_rate(flat_data, unit_bytes=128, lanes=8)

    # HBM bytes and L2 requests per launch of the dominant kernel come from rocprofv3 counters (separate
    # --pmc runs), not from this process: the committed summary carries the figures for the default workload
    # (traffic = 2.00 x FETCH_SIZE + WRITE_SIZE: the factor a plain copy gives, and the one the whole-line probe
    # above gives for scattered reads -- the counter books 64 bytes for a request that moves a 128-byte line)
    traffic = l2_requests = l2_misses = None
    traffic_source = None
    prof_rel = os.path.join("profiles", "hbm_traffic_sparse512_sh16.txt")
    prof = os.path.join(ROOT, prof_rel)
    stamp = kernel_source_stamp()
    if args.depth == 9 and args.size == 800 and args.poses == 8 and os.path.exists(prof):
        import re
        text = open(prof).read()
        m = re.search(r"kernel_sources_stamp:\s*([0-9a-f]+)", text)
        if m and m.group(1) == stamp:
            traffic_source = f"{prof_rel} (rocprofv3 --pmc runs on these kernel sources, stamp {stamp})"
            m = re.search(r"traffic_bytes_per_launch:\s*(\d+)", text)
            traffic = int(m.group(1)) if m else None
            m = re.search(r"l2_requests_per_launch:\s*(\d+)", text)
            l2_requests = int(m.group(1)) if m else None
            m = re.search(r"l2_misses_per_launch:\s*(\d+)", text)
            l2_misses = int(m.group(1)) if m else None
        else:
            traffic_source = (f"none: {prof_rel} was taken on other kernel sources (its stamp "
                              f"{m.group(1) if m else 'missing'}, these sources {stamp}); counters are not mixed with this run")

    # which forward kernel the launcher picks for this launch (its rule goes by tiles of 64 pixels: up to 49 152
    # where the marks decide the shading the two-wavefront kernel, beyond that the one-wavefront kernel that
    # builds its shade list from the marks alone)
    tiles = args.poses * ((W * H + 63) // 64)
    dominant = ("render_forward_split_kernel<OctreePolicy<SH,16>, ImageSource>" if tiles <= 49152 else
                "render_forward_kernel<OctreePolicy<SH,16>, ImageSource, all-shaded>")
    roofline = {
        "bound": "hbm", "kernel": dominant,
        "launch": f"{args.poses} poses x {W}x{H} in one launch",
        "achieved": round(achieved, 2), "peak": PEAK_HBM_GBS, "unit": "GB/s",
        "frac": round(achieved / PEAK_HBM_GBS, 5), "traffic": traffic, "traffic_source": traffic_source,
        # the same launch on the bytes it makes the memory move (`traffic`: whole 128-byte lines per L2 miss)
        "fetched_gbs": round(traffic / (float(durs.mean()) * 1e6), 1) if traffic else None,
        "frac_on_fetched_bytes": round(traffic / (float(durs.mean()) * 1e6) / PEAK_HBM_GBS, 4) if traffic else None,
        "algorithmic_bytes_per_launch": int(launch_bytes.mean()),
        "avg_launch_ms": round(float(durs.mean()), 4),
        "median_launch_ms": round(float(np.median(durs)), 4), "min_launch_ms": round(float(durs.min()), 4),
        "empty_leaves_marked_per_call": marks_made_in_call,
        # the reference's calling pattern beside it: one launch per pose (no marks), its own launch times and the
        # fraction of the roofline those launches reach on their algorithmic bytes
        "per_call": {
            "launch": f"one pose {W}x{H} per launch, {args.poses} launches",
            "avg_launch_ms": round(float(single_ms.mean()), 4), "median_launch_ms": round(float(np.median(single_ms)), 4),
            "min_launch_ms": round(float(single_ms.min()), 4),
            "algorithmic_bytes_per_launch": int(single_bytes / args.poses),
            "achieved": round(single_bytes / (float(single_ms.sum()) * 1e-3) / 1e9, 2),
            "frac": round(single_bytes / (float(single_ms.sum()) * 1e-3) / 1e9 / PEAK_HBM_GBS, 5),
        },
        "copy_ceiling_gbs": round(copy_gbs, 1),
        "rays_hit": int(sum(s["rays_hit"] for s in pose_stats)),
        "samples": int(sum(s["samples"] for s in pose_stats)),
        "samples_shaded": int(sum(s["samples_shaded"] for s in pose_stats)),
        # visits after the last shaded leaf of their ray (all visits of a ray that shades nothing)
        "samples_tail": int(sum(s["samples_tail"] for s in pose_stats)),
        "samples_per_ray": round(sum(s["samples"] for s in pose_stats) / n_rays_step, 2),
        "shaded_per_ray": round(sum(s["samples_shaded"] for s in pose_stats) / n_rays_step, 2),
        "msamples_s": round(sum(s["samples"] for s in pose_stats) / (durs.mean() * 1e3), 1),
        # the launch as a stream of scattered cache lines: its L2 requests (rocprofv3 TCC_REQ, from the
        # committed profile) per microsecond against a plain gather of random 128-byte lines measured here
        "scattered_lines": {
            "l2_requests_per_launch": l2_requests, "l2_misses_per_launch": l2_misses,
            "l2_hit_rate": round(1 - l2_misses / l2_requests, 4) if l2_requests and l2_misses else None,
            "l2_requests_per_us": round(l2_requests / (durs.mean() * 1e3), 1) if l2_requests else None,
            "l2_misses_per_us": round(l2_misses / (durs.mean() * 1e3), 1) if l2_misses else None,
            "torch_index_select_lines_per_us": round(gather_lines_per_us, 1),
            # the gather probe: 64-byte requests per microsecond that miss / hit L2, and the time the launch's
            # requests alone would take at those rates (misses at the one, the other requests at the other)
            "probe_whole_lines_per_us": round(probe_lines_per_us, 1),
            "probe_line_bandwidth_gbs": round(probe_lines_per_us * 128 / 1e3, 1),
            "probe_l2_miss_requests_per_us": round(probe_miss_per_us, 1),
            "probe_l2_hit_requests_per_us": round(probe_hit_per_us, 1),
            "launch_ms_at_probe_rates": round((l2_misses / probe_miss_per_us
                                               + (l2_requests - l2_misses) / probe_hit_per_us) / 1e3, 4)
            if l2_requests and l2_misses else None,
            "frac_of_probe_rates": round((l2_misses / probe_miss_per_us + (l2_requests - l2_misses) / probe_hit_per_us)
                                         / 1e3 / float(durs.mean()), 4) if l2_requests and l2_misses else None,
            # filled in by the query leg: what this library's own gather kernel reaches on random records
            "gather_ceiling_lines_per_us": None, "misses_over_gather_ceiling": None,
        },
    }
    per_call = {"value": round(n_rays_step / (per_call_ms * 1e-3) / 1e6, 3), "unit": "Mrays/s",
                "ms_per_step": round(per_call_ms, 4), "ms_per_pose": round(per_call_ms / args.poses, 4),
                "mrays_hit_s": round(roofline["rays_hit"] / (per_call_ms * 1e-3) / 1e6, 1),
                "note": "same step as one render_persp call (one launch) per pose, the reference's calling pattern"}
    log(f"[bench] forward {fwd_ms:.2f} ms/step, {fwd_mrays:.1f} Mrays/s (one call per pose: {per_call}), roofline {roofline}")

    # ---------------------------------------------------------------- the same step with the empty leaves marked
    # (opt-in, for a tree that is rendered as it is many times: tree.mark_empty_leaves() once, then
    # the renderer passes through empty leaves without reading their density; pictures are identical)
    auto_mark = C.AUTO_MARK_RAYS_PER_CELL
    C.AUTO_MARK_RAYS_PER_CELL = None          # no marks at all: the launch reads the density of every leaf it visits
    plain_imgs = forward_step()
    plain_ms = timed(forward_step, "forward_without_marks")
    C.AUTO_MARK_RAYS_PER_CELL = auto_mark
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    tree.mark_empty_leaves(sigma_thresh=opt.sigma_thresh)
    torch.cuda.synchronize()
    a.record()
    tree.mark_empty_leaves(sigma_thresh=opt.sigma_thresh)
    b.record()
    torch.cuda.synchronize()
    mark_ms = a.elapsed_time(b)
    marked_ms = timed(forward_step, "forward_marks_kept")
    marked_equal = bool(torch.equal(forward_step(), plain_imgs))
    del plain_imgs
    tree.clear_leaf_marks()
    # the density of a leaf marked empty is not read: count 4 bytes for it only where the leaf is shaded
    marked_bytes = sum(W * H * 12 + st["samples"] * 4 + st["samples_shaded"] * 4 * K for st in pose_stats)
    static_tree = {
        "value": round(n_rays_step / (marked_ms * 1e-3) / 1e6, 3), "unit": "Mrays/s", "ms_per_step": round(marked_ms, 4),
        "mark_empty_leaves_ms": round(mark_ms, 4), "pictures_identical": marked_equal,
        "ms_per_step_without_marks": round(plain_ms, 4),
        "algorithmic_gbs": round(marked_bytes / (marked_ms * 1e-3) / 1e9, 2),
        "frac_of_peak": round(marked_bytes / (marked_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 5),
        "note": "not the headline: N3Tree.mark_empty_leaves() is an explicit call outside the reference's interface, "
                "made once per version of the tree and not inside the timed region; `value` at the top is the "
                "stateless path, which makes the marks inside every call of this size"}
    log(f"[bench] forward with marked empty leaves {static_tree}")

    # ---------------------------------------------------------------- forward + backward + SGD
    fwd_bwd = None
    if not args.no_bwd:
        g = torch.Generator().manual_seed(7)
        B = args.train_rays
        per_pose = [svox.VolumeRenderer.persp_rays(p, W, H, fx) for p in poses]
        pick = torch.randint(0, n_rays_step, (B,), generator=g).to(dev)
        all_o = torch.cat([r.origins for r in per_pose])
        all_d = torch.cat([r.dirs for r in per_pose])
        rays = svox.Rays(all_o[pick].contiguous(), all_d[pick].contiguous(), all_d[pick].contiguous())
        del all_o, all_d, per_pose
        grad_out = (torch.randn(B, 3, generator=g) * 1e-2).to(dev)
        lr = 1e-3
        train_stats = C.volume_render_stats(spec, _rays_spec_from_rays(rays), opt)
        data_before = tree.data.data.clone()   # the SGD steps below change the tree; put back afterwards
        ev = []

        def train_step(record=False):
            tree.data.grad = None
            out = renderer(rays, fast=True)
            if record:
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
            out.backward(grad_out)
            if record:
                b.record()
                ev.append((a, b))
            with torch.no_grad():
                tree.data.data.add_(tree.data.grad, alpha=-lr)

        tb_ms = timed(train_step, "fwd_bwd")
        for _ in range(2):
            train_step(record=True)
        torch.cuda.synchronize()
        bwd_ms = float(np.mean([a.elapsed_time(b) for a, b in ev]))

        # the same step through the two stateless operators of the reference's interface
        rspec = _rays_spec_from_rays(rays)

        def separate_step():
            C.volume_render(spec, rspec, opt)
            grad = C.volume_render_backward(spec, rspec, opt, grad_out)
            with torch.no_grad():
                tree.data.data.add_(grad, alpha=-lr)

        sep_ms = timed(separate_step, "fwd_bwd_separate_calls")
        bbytes = backward_bytes(train_stats, B, K, 36 + 12, data_bytes)
        fbytes = forward_bytes(train_stats, B, K, 36 + 12)
        fwd_bwd = {
            "value": round(B / (tb_ms * 1e-3) / 1e6, 3), "unit": "Mrays/s", "rays": B,
            "ms_per_step": round(tb_ms, 3),
            "includes": "renderer(rays).backward(grad) + SGD update: the forward pass notes the leaves with sigma > 0 "
                        "of every ray in a 768 B/ray workspace (one march, no early stop), the backward pass "
                        "(zero-fill included) replays the notes instead of marching",
            "backward_ms": round(bwd_ms, 3),
            "algorithmic_gbs": round((fbytes + bbytes) / (tb_ms * 1e-3) / 1e9, 2),
            "frac_of_peak": round((fbytes + bbytes) / (tb_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 5),
            "separate_calls": {
                "value": round(B / (sep_ms * 1e-3) / 1e6, 3), "ms_per_step": round(sep_ms, 3),
                "note": "volume_render + volume_render_backward + SGD update as independent calls (the backward "
                        "walks every ray once, taking notes in a workspace of its own, and forms the gradient from the notes)"},
            "samples_per_ray": round(train_stats["samples_bwd"] / B, 2),
            "positive_per_ray": round(train_stats["samples_bwd_pos"] / B, 2),
        }
        # The gradient records reach memory as fp32 atomic adds, K scalars per leaf with density: what the
        # memory system takes of those is measured by the library's atomic probe (wavefronts adding to runs
        # of 16 consecutive floats, one 64-byte request each, at random places of a scratch the size of the
        # gradient).  A record of K floats at a K-float stride lies in (4 K + 60) / 64 such pieces on average.
        scratch = torch.zeros_like(tree.data).view(-1)
        bench_probes.atomic_probe(scratch, run_floats=16, iters=8)
        torch.cuda.synchronize()
        pa, pb = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        pa.record()
        _, probe_requests = bench_probes.atomic_probe(scratch, run_floats=16, iters=512)
        pb.record()
        torch.cuda.synchronize()
        atomic_requests_per_us = probe_requests / (pa.elapsed_time(pb) * 1e3)
        za, zb = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        za.record()
        scratch.zero_()
        zb.record()
        torch.cuda.synchronize()
        zero_ms = za.elapsed_time(zb)
        del scratch
        records = int(train_stats["samples_bwd_pos"])
        record_requests = records * (4 * K + 60) / 64
        fwd_bwd["atomics"] = {
            "probe_requests_per_us": round(atomic_requests_per_us, 1),
            "records": records, "requests_per_record": round((4 * K + 60) / 64, 2),
            "ms_at_probe_rate": round(record_requests / atomic_requests_per_us / 1e3, 4),
            "backward_ms_without_zero_fill": round(bwd_ms - zero_ms, 4),
            "frac_of_probe_rate": round(record_requests / atomic_requests_per_us / 1e3 / max(bwd_ms - zero_ms, 1e-9), 4),
            "note": "64-byte atomic-add requests per microsecond the memory system takes (the same for 1, 4 or 16 "
                    "floats per request and for a scratch of 2 MiB or 2 GiB), and the time the records of this "
                    "step's backward pass would take at that rate",
        }
        tree.data.grad = None
        # the squared-error step on the same rays: colour, gradient and Hessian diagonal in one call
        target = torch.rand(B, 3, generator=g).to(dev)

        def se_step(workspace):
            C.se_grad(spec, rspec, target, opt, workspace=workspace)

        se_ms = {}
        for workspace in (True, False):
            for _ in range(args.warmup):
                se_step(workspace)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                se_step(workspace)
            torch.cuda.synchronize()
            se_ms[workspace] = (time.perf_counter() - t0) * 1e3 / args.steps
        fwd_bwd["se_grad"] = {
            "ms": round(se_ms[True], 3), "mrays_s": round(B / (se_ms[True] * 1e-3) / 1e6, 1),
            "ms_marching_twice": round(se_ms[False], 3),
            "includes": "zero-fill of gradient and Hessian diagonal (2 x data); one march that takes notes, "
                        "then residual, gradient and Hessian from the notes"}
        del target
        with torch.no_grad():
            tree.data.data.copy_(data_before)
        del data_before
        # the gradient of one whole pose (every pixel a ray): neighbouring rays share leaves, unlike the random rays above
        igo = (torch.randn(H, W, 3, generator=g) * 1e-2).to(dev)
        icam = _make_camera_spec(poses[0].contiguous(), W, H, fx, fx)

        def image_step():
            tree.data.grad = None
            renderer.render_persp(poses[0], width=W, height=H, fx=fx, fast=True).backward(igo)

        def timed_median(fn, n=5):
            # median of n steps queued back to back, an event between every two (a process now and then
            # stalls for tens of milliseconds once, early on: a mean over a few steps would carry that)
            fn()
            torch.cuda.synchronize()
            marks = [torch.cuda.Event(enable_timing=True) for _ in range(n + 1)]
            marks[0].record()
            for i in range(n):
                fn()
                marks[i + 1].record()
            torch.cuda.synchronize()
            return float(np.median([marks[i].elapsed_time(marks[i + 1]) for i in range(n)]))

        itarget = torch.rand(H, W, 3, generator=g).to(dev)
        fwd_bwd["image_pose"] = {
            "forward_backward_ms": round(timed_median(image_step), 3),
            "se_grad_persp_ms": round(timed_median(lambda: renderer.se_grad_persp(poses[0], itarget, width=W, height=H,
                                                                           fx=fx)), 3),
            "backward_marching_ms": round(timed_median(lambda: C.volume_render_image_backward(spec, icam, opt, igo,
                                                                                        workspace=False)), 3),
            "note": f"render_persp of pose 0 ({W}x{H}) and its gradient through autograd; then the stateless "
                    "backward operator without a workspace (zero-fill of the gradient included in both)"}
        tree.data.grad = None
        del igo, itarget
        log(f"[bench] fwd+bwd {fwd_bwd}")

    # ---------------------------------------------------------------- point queries (dense 128^3 SH9 tree)
    query = None
    if not args.no_query:
        qtree = synth.dense_tree(6, "SH9", seed=0, sigma="lognormal", coeff_std=0.5, zero_fraction=0.5).to(dev)
        Q = 1 << 22
        pts = torch.rand(Q, 3, generator=torch.Generator().manual_seed(3)).to(dev)
        Kq, Lq = qtree.data_dim, 7

        def ev_time(fn, n=5):
            fn()
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(n):
                fn()
            b.record()
            torch.cuda.synchronize()
            return a.elapsed_time(b) / n

        qspec = qtree._spec()
        with torch.no_grad():
            q_ms = ev_time(lambda: C.query_vertical(qspec, pts))
        go = torch.randn(Q, Kq, device=dev)
        qb_ms = ev_time(lambda: C.query_vertical_backward(qspec, pts, go))
        leaves = qtree._all_leaves().to(dev)
        c_ms = ev_time(lambda: C.calc_corners(qspec, leaves))
        q_bytes = Q * (12 + 4 * Lq + 4 * Kq + 4 * Kq + 8)
        qb_bytes = Q * (12 + 4 * Lq + 4 * Kq + 8 * Kq) + qtree.data.numel() * 4
        c_bytes = leaves.shape[0] * (32 + 12 + 8 * (Lq - 1))
        query = {
            "workload": "dense 128^3 SH9 tree (268 MB), 4M uniform points",
            "query_vertical": {"mpoints_s": round(Q / q_ms / 1e3, 1), "ms": round(q_ms, 4),
                               "algorithmic_gbs": round(q_bytes / q_ms / 1e6, 1),
                               "frac_of_peak": round(q_bytes / q_ms / 1e6 / PEAK_HBM_GBS, 4)},
            "query_vertical_backward": {"mpoints_s": round(Q / qb_ms / 1e3, 1), "ms": round(qb_ms, 4),
                                        "algorithmic_gbs": round(qb_bytes / qb_ms / 1e6, 1),
                                        "frac_of_peak": round(qb_bytes / qb_ms / 1e6 / PEAK_HBM_GBS, 4),
                                        "includes": "zero-fill of the (M,2,2,2,28) gradient"},
            "calc_corners": {"mleaves_s": round(leaves.shape[0] / c_ms / 1e3, 1), "ms": round(c_ms, 4),
                             "algorithmic_gbs": round(c_bytes / c_ms / 1e6, 1)},
        }
        # the gather kernel as a ceiling for scattered lines: a 112-byte record at a 112-byte stride lies in
        # 1 + 111/128 lines of 128 bytes on average, and every point reads one (the child reads hit in L2)
        lines_per_point = 1.0 + (4 * Kq - 1) / 128.0
        sl = roofline["scattered_lines"]
        sl["gather_ceiling_lines_per_us"] = round(Q * lines_per_point / (q_ms * 1e3), 1)
        sl["gather_ceiling_note"] = (f"query_vertical, {Q} random points, {4 * Kq}-byte records of a 268 MB tree: "
                                     f"{lines_per_point:.2f} lines read per point")
        if sl["l2_misses_per_us"]:
            sl["misses_over_gather_ceiling"] = round(sl["l2_misses_per_us"] / sl["gather_ceiling_lines_per_us"], 4)
        # render_persp of the same dense tree: one 800x800 pose from the radius-4 orbit, thresholds 0
        # (every ray that hits shades some 57 leaves; the tree and its child table sit in the 256 MB
        # Infinity Cache, so bytes fetched from HBM are far below the algorithmic ones here)
        qrend = svox.VolumeRenderer(qtree)
        qopt = qrend._get_options(False)
        qcam = _make_camera_spec(poses[0].contiguous(), W, H, fx, fx)
        qstats = C.volume_render_stats(qspec, qcam, qopt)
        with torch.no_grad():
            qr_ms = ev_time(lambda: qrend.render_persp(poses[0], width=W, height=H, fx=fx))
            qimg = qrend.render_persp(poses[0], width=W, height=H, fx=fx)
        qgo = (torch.randn(H, W, 3, generator=torch.Generator().manual_seed(5)) * 1e-2).to(dev)

        def dense_train():
            qtree.data.grad = None
            qrend.render_persp(poses[0], width=W, height=H, fx=fx).backward(qgo)

        qrb_ms = ev_time(dense_train, n=3)
        qrm_ms = ev_time(lambda: C.volume_render_image_backward(qspec, qcam, qopt, qgo, workspace=False), n=3)
        # the same tree from close by (a finest voxel covers some 12x12 pixels): the rays of a wavefront
        # share their leaves, so the backward pass sums the records of a leaf before its atomics
        near = synth.orbit_poses(1, seed=3, radius=1.2)[0].to(dev)
        ncam = _make_camera_spec(near.contiguous(), W, H, fx, fx)
        with torch.no_grad():
            nr_ms = ev_time(lambda: qrend.render_persp(near, width=W, height=H, fx=fx), n=3)

        def near_train():
            qtree.data.grad = None
            qrend.render_persp(near, width=W, height=H, fx=fx).backward(qgo)

        # (the renderer gives the notes of later steps more room when those of a step ran out: a few
        # untimed steps let it settle, as the first steps of a training run would)
        for _ in range(5):
            near_train()
            torch.cuda.synchronize()
        nrb_ms = ev_time(near_train, n=3)
        near_notes = qrend.notes_budget.records_per_ray()
        nrm_ms = ev_time(lambda: C.volume_render_image_backward(qspec, ncam, qopt, qgo, workspace=False), n=3)
        qtree.data.grad = None
        qr_bytes = forward_bytes(qstats, W * H, Kq, 12)
        query["render_persp"] = {
            "workload": f"one {W}x{H} pose of the dense tree, radius-4 orbit, focal {fx:.0f}, thresholds 0",
            "ms": round(qr_ms, 4), "mrays_s": round(W * H / qr_ms / 1e3, 1),
            "rays_hit": qstats["rays_hit"], "mrays_hit_s": round(qstats["rays_hit"] / qr_ms / 1e3, 1),
            "msamples_s": round(qstats["samples"] / qr_ms / 1e3, 1),
            "samples_per_hit_ray": round(qstats["samples"] / max(qstats["rays_hit"], 1), 1),
            "shaded_per_hit_ray": round(qstats["samples_shaded"] / max(qstats["rays_hit"], 1), 1),
            "algorithmic_gbs": round(qr_bytes / qr_ms / 1e6, 1),
            "frac_of_peak": round(qr_bytes / qr_ms / 1e6 / PEAK_HBM_GBS, 4),
            "forward_backward_ms": round(qrb_ms, 4),
            "backward_marching_ms": round(qrm_ms, 4),
            "close_up": {"workload": "the same tree from radius 1.2: about 12 pixels across a finest voxel",
                         "ms": round(nr_ms, 4), "forward_backward_ms": round(nrb_ms, 4),
                         "notes_room_leaves_per_ray": near_notes,
                         "backward_marching_ms": round(nrm_ms, 4)},
        }
        if not args.no_cpu:
            from oracle import oracle as _oracle
            qot = _oracle.Tree.from_n3tree(qtree.cpu())
            qref = _oracle.volume_render_image(qot, poses[0].cpu(), fx, fx, W, H, qopt,
                                               n_threads=min(os.cpu_count() or 1, 16))
            query["render_persp"]["max_abs_err_vs_oracle"] = float(np.abs(qimg.cpu().numpy() - qref).max())
            del qot, qref
        del qtree, pts, go, leaves, qimg, qgo
        log(f"[bench] query {query}")

    # ---------------------------------------------------------------- what the generic kernels do
    # (fp64 data, spherical-Gaussian lobes, density_softplus: one ray per lane, the reference's loop)
    generic = None
    if not args.no_generic:
        def ev_time(fn, n=3):
            fn()
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(n):
                fn()
            b.record()
            torch.cuda.synchronize()
            return a.elapsed_time(b) / n

        generic = {"workload": f"dense 128^3 tree (SH9 / SG9 records), one {W}x{H} pose, thresholds 0; "
                               "4M-point query in fp64"}
        gtree = synth.dense_tree(6, "SH9", seed=0, sigma="lognormal", coeff_std=0.5, zero_fraction=0.5).to(dev)
        gcam = _make_camera_spec(poses[0].contiguous(), W, H, fx, fx)
        with torch.no_grad():
            base_ms = ev_time(lambda: C.volume_render_image(gtree._spec(), gcam, svox.VolumeRenderer(gtree)._get_options(False)))
            soft_opt = svox.VolumeRenderer(gtree, density_softplus=True)._get_options(False)
            soft_ms = ev_time(lambda: C.volume_render_image(gtree._spec(), gcam, soft_opt))
            C.set_debug_flags(1)
            try:
                forced_ms = ev_time(lambda: C.volume_render_image(gtree._spec(), gcam, svox.VolumeRenderer(gtree)._get_options(False)))
            finally:
                C.set_debug_flags(0)
        generic["fp32_sh9_octree_kernel_ms"] = round(base_ms, 4)
        generic["fp32_sh9_generic_kernel_ms"] = round(forced_ms, 4)
        generic["fp32_sh9_density_softplus_ms"] = round(soft_ms, 4)
        # SG lobes on the same records (extra_data: lambda, mu)
        lobes = torch.cat([torch.rand(9, 1, generator=torch.Generator().manual_seed(2)) * 4 + 0.5,
                           synth.unit_vectors(9, torch.Generator().manual_seed(3))], dim=1).to(dev)
        sgtree = svox.N3Tree(N=2, data_format="SG9", init_refine=0, extra_data=lobes, device=dev)
        sgtree.data, sgtree.child, sgtree.parent_depth = gtree.data, gtree.child, gtree.parent_depth
        sgtree._n_internal.fill_(gtree.n_internal)
        with torch.no_grad():
            sg_opt = svox.VolumeRenderer(sgtree)._get_options(False)
            generic["fp32_sg9_ms"] = round(ev_time(lambda: C.volume_render_image(sgtree._spec(), gcam, sg_opt)), 4)
            C.set_debug_flags(1)
            try:
                generic["fp32_sg9_generic_kernel_ms"] = round(
                    ev_time(lambda: C.volume_render_image(sgtree._spec(), gcam, sg_opt)), 4)
            finally:
                C.set_debug_flags(0)
        generic["note"] = ("fp32 SH, SG and ASG records of 1, 4, 9, 16 or 25 basis functions run on the wavefront-per-tile kernels, "
                           "for any branching factor and with or without density_softplus "
                           "(`..._generic_kernel_ms`: the same call forced onto the one-ray-per-lane kernels, which "
                           "serve fp64 and the other record shapes)")
        del sgtree
        gtree64 = gtree.double()
        g64cam = _make_camera_spec(poses[0].double().contiguous(), W, H, fx, fx)
        pts64 = torch.rand(1 << 22, 3, generator=torch.Generator().manual_seed(3), dtype=torch.float64).to(dev)
        with torch.no_grad():
            opt64 = svox.VolumeRenderer(gtree64)._get_options(False)
            generic["fp64_sh9_ms"] = round(ev_time(lambda: C.volume_render_image(gtree64._spec(), g64cam, opt64)), 4)
            generic["fp64_query_4M_ms"] = round(ev_time(lambda: C.query_vertical(gtree64._spec(), pts64)), 4)
        # gradient and se_grad of the fp64 pose (one-ray-per-lane kernels whose wavefronts add the records of a step
        # together; zero-fills of the fp64 gradient, 0.54 GB, included)
        g64 = torch.Generator().manual_seed(12)
        go64 = (torch.randn(H, W, 3, generator=g64, dtype=torch.float64) * 1e-2).to(dev)
        ref64 = torch.rand(H, W, 3, generator=g64, dtype=torch.float64).to(dev)
        generic["fp64_sh9_backward_ms"] = round(
            ev_time(lambda: C.volume_render_image_backward(gtree64._spec(), g64cam, opt64, go64), n=3), 4)
        generic["fp64_sh9_se_grad_ms"] = round(ev_time(lambda: C.se_grad_persp(gtree64._spec(), g64cam, opt64, ref64), n=3), 4)
        del go64, ref64
        # a tree with branching factor 3 (81^3 leaves, SH9 records): the wavefront-per-tile kernels with the reference's
        # floating-point walk, against the same calls forced onto the one-ray-per-lane kernels
        t3 = svox.N3Tree(N=3, data_format="SH9", init_refine=3, device=dev)
        g3 = torch.Generator().manual_seed(9)
        t3.data.data.copy_((torch.randn(t3.data.shape, generator=g3) * 0.5).to(dev))
        t3.data.data[..., -1] = (torch.exp(torch.randn(t3.child.shape, generator=g3))
                                 * (torch.rand(t3.child.shape, generator=g3) < 0.5)).to(dev)
        o3 = svox.VolumeRenderer(t3)._get_options(False)
        go3 = (torch.randn(H, W, 3, generator=g3) * 1e-2).to(dev)
        with torch.no_grad():
            generic["fp32_n3_sh9_ms"] = round(ev_time(lambda: C.volume_render_image(t3._spec(), gcam, o3)), 4)
        generic["fp32_n3_sh9_backward_ms"] = round(ev_time(lambda: C.volume_render_image_backward(t3._spec(), gcam, o3, go3)), 4)
        C.set_debug_flags(1)
        try:
            with torch.no_grad():
                generic["fp32_n3_sh9_generic_kernel_ms"] = round(ev_time(lambda: C.volume_render_image(t3._spec(), gcam, o3)), 4)
            generic["fp32_n3_sh9_backward_generic_kernel_ms"] = round(
                ev_time(lambda: C.volume_render_image_backward(t3._spec(), gcam, o3, go3)), 4)
        finally:
            C.set_debug_flags(0)
        del t3, go3
        generic["mrays_s"] = {k[:-3]: round(W * H / v / 1e3, 1) for k, v in generic.items() if k.endswith("_ms") and "query" not in k}
        del gtree, gtree64, pts64
        torch.cuda.empty_cache()
        log(f"[bench] generic kernels {generic}")

    # ---------------------------------------------------------------- depth-10 SH25 tree, NDC camera
    large = None
    free_bytes, _ = torch.cuda.mem_get_info()
    if not args.no_large and free_bytes > 100 * 2 ** 30:
        ltree = synth.shell_tree(depth=10, data_format="SH25", seed=5, device=dev, geometry="noise")
        ltree.invradius.data[:] = 0.5
        ltree.offset.data[:] = 0.5
        LW, LH, lfx = 1008, 756, 815.0
        lposes = torch.stack([torch.tensor([[1.0, 0, 0, 0.1 * i - 0.15], [0, 1, 0, 0.05 * i - 0.05],
                                            [0, 0, 1, 0.2 + 0.05 * i]]) for i in range(4)]).to(dev)
        lrend = svox.VolumeRenderer(ltree, step_size=5e-4, ndc=svox.NDCConfig(LW, LH, lfx))
        lopt = lrend._get_options(True)
        lspec = ltree._spec()
        lstats = [C.volume_render_stats(lspec, _make_camera_spec(p.contiguous(), LW, LH, lfx, lfx), lopt)
                  for p in lposes]
        l_bytes = sum(forward_bytes(st, LW * LH, 76, 12) for st in lstats)
        lcam = _make_camera_spec(lposes, LW, LH, lfx, lfx)

        def ev_time(fn, n=5):
            fn()
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(n):
                fn()
            b.record()
            torch.cuda.synchronize()
            return a.elapsed_time(b) / n

        with torch.no_grad():
            l_ms = ev_time(lambda: C.volume_render_images(lspec, lcam, lopt))
            # (a launch of 3 M rays does not pay for marking 48 M cells; with marks kept on the tree:)
            lmarked = ltree._spec()
            lmarked.child_marks = C.mark_empty_leaves(lspec, lopt.sigma_thresh)
            lmarked.child_marks_thresh = lopt.sigma_thresh
            l_marked_ms = ev_time(lambda: C.volume_render_images(lmarked, lcam, lopt))
            l_mark_ms = ev_time(lambda: C.mark_empty_leaves(lspec), n=2)
            del lmarked
            Ql = 1 << 24
            # uniform over the whole tree: world coordinates of this tree span [-1, 1]^3
            lpts = (torch.rand(Ql, 3, generator=torch.Generator().manual_seed(4)) * 2 - 1).to(dev)
            lq_ms = ev_time(lambda: C.query_vertical(lspec, lpts), n=3)
        lgo = torch.randn(Ql, 76, device=dev)
        lqb_ms = ev_time(lambda: C.query_vertical_backward(lspec, lpts, lgo), n=2)
        lq_bytes = Ql * (12 + 4 * 10 + 4 * 76 + 4 * 76 + 8)
        lqb_bytes = Ql * (12 + 4 * 10 + 4 * 76 + 8 * 76) + ltree.data.numel() * 4
        large = {
            "workload": "ndc1024_sh25: depth-10 octree, SH25, NDC camera, 4 poses x 1008x756 in one launch, "
                        "step 5e-4, thresholds 1e-2; queries on 16M uniform points",
            "nodes": ltree.info["nodes"], "leaves": ltree.info["leaves"],
            "occupancy": round(ltree.info["occupancy"], 5), "data_gib": round(ltree.data.numel() * 4 / 2 ** 30, 2),
            "forward": {"mrays_s": round(4 * LW * LH / l_ms / 1e3, 1), "ms": round(l_ms, 4),
                        "samples_per_ray": round(sum(st["samples"] for st in lstats) / (4 * LW * LH), 2),
                        "shaded_per_ray": round(sum(st["samples_shaded"] for st in lstats) / (4 * LW * LH), 2),
                        "algorithmic_gbs": round(l_bytes / l_ms / 1e6, 1),
                        "frac_of_peak": round(l_bytes / l_ms / 1e6 / PEAK_HBM_GBS, 4),
                        "ms_with_kept_marks": round(l_marked_ms, 4), "mark_empty_leaves_ms": round(l_mark_ms, 4)},
            "query_vertical": {"mpoints_s": round(Ql / lq_ms / 1e3, 1), "ms": round(lq_ms, 4),
                               "algorithmic_gbs": round(lq_bytes / lq_ms / 1e6, 1),
                               "frac_of_peak": round(lq_bytes / lq_ms / 1e6 / PEAK_HBM_GBS, 4)},
            "query_vertical_backward": {"mpoints_s": round(Ql / lqb_ms / 1e3, 1), "ms": round(lqb_ms, 4),
                                        "algorithmic_gbs": round(lqb_bytes / lqb_ms / 1e6, 1),
                                        "frac_of_peak": round(lqb_bytes / lqb_ms / 1e6 / PEAK_HBM_GBS, 4),
                                        "includes": "zero-fill of the 13.5 GB gradient"},
        }
        del ltree, lpts, lgo, lspec, lrend, lcam
        torch.cuda.empty_cache()
        log(f"[bench] large {large}")

    # ---------------------------------------------------------------- CPU baseline (this host)
    cpu = None
    if not args.no_cpu:
        from oracle import oracle, torch_fallback

        n_threads = os.cpu_count() or 1
        n_threads = min(n_threads, 16)
        torch.set_num_threads(n_threads)
        host = {k: getattr(tree, k).detach().cpu() for k in ("data", "child", "parent_depth", "invradius", "offset")}
        ot = oracle.Tree(host["data"], host["child"], host["parent_depth"], host["offset"], host["invradius"])
        cpu_poses = [p.cpu() for p in poses]
        # the OpenMP C++ oracle on the whole workload (every pixel of every pose), benchmark thresholds
        t0 = time.perf_counter()
        ref0 = None
        for i, p in enumerate(cpu_poses):
            img = oracle.volume_render_image(ot, p, fx, fx, W, H, opt, n_threads=n_threads)
            if i == 0:
                ref0 = img
        t_oracle = time.perf_counter() - t0
        n_oracle = len(cpu_poses) * W * H
        # the GPU result for pose 0, for the record
        with torch.no_grad():
            got = renderer.render_persp(poses[0], width=W, height=H, fx=fx, fast=True).cpu().numpy()
        check = float(np.abs(got - ref0).max())
        # the reference's CPU path: its PyTorch fallback (restated; it has no thresholds), whole frames
        # pose by pose until about 20 s have gone by
        n_fb, t_fb = 0, 0.0
        for p in cpu_poses:
            rays_p = svox.VolumeRenderer.persp_rays(p, W, H, fx)
            t0 = time.perf_counter()
            with torch.no_grad():
                torch_fallback.render(host["data"], host["child"], host["parent_depth"], host["invradius"],
                                      host["offset"], rays_p.origins, rays_p.dirs, rays_p.viewdirs, 16,
                                      step_size=5e-4)
            t_fb += time.perf_counter() - t0
            n_fb += W * H
            if t_fb > 20.0:
                break
        cpu = {
            "value": round(n_fb / t_fb / 1e6, 6), "unit": "Mrays/s", "cores": n_threads, "kind": "port",
            "sample": f"{n_fb // (W * H)} whole poses ({n_fb} rays) of the workload through the PyTorch restatement "
                      f"of the reference's fallback renderer (no thresholds: it has none), {t_fb:.1f}s",
            "scalar_oracle": {"value": round(n_oracle / t_oracle / 1e6, 4), "unit": "Mrays/s",
                              "cores": n_threads, "sample": f"all {len(cpu_poses)} poses ({n_oracle} rays), OpenMP "
                              f"C++ oracle with the benchmark's thresholds, {t_oracle:.1f}s"},
            "gpu_vs_oracle_max_abs_err": check,
            "host": f"{os.cpu_count()} logical cpus",
        }
        log(f"[bench] cpu baseline {cpu}")

    line = {
        "metric": "Mrays/s fwd, 512^3 sparse SH16 tree",
        "value": round(fwd_mrays, 3), "unit": "Mrays/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(fwd_ms, 4), "ms_per_step_median": step_spread["forward"]["median_ms"],
        "ms_per_step_min": step_spread["forward"]["min_ms"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "rays_hit": roofline["rays_hit"], "mrays_hit_s": round(roofline["rays_hit"] / (fwd_ms * 1e-3) / 1e6, 1),
        "msamples_s": round(roofline["samples"] / (fwd_ms * 1e-3) / 1e6, 1),
        "config": {"workload": "sparse512_sh16: 8 poses x 800x800, step 5e-4, sigma/stop thresh 1e-2",
                   "depth": args.depth, "image": [W, H], "poses": args.poses, "nodes": tree.info["nodes"],
                   "leaves": tree.info["leaves"], "occupancy": round(tree.info["occupancy"], 5),
                   "data_gib": round(data_bytes / 2**30, 3)},
        "roofline": roofline,
        "step_times": step_spread,
        "fwd_per_call": per_call,
        "fwd_static_tree": static_tree,
        "fwd_bwd": fwd_bwd,
        "query": query,
        "large": large,
        "generic_kernels": generic,
        "cpu_baseline": cpu,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
