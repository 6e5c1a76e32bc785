#!/usr/bin/env python3
"""Headline benchmark: forward + backward + fused Adam of the point splat on the 6M-point / 1920x1080 / 8-layer
scene, inputs resident in HBM. Prints ONE JSON line.

  python bench.py --gpus 1 --steps K --warmup W

A step is one pass of the hot path over one synthetic view: trips_splat_forward, trips_splat_backward (dL/dimage ~
N(0,1) on all layers, gradients to position, size, confidence, descriptors, background, pose, intrinsics) and one
trips_adam_step_fused over position, size, descriptors and confidence. `value` = points / second of that whole step.
The timed region holds nothing but the product's launches; the same K steps are then run once more with a pair of HIP
events around every kernel, recorded by the library on the launch stream (trips_profile_*): the per-kernel times. The
roofline object is for the kernel with the largest share of the step.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
DEFAULT_POINTS = 6_000_000

# HBM traffic per launch on the default workload, measured with `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE`
# (KiB per dispatch, one counter per run, same bench.py command with --steps 2 --warmup 1 --cpu-steps 0
# --calibration-copy). A plain 256 MiB device copy reads FETCH_SIZE = 131084 and WRITE_SIZE = 262144 for
# 262144 KiB each way, hence the scale factors. bench.py cannot run the profiler on itself; these are the figures
# of the committed summary of those two runs and apply to the default --points only. They belong to the kernel
# sources whose digest is PMC_SOURCES_SHA256 (kernel_sources_sha256 below): when the sources have changed since the
# profile, no traffic figure is reported.
PMC_FETCH_SCALE, PMC_WRITE_SCALE = 2.0, 1.0
PMC_SOURCES_SHA256 = "d9c026c0d3e07d77b1959417be03cf789c9f51952ba1a1782b13b9803885a19b"
PMC_KIB_DEFAULT_WORKLOAD = {
    "project_bin": (129117, 244115),
    "bin_scatter": (96028, 166743),
    "tile_count": (13152, 2296),
    "tile_scatter": (26691, 108508),
    "cell_sort": (35350, 42126),
    "blend": (317781, 195746),
    "backward_prologue": (55, 265170),
    "backward_tiles": (426000, 121572),
    "backward_points": (297376, 234503),
    "adam_fused": (383789, 498420),
}
SPLAT_KERNEL_SOURCES = ("splat_forward.hip", "splat_backward.hip", "misc_kernels.hip", "trips_splat_abi.hip",
                        "splat_internal.h", "trips_math.h", "row16.h")


def kernel_sources_sha256():
    """Digest of the sources of the splat and Adam kernels, as shipped next to this file."""
    import hashlib
    h = hashlib.sha256()
    for name in SPLAT_KERNEL_SOURCES:
        with open(os.path.join(ROOT, "trips_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


# The sort + blend of the forward runs as two launches (the lists of the cells sorted and cut, then the pixels merged
# and blended); the algorithmic bytes of the sort + blend are those of the pair, so the two are reported as one kernel
# with parts.
KERNEL_PARTS = {"sort_blend": ("cell_sort", "blend")}


def merge_parts(prof):
    """prof: name -> (ms summed over launches, launches). Returns the same with the parts of KERNEL_PARTS folded into
    one entry (its launches = those of the first part) and the parts' own average times."""
    prof = dict(prof)
    parts_ms = {}
    for whole, parts in KERNEL_PARTS.items():
        present = [k for k in parts if k in prof]
        if not present:
            continue
        launches = prof[present[0]][1]
        parts_ms[whole] = {k: prof[k][0] / max(prof[k][1], 1) for k in present}
        total = sum(prof.pop(k)[0] for k in present)
        prof[whole] = (total, launches)
    return prof, parts_ms


def measured_traffic_bytes(kernel, usable=True):
    """HBM bytes per launch from the committed counter profile; a kernel reported with parts is the sum of its parts."""
    parts = KERNEL_PARTS.get(kernel, (kernel,))
    if not usable or any(k not in PMC_KIB_DEFAULT_WORKLOAD for k in parts):
        return None
    return sum(int((PMC_KIB_DEFAULT_WORKLOAD[k][0] * PMC_FETCH_SCALE + PMC_KIB_DEFAULT_WORKLOAD[k][1] * PMC_WRITE_SCALE) * 1024)
               for k in parts)


def algorithmic_bytes(c, n_points, channels=4, adam_nonzero=0, adam_zero=0, adam_step_bytes=4):
    """Algorithmic HBM bytes per launch of each kernel, from the run's own counters
    (N points, E list entries, R retained entries, P pyramid pixels). Adam: an updated element reads w, g, m, v and its
    step counter and writes w, m, v and the counter (28 + 2 x counter bytes: 44 with the reference's int64 counters,
    36 with int32 ones); an element with zero gradient is counted with 8 bytes in both."""
    N, E, R, P, C = n_points, c["E"], c["R"], c["P"], channels
    return {
        "project_bin": 24 * N,                                    # position 16 + size 4 + index 4
        "tile_scatter": 8 * E,                                    # one 64-bit key written per entry
        "sort_blend": 8 * E + (20 + 4 + 4 * C + 28) * R + 4 * C * P,  # keys read, record+conf+descriptor, saved, image
        # the backward's bytes split as its two passes split the work: the compositing (tile pass) reads dL/dimage, the
        # saved entry, descriptor and confidence; the geometry (point pass) reads position + size again (20 B per entry)
        # and makes the one write per accumulated gradient float. (The prologue that clears the pair rows has no
        # algorithmic bytes: its time counts, its bytes do not.)
        "backward_tiles": 4 * C * P + (28 + 4 * C + 4) * R,
        "backward_points": (20 + 4 * C + 4 + 12 + 4) * R,
        "adam_fused": (28 + 2 * adam_step_bytes) * adam_nonzero + 8 * adam_zero,
    }


def measure_other_config(ctx, name, steps):
    """One of the other BASELINE configurations (1, 2, 4) at its full size, beside the headline: wall time of the forward
    and of forward + backward with inputs resident, per-kernel times, the run's counters, the algorithmic bytes that
    follow from them and the fraction of the HBM peak they stand for. Configuration 1 is forward-only by definition."""
    import numpy as np
    import torch
    from trips_amd import abi, scenes
    from trips_amd.renderer import SplatContext
    dev = ctx.device
    sc = getattr(scenes, name)()
    backward = name != "config1"
    desc = abi.desc_for_scene(sc, train=backward)
    f = lambda a, dt=torch.float32: torch.as_tensor(np.ascontiguousarray(a), dtype=dt).to(dev).contiguous()
    t = dict(position=f(sc.position), point_size=f(sc.point_size), index=f(sc.index, torch.int32), texture=f(sc.texture),
             confidence=f(sc.confidence), background=f(sc.background), poses_se3=f(sc.poses_se3, torch.float64),
             intrinsics=f(sc.intrinsics), dropout=None)
    tin = SplatContext.make_in(**t)
    workspace = ctx.alloc_bytes(ctx.workspace_size(desc))
    saved = ctx.alloc_bytes(ctx.saved_size(desc)) if backward else None
    images = ctx.alloc_images(desc)
    N, C, B = desc.num_points, desc.num_channels, desc.num_views
    grads = grad_images = None
    if backward:
        gen = torch.Generator(device=dev)
        gen.manual_seed(4321)
        grad_images = [torch.randn(im.shape, generator=gen, device=dev, dtype=torch.float32) for im in images]
        grads = dict(d_texture=torch.zeros((C, N), device=dev), d_confidence=torch.zeros(N, device=dev),
                     d_background=torch.zeros(C, device=dev), d_position=torch.zeros((N, 4), device=dev),
                     d_point_size=torch.zeros(N, device=dev),
                     d_pose=torch.zeros((desc.num_images, 6), dtype=torch.float64, device=dev),
                     d_intrinsics=torch.zeros((desc.num_cameras, 13), device=dev))

    def fwd():
        ctx.forward(desc, tin, images, saved, workspace)

    def both():
        ctx.forward(desc, tin, images, saved, workspace)
        ctx.backward(desc, tin, saved, grad_images, grads, workspace, overwrite_point_grads=True, clear_block_sums=True)

    def wall(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps

    out = {"workload": sc.name + ": " + " ".join((getattr(scenes, name).__doc__ or "").split()),
           "points": N, "views": B, "width": sc.width, "height": sc.height, "layers": desc.num_layers,
           "list_depth": desc.list_depth, "ms_forward": round(wall(fwd), 4)}
    if backward:
        out["ms_forward_backward"] = round(wall(both), 4)
        ctx.check(workspace)
        per_view = [ctx.counters(desc, saved, b) for b in range(B)]
        c = {k: sum(v[k] for v in per_view) for k in ("valid", "E", "R", "P")}
        out["counters"] = c
        ctx.profile_enable(True)
        ctx.profile_read()
        for _ in range(steps):
            both()
        torch.cuda.synchronize()
        prof, _parts = merge_parts(ctx.profile_read())
        ctx.profile_enable(False)
        kern = {k: round(ms / steps, 4) for k, (ms, n) in prof.items()}  # per step: all views
        out["kernels_ms_per_step"] = kern
        alg = algorithmic_bytes(c, N * B, C)
        alg_fb = sum(v for k, v in alg.items() if k != "adam_fused")
        k_ms = sum(kern.values())
        out["fwd_bwd_kernels_ms"] = round(k_ms, 4)
        out["alg_bytes_fwd_bwd"] = int(alg_fb)
        out["hbm_frac_fwd_bwd"] = round(alg_fb / (k_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4) if k_ms > 0 else None
        out["points_per_s_fwd_bwd"] = round(N * B / (out["ms_forward_backward"] * 1e-3), 1)
    else:
        out["points_per_s_forward"] = round(N * B / (out["ms_forward"] * 1e-3), 1)
    del workspace, saved, images, grads, grad_images, t, tin
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--points", type=int, default=DEFAULT_POINTS)
    ap.add_argument("--point-order", choices=("random", "morton_blocks"), default="random",
                    help="memory order of the synthetic cloud: random (default, the workload the metric is quoted on) or "
                         "the order the reference's scene preprocessing produces")
    ap.add_argument("--no-order-variant", action="store_true",
                    help="skip the second splat measurement with the points in the reference's preprocessing order")
    ap.add_argument("--no-graph", action="store_true", help="skip the HIP-graph replay of the step that is reported beside the eager one")
    ap.add_argument("--cpu-steps", type=int, default=3, help="oracle steps for the cpu_baseline sample (0 = skip)")
    ap.add_argument("--no-net", action="store_true", help="skip the reconstruction-net forward that is reported beside the splat")
    ap.add_argument("--no-adam-variants", action="store_true",
                    help="skip the separate timing of the optimiser kernel with int32 and int64 step counters")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip the block that measures BASELINE configurations 1, 2 and 4 beside the headline workload")
    ap.add_argument("--only-config", choices=("config1", "config2", "config4"), default=None,
                    help="measure that BASELINE configuration alone and print its block (for profiler runs; no headline line)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run three plain 256 MiB device copies, the yardstick for rocprofv3 FETCH_SIZE / WRITE_SIZE")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (--gpus 1); nothing here shards across devices",
              file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from trips_amd import abi, scenes
    from trips_amd.adam import MyAdam, MyAdamPoints
    from trips_amd.renderer import SplatContext, get_context

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    ctx = get_context(0)
    dev = ctx.device
    if args.only_config:
        print(json.dumps({args.only_config: measure_other_config(ctx, args.only_config, args.steps)}))
        return

    def splat_run(order):
        """Builds config 3 with the given memory order of the points and times warm-up + steps of the splat step."""
        sc = scenes.config3(n=args.points, order=order)
        desc = abi.desc_for_scene(sc)
        f = lambda a, dt=torch.float32: torch.as_tensor(np.ascontiguousarray(a), dtype=dt).to(dev).contiguous()
        t = dict(position=f(sc.position), point_size=f(sc.point_size), index=f(sc.index, torch.int32),
                 texture=f(sc.texture), confidence=f(sc.confidence), background=f(sc.background),
                 poses_se3=f(sc.poses_se3, torch.float64), intrinsics=f(sc.intrinsics), dropout=None)
        tin = SplatContext.make_in(**t)
        workspace = ctx.alloc_bytes(ctx.workspace_size(desc))
        saved = ctx.alloc_bytes(ctx.saved_size(desc))
        images = ctx.alloc_images(desc)
        gen = torch.Generator(device=dev)
        gen.manual_seed(1234)
        grad_images = [torch.randn(im.shape, generator=gen, device=dev, dtype=torch.float32) for im in images]
        N, C = desc.num_points, desc.num_channels
        grads = dict(d_texture=torch.zeros((C, N), device=dev), d_confidence=torch.zeros(N, device=dev),
                     d_background=torch.zeros(C, device=dev), d_position=torch.zeros((N, 4), device=dev),
                     d_point_size=torch.zeros(N, device=dev), d_pose=torch.zeros((1, 6), dtype=torch.float64, device=dev),
                     d_intrinsics=torch.zeros((1, 13), device=dev))
        params = [torch.nn.Parameter(t[k]) for k in ("position", "point_size", "texture", "confidence")]
        gkeys = ("d_position", "d_point_size", "d_texture", "d_confidence")
        for p, k in zip(params, gkeys):
            p.grad = grads[k]
        # the optimiser of the point parameters, its state packed per point (int32 step counters): a point that the view
        # culls costs it the read of its zero gradients and nothing else
        opt = MyAdamPoints(params, *params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8)

        def step():
            # the per-point gradients are written by the backward, every element; the block sums (background, pose,
            # intrinsics) are cleared by the backward itself before it adds to them
            ctx.forward(desc, tin, images, saved, workspace)
            ctx.backward(desc, tin, saved, grad_images, grads, workspace, overwrite_point_grads=True, clear_block_sums=True)
            opt.step()

        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        ctx.check(workspace)
        counters = ctx.counters(desc, saved, 0)
        nz = sum(int((grads[k] != 0).sum().item()) for k in gkeys)
        total_el = sum(int(grads[k].numel()) for k in gkeys)

        # the timed region: exactly `steps` steps, nothing but the product's own launches on the stream
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        ms_per_step = (t1 - t0) * 1e3 / args.steps
        # the same steps once more with a pair of HIP events around every kernel, on the launch stream: the per-kernel
        # durations (the events and the gaps they open cost about 4 % of the step, which is why they are not part of
        # the region that `value` is taken from)
        ctx.profile_enable(True)
        ctx.profile_read()
        torch.cuda.synchronize()
        e0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        e1 = time.perf_counter()
        prof = ctx.profile_read()
        ctx.profile_enable(False)
        ms_per_step_events = (e1 - e0) * 1e3 / args.steps
        # the same step captured once into a HIP graph and replayed: the launch gaps of the eager loop are gone
        graph_ms = None
        if not args.no_graph:
            side = torch.cuda.Stream()
            with torch.cuda.stream(side):
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=side):
                    step()
            torch.cuda.synchronize()
            for _ in range(2):
                graph.replay()
            torch.cuda.synchronize()
            g0 = time.perf_counter()
            for _ in range(args.steps):
                graph.replay()
            torch.cuda.synchronize()
            graph_ms = (time.perf_counter() - g0) * 1e3 / args.steps
            del graph
        # the forward as a viewer runs it: eval mode, nothing kept for a backward
        desc_eval = abi.desc_for_scene(sc, train=False)
        ws_eval = ctx.alloc_bytes(ctx.workspace_size(desc_eval))
        for _ in range(3):
            ctx.forward(desc_eval, tin, images, None, ws_eval)
        torch.cuda.synchronize()
        v0 = time.perf_counter()
        for _ in range(args.steps):
            ctx.forward(desc_eval, tin, images, None, ws_eval)
        torch.cuda.synchronize()
        eval_ms = (time.perf_counter() - v0) * 1e3 / args.steps
        del ws_eval
        # the same step with the optimiser state laid out as the reference lays it out (one array per tensor, int64 step
        # counters): what a caller gets who keeps the reference's optimiser structure
        ref_layout_ms = None
        if not args.no_adam_variants:
            o3 = MyAdam(params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, param_steps_dtype=torch.int64)

            def step_ref_layout():
                ctx.forward(desc, tin, images, saved, workspace)
                ctx.backward(desc, tin, saved, grad_images, grads, workspace, overwrite_point_grads=True, clear_block_sums=True)
                o3.step()

            for _ in range(max(args.warmup, 2)):
                step_ref_layout()
            torch.cuda.synchronize()
            r0 = time.perf_counter()
            for _ in range(args.steps):
                step_ref_layout()
            torch.cuda.synchronize()
            ref_layout_ms = (time.perf_counter() - r0) * 1e3 / args.steps
            del o3
        # Adam on its own, with the step counters the product uses (int32) and with the reference's int64 state tensor
        adam_ms = {}
        for name, dt in (() if args.no_adam_variants else (("int32_counters", torch.int32), ("int64_counters", torch.int64))):
            o2 = MyAdam(params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, param_steps_dtype=dt)
            for _ in range(2):
                o2.step()
            torch.cuda.synchronize()
            ctx.profile_enable(True)
            ctx.profile_read()
            for _ in range(args.steps):
                o2.step()
            torch.cuda.synchronize()
            ms, launches = ctx.profile_read()["adam_fused"]  # HIP events around the launch, as for the step's kernels
            ctx.profile_enable(False)
            adam_ms[name] = ms / max(launches, 1)
            del o2
        return dict(ref_layout_ms=ref_layout_ms, graph_ms=graph_ms, events_ms=ms_per_step_events, eval_ms=eval_ms, adam_ms=adam_ms, sc=sc, desc=desc, t=t, tin=tin, workspace=workspace, saved=saved, images=images, gen=gen,
                    grad_images=grad_images, grads=grads, opt=opt, counters=counters, nz=nz, total_el=total_el,
                    prof=prof, ms_per_step=ms_per_step)

    other_order = None
    if args.point_order == "random" and not args.no_order_variant:
        # the same cloud in the memory order real TRIPS scenes have after the reference's preprocessing
        r = splat_run("morton_blocks")
        ms_k = {k: ms / max(n, 1) * (n / args.steps) for k, (ms, n) in merge_parts(r["prof"])[0].items()}
        other_order = {"point_order": "morton_blocks (Morton curve, blocks of 256 shuffled: SceneData.cpp:115-116)",
                       "ms_per_step": round(r["ms_per_step"], 4),
                       "ms_per_step_hip_graph": None if r["graph_ms"] is None else round(r["graph_ms"], 4),
                       "forward_eval_mode_ms": round(r["eval_ms"], 4),
                       "fwd_bwd_kernels_ms": round(sum(v for k, v in ms_k.items() if k != "adam_fused"), 4),
                       "points_per_s": round(r["desc"].num_points / (r["ms_per_step"] * 1e-3), 1),
                       "kernels_ms": {k: round(v, 4) for k, v in ms_k.items()}}
        del r
        torch.cuda.empty_cache()

    r = splat_run(args.point_order)
    sc, desc, t, tin, workspace, saved, images = (r[k] for k in ("sc", "desc", "t", "tin", "workspace", "saved", "images"))
    gen, grad_images, grads, opt, counters = (r[k] for k in ("gen", "grad_images", "grads", "opt", "counters"))
    nz, total_el, prof, ms_per_step = r["nz"], r["total_el"], r["prof"], r["ms_per_step"]
    N, C = desc.num_points, desc.num_channels

    # the timed step runs the product's optimiser state: int32 step counters, 36 bytes per updated element
    alg = algorithmic_bytes(counters, N, C, adam_nonzero=nz, adam_zero=total_el - nz, adam_step_bytes=4)
    alg_adam_i64 = algorithmic_bytes(counters, N, C, adam_nonzero=nz, adam_zero=total_el - nz, adam_step_bytes=8)["adam_fused"]
    pmc_usable = (args.points == DEFAULT_POINTS and args.point_order == "random" and
                  kernel_sources_sha256() == PMC_SOURCES_SHA256)
    kernels = {}
    prof, parts_ms = merge_parts(prof)
    for name, (ms, launches) in prof.items():
        avg = ms / max(launches, 1)
        entry = {"avg_ms": round(avg, 4), "launches_per_step": launches / args.steps}
        if name in parts_ms:
            entry["parts_ms"] = {k: round(v, 4) for k, v in parts_ms[name].items()}
        if name in alg and avg > 0:
            entry["alg_bytes"] = int(alg[name])
            entry["alg_GBs"] = round(alg[name] / (avg * 1e-3) / 1e9, 1)
            entry["roofline_frac"] = round(alg[name] / (avg * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
        traffic = measured_traffic_bytes(name, pmc_usable)
        if traffic is not None:
            entry["traffic_bytes"] = traffic
            if name in alg:
                entry["traffic_over_alg"] = round(traffic / alg[name], 2)
        kernels[name] = entry
    dom = max((k for k in kernels if k in alg), key=lambda k: kernels[k]["avg_ms"] * kernels[k]["launches_per_step"])
    achieved = kernels[dom]["alg_GBs"]
    kernel_ms = sum(v["avg_ms"] * v["launches_per_step"] for v in kernels.values())
    fwd_bwd_ms = sum(v["avg_ms"] * v["launches_per_step"] for k, v in kernels.items() if k != "adam_fused")

    if args.calibration_copy:
        src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()

    # The reconstruction net that consumes the pyramid (next row after the splat): forward only, on the images
    # the splat just rendered. 4 levels, filters 16/32/64/64, fp16 operands on the matrix cores.
    unet = None
    if not args.no_net:
        from trips_amd.unet import MultiScaleUnet2dDecOnlySmallFixed, MultiScaleUnet2dParams
        np_ = MultiScaleUnet2dParams(num_input_layers=desc.num_layers, num_layers=4, filters_network=[16, 32, 64, 64])
        net = MultiScaleUnet2dDecOnlySmallFixed(np_).he_normal_(torch.Generator().manual_seed(5)).to(dev)
        with torch.no_grad():
            # as a viewer runs it: the weights do not change between frames, so their fp16 packing (one small launch)
            # is done by the first frame only; then the same with the packing in every call, as a training step has it
            net.reuse_packed_weights = True
            for _ in range(3):
                rgb = net.forward(images)
            torch.cuda.synchronize()
            ctx.profile_enable(True)
            ctx.profile_read()
            for _ in range(args.steps):
                rgb = net.forward(images)
            torch.cuda.synchronize()
            nprof = ctx.profile_read()
            net.reuse_packed_weights = False
            net.invalidate_packed_weights()
            for _ in range(args.steps):
                rgb = net.forward(images)
            torch.cuda.synchronize()
            nprof_packing = ctx.profile_read()
            ctx.profile_enable(False)
        net_ms = sum(ms for ms, _ in nprof.values()) / args.steps
        net_ms_packing = sum(ms for ms, _ in nprof_packing.values()) / args.steps
        flops = net.flops(images)
        unet = {"workload": "MultiScaleUnet2dDecOnlySmallFixed forward, 4 levels 16/32/64/64, 1920x1080, fp16 operands / "
                            "fp32 accumulate, He-normal weights, input = the splat's pyramid",
                "ms_forward": round(net_ms, 4), "ms_forward_packing_weights_every_call": round(net_ms_packing, 4),
                "gflop": round(flops / 1e9, 2),
                "tflops": round(flops / (net_ms * 1e-3) / 1e12, 1),
                "mfma_frac_of_fp16_dense_peak": round(flops / (net_ms * 1e-3) / 2.5e15, 4),
                "kernels": {k: round(ms / max(n, 1), 4) for k, (ms, n) in nprof.items()}}

        # The full training step of the fifth configuration: splat forward, net forward, L1 loss against a uniform
        # target, net backward, splat backward with the net's input gradients, fused Adam over point and net
        # parameters.
        target = torch.rand(rgb.shape, generator=gen, device=dev)
        net_params = [q for q in net.parameters()]
        net_opt = MyAdam(net_params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8)
        zero_tail = [torch.zeros_like(im) for im in images[np_.num_layers:]]

        def train_step():
            net_opt.zero_grad(set_to_none=True)
            ctx.forward(desc, tin, images, saved, workspace)
            ins = [im.detach().requires_grad_(True) for im in images]
            loss = (net.forward(ins) - target).abs().mean()
            loss.backward()
            gi = [t.grad for t in ins[:np_.num_layers]] + zero_tail
            ctx.backward(desc, tin, saved, gi, grads, workspace, overwrite_point_grads=True, clear_block_sums=True)
            opt.step()
            net_opt.step()
            return loss

        for _ in range(3):
            train_step()
        torch.cuda.synchronize()
        c0 = time.perf_counter()
        for _ in range(args.steps):
            train_step()
        torch.cuda.synchronize()
        c1 = time.perf_counter()
        # (once more with the events around every kernel, for the per-kernel figures)
        ctx.profile_enable(True)
        ctx.profile_read()
        for _ in range(args.steps):
            train_step()
        torch.cuda.synchronize()
        tprof = ctx.profile_read()
        ctx.profile_enable(False)
        # the same training step captured once into a HIP graph and replayed (autograd included: every tensor it
        # creates comes out of the graph's own memory pool, so the replays run on the addresses of the capture)
        train_graph_ms = None
        if not args.no_graph:
            try:
                side = torch.cuda.Stream()
                with torch.cuda.stream(side):
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph, stream=side):
                        train_step()
                torch.cuda.synchronize()
                for _ in range(2):
                    graph.replay()
                torch.cuda.synchronize()
                g0 = time.perf_counter()
                for _ in range(args.steps):
                    graph.replay()
                torch.cuda.synchronize()
                train_graph_ms = (time.perf_counter() - g0) * 1e3 / args.steps
                del graph
            except Exception as e:  # the eager figure above stands on its own
                print(f"bench.py: graph capture of the config-5 step failed: {e}", file=sys.stderr)
        net_bwd_ms = sum(ms for k, (ms, _) in tprof.items() if k.startswith("unet_bwd")) / args.steps
        net_fwd_ms = sum(ms for k, (ms, _) in tprof.items() if k.startswith("unet_") and not k.startswith("unet_bwd")) / args.steps
        unet["train_step"] = {
            "workload": "config5: splat forward + net forward + L1 loss + net backward + splat backward + fused Adam "
                        "(point parameters and net weights), 6M points, 1920x1080",
            "ms_per_step_wall": round((c1 - c0) * 1e3 / args.steps, 4),
            "ms_per_step_hip_graph": None if train_graph_ms is None else round(train_graph_ms, 4),
            "ms_all_kernels": round(sum(ms for ms, _ in tprof.values()) / args.steps, 4),
            "ms_net_forward": round(net_fwd_ms, 4), "ms_net_backward": round(net_bwd_ms, 4),
            "net_backward_tflops": round(2 * flops / (net_bwd_ms * 1e-3) / 1e12, 1) if net_bwd_ms > 0 else None,
            "kernels": {k: round(ms / max(n, 1), 4) for k, (ms, n) in tprof.items() if k.startswith("unet_bwd")}}

    # the other BASELINE configurations, each at its full size, outside the region that `value` is timed in
    other_configs = None
    if not args.no_other_configs:
        other_configs = {name: measure_other_config(ctx, name, max(5, args.steps // 2)) for name in ("config1", "config2", "config4")}

    cpu = None
    if args.cpu_steps > 0:
        from tests import oracle_lib
        oracle = oracle_lib.load()
        ref = oracle.forward(sc, desc, want_points=False)  # warm-up, also allocates
        gi = [g.cpu().numpy() for g in grad_images]
        c0 = time.perf_counter()
        for _ in range(args.cpu_steps):
            ref = oracle.forward(sc, desc, want_points=False)
            oracle.backward(sc, desc, ref, gi)
        c1 = time.perf_counter()
        cpu_ms = (c1 - c0) * 1e3 / args.cpu_steps
        cpu = {"value": round(N / (cpu_ms * 1e-3), 1), "unit": "points/s", "cores": oracle.num_threads(),
               "kind": "port", "ms_per_step": round(cpu_ms, 1),
               "sample": f"{args.cpu_steps} forward+backward passes (no Adam) of the same {N}-point 1920x1080 view "
                         "with the OpenMP C++ oracle"}

    out = {
        "metric": "splatted points/s fwd+bwd (6M pts, 1080p); frame ms; % HBM peak",
        "value": round(N / (ms_per_step * 1e-3), 1),
        "unit": "points/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        # the same step with the reference's optimiser state layout (per-tensor arrays, int64 step counters) instead of
        # the packed per-point rows that `value` is timed with
        "ms_per_step_reference_adam_layout": None if r["ref_layout_ms"] is None else round(r["ref_layout_ms"], 4),
        "value_reference_adam_layout": None if r["ref_layout_ms"] is None else round(N / (r["ref_layout_ms"] * 1e-3), 1),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "config3: 6M points (80% noisy ground plane, 20% box), 1920x1080, 8 layers, K=16, "
                               "4-ch f32 descriptors; forward + backward + fused Adam, 1 view",
                   "point_order": args.point_order, "points": N, "width": sc.width, "height": sc.height, "layers": desc.num_layers,
                   "list_depth": desc.list_depth, "counters": counters},
        "frame_ms": {"fwd_bwd_kernels": round(fwd_bwd_ms, 4), "all_kernels": round(kernel_ms, 4),
                     "wall_per_step": round(ms_per_step, 4), "wall_per_step_with_kernel_events": round(r["events_ms"], 4),
                     "wall_per_step_hip_graph": None if r["graph_ms"] is None else round(r["graph_ms"], 4),
                     "forward_eval_mode": round(r["eval_ms"], 4),
                     "kernel_times_from": "a second pass of the same steps with HIP events around every kernel; the timed "
                                          "region that value comes from carries no events"},
        "hbm_frac_fwd_bwd": round(sum(alg[k] for k in alg if k != "adam_fused") / (fwd_bwd_ms * 1e-3) / 1e9 /
                                  HBM_PEAK_GBS, 4) if fwd_bwd_ms > 0 else None,
        # How busy the memory system was, NOT the target metric: the HBM traffic rocprofv3 measured (committed summary
        # under profiles/; wasted re-reads included) per second of forward + backward kernels over the peak. null when
        # the kernel sources have changed since that profile.
        "hbm_busy_frac": round(
            sum(measured_traffic_bytes(k) for k in PMC_KIB_DEFAULT_WORKLOAD if k != "adam_fused") / (fwd_bwd_ms * 1e-3) / 1e9 /
            HBM_PEAK_GBS, 4) if (fwd_bwd_ms > 0 and pmc_usable) else None,
        "traffic_profile": {"sources_sha256": PMC_SOURCES_SHA256, "matches_these_sources": pmc_usable},
        "roofline": {"kernel": dom, "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": measured_traffic_bytes(dom, pmc_usable),
                     "algorithmic_bytes": int(alg[dom]), "avg_ms": kernels[dom]["avg_ms"]},
        # the kernel whose measured traffic is furthest above its algorithmic bytes
        "worst_traffic_ratio": (lambda c: {"kernel": c[0], "traffic_over_alg": c[1]} if c else None)(
            max(((k, v["traffic_over_alg"]) for k, v in kernels.items() if "traffic_over_alg" in v),
                key=lambda kv: kv[1], default=None)),
        "adam": None if not r["adam_ms"] else {
            "timed_step_state": "packed per point: {first moment, second moment, int32 step counter} of a point's 10 "
                                "elements in one 128-byte row (36 B per updated element)",
            "kernel_ms_packed_state_in_step": round(kernels["adam_fused"]["avg_ms"], 4),
            "per_tensor_state": "the same step with the reference's state layout (one array per tensor), kernel alone, "
                                "gradients of the last step",
            "kernel_ms_int32_counters": round(r["adam_ms"]["int32_counters"], 4),
            "kernel_ms_int64_counters": round(r["adam_ms"]["int64_counters"], 4),
            "alg_bytes_int32": int(alg["adam_fused"]), "alg_bytes_int64": int(alg_adam_i64),
            "alg_GBs_int32": round(alg["adam_fused"] / (r["adam_ms"]["int32_counters"] * 1e-3) / 1e9, 1),
            "alg_GBs_int64": round(alg_adam_i64 / (r["adam_ms"]["int64_counters"] * 1e-3) / 1e9, 1)},
        "kernels": kernels,
        "other_point_order": other_order,
        "other_configs": other_configs,
        "unet": unet,
        "cpu_baseline": cpu,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
