"""Headline benchmark: TV inpainting forward + backward, 4 x 2 x 384 x 1248, 100 FISTA iterations.

One "step" is one forward and one backward call of the layer on the whole batch, inputs resident
in HBM.  Prints ONE JSON line.  The metric is pixel-iterations per second (one pixel of one sample,
all channels, advanced through one iteration of the forward and its share of the backward).
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# Peak LDS rate: 128 B per clock and CU x 256 CUs x 2.4 GHz.
LDS_PEAK_GBS = 128 * 256 * 2.4


def sources_sha16(files):
    """First 16 hex digits of the SHA-256 over the named source files (paths relative to the repository root)."""
    import hashlib

    h = hashlib.sha256()
    for f in sorted(files):
        with open(os.path.join(ROOT, f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def load_counters(config):
    """Counter figures that no bench run can take itself (rocprofv3 --pmc needs a run of its own), from
    profiles/counters.json -- the same file the text summaries under profiles/ are written from.  Per workload:
      traffic_bytes   HBM bytes per launch of the dominant kernel: FETCH_SIZE (scaled by the copy-kernel calibration
                      of the same run) + WRITE_SIZE
      step_bytes      HBM bytes of one whole forward+backward (every kernel and copy)
      lds_bytes       LDS bytes per launch of the dominant kernel (SQ_INSTS_LDS x 64 lanes x 8 B; the TV strip kernels
                      issue no LDS instruction at all -- neighbours are exchanged through DPP in registers)
      rocprof_avg_us  average duration of the dominant kernel in the rocprofv3 --kernel-trace --stats summary
      sources, sources_sha16   the kernel sources the figures were read at; `stale` is set when they have changed since
    Returns None when the file has no entry for the workload."""
    path = os.path.join(ROOT, "profiles", "counters.json")
    if not os.path.exists(path):
        return None
    with open(path) as fh:
        entry = json.load(fh).get("configs", {}).get(str(config))
    if entry is None:
        return None
    entry = dict(entry)
    entry["stale"] = sources_sha16(entry["sources"]) != entry["sources_sha16"]
    return entry


def physical_roofline(roof, cnt, kernel_ms, key="traffic_bytes"):
    """Fills the roofline entry: `achieved` / `frac` are the bytes the kernel really moves (counters) over its launch
    time, a rate that cannot exceed the peak; `model_achieved` / `model_frac` are the algorithmic bytes (what
    `bytes_per_launch` counts) over the same time, which can: a launch that fuses two steps keeps the value between them
    in registers, and the model charges it a round trip.  Without counters only the model figures are given."""
    model = roof["bytes_per_launch"] / (kernel_ms * 1e-3) / 1e9 if kernel_ms > 0 else 0.0
    roof["model_achieved"] = round(model, 1)
    roof["model_frac"] = round(model / HBM_PEAK_GBS, 4)
    if cnt and key in cnt and kernel_ms > 0:
        gbs = cnt[key] / (kernel_ms * 1e-3) / 1e9
        roof["achieved"] = round(gbs, 1)
        roof["frac"] = round(gbs / HBM_PEAK_GBS, 4)
        roof["traffic"] = cnt[key]
        roof["counters_from"] = {"files": cnt["files"], "library_commit": cnt["library_commit"]}
        roof["counters_stale"] = cnt["stale"]
    else:
        roof["achieved"] = None
        roof["frac"] = None
        roof["traffic"] = None
    roof["basis"] = ("achieved, frac: HBM bytes per launch read off FETCH_SIZE + WRITE_SIZE (profiles/counters.json) / launch time; "
                     "model_achieved, model_frac: algorithmic bytes per launch (bytes_per_launch) / the same time")
    return roof


def algorithmic_bytes_per_pixel(c, kind="tv"):
    """One HBM round trip per iteration, fp32.  TV: forward 5C+3, recompute 6C+3, adjoint 10C+9
    floats.  TGV (three state variables, four weight fields): forward 13C+5, recompute 16C+5,
    adjoint 22C+15 floats."""
    if kind == "tgv":
        return dict(forward=4 * (13 * c + 5), recompute=4 * (16 * c + 5), adjoint=4 * (22 * c + 15),
                    total=4 * (51 * c + 25))
    return dict(forward=4 * (5 * c + 3), recompute=4 * (6 * c + 3), adjoint=4 * (10 * c + 9),
                total=4 * (21 * c + 15))


def layer_of(kind):
    """(binding module, C-ABI prefix, input generator, oracle class name, dominant kernel)."""
    from customnetworklayers_amd import workloads
    if kind == "tgv":
        from customnetworklayers_amd.cudaTGV import tgvInpaint_cuda_ext as ext
        return ext, "tgvinpaint", workloads.tgv_inputs, "TGVOracle", "tgvstrip::tgv_adjoint_strip2w<2,false,false>"
    from customnetworklayers_amd.cudaTV import tvInpaint_cuda_ext as ext
    return ext, "tvinpaint", workloads.tv_inputs, "TVOracle", "tvstrip::tv_adjoint_strip2<2,false,false>"


def cpu_baseline(cfg, whole=False):
    """The CPU oracle on a bounded sample of the same workload: ONE sample of the batch, all
    iterations, forward + backward, all host cores (best of 2 after a warm-up) and one core.
    `whole`: the workload has one sample, so the sample is the workload."""
    import oracle.oracle_lib as oracle_lib

    _, _, make_inputs, oracle_name, _ = layer_of(cfg["kind"])
    o = getattr(oracle_lib, oracle_name)()
    o.set_quirks()
    d = make_inputs(1, cfg["c"], cfg["h"], cfg["w"], seed=0, **cfg["gen"])
    its = cfg["its"]
    pxit = cfg["h"] * cfg["w"] * 2 * (its // 2)

    def once():
        o.reset_id(9)
        t0 = time.perf_counter()
        o.forward(d["dx"], d["dy"], d["dc"], d["db"], d["di"], its, 9)
        o.backward(d["grad"].copy(), d["dx"], d["dy"], d["dc"], d["db"], its, 9)
        return time.perf_counter() - t0

    import multiprocessing
    avail = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else multiprocessing.cpu_count()
    cores = min(avail, int(os.environ.get("OMP_NUM_THREADS", "0") or avail))
    o.set_threads(cores)
    once()
    t_all = min(once(), once())
    o.set_threads(1)
    t_one = once()
    o.set_threads(cores)
    return dict(value=round(pxit / t_all / 1e6, 3), unit="Mpixel-iter/s", cores=cores, kind="port",
                sample=("the whole workload (1 x %dx%dx%d), %d iterations, fwd+bwd, best of 2" % (cfg["c"], cfg["h"], cfg["w"], its)) if whole
                       else "1 of %d samples (%dx%dx%d), %d iterations, fwd+bwd, best of 2" % (cfg["n"], cfg["c"], cfg["h"], cfg["w"], its),
                one_core_value=round(pxit / t_one / 1e6, 3), host_cpu_count=os.cpu_count())


def flowaux_cpu_baseline(cfg, d):
    """The CPU oracle on ONE sample of the batch, forward + backward, all host cores (best of 2) and one core."""
    import multiprocessing

    from oracle.oracle_lib import FlowAuxOracle

    o = FlowAuxOracle()
    one = {k: v[:1] for k, v in d.items()}

    def once():
        t0 = time.perf_counter()
        if cfg["kind"] == "quadfit":
            o.quadfit_forward(one["feat0"], one["feat1"], one["flow"])
            o.quadfit_backward(one["grad"], one["feat0"], one["feat1"], one["flow"])
        else:
            o.median_forward(one["vol"])
            o.median_backward(one["grad"], one["vol"])
        return time.perf_counter() - t0

    avail = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else multiprocessing.cpu_count()
    cores = min(avail, int(os.environ.get("OMP_NUM_THREADS", "0") or avail))
    o.set_threads(cores)
    once()
    t_all = min(once(), once())
    o.set_threads(1)
    t_one = once()
    px = cfg["h"] * cfg["w"]
    # the quadratic fit's backward scatter runs one thread per sample in the oracle
    used = 1 if cfg["kind"] == "quadfit" else cores
    return dict(value=round(px / t_all / 1e6, 3), unit="Mpixel/s", cores=cores, kind="port",
                sample="1 of %d samples, fwd+bwd, best of 2%s" % (cfg["n"], " (backward scatter on %d core)" % used
                                                                  if cfg["kind"] == "quadfit" else ""),
                one_core_value=round(px / t_one / 1e6, 3), host_cpu_count=os.cpu_count())


def bench_flowaux(args, cfg, d):
    """Configs 5 and 6: the quadratic fit and the median, forward + backward per step."""
    import torch

    from customnetworklayers_amd._lib import lib

    dev = torch.device("cuda:0")
    t = {k: torch.from_numpy(v).to(dev) for k, v in d.items()}
    n, h, w = cfg["n"], cfg["h"], cfg["w"]
    px = n * h * w
    if cfg["kind"] == "quadfit":
        from customnetworklayers_amd.cudaQuadFit import QuadFit_cuda_ext as ext
        c = cfg["c"]
        fwd = lambda: ext.forward(t["feat0"], t["feat1"], t["flow"])  # noqa: E731
        bwd = lambda: ext.backward(t["grad"], t["feat0"], t["feat1"], t["flow"])  # noqa: E731
        # floats per pixel: forward reads both feature maps and the flow, writes 3; backward reads both maps,
        # flow and upstream, writes g0, zero-fills g1 and read-modify-writes it
        # per-source pass of the backward (the dominant kernel): both maps, flow, upstream in; g0 and 5 coefficients out
        # per-source pass of the backward: both maps, flow, upstream in; g0 and 5 coefficients out (the inverse map not counted)
        # gather pass (the dominant kernel): first map, 5 coefficients, list length and up to 4 list entries in; g1 out
        bpp = dict(forward=4 * (2 * c + 5), backward=4 * (5 * c + 5), kernel=4 * (2 * c + 10), sources=4 * (3 * c + 10))
        kernel = "quadfit_gather_tiles<2> (backward, gather pass)"
        shape = "features %dx%dx%d" % (c, h, w)
    else:
        from customnetworklayers_amd.cudaMedian import median_cuda_ext as ext
        dd = cfg["d"]
        fwd = lambda: ext.forward(t["vol"])  # noqa: E731
        bwd = lambda: ext.backward(t["grad"], t["vol"])  # noqa: E731
        # forward reads the histogram once (it may stop early) and writes 2; backward reads it, the upstream and writes it
        bpp = dict(forward=4 * (dd + 2), backward=4 * (2 * dd + 2), kernel=4 * (2 * dd + 2))
        kernel = "median_stream_kernel<10,true> (backward)"
        shape = "histograms %dx%dx%d" % (h, w, dd)
    bpp["total"] = bpp["forward"] + bpp["backward"]  # "kernel": the dominant kernel alone
    for _ in range(args.warmup):
        fwd(), bwd()
    torch.cuda.synchronize()
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    t0 = time.perf_counter()
    for e in ev:  # events on the stream the kernels are launched on (torch's current stream)
        e[0].record(); fwd(); e[1].record(); bwd(); e[2].record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    f_ms = sum(e[0].elapsed_time(e[1]) for e in ev) / args.steps
    b_ms = sum(e[1].elapsed_time(e[2]) for e in ev) / args.steps

    def kernel_ms(which):
        """HIP events around one kernel of the backward pass, on the stream it is launched on; steps outside the timed region."""
        lib.flowaux_profile(which)
        for _ in range(args.steps):
            bwd()
        torch.cuda.synchronize()
        tot_ms, launches = ctypes.c_double(0), ctypes.c_int(0)
        lib.flowaux_profile_read(ctypes.byref(tot_ms), ctypes.byref(launches))
        lib.flowaux_profile(0)
        return tot_ms.value / max(launches.value, 1), launches.value

    k_ms, launches_timed = kernel_ms(2 if cfg["kind"] == "quadfit" else 1)
    src_ms = kernel_ms(1)[0] if cfg["kind"] == "quadfit" else None
    value = px / (elapsed / args.steps) / 1e6
    cnt = load_counters(args.config)
    out = {
        "metric": "%s fwd+bwd Mpixel/s at %d x %s; achieved HBM GB/s vs peak" % (cfg["kind"], n, shape),
        "value": round(value, 2), "unit": "Mpixel/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(elapsed * 1e3 / args.steps, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "%s fwd+bwd, N=%d, %s fp32 (config %d)" % (cfg["kind"], n, shape, args.config), "pixels_per_step": px},
        "whole_job": {"model_bytes_per_pixel": bpp["total"], "model_GBps": round(bpp["total"] * px / (elapsed / args.steps) / 1e9, 1),
                      "forward_ms": round(f_ms, 4), "backward_ms": round(b_ms, 4),
                      "forward_model_GBps": round(bpp["forward"] * px / (f_ms * 1e-3) / 1e9, 1),
                      "backward_model_GBps": round(bpp["backward"] * px / (b_ms * 1e-3) / 1e9, 1)},
        "roofline": physical_roofline({"bound": "hbm", "kernel": kernel, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                       "bytes_per_launch": bpp["kernel"] * px, "avg_launch_ms": round(k_ms, 5),
                                       "launches_timed": launches_timed}, cnt, k_ms),
    }
    if src_ms is not None:  # the second kernel of the backward pass
        out["roofline"]["per_source_pass"] = physical_roofline(
            {"kernel": "quadfit_sources_resident<32,true>", "avg_launch_ms": round(src_ms, 5), "bytes_per_launch": bpp["sources"] * px},
            cnt, src_ms, key="sources_traffic_bytes")
        out["roofline"]["per_source_pass"].pop("basis")
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = flowaux_cpu_baseline(cfg, d)
    print(json.dumps(out))


def hierarchy_inputs(cfg, n, seed=0):
    """Config 3: per level the confidence / flow of tv_inputs, one guidance-image pyramid per sample."""
    import numpy as np

    from customnetworklayers_amd import workloads

    rng = np.random.default_rng(seed)
    top = cfg["levels"][-1]
    imgs_top = [workloads.smooth_image(rng, *top) for _ in range(n)]
    levels = []
    for lvl, (h, w) in enumerate(cfg["levels"]):
        d = workloads.tv_inputs(n, cfg["c"], h, w, seed=seed + 10 + lvl, **cfg["gen"])
        f = top[0] // h
        d["img"] = np.stack([im[::f, ::f] for im in imgs_top])[:, None].astype(np.float32)
        levels.append(d)
    return levels


def bench_hierarchy(args, cfg):
    """Config 3: three TV layers (ids 0,1,2) coarse to fine with the glue between the levels on the device, then the
    backward passes fine to coarse.  One step = all of it."""
    import torch

    from customnetworklayers_amd import hierarchy
    from customnetworklayers_amd._lib import lib
    from customnetworklayers_amd.cudaTV import tvInpaint_cuda_ext as ext

    dev = torch.device("cuda:0")
    n, c, its = cfg["n"], cfg["c"], cfg["its"]
    levels = hierarchy_inputs(cfg, n)
    t = [{k: torch.from_numpy(v).to(dev) for k, v in d.items()} for d in levels]
    nl = len(t)
    h0, w0 = cfg["levels"][0]
    _, wx0, wy0 = hierarchy.next_level_forward(torch.zeros((n, c, h0 // 2, w0 // 2), dtype=torch.float32, device=dev), t[0]["img"])
    pxit = sum(n * h * w * 2 * (its // 2) for h, w in cfg["levels"])
    glue_ev = []

    def step(time_glue=False, per_level=None):
        feeds, b, wx, wy = [], t[0]["db"], wx0, wy0
        for lvl in range(nl):
            feeds.append((wx, wy, b))
            (sol,) = ext.forward(wx, wy, t[lvl]["dc"], b, b, its, lvl)
            if lvl + 1 < nl:
                if time_glue:
                    e = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
                    e[0].record()
                b, wx, wy = hierarchy.next_level_forward(sol, t[lvl + 1]["img"])
                if time_glue:
                    e[1].record()
                    glue_ev.append(("fwd", lvl, e))
        up = t[-1]["grad"]
        for lvl in reversed(range(nl)):
            wx, wy, b = feeds[lvl]
            g = ext.backward(up, wx, wy, t[lvl]["dc"], b, its, lvl)
            if per_level is not None:
                ms, cnt = ctypes.c_double(0), ctypes.c_int(0)
                lib.tvinpaint_profile_read(ctypes.byref(ms), ctypes.byref(cnt))
                per_level[lvl] = (ms.value, cnt.value)
            if lvl > 0:
                if time_glue:
                    e = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
                    e[0].record()
                up = hierarchy.next_level_backward(g[3], g[4])
                if time_glue:
                    e[1].record()
                    glue_ev.append(("bwd", lvl, e))
        return g

    for lvl in range(nl):
        ext.reset_id(lvl)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    # one more, untimed step with event pairs around the glue launches and around each level's adjoint pair launches
    per_level = {}
    lib.tvinpaint_profile(1)
    step(time_glue=True, per_level=per_level)
    torch.cuda.synchronize()
    lib.tvinpaint_profile(0)
    glue_ms = {"fwd": 0.0, "bwd": 0.0}
    for kind, lvl, e in glue_ev:
        glue_ms[kind] += e[0].elapsed_time(e[1])
    # glue bytes: forward reads sol and the fine image, writes up, wx, wy; backward reads two fine gradients, writes one coarse
    fine = [n * h * w for h, w in cfg["levels"][1:]]
    glue_bytes = {"fwd": sum(4 * (p // 4 * c + p + p * c + 2 * p) for p in fine), "bwd": sum(4 * (2 * p * c + p // 4 * c) for p in fine)}
    bpp = algorithmic_bytes_per_pixel(c, "tv")
    top_ms, top_cnt = per_level[nl - 1]
    h, w = cfg["levels"][-1]
    k_ms = top_ms / max(top_cnt, 1)
    k_bytes = 2 * bpp["adjoint"] * n * h * w
    # the finest level runs the headline's dominant kernel: its counter bytes per pixel, times this level's pixels
    cnt = load_counters(1)
    if cnt:
        cnt = dict(cnt, traffic_bytes=int(cnt["traffic_bytes"] / cnt["pixels"] * n * h * w))
    sec = elapsed / args.steps
    out = {
        "metric": "TV-FISTA hierarchy fwd+bwd Mpixel-iter/s, %d levels up to %dx%dx%dx%d; achieved HBM GB/s vs peak" % (nl, n, c, h, w),
        "value": round(pxit / sec / 1e6, 2), "unit": "Mpixel-iter/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(sec * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "three TV layers coarse to fine with device glue, N=%d, C=%d, levels %s, %d iterations each (config 3)"
                               % (n, c, "/".join("%dx%d" % l for l in cfg["levels"]), its), "pixel_iterations_per_step": pxit},
        "whole_job": {"model_bytes_per_pixel_iteration": bpp["total"], "model_GBps": round(bpp["total"] * pxit / sec / 1e9, 1),
                      "model_frac_of_hbm_peak": round(bpp["total"] * pxit / sec / 1e9 / HBM_PEAK_GBS, 4),
                      "glue_forward_ms": round(glue_ms["fwd"], 4), "glue_backward_ms": round(glue_ms["bwd"], 4),
                      "glue_forward_GBps": round(glue_bytes["fwd"] / (glue_ms["fwd"] * 1e-3) / 1e9, 1),
                      "glue_backward_GBps": round(glue_bytes["bwd"] / (glue_ms["bwd"] * 1e-3) / 1e9, 1)},
        "roofline": physical_roofline({"bound": "hbm", "kernel": "tvstrip::tv_adjoint_strip2<2,false,false> at the finest level",
                                       "peak": HBM_PEAK_GBS, "unit": "GB/s", "bytes_per_launch": k_bytes, "adjoint_steps_per_launch": 2,
                                       "avg_launch_ms": round(k_ms, 5), "launches_timed": top_cnt,
                                       "traffic_scaled_from": "the same kernel on the headline workload, per pixel"}, cnt, k_ms),
    }
    if not args.no_cpu_baseline:
        import oracle.oracle_lib as oracle_lib

        tv, aux = oracle_lib.TVOracle(), oracle_lib.FlowAuxOracle()
        tv.set_quirks()
        one = [{k: v[:1] for k, v in d.items()} for d in levels]

        def once():
            t1 = time.perf_counter()
            feeds, b = [], one[0]["db"]
            wx, wy = aux.edge_weights(one[0]["img"], 10.0)
            for lvl in range(nl):
                feeds.append((wx, wy, b))
                tv.reset_id(lvl)
                sol = tv.forward(wx, wy, one[lvl]["dc"], b, b, its, lvl)
                if lvl + 1 < nl:
                    b = aux.upsample2x(sol, 2.0)
                    wx, wy = aux.edge_weights(one[lvl + 1]["img"], 10.0)
            up = one[-1]["grad"].copy()
            for lvl in reversed(range(nl)):
                wx, wy, b = feeds[lvl]
                g = tv.backward(up.copy(), wx, wy, one[lvl]["dc"], b, its, lvl)
                if lvl > 0:
                    up = aux.upsample2x_adjoint(g[3], g[4], 2.0)
            return time.perf_counter() - t1

        import multiprocessing
        avail = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else multiprocessing.cpu_count()
        cores = min(avail, int(os.environ.get("OMP_NUM_THREADS", "0") or avail))
        tv.set_threads(cores)
        aux.set_threads(cores)
        once()
        t_all = min(once(), once())
        out["cpu_baseline"] = dict(value=round(pxit / n / t_all / 1e6, 3), unit="Mpixel-iter/s", cores=cores, kind="port",
                                   sample="1 of %d samples, all levels, fwd+bwd, best of 2" % n, host_cpu_count=os.cpu_count())
    return out


def event_median_ms(step, steps):
    """Median duration of `steps` more calls of step(), each bracketed by its own pair of HIP events on the stream
    the layers launch on (torch's current stream)."""
    import torch

    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for a, b in ev:
        a.record()
        step()
        b.record()
    torch.cuda.synchronize()
    ms = sorted(a.elapsed_time(b) for a, b in ev)
    return ms[len(ms) // 2]


def bench_layer(config, steps, warmup, corrected=False, keep=None, detail=True):
    """Configs 0, 1, 2, 4: one TV or TGV layer, forward + backward per step.  Returns the result dict."""
    import torch

    from customnetworklayers_amd._lib import lib
    from customnetworklayers_amd.workloads import config_inputs

    dev = torch.device("cuda:0")
    cfg, d = config_inputs(config, seed=0)
    ext, prefix, _, _, kernel_name = layer_of(cfg["kind"])
    if cfg["kind"] == "tv" and (os.environ.get("INPAINT_TV_FUSE", "1") == "0" or os.environ.get("INPAINT_TV_FUSE_ADJ", "1") == "0"):
        kernel_name = "tvstrip::tv_adjoint_strip<2,false,false>"
    if cfg["kind"] == "tgv" and (os.environ.get("INPAINT_TGV_FUSE", "1") == "0" or os.environ.get("INPAINT_TGV_FUSE_ADJ", "1") == "0"):
        kernel_name = "tgvstrip::tgv_adjoint_strip<2,false,false>"
    if corrected:
        kernel_name = kernel_name.replace(">", ",true>")
    profile, profile_read = getattr(lib, prefix + "_profile"), getattr(lib, prefix + "_profile_read")
    t = {k: torch.from_numpy(v).to(dev) for k, v in d.items()}
    its, pid = cfg["its"], 0
    n, c, h, w = cfg["n"], cfg["c"], cfg["h"], cfg["w"]
    pxit = n * h * w * 2 * (its // 2)

    def step():
        (sol,) = ext.forward(t["dx"], t["dy"], t["dc"], t["db"], t["di"], its, pid)
        return ext.backward(t["grad"], t["dx"], t["dy"], t["dc"], t["db"], its, pid)

    ext.reset_id(pid)
    if corrected:
        ext.gradient_mode(pid, 1)
    if keep is not None:
        ext.keep_iterates(pid, keep)
    for _ in range(warmup):
        step()
    # the timed region: exactly `steps` steps between two synchronisations, nothing else inside
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    sec = elapsed / steps
    med_ms = event_median_ms(step, steps)
    slot_bytes = int(getattr(lib, prefix + "_slot_bytes")(pid))
    label = cfg["kind"].upper() + (" (corrected gradient)" if corrected else "")
    out = {
        "metric": "%s-FISTA fwd+bwd Mpixel-iter/s at %dx%dx%dx%d; achieved HBM GB/s vs peak" % (label, n, c, h, w),
        "value": round(pxit / sec / 1e6, 2), "unit": "Mpixel-iter/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(sec * 1e3, 4), "ms_per_step_event_median": round(med_ms, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": label + " inpainting fwd+bwd, N=%d, flow %dx%dx%d fp32, %d FISTA iterations (config %d)"
                               % (n, c, h, w, its, config), "pixel_iterations_per_step": pxit,
                   "keep_mode": 2 if keep is None else keep, "slot_bytes": slot_bytes},
    }
    if not detail:
        ext.reset_id(pid)
        return out, cfg
    # one more, untimed run of steps with event pairs around each reverse sweep's launches of the dominant kernel
    profile(1)
    for _ in range(min(steps, 5)):
        step()
    torch.cuda.synchronize()
    tot_ms, launches = ctypes.c_double(0), ctypes.c_int(0)
    profile_read(ctypes.byref(tot_ms), ctypes.byref(launches))
    profile(0)
    ext.reset_id(pid)
    bpp = algorithmic_bytes_per_pixel(c, cfg["kind"])
    kernel_ms = tot_ms.value / max(launches.value, 1)
    steps_per_launch = 1 if kernel_name.split("<")[0].endswith("_strip") else 2  # the pair kernels run two adjoint steps
    cnt = load_counters(config) if not corrected and keep is None else None  # the counters were read on the default path
    kernel_bytes = steps_per_launch * bpp["adjoint"] * n * h * w
    model_gbs = bpp["total"] * pxit / sec / 1e9
    have_step = bool(cnt) and "step_bytes" in cnt
    out["whole_job"] = {
        # what the job really moves (every kernel and copy of a step, from the counters) ...
        "effective_bytes_per_pixel_iteration": round(cnt["step_bytes"] / pxit, 1) if have_step else None,
        "effective_GBps": round(cnt["step_bytes"] / sec / 1e9, 1) if have_step else None,
        "effective_frac_of_hbm_peak": round(cnt["step_bytes"] / sec / 1e9 / HBM_PEAK_GBS, 4) if have_step else None,
        # ... and the one-round-trip-per-iteration model, which counts a recompute this build does not execute (keep
        # mode 2) and one round trip per iteration where a pair launch makes one per two: its rate may exceed the peak
        "model_bytes_per_pixel_iteration": bpp["total"], "model_GBps": round(model_gbs, 1),
        "model_frac_of_hbm_peak": round(model_gbs / HBM_PEAK_GBS, 4)}
    roof = physical_roofline({"bound": "hbm", "kernel": kernel_name, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                              "bytes_per_launch": kernel_bytes, "adjoint_steps_per_launch": steps_per_launch,
                              "avg_launch_ms_events": round(kernel_ms, 5), "launches_timed": launches.value}, cnt, kernel_ms)
    if cnt:
        if "rocprof_avg_us" in cnt:
            r_ms = cnt["rocprof_avg_us"] * 1e-3
            roof["rocprof"] = {"avg_launch_ms": round(r_ms, 5), "achieved": round(cnt["traffic_bytes"] / (r_ms * 1e-3) / 1e9, 1),
                               "frac": round(cnt["traffic_bytes"] / (r_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                               "model_frac": round(kernel_bytes / (r_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
        if "lds_bytes" in cnt and kernel_ms > 0:
            lds_gbs = cnt["lds_bytes"] / (kernel_ms * 1e-3) / 1e9
            roof["lds"] = {"bytes_per_launch": cnt["lds_bytes"], "achieved_GBps": round(lds_gbs, 1), "peak_GBps": round(LDS_PEAK_GBS, 1),
                           "frac": round(lds_gbs / LDS_PEAK_GBS, 4)}
    out["roofline"] = roof
    return out, cfg


def bench_channels(kind, c, steps, warmup):
    """One TV or TGV layer at the headline's image size with c channels (the reference accepts any channel count)."""
    import torch

    from customnetworklayers_amd import workloads

    ext = layer_of(kind)[0]
    n, h, w, its = 4, 384, 1248, 100
    make = workloads.tv_inputs if kind == "tv" else workloads.tgv_inputs
    d = make(n, c, h, w, seed=0, conf_density=0.2)
    t = {k: torch.from_numpy(v).to("cuda:0") for k, v in d.items()}

    def step():
        ext.forward(t["dx"], t["dy"], t["dc"], t["db"], t["di"], its, 0)
        return ext.backward(t["grad"], t["dx"], t["dy"], t["dc"], t["db"], its, 0)

    ext.reset_id(0)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    sec = (time.perf_counter() - t0) / steps
    ext.reset_id(0)
    return {"value": round(n * h * w * its / sec / 1e6, 2), "unit": "Mpixel-iter/s", "ms_per_step": round(sec * 1e3, 4), "steps": steps,
            "warmup": warmup, "workload": "%s inpainting fwd+bwd, N=%d, flow %dx%dx%d fp32, %d FISTA iterations" % (kind.upper(), n, c, h, w, its)}


def copy_ceiling():
    """What a plain copy kernel over 1 GiB reaches on this GPU (read + written bytes per second)."""
    import torch

    from customnetworklayers_amd._lib import lib

    g = ctypes.c_double(0)
    rc = lib.inpaint_copy_bandwidth(1 << 30, 10, ctypes.byref(g), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    return round(g.value, 1) if rc == 0 else None


def stream_ceiling(planes_read=2, planes_written=1):
    """What a streaming kernel that reads two bytes for each one it writes (the strip kernels' mix) reaches on this GPU."""
    import torch

    from customnetworklayers_amd._lib import lib

    g = ctypes.c_double(0)
    rc = lib.inpaint_stream_bandwidth(1 << 29, planes_read, planes_written, 10, ctypes.byref(g),
                                      ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    return {"planes_read": planes_read, "planes_written": planes_written, "GBps": round(g.value, 1)} if rc == 0 else None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="config 1 only: skip the short legs of configs 2, 3, 4 and of keep mode 0 after the headline's timed region")
    ap.add_argument("--config", type=int, default=1,
                    help="workload index (1 = headline TV layer, 2 = TGV layer, 3 = three-level TV hierarchy, 4 = stress shape, "
                         "5 = quadratic fit, 6 = median)")
    ap.add_argument("--keep", type=int, default=None, choices=[0, 1, 2],
                    help="configs 1, 2, 4: which half-step iterates the forward pass keeps (default 2 = all; 0 = the reference's footprint)")
    ap.add_argument("--corrected-gradient", action="store_true",
                    help="configs 1 and 2: time the opt-in corrected gradient instead of the reference's (not the headline)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus %d is not supported (the samples of a batch are "
              "independent: more GPUs would each take a share of them, with no communication)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    from customnetworklayers_amd.workloads import CONFIGS, config_inputs

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    kind = CONFIGS[args.config]["kind"]
    if kind == "tv_hierarchy":
        print(json.dumps(bench_hierarchy(args, CONFIGS[args.config])))
        return
    if kind in ("quadfit", "median"):
        cfg, d = config_inputs(args.config, seed=0)
        return bench_flowaux(args, cfg, d)
    out, cfg = bench_layer(args.config, args.steps, args.warmup, corrected=args.corrected_gradient, keep=args.keep)
    out["roofline"]["hbm_copy_ceiling_GBps"] = copy_ceiling()
    out["roofline"]["hbm_stream_ceiling"] = stream_ceiling()
    if out["roofline"]["hbm_stream_ceiling"] and out["roofline"].get("achieved"):
        # the physical rate of the dominant kernel against what a plain stream with its mix of reads and writes reaches
        out["roofline"]["frac_of_stream_ceiling"] = round(out["roofline"]["achieved"] / out["roofline"]["hbm_stream_ceiling"]["GBps"], 4)
    if args.config == 1 and not args.no_other_configs and not args.corrected_gradient and args.keep is None:
        # after the headline's timed region: short legs of the other workloads, so that one run witnesses them all
        other = {}
        leg = lambda o: {k: o[k] for k in ("value", "unit", "ms_per_step", "ms_per_step_event_median", "steps", "warmup")}  # noqa: E731
        o, _ = bench_layer(1, 5, 2, keep=0, detail=False)
        other["config1_keep_mode_0"] = dict(leg(o), workload=o["config"]["workload"] + ", nothing kept: every segment recomputed (the reference's footprint)",
                                            slot_bytes=o["config"]["slot_bytes"])
        o, _ = bench_layer(2, 4, 2, detail=False)
        other["config2_tgv"] = dict(leg(o), workload=o["config"]["workload"], slot_bytes=o["config"]["slot_bytes"])
        hargs = argparse.Namespace(steps=30, warmup=5, no_cpu_baseline=True)  # (2 ms steps: a short leg would time the empty queue at its start)
        o = bench_hierarchy(hargs, CONFIGS[3])
        other["config3_hierarchy"] = dict({k: o[k] for k in ("value", "unit", "ms_per_step", "steps", "warmup")}, workload=o["config"]["workload"])
        o, _ = bench_layer(4, 3, 1, detail=False)
        other["config4_stress"] = dict(leg(o), workload=o["config"]["workload"], slot_bytes=o["config"]["slot_bytes"])
        # more channels than the two of the configurations: time per step against (C/2) x the two-channel time
        two = {"tv": out["ms_per_step"], "tgv": other["config2_tgv"]["ms_per_step"]}
        for kind, c in (("tv", 4), ("tv", 8), ("tgv", 4)):
            o = bench_channels(kind, c, 3, 1)
            o["x_of_two_channel_time_per_channel_pair"] = round(o["ms_per_step"] / (two[kind] * c / 2), 3)
            other["%s_%d_channels" % (kind, c)] = o
        out["other_configs"] = other
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg)
        if args.config == 1:  # the reference's own CPU-sized case, whole (milliseconds)
            out["cpu_baseline_config0"] = cpu_baseline(CONFIGS[0], whole=True)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
