#!/usr/bin/env python3
"""Benchmark of the differentiable Gaussian ray-march path on one MI355X.

One step = one training view through the reference's operator API:
``RenderOptixFunction.apply`` (k-sigma boxes + LBVH build + SH colour + prim packing +
forward march) followed by the backward of an MSE loss (backward march + SH backward),
exactly what scripts/train.py:119-148 runs per iteration (the reference rebuilds its
acceleration structure on every forward, ``update=False``).

Workload (``config.workload``): the 1 M-Gaussian scene of the training-stress configuration
(centres uniform in a ball of radius 2) rendered at 800x800 -- the configuration the headline
metric "Mrays/s fwd+bwd @1M Gaussians 800x800" is quoted on -- one camera of the
upper-hemisphere orbit per step.  Inputs are resident in HBM before the timed region.

Prints ONE JSON line.  ``roofline`` prices the dominant kernel (the backward march) with its
algorithmic bytes (64+56 B per ray-slab-hit + 24 B per ray) over its own HIP-event time;
``cpu_baseline`` times the CPU oracle on a bounded ray sample of the same workload.
``fwd_fps_c3`` is the other half of the headline metric, measured in the same run: frames per second
of the forward-only render of the 3 M-Gaussian scene at 1920x1080 along its orbit, tree built once,
with a roofline of its own.  ``hbm_measured`` is the bandwidth a plain 1 GiB device-to-device copy
reaches on this GPU (read + written bytes), the practical ceiling beside the 8 TB/s peak;
``memory`` reports the peak device memory of the run and the record's allocated and used bytes.
Beside the contract's keys: ``atomics`` (the gradient scatter's atomic adds per backward launch,
counted by the kernels, over the launch's time) and ``views_in_flight`` (the same steps timed once
more with two views in flight on two streams, as a loop that accumulates gradients over several
views can run them; ``value`` itself is always one view at a time).  ``other_workloads``: the other
benchmark configurations (300 k Gaussians at 800x800, 3 M at 1237x822, 1 M at 1024x1024), five steps each,
with their own step and kernel rooflines.  ``valu_measured``: the rate at which this card issues VALU
instructions, from a kernel of independent multiply-adds run here; it is the ``peak`` of every
``valu_issue`` figure (whose instruction counts are stored figures of a profiler run, see ``valu_issue``).
``--workload coherent_512_800x800`` is not a benchmark configuration but the kernels' best case (every ray
of a tile hits the same few large Gaussians for whole slabs); ``--sections`` reads the per-section cycle
census of a diagnostic build of the library (``python -m raygaussx_amd.build --sections``, selected with
``RGX_LIB_PATH``).
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from raygaussx_amd import _lib as L  # noqa: E402
from raygaussx_amd import optix_utils as u_ox  # noqa: E402
from raygaussx_amd import scenes  # noqa: E402
from raygaussx_amd.render_optix import RenderOptixFunction, default_settings  # noqa: E402

HBM_PEAK_GBPS = 8000.0

PROFILES = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles")


def _stored(tag, workload, kernel_key):
    import glob
    import re
    for path in sorted(glob.glob(os.path.join(PROFILES, "*.md"))):
        for line in open(path):
            m = re.match(r"\s*" + tag + r"\s+(\S+)\s+(\S+)\s+([0-9.eE+]+)", line)
            if m and m.group(1) == workload and m.group(2) == kernel_key:
                return float(m.group(3)), os.path.relpath(path, os.path.dirname(PROFILES))
    return None, None


# wave instructions per second all SIMDs could issue at the nominal clock: 256 CUs x 4 SIMDs x 2.4 GHz, one VALU
# instruction per 4 clocks.  Reported beside the measured rate; the measured rate is the one fractions are taken of.
VALU_NOMINAL_GINST = 256 * 4 * 2.4 / 4.0
_valu_measured = None


PROBE_KINDS = ("v_fma_f32", "v_add_f32", "v_mov_b32", "v_and_b32", "v_cmp_lt_f32", "v_cndmask_b32", "v_max_f32",
               "v_add_f32_dpp", "v_lshlrev_b32", "v_exp_f32")
# kinds 10..13 name their registers (160 of them: three wavefronts per SIMD at most): where the operands live matters
BANK_KINDS = ("v_fma_f32 acc = x * k + acc, fresh x from the other register bank", "v_fma_f32 d = a * b + c, all fresh, banks mixed",
              "v_fma_f32 d = a * b + c, all fresh, one bank", "v_mul_f32 d = a * b, both fresh")


def probe_rate(dev, kind, waves_per_simd, iters=1024, reps=5):
    """(G wave instructions/s, launch ms, instructions) of rgx_probe_valu_rate: one instruction class, sixteen
    independent registers per lane, ``waves_per_simd`` wavefronts on each of the 1024 SIMDs; best of ``reps``."""
    sink = torch.zeros(4, device=dev)
    count = C.c_uint64(0)
    best = float("inf")
    for rep in range(reps + 2):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        L.check(L.lib().rgx_probe_valu_rate(C.c_int32(256 * 4 * waves_per_simd), C.c_int32(iters), C.c_int32(kind), L.ptr(sink),
                                            C.byref(count), L.stream(dev)))
        b.record()
        torch.cuda.synchronize()
        if rep >= 2:
            best = min(best, a.elapsed_time(b))
    return count.value / (best * 1e-3) / 1e9, best, count.value


def valu_measured(dev):
    """G VALU wave instructions per second this card issues, measured: independent v_fma_f32 (rgx_probe_valu_rate,
    8 wavefronts per SIMD, nothing but the multiply-adds and a loop counter), the instruction count known from the
    kernel's shape, timed with events on the launch stream.  Also at the three wavefronts per SIMD the march kernels
    run with, and for a compare (the slower class of VALU instruction: compares, selects, min / max, DPP, shifts)."""
    global _valu_measured
    if _valu_measured is None:
        rate, ms, count = probe_rate(dev, 0, 8, iters=2048)
        _valu_measured = dict(value=round(rate, 1), unit="G wave instructions/s", nominal=round(VALU_NOMINAL_GINST, 1),
                              instructions=count, kernel_ms=round(ms, 4), what="independent v_fma_f32, 8 wavefronts per SIMD",
                              fma_at_3_waves_per_simd=round(probe_rate(dev, 0, 3)[0], 1),
                              fma_accumulate_at_3_waves_per_simd=round(probe_rate(dev, 10, 3)[0], 1),
                              cmp_at_3_waves_per_simd=round(probe_rate(dev, 4, 3)[0], 1),
                              exp_at_3_waves_per_simd=round(probe_rate(dev, 9, 3)[0], 1))
    return _valu_measured


def valu_cost_table(dev):
    """Clocks per wave instruction and SIMD (1024 SIMDs at 2.4 GHz over the measured rate) of every probe kind at
    1, 2, 3, 4 and 8 wavefronts per SIMD."""
    table = {}
    for kind, name in enumerate(PROBE_KINDS):
        table[name] = {str(w): round(1024 * 2.4 / probe_rate(dev, kind, w, reps=3)[0], 2) for w in (1, 2, 3, 4, 8)}
    for kind, name in enumerate(BANK_KINDS, start=len(PROBE_KINDS)):
        table[name] = {str(w): round(1024 * 2.4 / probe_rate(dev, kind, w, reps=3)[0], 2) for w in (1, 2, 3)}
    return table


def valu_issue(workload, kernel_key, kernel_ms, dev):
    """The march kernels are bound by VALU instruction issue, not by bytes.  ``instructions_per_launch`` is a STORED
    figure: VALU wave instructions per launch as a profiler run of this script counted them (rocprofv3 --pmc
    SQ_INSTS_VALU; the summary under profiles/ holds it in a line `valu_instructions_per_launch <workload> <kernel
    key> <count>`), divided by THIS run's kernel time; ``peak`` is the issue rate measured on this card in this run
    (``valu_measured``).  The stored count and this run's time belong to different launches of the same
    deterministic kernel on the same inputs; should the pairing ever read above the measured peak it is reported as
    such (``above_peak``) and ``frac`` is capped at 1.  None without a stored line."""
    count, source = _stored("valu_instructions_per_launch", workload, kernel_key)
    if count is None or kernel_ms <= 0:
        return None
    peak = valu_measured(dev)["value"]
    rate = count / (kernel_ms * 1e-3) / 1e9
    return dict(instructions_per_launch=count, count_is="stored (profiler run)", source=source, achieved=round(rate, 1),
                peak=peak, peak_is="measured in this run", unit="G wave instructions/s", frac=round(min(rate / peak, 1.0), 4),
                above_peak=bool(rate > peak))


def stored_traffic(workload, kernel_key):
    """HBM bytes per launch of a march kernel as a profiler run measured them: rocprofv3 --pmc FETCH_SIZE /
    WRITE_SIZE of this script, scaled by the same counters' reading for a 1 GiB copy (--calibrate-copy).
    The summary under profiles/ holds the figure in a line `traffic_bytes_per_launch <workload> <kernel key> <bytes>`;
    this run does not measure it (counters need the profiler), so the JSON line names the file it came from.
    None when there is no such line."""
    return _stored("traffic_bytes_per_launch", workload, kernel_key)

WORKLOADS = {
    # name: (scene config, n, width, height)
    "c4_1M_800x800": (4, 1_000_000, 800, 800),
    "c1_300k_800x800": (1, 300_000, 800, 800),
    "c4_1M_1024x1024": (4, 1_000_000, 1024, 1024),
    "c2_3M_1237x822": (2, 3_000_000, 1237, 822),
    "c0_4096_128x128": (0, 4096, 128, 128),
    # not a benchmark configuration: the kernels' best case (see scenes.CONFIGS["coherent"])
    "coherent_512_800x800": ("coherent", 512, 800, 800),
    # inference along a camera path, tree built once (scripts/test.py:60-126): frames per second
    "c3_3M_1920x1080_fwd": (3, 3_000_000, 1920, 1080),
}


def cpu_baseline(scene, cam, cfg, n_sample, threads, backward=True):
    """The same step on the host cores: the CPU oracle's forward (+ backward) march on a strided ray sample
    of the same view, candidates culled by its bounding-volume tree over the Gaussians' boxes (same results
    as its brute force, see tests/test_oracle_geometry.py).  Timed: tree build + march of the sample; the
    per-Gaussian colour / packing / SH gradient passes run once per view whatever the sample and are left out."""
    from oracle import oracle as orc
    orc.build()
    orc.set_num_threads(threads)
    sc = scenes.scene_to_numpy(scene)
    n_rays = cam.image_width * cam.image_height
    ids = np.linspace(0, n_rays - 1, n_sample).astype(np.int64)
    few = ids[:: max(1, n_sample // 64)]
    _, _, ctx = orc.render_forward(sc, cam, cfg["dt_step"], cfg["dynamic_sampling"], cfg["max_prim_slice"],
                                   t_eps=cfg["t_eps"], ray_ids=few[:1])      # boxes, colours, primitive records
    t0 = time.perf_counter()
    orc.cull_build(ctx["prims"])
    t_build = time.perf_counter() - t0
    try:
        img, _ = orc.march_forward(ctx["cs"], ctx["ms"], ctx["bmin"], ctx["bmax"], ctx["prims"], ids)
        if backward:
            dloss = np.full(img.shape, 1.0 / img.size, np.float32)
            orc.march_backward(ctx["cs"], ctx["ms"], ctx["bmin"], ctx["bmax"], ctx["prims"], img, dloss, ids)
    finally:
        orc.cull_free()
    dt = time.perf_counter() - t0
    return dict(value=round(n_sample / dt / 1e6, 6), unit="Mrays/s", cores=threads, kind="port",
                sample=f"{n_sample} strided rays of camera 0, {'fwd+bwd' if backward else 'fwd'} march, all {sc['positions'].shape[0]} "
                       f"Gaussians behind a CPU bounding-volume tree ({t_build:.2f} s to build, included), {dt:.1f} s")


def copy_bandwidth(dev, reps=10):
    """GB/s (bytes read + bytes written) of a 1 GiB device-to-device copy: what a plain streaming kernel
    reaches on this GPU, the practical ceiling beside the published peak."""
    src = torch.full((1 << 28,), 1.0, dtype=torch.float32, device=dev)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        dst.copy_(src)
    b.record()
    torch.cuda.synchronize()
    ms = a.elapsed_time(b) / reps
    del src, dst
    torch.cuda.empty_cache()
    return round(2 * (1 << 30) / (ms * 1e-3) / 1e9, 1)


def inference_leg(dev, frames, warmup):
    """The headline metric's second figure: forward-only frames per second of the 3 M-Gaussian scene at
    1920x1080 along its 300-camera orbit (every 7th camera), rays ended at T < 1e-4, tree built once and
    reused (scripts/test.py:60-126).  A frame is view-dependent colour + primitive records + march."""
    from raygaussx_amd.render_optix import compute_rgb
    name = "c3_3M_1920x1080_fwd"
    config, n, width, height = WORKLOADS[name]
    cfg = scenes.CONFIGS[config]
    d = {k: v.to(dev) for k, v in scenes.make_scene(config, n=n).items()}
    cams = [scenes.make_camera(config, (7 * i) % cfg["n_cameras"], width=width, height=height).to(dev) for i in range(frames + warmup)]
    structs = [u_ox.camera_struct(c) for c in cams]       # host copies of the camera constants: no sync per frame
    t0 = time.perf_counter()
    tree = u_ox.AccelerationStructure(n, dev).build_from_gaussians(d["positions"], d["scales"], d["quaternions"], d["densities"])
    torch.cuda.synchronize()
    stats = u_ox.new_stats(dev)

    def frame(i, census=False):
        rgb = compute_rgb(structs[i].eye, d["positions"], d["color_features"], None, None, None, 0, 3)
        return u_ox.launch_pipeline_test(None, None, tree, None, None, cfg["dt_step"], cfg["dynamic_sampling"], cams[i],
                                         d["densities"], rgb, d["positions"], d["scales"], d["quaternions"],
                                         cfg["max_prim_slice"], t_eps=cfg["t_eps"], stats=stats if census else None)
    for i in range(warmup):
        frame(i)
    torch.cuda.synchronize()
    L.timing_enable(True)
    t0 = time.perf_counter()
    for i in range(frames):
        frame(warmup + i)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    timing = L.timing_read()
    L.timing_enable(False)
    for i in range(frames):
        frame(warmup + i, census=True)
    torch.cuda.synchronize()
    st = u_ox.read_stats(stats)
    hits = st["hit_pairs"] / frames
    n_rays = width * height
    ms_kernel = timing["march_forward"][0] / max(timing["march_forward"][1], 1)
    nbytes = 64.0 * hits + 12.0 * n_rays
    gbps = nbytes / (ms_kernel * 1e-3) / 1e9
    frame_bytes = nbytes + 300.0 * n
    ms_frame = elapsed / frames * 1e3
    traffic, source = stored_traffic(name, "march_forward")
    return dict(value=round(frames / elapsed, 3), unit="frames/s", frames=frames, warmup=warmup, ms_per_frame=round(ms_frame, 4),
                workload=name, gaussians=n, width=width, height=height, t_eps=cfg["t_eps"], dynamic_sampling=cfg["dynamic_sampling"],
                frame="sh + pack + march fwd, 1 view, tree built once and reused",
                roofline=dict(bound="hbm", kernel="k_march_fwd", achieved=round(gbps, 2), peak=HBM_PEAK_GBPS, unit="GB/s",
                              frac=round(gbps / HBM_PEAK_GBPS, 5), traffic=traffic, traffic_source=source,
                              kernel_ms=round(ms_kernel, 4), algorithmic_bytes=int(nbytes), hit_pairs_per_launch=int(hits),
                              valu_issue=valu_issue(name, "march_forward", ms_kernel, dev)),
                frame_roofline=dict(bytes_per_frame=int(frame_bytes), frac=round(frame_bytes / (ms_frame * 1e-3) / 1e9 / HBM_PEAK_GBPS, 5),
                                    roofline_fps=round(HBM_PEAK_GBPS * 1e9 / frame_bytes, 2)),
                kernels_ms={k: round(v[0] / max(v[1], 1), 4) for k, v in timing.items() if v[1]})


def _timed(fn, reps):
    fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / reps * 1e3


def side_kernels(dev, reps):
    """The entry points either side of the march, each on its benchmark-size input: ms per call and, for
    the streaming ones, algorithmic bytes moved per second against the 8 TB/s of HBM."""
    from raygaussx_amd.general_utils import reduce_supersampling
    from raygaussx_amd.reordering import morton_order, reorder_tensors
    from raygaussx_amd.render_optix import compute_rgb
    from raygaussx_amd.simple_knn import distCUDA2
    out = {}
    # image epilogue: 1920x1080 at 2x2 supersampling -> float image + 8-bit image
    w, h, f = 1920, 1080, (2, 2)
    rays = torch.rand(w * f[0] * h * f[1], 3, device=dev)
    ms = _timed(lambda: reduce_supersampling(w, h, rays, f, clip=True, to_uint8=True), reps)
    nbytes = rays.numel() * 4 + w * h * 3 * 5
    out["reduce_supersampling_1080p_2x2"] = dict(ms=round(ms, 4), GBps=round(nbytes / ms / 1e6, 1), frac_hbm=round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4))
    # reordering of a 1 M point cloud: parameters + two Adam moments each (classes/point_cloud.py:1031-1044)
    sc = {k: v.to(dev) for k, v in scenes.make_scene(4, n=1_000_000).items()}
    tensors = [sc[k] for k in ("positions", "scales", "quaternions", "densities", "color_features")]
    tensors = tensors + [t.clone() for t in tensors] + [t.clone() for t in tensors]
    out["morton_order_1M"] = dict(ms=round(_timed(lambda: morton_order(sc["positions"]), reps), 4))
    order = morton_order(sc["positions"])
    ms = _timed(lambda: reorder_tensors(order, tensors), reps)
    nbytes = 2 * sum(t.numel() * 4 for t in tensors) + order.numel() * 8
    out["reorder_tensors_1M_x15"] = dict(ms=round(ms, 4), GBps=round(nbytes / ms / 1e6, 1), frac_hbm=round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 4))
    ms_torch = _timed(lambda: [t.index_select(0, order) for t in tensors], reps)
    out["reorder_tensors_1M_x15"]["torch_index_select_ms"] = round(ms_torch, 4)
    # distCUDA2 at 1 M and 3 M points
    out["distCUDA2_1M"] = dict(ms=round(_timed(lambda: distCUDA2(sc["positions"]), reps), 4))
    big = scenes.make_scene(3)
    pos3 = big["positions"].to(dev)
    out["distCUDA2_3M"] = dict(ms=round(_timed(lambda: distCUDA2(pos3), reps), 4))
    # viewer launch on the 3 M scene at 1920x1080 (tree built once)
    cfg = scenes.CONFIGS[3]
    d3 = {k: v.to(dev) for k, v in big.items()}
    tree = u_ox.AccelerationStructure(d3["positions"].shape[0], dev).build_from_gaussians(d3["positions"], d3["scales"],
                                                                                            d3["quaternions"], d3["densities"])
    cam = scenes.make_camera(3, 0).to(dev)
    cs = u_ox.camera_struct(cam)
    rgb = compute_rgb(cam.camera_center, d3["positions"], d3["color_features"], None, None, None, 0, 3)
    prims = u_ox.pack_prims(tree, cs, d3["positions"], d3["scales"], d3["quaternions"], d3["densities"], rgb)
    ms = _timed(lambda: u_ox.march_viewer(tree, cs, prims, cfg["dt_step"], cfg["dynamic_sampling"], cfg["max_prim_slice"], cfg["t_eps"]), reps)
    out["march_viewer_c3_1080p"] = dict(ms=round(ms, 4), frames_per_s=round(1e3 / ms, 2))
    return dict(side_kernels=out, reps=reps, data="synthetic")


SECTION_NAMES = ("sweep", "filter", "shade_or_gradient_trips", "record_lists", "blend_or_prefix", "sample_sums_io",
                 "tile_setup", "iteration_top", "iteration_end", "epilogue", "walk_and_parse", "flush_gradients")
SECTION_KERNELS = ("k_march_fwd<record>", "k_march_fwd<plain>", "k_march_bwd_replay_sums", "k_march_bwd_replay", "k_march_bwd")
# the replaying backward sweeps and filters nothing: it files the parts of its walk under those sections
REPLAY_SECTION_NAMES = {"sweep": "parse_items", "filter": "count_hits_and_set_windows_up", "record_lists": "first_words_of_the_lists"}


def read_sections(reset=False):
    """The per-section cycle census of a diagnostic build (python -m raygaussx_amd.build --sections): per march kernel
    the share of its waves' lifetimes spent in each section, or None when the loaded library has no census."""
    lib = L.lib()
    if not hasattr(lib, "rgx_debug_section_cycles"):
        return None
    nsec = len(SECTION_NAMES)
    raw = (C.c_uint64 * (len(SECTION_KERNELS) * (nsec + 1)))()
    L.check(lib.rgx_debug_section_cycles(raw, int(reset)))
    out = {}
    for k, kernel in enumerate(SECTION_KERNELS):
        row = [int(raw[k * (nsec + 1) + i]) for i in range(nsec + 1)]
        total = sum(row[:nsec])
        if row[nsec] and total:
            out[kernel] = dict(waves=row[nsec], cycles_per_wave=round(total / row[nsec]),
                               shares={(REPLAY_SECTION_NAMES.get(name, name) if "replay" in kernel else name): round(c / total, 4)
                                       for name, c in zip(SECTION_NAMES, row[:nsec]) if c})
    return out


def training_leg(dev, workload, steps, warmup, opts, in_flight=1):
    """``steps`` timed training steps (or frames) of one workload; returns (JSON fields, the CPU scene, cfg)."""
    config, n, width, height = WORKLOADS[workload]
    cfg = dict(scenes.CONFIGS[config])
    scene = scenes.make_scene(config, n=n)
    dscene = {k: v.to(dev) for k, v in scene.items()}
    names = ("positions", "scales", "quaternions", "densities", "color_features", "sph_gauss_features",
             "bandwidth_sharpness", "lobe_axis")
    inference = workload.endswith("_fwd")
    forward_only = opts.forward_only or inference
    params = [dscene[k].clone().requires_grad_(not forward_only) for k in names]
    n_cams = min(cfg["n_cameras"], 100)
    cams = [scenes.make_camera(config, i, width=width, height=height).to(dev) for i in range(n_cams)]
    cam_structs = [u_ox.camera_struct(c) for c in cams]   # also caches each camera's host constants: no sync per step
    n_rays = width * height
    target = torch.rand(n_rays, 3, device=dev, generator=torch.Generator(dev).manual_seed(1))
    stats = u_ox.new_stats(dev)
    gas = None
    if inference:
        from raygaussx_amd.render_optix import compute_rgb
        tree = u_ox.AccelerationStructure(n, dev).build_from_gaussians(dscene["positions"], dscene["scales"],
                                                                        dscene["quaternions"], dscene["densities"])

    def step(i, census=False, lane=None):
        """One step.  Timed steps run the kernels as a training loop does, without a statistics block;
        the census pass afterwards repeats the same views with one to count the hit pairs.  ``lane``:
        (stream, one-element list holding that stream's tree) for the views-in-flight pass."""
        nonlocal gas
        if lane is not None:
            with torch.cuda.stream(lane[0]):
                keep, gas = gas, lane[1][0]
                out = step(i)
                lane[1][0], gas = gas, keep
            return out
        if inference:   # per frame: view-dependent colour, primitive records, march
            cam = cams[(7 * i) % n_cams]
            rgb = compute_rgb(cam_structs[(7 * i) % n_cams].eye, dscene["positions"], dscene["color_features"], None, None, None, 0, 3)
            return u_ox.launch_pipeline_test(None, None, tree, None, None, cfg["dt_step"], cfg["dynamic_sampling"], cam,
                                             dscene["densities"], rgb, dscene["positions"], dscene["scales"],
                                             dscene["quaternions"], cfg["max_prim_slice"], t_eps=cfg["t_eps"],
                                             stats=stats if census else None)
        s = default_settings(cams[i % n_cams], cfg["dt_step"], cfg["dynamic_sampling"], cfg["max_prim_slice"],
                             t_eps=cfg["t_eps"], gas=gas)
        s.stats = stats if census else None
        s.record_hits = not opts.no_records
        if opts.rec_tile_words is not None:
            s.rec_tile_words = opts.rec_tile_words
        s.rec_half_sums = opts.half_sums
        img = RenderOptixFunction.apply(*params, s)
        gas = s.gas
        if not forward_only:
            loss = ((img - target) ** 2).mean()
            loss.backward()
            for p in params:
                p.grad = None
        return img

    torch.cuda.reset_peak_memory_stats(dev)
    base_mem = torch.cuda.memory_allocated(dev)
    step(0)                        # the first view of a shape: its record is sized before anything is known of its use
    torch.cuda.synchronize()
    first_peak = torch.cuda.max_memory_allocated(dev)
    for i in range(1, warmup):
        step(i)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats(dev)
    if opts.sections:
        read_sections(reset=True)
    L.timing_enable(True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(warmup + i)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    timing = L.timing_read()
    L.timing_enable(False)
    sections = read_sections() if opts.sections else None
    if opts.sections and opts.dump_tile_times:
        # per workgroup (launch order): cycles per section, waves, kernel, start and end of its last wave (100 MHz ticks)
        rows = np.zeros((2, 65536, 16), np.uint32)
        L.check(L.lib().rgx_debug_section_rows(rows.ctypes.data_as(C.c_void_p)))
        used = int(max(np.nonzero(rows[:, :, 12].sum(0))[0], default=0)) + 1
        np.save(opts.dump_tile_times, rows[:, :used])
    steady_peak = torch.cuda.max_memory_allocated(dev)
    for i in range(steps):     # census: the same views once more, counted, not timed
        step(warmup + i, census=True)
    torch.cuda.synchronize()
    st = u_ox.read_stats(stats)
    flight = None
    if in_flight > 1:     # views of one accumulation window are independent: keep several in flight
        lanes = [(torch.cuda.Stream(dev), [None]) for _ in range(in_flight)]
        for i in range(max(warmup, in_flight)):
            step(i, lane=lanes[i % len(lanes)])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            step(warmup + i, lane=lanes[i % len(lanes)])
        torch.cuda.synchronize()
        el = time.perf_counter() - t0
        flight = dict(views=in_flight, value=round(n_rays * steps / el / 1e6, 4), unit="Mrays/s",
                      ms_per_step=round(el / steps * 1e3, 4))
        if inference:
            flight["frames_per_s"] = round(steps / el, 3)

    ms_per_step = elapsed / steps * 1e3
    mrays = n_rays * steps / elapsed / 1e6
    passes = 1 if forward_only else 2
    hits_per_launch = st["hit_pairs"] / (steps * passes)   # H: fwd and bwd march the same slabs
    # the dominant kernel: the march launch (forward or backward) that takes longer
    bwd_name = "k_march_bwd" if opts.no_records else (
        "k_march_bwd_replay" if (opts.rec_tile_words or 1 << 30) < 16384 + 8192 else "k_march_bwd_replay_sums")
    cand = [("march_forward", "k_march_fwd", 64.0 * hits_per_launch + 12.0 * n_rays)]
    if not forward_only:
        cand.append(("march_backward", bwd_name, (64.0 + 56.0) * hits_per_launch + 24.0 * n_rays))
    per_kernel = {}
    default_record = not (opts.no_records or opts.rec_tile_words is not None or opts.half_sums)
    for key, name, nbytes in cand:
        ms, cnt = timing[key]
        avg = ms / max(cnt, 1)
        gbps = nbytes / (avg * 1e-3) / 1e9 if avg > 0 else 0.0
        per_kernel[key] = dict(kernel=name, kernel_ms=round(avg, 4), algorithmic_bytes=int(nbytes), achieved=round(gbps, 2),
                               frac=round(gbps / HBM_PEAK_GBPS, 5),
                               valu_issue=valu_issue(workload, key, avg, dev) if default_record else None)
    kname = max(per_kernel, key=lambda k: per_kernel[k]["kernel_ms"])
    dom = per_kernel[kname]
    traffic, traffic_source = stored_traffic(workload, kname) if default_record else (None, None)
    roofline = dict(bound="hbm", kernel=dom["kernel"], achieved=dom["achieved"], peak=HBM_PEAK_GBPS, unit="GB/s", frac=dom["frac"],
                    traffic=traffic, traffic_source=traffic_source,
                    kernel_ms=dom["kernel_ms"], algorithmic_bytes=dom["algorithmic_bytes"],
                    hit_pairs_per_launch=int(hits_per_launch), march_kernels=per_kernel)
    # whole-step roofline-derived rate: all algorithmic bytes of one step at peak bandwidth
    step_bytes = (64.0 * hits_per_launch + 12.0 * n_rays + 300.0 * n
                  + (0 if forward_only else (120.0 * hits_per_launch + 24.0 * n_rays + 464.0 * n)))
    out = dict(metric="Mrays/s fwd" + ("" if forward_only else "+bwd"), value=round(mrays, 4), unit="Mrays/s",
               n_gpus=1, steps=steps, warmup=warmup, ms_per_step=round(ms_per_step, 4),
               higher_is_better=True, scaling="weak", vs_baseline=None, dtype="f32", data="synthetic",
               config=dict(workload=workload, gaussians=n, width=width, height=height, sh_degree=3,
                           dt_step=cfg["dt_step"], dynamic_sampling=cfg["dynamic_sampling"],
                           max_prim_slice=cfg["max_prim_slice"], t_eps=cfg["t_eps"],
                           step=("sh + pack + march fwd, 1 view, tree built once" if inference else
                                 "bvh build + sh + pack + march fwd"
                                 + ("" if forward_only else " + march bwd + sh bwd") + ", 1 view")),
               roofline=roofline,
               step_roofline=dict(bytes_per_step=int(step_bytes),
                                  achieved=round(step_bytes / (ms_per_step * 1e-3) / 1e9, 2), unit="GB/s",
                                  frac=round(step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS, 5),
                                  roofline_mrays=round(HBM_PEAK_GBPS * 1e9 * n_rays / step_bytes / 1e6, 2)),
               kernels_ms={k: round(v[0] / max(v[1], 1), 4) for k, v in timing.items() if v[1]},
               stats_per_step={k: v / steps for k, v in st.items()})
    if inference:
        out["frames_per_s"] = round(1e3 / ms_per_step, 3)
    if not forward_only:   # the gradient scatter: fp32 atomic adds to memory per backward launch (census) over its time
        adds = st["grad_atomics"] / steps
        out["atomics"] = dict(per_backward_launch=int(adds), unit="G atomic adds/s",
                              value=round(adds / (per_kernel["march_backward"]["kernel_ms"] * 1e-3) / 1e9, 3))
    # lane-slots per ray-slab-hit pair from this run's kernel time: what the launch could have issued at the measured
    # VALU rate, per pair -- an upper bound of the instructions actually issued (the profiler's count is in valu_issue)
    rate = valu_measured(dev)["value"] * 1e9
    for key in per_kernel:
        per_kernel[key]["lane_slots_per_pair_at_measured_issue_rate"] = (
            round(per_kernel[key]["kernel_ms"] * 1e-3 * rate * 64.0 / hits_per_launch, 1) if hits_per_launch else None)
    out["views_in_flight"] = flight
    if sections is not None:
        out["sections"] = sections
    rec_use = None if forward_only else u_ox.record_use(cam_structs[0], dev, n, 1 if opts.half_sums else 0)
    out["memory"] = dict(first_view_peak_GB=round(first_peak / 1e9, 3), steady_peak_GB=round(steady_peak / 1e9, 3),
                         first_over_steady=round(first_peak / max(steady_peak, 1), 3),
                         resident_before_GB=round(base_mem / 1e9, 3),
                         record_allocated_GB=None if rec_use is None else round(rec_use[0] / 1e9, 3),
                         record_used_GB=None if rec_use is None else round(rec_use[1] / 1e9, 3))
    del params, dscene, target, stats
    gas = None
    torch.cuda.empty_cache()
    return out, scene, cfg


OTHER_WORKLOADS = ("c1_300k_800x800", "c2_3M_1237x822", "c4_1M_1024x1024")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c4_1M_800x800", choices=sorted(WORKLOADS))
    ap.add_argument("--cpu-rays", type=int, default=262144, help="ray sample of the CPU baseline (0 = skip)")
    ap.add_argument("--fps-frames", type=int, default=20,
                    help="after the headline pass, frames of the 3 M-Gaussian 1920x1080 forward-only orbit to time for "
                         "`fwd_fps_c3` (0 = skip; skipped for workloads other than the default)")
    ap.add_argument("--other-steps", type=int, default=5,
                    help="after the headline pass, timed steps of each other benchmark configuration for `other_workloads` "
                         "(0 = skip; skipped for workloads other than the default)")
    ap.add_argument("--forward-only", action="store_true")
    ap.add_argument("--no-records", action="store_true",
                    help="backward searches the tree again instead of replaying the forward's hit-list record")
    ap.add_argument("--rec-tile-words", type=int, default=None,
                    help="record size per tile in 32-bit words (16384: hit lists only, no per-sample sums); "
                         "default: the renderer's own")
    ap.add_argument("--half-sums", action="store_true",
                    help="the record keeps the per-sample colour sums in half precision (settings.rec_half_sums)")
    ap.add_argument("--in-flight", type=int, default=2,
                    help="after the timed steps, time the same steps again with this many views in flight, each on "
                         "a stream of its own (reported beside the headline figure; 1 = skip)")
    ap.add_argument("--sections", action="store_true",
                    help="also report the march kernels' per-section cycle census; needs the diagnostic build "
                         "(python -m raygaussx_amd.build --sections; RGX_LIB_PATH=raygaussx_amd/librgx_sections.so)")
    ap.add_argument("--dump-tile-times", default=None,
                    help="with --sections: write the per-workgroup table of the timed steps (cycles per section, start and "
                         "end of the workgroup's last wave) to this .npy file")
    ap.add_argument("--side-kernels", action="store_true",
                    help="time the entry points around the march (image epilogue, reorder gather, distCUDA2, viewer launch) "
                         "instead of the training step; one JSON line")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run a 1 GiB device-to-device copy (reference reading for the FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--calibrate-valu", action="store_true",
                    help="only run the multiply-add kernel of `valu_measured` (reference reading for the SQ_INSTS_VALU counter)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (--gpus 1); the path would shard by views or bands "
                 "of tiles with one gradient all-reduce per step, but no multi-GPU figure is produced")
    if not torch.cuda.is_available():
        sys.exit("bench.py: needs a GPU (librgx has no CPU path)")
    dev = "cuda:0"
    if args.calibrate_copy:
        src = torch.full((1 << 28,), 1.0, dtype=torch.float32, device=dev)     # 1 GiB
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps(dict(calibration="copy", bytes_read=src.numel() * 4, bytes_written=dst.numel() * 4, launches=3)))
        return
    L.lib()
    if args.calibrate_valu:
        print(json.dumps(dict(calibration="valu", **valu_measured(dev), clocks_per_instruction_per_simd=valu_cost_table(dev))))
        return
    if args.side_kernels:
        print(json.dumps(side_kernels(dev, args.steps)), flush=True)
        return
    if args.sections and read_sections() is None:
        sys.exit("bench.py --sections: the loaded library has no section census; build it with "
                 "`python -m raygaussx_amd.build --sections` and set RGX_LIB_PATH=raygaussx_amd/librgx_sections.so")
    out, scene, cfg = training_leg(dev, args.workload, args.steps, args.warmup, args, in_flight=args.in_flight)
    config, n, width, height = WORKLOADS[args.workload]
    out["valu_measured"] = valu_measured(dev)
    bw = copy_bandwidth(dev)
    out["hbm_measured"] = dict(copy_GBps=bw, what="1 GiB device-to-device copy, bytes read + written",
                               roofline_frac_of_measured=round(out["roofline"]["achieved"] / bw, 5),
                               step_frac_of_measured=round(out["step_roofline"]["achieved"] / bw, 5))
    headline = args.workload == "c4_1M_800x800" and not args.forward_only
    if args.fps_frames > 0 and headline:
        out["fwd_fps_c3"] = inference_leg(dev, args.fps_frames, 3)
    if args.other_steps > 0 and headline:
        others = {}
        for name in OTHER_WORKLOADS:
            o, _, _ = training_leg(dev, name, args.other_steps, 2, args, in_flight=1)
            dom = o["roofline"]
            others[name] = dict(value=o["value"], unit="Mrays/s", ms_per_step=o["ms_per_step"], steps=o["steps"], warmup=o["warmup"],
                                step_roofline_frac=o["step_roofline"]["frac"], roofline_mrays=o["step_roofline"]["roofline_mrays"],
                                dominant_kernel=dom["kernel"], dominant_kernel_ms=dom["kernel_ms"], dominant_kernel_frac=dom["frac"],
                                march_kernels={k: dict(kernel_ms=v["kernel_ms"], frac=v["frac"],
                                                       lane_slots_per_pair_at_measured_issue_rate=v["lane_slots_per_pair_at_measured_issue_rate"])
                                               for k, v in dom["march_kernels"].items()},
                                hit_pairs_per_launch=dom["hit_pairs_per_launch"], kernels_ms=o["kernels_ms"], memory=o["memory"],
                                config=o["config"])
        out["other_workloads"] = others
    if args.cpu_rays > 0:
        # the box grants a job 16 host threads whatever os.cpu_count() shows: the baseline uses those, and says so
        threads = min(16, os.cpu_count() or 1)
        out["cpu_baseline"] = cpu_baseline(scene, scenes.make_camera(config, 0, width=width, height=height), cfg,
                                           args.cpu_rays if n <= 1_000_000 else min(args.cpu_rays, 16384), threads,
                                           backward=not (args.forward_only or args.workload.endswith("_fwd")))
        out["cpu_baseline"]["host_cpus"] = os.cpu_count()
        out["cpu_baseline"]["threads_note"] = "min(16, host cpus): 16 is this GPU box's CPU share per job"
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
