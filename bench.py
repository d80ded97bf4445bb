#!/usr/bin/env python3
"""Frame-rate benchmark of the forward rasterizer on one MI355X.

A step is one full frame of the FlashGS forward sequence (``example.py:67-94`` of the reference):
zero the pair counter, preprocess + key emission, the pair count on the host (polled in pinned
memory, where the launch stores it; ``blocking_readback_ms_per_frame`` is the same frame with the
reference driver's blocking 4-byte copy), sort, tile ranges, blend - on a synthetic scene that is
resident in HBM before timing starts.  All calls go through the C ABI of libflashgs_hip.so on
torch's current HIP stream; the output image and every work buffer are allocated once, outside
the timed region.  The K steps are timed between two synchronisations; the per-stage times and
the blend launch's duration come from a second pass over the same steps with HIP events.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 0..4] [--no-cpu-baseline] [--headline-only]

Prints one JSON line.  ``value`` is frames per second of the whole frame on the headline workload
(``--config``, default the 4K / 3M one) with the library's default arithmetic, fp32 throughout as
the reference computes; the same frame with the opt-in colour sums on the matrix unit (f16
operands) is reported beside it as ``fast_mode_*``.  ``roofline`` describes the dominant kernel (the blend),
``stages`` every stage with its algorithmic bytes against the 8 TB/s HBM peak, ``cpu_baseline`` the
same frame computed by the multithreaded CPU oracle on this machine's host cores,
``ops_surface_ms_per_frame`` the same frame through ``flash_gaussian_splatting.ops`` the way
``example.py:130-141`` times it (``ops_surface_batch_ms_per_frame``: as one batch through
``BatchRasterizer``, two frames in flight; ``two_frames_in_flight_*``: the same through the C ABI), and ``configs`` the same figures for every other benchmark
configuration (the 60-pose orbit at both frame sizes with per-frame p50 / p99).
"""
import argparse
import json
import os
import re
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0            # MI355X HBM3E, published
FP32_PEAK_TFLOPS = 157.3         # MI355X fp32 vector, published (packed FMA)
FLOP_PER_EVAL = 19               # render.cu:40-52: 2 sub, 6 mul + 3 add, 1 mul, 3 FMA, 1 sub
EXEC_SLOTS_PER_EVAL = 8.1        # non-transcendental VALU instructions the fp32 blend kernel issues per evaluation (SQ counters,
                                 # profiles/frame_cfg2_3M_4K_sq_counters.txt): 2 for the exponent from its tables, alpha*T, T -=,
                                 # 3 colour FMAs, 1.1 for staging, stop tests and loop; the v_exp_f32 issues beside them
ATTAINED_FMA_LANE_OPS = 38.05e12 # v_fma_f32 lane-operations/s measured on this part without packed math (bench.py --calibrate)
CAPACITY = {0: 1 << 20, 1: 1 << 22, 2: 1 << 24, 3: 1 << 25, 4: 1 << 25, 5: 1 << 27, 6: 1 << 25}
FAST_MODE_DTYPE = "f32 (colour sums: f16 operands on the matrix unit, fp32 products and sums)"


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=50,
                    help="untimed frames first; the clocks of an idle GPU take about 50 frames of the 4K workload to settle")
    ap.add_argument("--config", type=int, default=2,
                    help="index into BASELINE.json configs (default: the 4K / 3M headline); 5 = the 8K scene with every "
                         "splat five times as large (more than 100M pairs); 6 = the orbit scene with its anisotropic "
                         "tenth stored last")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-reps", type=int, default=3)
    ap.add_argument("--headline-only", action="store_true", help="skip the other configurations (field \"configs\")")
    ap.add_argument("--sequential-only", action="store_true",
                    help="skip the pass with two frames in flight (for kernel traces: launches that run beside another "
                         "frame's kernels take longer and would blur the per-kernel averages)")
    ap.add_argument("--other-steps", type=int, default=20, help="timed frames per other configuration")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one 256 MiB device-to-device copy, as the known-size reference for FETCH_SIZE / WRITE_SIZE")
    ap.add_argument("--size", default=None, metavar="WxH",
                    help="frame size for the trajectory workload (config 4), e.g. 3840x2160; default 1920x1080")
    ap.add_argument("--calibrate", action="store_true",
                    help="also measure what this GPU attains on a stream copy, a stream read and fp32 FMA / exp2 issue "
                         "(libflashgs_calibrate.so) and report it under \"calibration\"")
    return ap.parse_args()


def calibrate(torch, dev):
    """Attained rates of this GPU on the resources the rooflines are priced against."""
    import ctypes as C
    from flashgs_amd import build
    if not os.path.exists(build.CAL_PATH):
        raise ImportError("%s is missing: run `python -m flashgs_amd.build` first" % build.CAL_PATH)
    lib = C.CDLL(build.CAL_PATH)
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    nbytes = 1 << 30
    src = torch.ones(nbytes // 4, device=dev, dtype=torch.float32)
    dst = torch.empty_like(src)
    sink = torch.zeros(4, device=dev, dtype=torch.float32)
    out = C.c_double(0.0)

    def call(fn, *a):
        rc = fn(*a, C.byref(out), st)
        if rc != 0:
            raise RuntimeError("calibration kernel failed: HIP error %d" % rc)
        return out.value

    copy = call(lib.fgs_cal_copy, C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr()), C.c_size_t(nbytes))
    read = call(lib.fgs_cal_read, C.c_void_p(src.data_ptr()), C.c_void_p(sink.data_ptr()), C.c_size_t(nbytes))
    fma = call(lib.fgs_cal_alu, C.c_int(0), C.c_void_p(sink.data_ptr()))
    mix4 = call(lib.fgs_cal_alu, C.c_int(1), C.c_void_p(sink.data_ptr()))
    mix8 = call(lib.fgs_cal_alu, C.c_int(2), C.c_void_p(sink.data_ptr()))
    exp = call(lib.fgs_cal_alu, C.c_int(3), C.c_void_p(sink.data_ptr()))
    torch.cuda.synchronize()
    return {
        "copy_GBs_read_plus_write": round(copy / 1e9, 1), "read_GBs": round(read / 1e9, 1),
        "fma_T_lane_ops_per_s": round(fma / 1e12, 2), "fma_TFLOPs": round(2 * fma / 1e12, 2),
        "exp2_plus_sub_T_lane_ops_per_s": round(exp / 1e12, 2),
        "fma_and_exp2_4to1_T_lane_ops_per_s": round(mix4 / 1e12, 2),
        "fma_and_exp2_8to1_T_lane_ops_per_s": round(mix8 / 1e12, 2),
        "note": "1 GiB buffers; lane-ops = wave64 instructions x 64; packed fp32 is switched off, so the FMA figure "
                "is the non-packed issue rate (the published 157.3 TFLOP/s counts packed FMA)",
    }


def cpu_baseline(sc, cam, capacity, reps):
    """The CPU oracle (a port of the reference algorithm, OpenMP) on the same frame."""
    from oracle import fgs_oracle as orc
    threads = orc.default_threads()
    W, H = cam.width, cam.height
    gx, gy = (W + 15) // 16, (H + 15) // 16
    totals, per_stage, counts, walked = [], None, None, 0
    for _ in range(max(1, reps)):
        t0 = time.perf_counter()
        pre = orc.preprocess(sc.position, sc.shs, sc.opacity, sc.cov3d, W, H, 16, 16, cam.position, cam.rotation,
                             cam.focal_x, cam.focal_y, cam.zFar, cam.zNear, capacity, threads=threads)
        t1 = time.perf_counter()
        K = pre["num_rendered"]
        ks, vs = orc.sort(K, W, H, 16, 16, pre["keys"], pre["values"], threads=threads)
        t2 = time.perf_counter()
        rg = orc.ranges(K, ks, gx * gy)
        t3 = time.perf_counter()
        _, _, walked = orc.render(W, H, 16, 16, pre["points_xy"], pre["rgb_depth"], pre["conic_opacity"], vs, rg,
                                  [0, 0, 0], want_f32=False, threads=threads)
        t4 = time.perf_counter()
        totals.append(t4 - t0)
        if per_stage is None or (t4 - t0) <= min(totals):
            per_stage = dict(preprocess=round((t1 - t0) * 1e3, 2), sort=round((t2 - t1) * 1e3, 2),
                             ranges=round((t3 - t2) * 1e3, 2), blend=round((t4 - t3) * 1e3, 2))
        counts = pre["counts"]
    med = statistics.median(totals)
    return dict(value=round(1.0 / med, 3), unit="frames/s", cores=threads, kind="port",
                sample="%d full frame(s) of this workload (first pose), median" % len(totals),
                ms_per_frame=round(med * 1e3, 2), stages_ms=per_stage), counts, walked


def profiled_traffic(workload, kernel):
    """HBM bytes per launch of `kernel` on `workload` from the committed counter summary
    profiles/frame_<workload>_hbm_traffic.txt (line "traffic_bytes <kernel>: <bytes>"), with the
    summary's date; None where no summary covers it."""
    path = os.path.join(ROOT, "profiles", "frame_%s_hbm_traffic.txt" % workload)
    if not os.path.exists(path):
        return None, None
    text = open(path).read()
    date = re.search(r"^measured: *(\S+)", text, re.M)
    for m in re.finditer(r"^traffic_bytes +(.+?): *(\d+)", text, re.M):
        if m.group(1).strip() == kernel:
            return int(m.group(2)), "profiles/%s%s" % (os.path.basename(path), " (%s)" % date.group(1) if date else "")
    return None, None


class Frame:
    """One configuration resident on the GPU with every buffer a frame needs."""

    def __init__(self, torch, np, cabi, scenes, config, size=None, base=None):
        kw = {}
        if size:
            kw["width"], kw["height"] = size
        if base is not None:
            kw["base"] = base
        self.torch, self.np, self.cabi = torch, np, cabi
        self.sc = scenes.make(config, **kw)
        self.cams = self.sc.cameras
        cam = self.cams[0]
        self.W, self.H = cam.width, cam.height
        self.n = n = self.sc.num_vertex
        self.capacity = capacity = CAPACITY.get(config, 1 << 24)
        dev = torch.device("cuda:0")
        gx, gy = (self.W + 15) // 16, (self.H + 15) // 16
        self.tiles = gx * gy

        def up(a):
            return torch.from_numpy(np.ascontiguousarray(a)).to(dev)

        self.position, self.shs, self.opacity, self.cov3d = up(self.sc.position), up(self.sc.shs), up(self.sc.opacity), up(self.sc.cov3d)
        self.points_xy = torch.zeros((n, 2), device=dev)
        self.rgb_depth = torch.zeros((n, 4), device=dev)
        self.conic_opacity = torch.zeros((n, 4), device=dev)
        self.keys_u = torch.zeros(capacity, device=dev, dtype=torch.int64)
        self.vals_u = torch.zeros(capacity, device=dev, dtype=torch.int32)
        self.keys_s = torch.zeros(capacity, device=dev, dtype=torch.int64)
        self.vals_s = torch.zeros(capacity, device=dev, dtype=torch.int32)
        self.sort_size = cabi.get_sort_buffer_size(capacity)
        self.sort_space = torch.zeros(self.sort_size, device=dev, dtype=torch.int8)
        self.ranges = torch.zeros((self.tiles, 2), device=dev, dtype=torch.int32)
        self.curr_offset = torch.zeros(1, device=dev, dtype=torch.int32)
        self.offset_host = torch.zeros(1, dtype=torch.int32, pin_memory=True)
        self.count_mirror = torch.zeros(1, dtype=torch.int32, pin_memory=True)    # polled for the pair count
        self.count_word = self.count_mirror.numpy()
        self.blocking_readback = False
        self.out_color = torch.zeros((self.H, self.W, 3), device=dev, dtype=torch.uint8)
        self.bg = np.zeros(3, np.float32)
        self.stream = torch.cuda.current_stream().cuda_stream
        self.P = {k: getattr(self, k).data_ptr() for k in (
            "position", "shs", "opacity", "cov3d", "points_xy", "rgb_depth", "conic_opacity", "keys_u", "vals_u",
            "keys_s", "vals_s", "sort_space", "ranges", "curr_offset", "out_color")}

    def twin(self):
        """A second set of work buffers and output image for the same scene (the scene tensors are shared)."""
        import copy
        torch, cabi = self.torch, self.cabi
        t = copy.copy(self)
        dev = self.position.device
        for name in ("points_xy", "rgb_depth", "conic_opacity", "keys_u", "vals_u", "keys_s", "vals_s", "sort_space", "ranges",
                     "curr_offset", "out_color"):
            setattr(t, name, torch.zeros_like(getattr(self, name)))
        t.offset_host = torch.zeros(1, dtype=torch.int32, pin_memory=True)
        t.count_mirror = torch.zeros(1, dtype=torch.int32, pin_memory=True)
        t.count_word = t.count_mirror.numpy()
        t.P = {k: getattr(t, k).data_ptr() for k in self.P}
        return t

    def in_flight(self, cams, steps, warmup, sets=2):
        """ms per frame with `sets` frames in flight: every set of work buffers has a stream of its own and
        the frames go to the sets in turn, so that one frame's blend (bound by instruction issue) runs beside
        the next frame's preprocess and sort (bound by memory).  Frame i + sets waits for frame i's image."""
        torch = self.torch
        frames = [self] + [self.twin() for _ in range(sets - 1)]
        streams = [torch.cuda.Stream() for _ in frames]
        saved = self.stream
        for f, s in zip(frames, streams):
            f.stream = s.cuda_stream

        def run(n):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(n):
                j = i % sets
                with torch.cuda.stream(streams[j]):
                    frames[j].frame(cams[i % len(cams)])
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) * 1e3 / n
        try:
            run(max(warmup, sets))
            ms = run(steps)
            same = all(bool(torch.equal(frames[0].out_color, f.out_color)) for f in frames[1:]) if len(cams) == 1 else None
        finally:
            self.stream = saved
        return ms, same

    def frame(self, c, ev=None, flags=None):
        """One frame; `flags` (cabi.BLEND_*) chooses the blend's colour-sum mode for this call, None = the library default."""
        cabi, P, W, H, st = self.cabi, self.P, self.W, self.H, self.stream
        if ev: ev[0].record()
        self.curr_offset.zero_()
        mirror = None
        if not self.blocking_readback:
            self.count_word[0] = cabi.COUNT_PENDING
            mirror = self.count_mirror.data_ptr()
        cabi.preprocess(self.n, P["position"], P["shs"], P["opacity"], P["cov3d"], W, H, 16, 16, c.position, c.rotation,
                        c.focal_x, c.focal_y, c.zFar, c.zNear, P["points_xy"], P["rgb_depth"], P["conic_opacity"],
                        P["keys_u"], P["vals_u"], P["curr_offset"], self.capacity, st, count_mirror=mirror)
        if ev: ev[1].record()
        if self.blocking_readback:
            self.offset_host.copy_(self.curr_offset)      # blocking read of the pair count (example.py:79)
            K = int(self.offset_host[0])
        else:
            K = cabi.wait_count(mirror)                   # the launch stores the count into pinned memory as soon as it has it
        if K < 0 or K >= self.capacity:
            raise RuntimeError("too many pairs: %d (capacity %d)" % (K, self.capacity))
        if ev: ev[2].record()
        cabi.sort_gaussian(K, W, H, 16, 16, P["sort_space"], self.sort_size, P["keys_u"], P["vals_u"], P["keys_s"], P["vals_s"], st)
        if ev: ev[3].record()
        cabi.tile_ranges(16, 16, K, W, H, P["keys_s"], P["ranges"], st)
        if ev: ev[4].record()
        cabi.blend(16, 16, W, H, P["points_xy"], P["rgb_depth"], P["conic_opacity"], P["vals_s"], P["ranges"], self.bg,
                   P["out_color"], None, st, flags=flags)
        if ev: ev[5].record()
        return K

    def timed(self, cams, steps, warmup, per_frame_sync, flags=None):
        """steps frames over `cams` in turn: (ms per step, per-stage mean ms, per-frame ms or [], pair count of the first).

        The steps are timed between two synchronisations with nothing else in the stream.  The
        per-stage times come from a second pass over the same steps with a HIP event in front of
        every stage: six event records cost about 0.02 ms per frame, a fifth of a 720p frame, so
        they stay out of the pass the frame time is taken from (`self.instrumented_ms` is the
        frame time of the pass that carries them)."""
        torch = self.torch
        for i in range(warmup):
            self.frame(cams[i % len(cams)], flags=flags)
        torch.cuda.synchronize()
        frame_ms, Ks = [], []
        t_start = time.perf_counter()
        for i in range(steps):
            t0 = time.perf_counter()
            Ks.append(self.frame(cams[i % len(cams)], None, flags))
            if per_frame_sync:            # per-frame latency only matters for the trajectory workload
                torch.cuda.synchronize()
                frame_ms.append((time.perf_counter() - t0) * 1e3)
        torch.cuda.synchronize()
        t_end = time.perf_counter()
        events = [[torch.cuda.Event(enable_timing=True) for _ in range(6)] for _ in range(steps)]
        torch.cuda.synchronize()
        t_events = time.perf_counter()
        for i in range(steps):
            self.frame(cams[i % len(cams)], events[i], flags)
            if per_frame_sync:
                torch.cuda.synchronize()
        torch.cuda.synchronize()
        self.instrumented_ms = (time.perf_counter() - t_events) * 1e3 / steps
        names = ["preprocess", "readback", "sort", "ranges", "blend"]
        stage_ms = {nm: statistics.mean(ev[j].elapsed_time(ev[j + 1]) for ev in events) for j, nm in enumerate(names)}
        return (t_end - t_start) * 1e3 / steps, stage_ms, frame_ms, Ks[0]


def stage_report(fr, stage_ms, K, counts, walked):
    """Per-stage figures against the rooflines that bound them, and the roofline block of the blend."""
    n, W, H, tiles = fr.n, fr.W, fr.H, fr.tiles
    passes = (32 + int(tiles).bit_length() + 7) // 8
    stages = {}

    def hbm(name, nbytes):
        ms = stage_ms[name]
        gbs = nbytes / (ms * 1e-3) / 1e9 if ms > 0 else 0.0
        stages[name] = dict(ms=round(ms, 4), bound="hbm", algorithmic_bytes=int(nbytes),
                            achieved_GBs=round(gbs, 1), peak_GBs=HBM_PEAK_GBS, frac=round(gbs / HBM_PEAK_GBS, 4))

    if counts is not None:
        hbm("preprocess", 16 * n + 24 * counts["n_pass"] + 232 * counts["visible"] + 12 * K)
    else:
        stages["preprocess"] = dict(ms=round(stage_ms["preprocess"], 4), bound="hbm")
    hbm("sort", K * (8 + 24 * passes))
    tile_passes = (int(tiles).bit_length() + 7) // 8
    stages["sort"]["design_bytes"] = int(K * (32 * tile_passes + 8 + 24))   # count + scatter per tile digit, starts, segment sort
    hbm("ranges", 8 * K + 16 * tiles)
    stages["readback"] = dict(ms=round(stage_ms["readback"], 4), bound="host latency: GPU time between the preprocess launch and the first sort launch (the host polls "
                                   "the pair count in pinned memory and enqueues the sort while the launch still writes keys)")

    blend_ms = stage_ms["blend"]
    kernel = fr.cabi.blend_kernel_name(16, 16, W, H)        # of the library default, which is what was timed
    traffic, source = profiled_traffic(fr.sc.name, kernel)
    roofline = dict(kernel=kernel, bound="valu", achieved=None, peak=FP32_PEAK_TFLOPS, unit="TFLOP/s", frac=None,
                    traffic=traffic, traffic_source=source, launch_ms=round(blend_ms, 4))
    stages["blend"] = dict(ms=round(blend_ms, 4), bound="valu", kernel=kernel)
    if walked is not None:
        evals = 256 * walked
        # reference-equivalent work: the 19 flop of render.cu:40-52 per pixel-Gaussian evaluation over the
        # published fp32 vector peak (which counts packed FMA; this library issues none)
        tflops = FLOP_PER_EVAL * evals / (blend_ms * 1e-3) / 1e12
        # executed work: the kernel's own VALU instructions per evaluation over the v_fma_f32 rate this part attains
        floor_ms = EXEC_SLOTS_PER_EVAL * evals / ATTAINED_FMA_LANE_OPS * 1e3
        roofline.update(achieved=round(tflops, 2), frac=round(tflops / FP32_PEAK_TFLOPS, 4),
                        achieved_is="reference-equivalent flop (19 per evaluation, render.cu:40-52) per second",
                        evaluations=int(evals), flop_per_evaluation=FLOP_PER_EVAL,
                        executed_valu_instructions_per_evaluation=EXEC_SLOTS_PER_EVAL,
                        issue_bound_ms=round(floor_ms, 4), frac_of_attained_issue_rate=round(floor_ms / blend_ms, 4),
                        hbm_bytes=int(8 * tiles + 44 * walked + 3 * W * H))
        stages["blend"].update(achieved_TFLOPs=roofline["achieved"], frac=roofline["frac"])
    return stages, roofline


def ops_surface_ms(torch, np, fr, steps):
    """The same frame through flash_gaussian_splatting.ops, timed as example.py:130-141 does: one
    untimed frame, then the mean over `steps` frames between two synchronisations."""
    from flashgs_amd.rasterizer import Camera, Rasterizer, Scene
    scene = Scene(torch.device("cuda:0"))
    scene.num_vertex = fr.n
    scene.position, scene.shs, scene.opacity, scene.cov3d = fr.position, fr.shs, fr.opacity, fr.cov3d
    cam = Camera.from_synthetic(fr.cams[0])
    rast = Rasterizer(scene, fr.capacity, fr.tiles, max_width=fr.W, max_height=fr.H)
    bg = torch.zeros(3, dtype=torch.float32)
    img = rast.forward(scene, cam, bg)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        img = rast.forward(scene, cam, bg)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    fr.frame(fr.cams[0])                        # the same frame through the C ABI, library default like the ops
    torch.cuda.synchronize()
    same = bool(torch.equal(img, fr.out_color))
    del rast
    # the same frames as one batch through BatchRasterizer: two frames in flight, every image kept
    from flashgs_amd.rasterizer import BatchRasterizer
    frames = min(steps, 64)
    batch = BatchRasterizer(scene, fr.capacity, fr.tiles, frames_in_flight=2)
    out = batch.render(scene, [cam] * frames, bg)
    batch.render(scene, [cam] * frames, bg, out=out)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(2):
        batch.render(scene, [cam] * frames, bg, out=out)
    torch.cuda.synchronize()
    batch_ms = (time.perf_counter() - t0) * 1e3 / (2 * frames)
    same = same and bool(torch.equal(out[0], fr.out_color)) and bool(torch.equal(out[-1], fr.out_color))
    del batch, out
    return round(ms, 4), same, round(batch_ms, 4)


def run_config(mods, config, size, steps, warmup, cpu_reps, with_cpu, with_ops, base=None, in_flight=True):
    torch, np, cabi, scenes = mods
    fr = Frame(torch, np, cabi, scenes, config, size, base)
    ms_per_step, stage_ms, _, K = fr.timed(fr.cams[:1], steps, warmup, False)
    instrumented_ms = fr.instrumented_ms
    # the same frame with the opt-in colour sums on the matrix unit, chosen per call
    fast_ms, fast_stage, _, _ = fr.timed(fr.cams[:1], max(5, steps // 2), 2, False, flags=cabi.BLEND_MATRIX_F16)
    # ... and with the reference driver's blocking read of the pair count instead of the polled mirror
    fr.blocking_readback = True
    blocking_ms, _, _, _ = fr.timed(fr.cams[:1], max(5, steps // 2), 2, False)
    fr.blocking_readback = False
    # ... and with two frames in flight, each on a stream and a set of work buffers of its own
    flight_ms, flight_same = fr.in_flight(fr.cams[:1], steps, min(warmup, 20)) if in_flight else (None, None)
    cpu, counts, walked = (None, None, None)
    if with_cpu:
        cpu, counts, walked = cpu_baseline(fr.sc, fr.cams[0], fr.capacity, cpu_reps)
    stages, roofline = stage_report(fr, stage_ms, K, counts, walked)
    rep = dict(workload=fr.sc.name, gaussians=fr.n, width=fr.W, height=fr.H, pairs=int(K), poses=len(fr.cams),
               ms_per_frame=round(ms_per_step, 4), fps=round(1000.0 / ms_per_step, 2), dtype="f32", stages=stages,
               roofline=roofline, cpu_baseline=cpu,
               pair_count="stored into pinned host memory by the launch as soon as it is known and polled there "
                          "(fgs_preprocess_mirrored / fgs_wait_count)",
               blocking_readback_ms_per_frame=round(blocking_ms, 4),
               two_frames_in_flight=None if flight_ms is None else dict(
                   ms_per_frame=round(flight_ms, 4), fps=round(1000.0 / flight_ms, 2), images_identical=flight_same,
                   what="the same frames sent in turn to two streams, each with work buffers and an image of its own: "
                        "one frame's blend runs beside the next frame's preprocess and sort"),
               stage_timing="a second pass over the same steps with a HIP event in front of every stage",
               ms_per_frame_with_stage_events=round(instrumented_ms, 4),
               fast_mode=dict(dtype=FAST_MODE_DTYPE, ms_per_frame=round(fast_ms, 4), fps=round(1000.0 / fast_ms, 2),
                              blend_ms=round(fast_stage["blend"], 4),
                              kernel=cabi.blend_kernel_name(16, 16, fr.W, fr.H, cabi.BLEND_MATRIX_F16)))
    if counts is not None:
        rep.update(n_pass=counts["n_pass"], visible=counts["visible"], walked=int(walked))
    if len(fr.cams) > 1:
        # the trajectory: every pose once, the per-frame pipeline re-run, host-timed with a sync per frame
        traj_ms, traj_stage, frame_ms, _ = fr.timed(fr.cams, len(fr.cams), min(warmup, 3), True)
        frame_ms.sort()
        rep["trajectory"] = dict(poses=len(fr.cams), ms_per_frame_mean=round(traj_ms, 4),
                                 frame_ms_p50=round(frame_ms[len(frame_ms) // 2], 4),
                                 frame_ms_p99=round(frame_ms[min(len(frame_ms) - 1, int(0.99 * len(frame_ms)))], 4),
                                 stages_ms_mean={k: round(v, 4) for k, v in traj_stage.items()})
        # the whole orbit as a batch: the poses in turn on two streams, no synchronisation between frames
        if in_flight:
            batch_ms, _ = fr.in_flight(fr.cams, 2 * len(fr.cams), len(fr.cams) // 2)
            rep["trajectory"]["batch_two_frames_in_flight_ms_per_frame"] = round(batch_ms, 4)
    if with_ops:
        (rep["ops_surface_ms_per_frame"], rep["ops_surface_image_identical"],
         rep["ops_surface_batch_ms_per_frame"]) = ops_surface_ms(torch, np, fr, steps)
    return rep, fr


def main():
    args = parse()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build renders on one GPU only; --gpus %d is not supported "
              "(a frame shards by poses or by bands of tiles, with no exchange but the final image)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from flashgs_amd import cabi, scenes

    cabi.load()   # no library, no benchmark: there is no fallback path
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    mods = (torch, np, cabi, scenes)

    size = None
    if args.size:
        if args.config not in (4, 6):
            sys.exit("bench.py: --size applies to the trajectory workload (--config 4 or 6) only")
        size = tuple(int(v) for v in args.size.lower().split("x"))
    with_cpu = not args.no_cpu_baseline

    head, fr = run_config(mods, args.config, size, args.steps, args.warmup, args.cpu_reps, with_cpu, not args.sequential_only,
                          in_flight=not args.sequential_only)
    if args.copy_calibration:
        src = torch.ones(64 << 20, device=dev, dtype=torch.float32)      # 256 MiB read + 256 MiB written
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    result = {
        "metric": "frames/s, full forward frame (preprocess + sort + ranges + blend)",
        "value": head["fps"], "unit": "frames/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": head["ms_per_frame"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": head["dtype"],
        "dtype_note": "every stage in fp32 as the reference (ndc2Pix in fp64 as its literals make it); the timed blend "
                      "kernel is the one named in roofline.kernel",
        "data": "synthetic",
        "config": {"workload": head["workload"], "gaussians": head["gaussians"], "width": head["width"], "height": head["height"],
                   "tile": "16x16", "sh_degree": 3, "pairs": head["pairs"], "poses": head["poses"],
                   "stages_ms": {k: v["ms"] for k, v in head["stages"].items()},
                   "fast_mode": head["fast_mode"],
                   "blocking_readback_ms_per_frame": head["blocking_readback_ms_per_frame"],
                   "two_frames_in_flight": head["two_frames_in_flight"]},
        "target_fps": 400 if args.config == 2 else None,
        "fast_mode_ms_per_frame": head["fast_mode"]["ms_per_frame"],
        "fast_mode_fps": head["fast_mode"]["fps"],
        "fast_mode_dtype": FAST_MODE_DTYPE,
        "pair_count": head["pair_count"],
        "blocking_readback_ms_per_frame": head["blocking_readback_ms_per_frame"],
        "two_frames_in_flight_ms_per_frame": (head["two_frames_in_flight"] or {}).get("ms_per_frame"),
        "two_frames_in_flight_fps": (head["two_frames_in_flight"] or {}).get("fps"),
        "stage_timing": head["stage_timing"],
        "ms_per_frame_with_stage_events": head["ms_per_frame_with_stage_events"],
        "stages": head["stages"],
        "roofline": head["roofline"],
        "cpu_baseline": head["cpu_baseline"],
        "ops_surface_ms_per_frame": head.get("ops_surface_ms_per_frame"),
        "ops_surface_image_identical": head.get("ops_surface_image_identical"),
        "ops_surface_batch_ms_per_frame": head.get("ops_surface_batch_ms_per_frame"),
    }
    for k in ("n_pass", "visible", "walked"):
        if k in head:
            result["config"][k] = head[k]
    if "trajectory" in head:
        result["trajectory"] = head["trajectory"]
        result["frame_ms_p50"] = head["trajectory"]["frame_ms_p50"]
        result["frame_ms_p99"] = head["trajectory"]["frame_ms_p99"]
    if args.calibrate:
        result["calibration"] = calibrate(torch, dev)
    del fr
    torch.cuda.empty_cache()

    if not args.headline_only:
        others = {}
        big = None          # the 8M scene, generated once for the 8K configuration and its dense variant
        for config, sz in ((0, None), (1, None), (2, None), (3, None), (5, None), (4, None), (4, (3840, 2160)), (6, (3840, 2160))):
            if config == args.config and sz == size:
                continue
            rep, fr_o = run_config(mods, config, sz, args.other_steps, min(args.warmup, 3), 1, with_cpu, False,
                                   base=big if config == 5 else None)
            others[rep["workload"]] = rep
            big = fr_o.sc if config == 3 else (None if config == 5 else big)
            del fr_o
            torch.cuda.empty_cache()
        result["configs"] = others
    print(json.dumps(result))


if __name__ == "__main__":
    main()
