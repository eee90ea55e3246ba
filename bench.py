"""Benchmark of the Visual Mesh inference hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2] [--frames F] [--no-cpu] [--no-pcie] [--no-configs]

A step is one pass of the whole device path (projection, filter/compaction, sampling, neighbourhood, all
graph-convolution layers) over one staged batch of synthetic frames whose inputs are already resident in
device memory. Prints one JSON line: nodes classified per second (`value`, configuration 2 unless --config says
otherwise), frames per second, the roofline position of the dominant kernel (timed live with HIP events on the
engine's stream), the reference's CPU engine timed on the host's cores as a baseline, the end-to-end figure (host
images to classified mesh in host arrays, pipelined over three engines) next to the serial one, and a short run of
each of the other configurations (`configs`).
"""
import argparse
import json
import os
import sys
import threading
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# Every engine owns a HIP stream, and the HIP runtime spreads a process's streams over GPU_MAX_HW_QUEUES hardware queues
# (4 unless the environment says otherwise). This process has up to five streams alive at a time (the engine of the timed
# passes, three engines in rotation for the end-to-end figure, the default stream); two streams on one hardware queue
# take turns, and the rotation then needs 2.55 ms per batch instead of 1.82 (measured both ways, and with 2 queues and no
# extra engine: 2.55 ms as well). Read by the runtime when it starts, so it is set before anything touches HIP - unless a
# profiler has already started the runtime's lower layers in this process with the value it found (rocprofv3's preloaded
# tool does; a different value afterwards crashes it in the first graph launch): then the environment is left alone, and
# a command line that wants the setting exports it before the profiler.
if not any(k.startswith(("ROCPROF", "ROCP_")) for k in os.environ) and "rocprof" not in os.environ.get("LD_PRELOAD", ""):
    try:
        queues_now = int(os.environ.get("GPU_MAX_HW_QUEUES", "4"))
    except ValueError:
        queues_now = 4
    if queues_now < 8:  # an environment that names the runtime's default of 4 is raised too: five streams need five queues
        os.environ["GPU_MAX_HW_QUEUES"] = "8"

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E
FP32_PEAK_TFLOPS = 157.3   # MI355X dense fp32 matrix
BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 matrix
# the arithmetic a configuration's engine computes its 64-wide layers in ("split": every value a pair of bf16, three
# products per pair of values on the bf16 matrix instructions, fp32 accumulation; parity bar as for fp32)
DTYPE = {"fp32": "f32", "bf16": "bf16", "split": "bf16 pairs"}

def measured_traffic(workload, kernel):
    """HBM bytes per launch of `kernel` on `workload` from the rocprofv3 FETCH_SIZE / WRITE_SIZE summaries under
    profiles/: each summary carries lines
        <!-- traffic: workload=cfg2 kernel=conv_flow_32x32s7 bytes_per_launch=N source=<kernel source file> sha256=<of that file> -->
    written when the counters were read. A figure counts only while the kernel's source is still the file that was
    measured; otherwise (or without a summary) -> (None, why)."""
    import glob
    import hashlib
    import re
    found = None
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*.md"))):
        for m in re.finditer(r"<!-- traffic: workload=(\S+) kernel=(\S+) bytes_per_launch=(\d+) source=(\S+) sha256=([0-9a-f]+) -->", open(path).read()):
            if m.group(1) == workload and m.group(2) == kernel:
                found = (int(m.group(3)), m.group(4), m.group(5), os.path.basename(path))
    if found is None:
        return None, "no counter summary under profiles/ for this kernel and workload"
    nbytes, source, sha, where = found
    try:
        now = hashlib.sha256(open(os.path.join(ROOT, source), "rb").read()).hexdigest()
    except OSError:
        return None, "the measured source file %s is gone" % source
    if now != sha:
        return None, "profiles/%s was measured on another version of %s" % (where, source)
    return nbytes, "profiles/" + where


def layer_table(cfg, n_neighbours):
    """per layer: (c_in, c_out, slots, algorithmic bytes per row, flops per row) for fp32 activations"""
    out = []
    c_in = 4
    for group in cfg.network:
        for li, (w, b, act) in enumerate(group):
            slots = n_neighbours + 1 if li == 0 else 1
            c_out = w.shape[1]
            nbytes = c_in * 4 + (4 * n_neighbours if li == 0 else 0) + c_out * 4
            flops = 2 * slots * c_in * c_out
            out.append((c_in, c_out, slots, nbytes, flops))
            c_in = c_out
    return out


def conv_roofline(name, avg_ms, rows):
    """Roofline entry of one launch of a graph-convolution kernel over `rows` rows: the layer shape is in the kernel
    name, conv_<kind>_<cin>x<cout>s<slots>, and so are storage and arithmetic: conv_bf16_<in>_to<out>_* runs on the
    bf16 matrix instructions and reads / writes rows as bf16 (2 bytes per channel), x2 (hi + lo pairs of bf16, 4 bytes)
    or f32; conv_lds_tox2_* writes x2 rows. Flops are the layer's algorithmic ones, not the hi/lo extras.
    -> (dict, algorithmic bytes per row, flops per row)"""
    shape = name.split("_")[-1]
    c_in, rest = shape.split("x")
    c_out, slots = rest.split("s")
    c_in, c_out, slots = int(c_in), int(c_out), int(slots)
    bf16_arith = name.startswith("conv_bf16")
    s_in = 2 if name.startswith("conv_bf16_bf16_") else 4
    s_out = 2 if "_tobf16_" in name else 4
    bytes_per_row = c_in * s_in + 4 * (slots - 1) + c_out * s_out
    if name.startswith("neighbourhood_conv_"):
        # the neighbourhood kernel with the first layer in it: the mesh's neighbour table read, the reverse-lookup gathers
        # and the row's table written (4 bytes per neighbour each), then the layer's input and output rows; the table
        # the layer gathers through is the one just written, so it is counted once
        bytes_per_row = 12 * (slots - 1) + c_in * 4 + c_out * 4
    flops_per_row = 2 * slots * c_in * c_out
    intensity = flops_per_row / bytes_per_row
    matrix_peak = BF16_PEAK_TFLOPS if bf16_arith else FP32_PEAK_TFLOPS
    ridge = matrix_peak * 1e12 / (HBM_PEAK_GBS * 1e9)
    if intensity > ridge:
        achieved = flops_per_row * rows / (avg_ms * 1e-3) / 1e12
        entry = dict(bound="mfma", achieved=achieved, peak=matrix_peak, unit="TFLOP/s", frac=achieved / matrix_peak)
    else:
        achieved = bytes_per_row * rows / (avg_ms * 1e-3) / 1e9
        entry = dict(bound="hbm", achieved=achieved, peak=HBM_PEAK_GBS, unit="GB/s", frac=achieved / HBM_PEAK_GBS)
    return entry, bytes_per_row, flops_per_row


def cpu_baseline(cfg, threads, passes):
    """The reference's CPU engine, compiled from its own headers behind the oracle's interface, where that library was
    built (kind "reference"); otherwise the CPU oracle, a port of it (kind "port"). `threads` host threads, one frame
    per task, a fresh engine per frame, the mesh shared - the reference benchmark's own pattern. The batch is
    worked through `passes` times so that the sample is several seconds of CPU work."""
    from oracle import vmo
    O = vmo.load("reference")
    kind = "reference"
    if O is None:
        O, kind = vmo.load("oracle"), "port"
    lens = vmo.make_lens(*cfg.lens_tuple())
    if cfg.visualmesh is None:
        mesh = O.mesh(cfg.model, cfg.shape, cfg.radius, cfg.mesh_h, cfg.k, cfg.max_distance)
        pick = lambda H: mesh
    else:
        v = cfg.visualmesh
        vm = O.visualmesh(cfg.model, cfg.shape, cfg.radius, v["min_h"], v["max_h"], cfg.k, v["max_error"], cfg.max_distance)
        pick = lambda H: vm.height(float(H[2][3]))
    net = vmo.Network(cfg.network)
    frames = cfg.frames
    visible = [0] * len(frames)
    todo = list(range(len(frames))) * passes
    lock = threading.Lock()

    def worker():
        while True:
            with lock:
                if not todo:
                    return
                i = todo.pop()
            f = frames[i]
            r = pick(f["Hoc"]).classify(f["Hoc"], lens, f["image"], cfg.fourcc, net)  # ctypes releases the GIL
            visible[i] = len(r["gidx"])

    t0 = time.perf_counter()
    pool = [threading.Thread(target=worker) for _ in range(threads)]
    for t in pool:
        t.start()
    for t in pool:
        t.join()
    dt = time.perf_counter() - t0
    return sum(visible) * passes / dt, len(frames) * passes / dt, dt, kind


def build_workload(index, n_frames=None):
    """configuration `index` staged on a fresh engine -> (cfg, engine, mesh, lens, frames)"""
    from visualmesh_amd import engine as eng
    from visualmesh_amd import native
    from visualmesh_amd import workloads as wl
    cfg = wl.config(index, n_frames=n_frames)
    lens = native.make_lens(*cfg.lens_tuple())
    if cfg.visualmesh is None:
        mesh = eng.Mesh(cfg.model, cfg.shape, cfg.radius, cfg.mesh_h, cfg.k, cfg.max_distance)
    else:
        v = cfg.visualmesh
        mesh = eng.VisualMesh(cfg.model, cfg.shape, cfg.radius, v["min_h"], v["max_h"], cfg.k, v["max_error"], cfg.max_distance)
    precision = {"bf16": native.BF16, "split": native.SPLIT}.get(cfg.precision, native.FP32)
    engine = eng.Engine(cfg.network, cfg.model, precision)
    frames = [dict(mesh=mesh, Hoc=f["Hoc"], lens=lens, image=f["image"], fourcc=cfg.fourcc) for f in cfg.frames]
    return cfg, engine, mesh, lens, frames


def workload_name(cfg, n_frames, table):
    from visualmesh_amd import workloads as wl
    return "%s: %d frames of %dx%d %s, %s lens, %s mesh, network %s" % (
        cfg.name, n_frames, cfg.width, cfg.height, "RGBA8" if cfg.fourcc == wl.fourcc("RGBA") else "GRBG8",
        {0: "rectilinear", 1: "equisolid", 2: "equidistant"}[cfg.projection],
        {0: "Ring6", 1: "NMGrid8"}[cfg.model], "->".join(["4"] + [str(t[1]) for t in table]))


def measure(cfg, engine, frames, steps, warmup, settle_s, events=True, stream_ceiling=True):
    """Stages `frames` (inputs resident in HBM from then on), lets the clocks settle, then W untimed and K timed passes.
    -> dict with the throughput, the dominant kernel's roofline (timed live with HIP events on the engine's stream in the
    timed passes) and every graph-convolution kernel's (from one fully bracketed, untimed pass)."""
    from visualmesh_amd import workloads as wl
    nn = wl.N_NEIGHBOURS[cfg.model]
    engine.stage(frames)
    # The GPU's clocks need some tens of milliseconds of work to settle (20 timed passes right after staging read 4-8 %
    # slower): an untimed pre-roll of the same pass, stated in the result, comes before the warm-up passes.
    settle_passes, t0 = 0, time.perf_counter()
    while settle_s > 0 and (time.perf_counter() - t0 < settle_s or settle_passes < 3):
        engine.run()
        settle_passes += 1
    settle_ms = (time.perf_counter() - t0) * 1e3
    for _ in range(warmup):
        engine.run()
    visible = engine.counts()
    nodes = int(visible.sum())

    # One pass with HIP events around every kernel launch (untimed, launched kernel by kernel) finds the kernel that takes
    # longest and gives the per-kernel table; in the timed passes only that kernel's launches are bracketed with events,
    # on the engine's own stream. The timed passes replay the captured HIP graph of the pass, as a caller's do, and the
    # event records are nodes of that graph (they cost 0.4 % of a pass; events between all kernels, which keep the pass
    # out of a graph, cost 4 %).
    engine.profile(1)
    engine.run()
    kernel_ms_per_step, launches_per_step = {}, {}
    for name, ms, units in engine.profile_read():
        kernel_ms_per_step[name] = kernel_ms_per_step.get(name, 0.0) + ms
        launches_per_step[name] = launches_per_step.get(name, 0) + 1
    engine.profile(2 if events else 0)
    for _ in range(2):
        engine.run()              # untimed: the first run after a change of timing mode goes kernel by kernel, the second is captured
    kernel_ms, kernel_launches = {}, {}
    dominant_ms_total = 0.0
    t0 = time.perf_counter()
    for _ in range(steps):
        engine.run()              # launches the whole path and waits for it
        if not events:
            continue
        for name, ms, units in engine.profile_read():
            kernel_ms[name] = kernel_ms.get(name, 0.0) + ms
            kernel_launches[name] = kernel_launches.get(name, 0) + 1
    elapsed = time.perf_counter() - t0
    engine.profile(0)

    # roofline of the dominant kernel: a graph-convolution kernel, or (small single-frame workloads) one of the
    # kernels before the network, which move bytes only
    rows = nodes + len(frames)    # visible nodes + one null row per frame
    conv = {k: v for k, v in kernel_ms.items() if k.startswith(("conv", "neighbourhood_conv"))}
    dominant = max(conv, key=conv.get) if conv else None
    roofline = None
    if not dominant and kernel_ms:
        dominant = max(kernel_ms, key=kernel_ms.get)
        avg_ms = kernel_ms[dominant] / kernel_launches[dominant]
        candidates = sum(int((r[:, 1] - r[:, 0]).sum()) for r in (engine.staged_ranges(i) for i in range(len(frames))))
        texel_bytes = 16 if cfg.fourcc == wl.fourcc("RGBA") else 36   # four RGBA8 texels / the 6x6 union of four Bayer patches
        algorithmic = {"project": 12 * candidates + 12 * nodes,            # rays read; pixel and index written per visible node
                       "compact_sample": (texel_bytes + 16) * nodes,       # texels read, four floats written
                       "neighbourhood": 12 * nn * nodes,                   # table read, reverse-lookup gathers, table written
                       "half_tables": (4 * nn + 16) * nodes}[dominant]     # table read, half-tile positions written
        achieved = algorithmic / (avg_ms * 1e-3) / 1e9
        roofline = dict(bound="hbm", achieved=achieved, peak=HBM_PEAK_GBS, unit="GB/s", frac=achieved / HBM_PEAK_GBS, kernel=dominant,
                        avg_launch_ms=avg_ms, launches_per_step=kernel_launches[dominant] // steps, algorithmic_bytes_per_launch=algorithmic)
    elif dominant:
        avg_ms = kernel_ms[dominant] / kernel_launches[dominant]
        roofline, bytes_per_row, flops_per_row = conv_roofline(dominant, avg_ms, rows)
        roofline.update(kernel=dominant, avg_launch_ms=avg_ms, launches_per_step=kernel_launches[dominant] // steps,
                        rows_per_launch=rows, algorithmic_bytes_per_row=bytes_per_row, flops_per_row=flops_per_row)
    if roofline is not None:
        roofline["traffic"], roofline["traffic_source"] = measured_traffic(cfg.name, dominant)

    # every graph-convolution kernel against its own roofline, from the one fully bracketed (untimed) pass
    conv_rooflines = {}
    for name, ms in sorted(kernel_ms_per_step.items()):
        if name.startswith(("conv", "neighbourhood_conv")):
            entry, bytes_per_row, flops_per_row = conv_roofline(name, ms / launches_per_step[name], rows)
            conv_rooflines[name] = dict(bound=entry["bound"], achieved=entry["achieved"], unit=entry["unit"], frac=entry["frac"],
                                        avg_launch_ms=ms / launches_per_step[name], algorithmic_bytes_per_row=bytes_per_row,
                                        flops_per_row=flops_per_row)
            if name.startswith("neighbourhood_conv"):
                nn = int(name.split("s")[-1]) - 1
                conv_rooflines[name]["bytes_per_row_is"] = (
                    "%d for the neighbourhood stage (mesh neighbours, reverse-lookup gathers and the table written, 4 bytes per "
                    "neighbour each) + %d for the layer (input row, neighbour table, output row) - %d: the layer gathers through "
                    "the table the same kernel has just written" % (12 * nn, bytes_per_row - 12 * nn + 4 * nn, 4 * nn))
    # The layers bound by memory, against what the memory system gives a kernel that does nothing but read and write
    # their bytes (same rows, same bytes per row in and out, whole cache lines, no gather, no arithmetic): the ceiling
    # that a copy-like kernel of that shape reaches on this device, next to the 8 TB/s on the data sheet.
    if stream_ceiling:
        from visualmesh_amd import native
        for name, entry in conv_rooflines.items():
            if entry["bound"] != "hbm" or name.startswith("neighbourhood_conv"):
                continue
            shape = name.split("_")[-1]
            c_in, rest = shape.split("x")
            c_out, slots = rest.split("s")
            s_in = 2 if name.startswith("conv_bf16_bf16_") else 4
            s_out = 2 if "_tobf16_" in name else 4
            read_b, write_b = int(c_in) * s_in + 4 * (int(slots) - 1), int(c_out) * s_out
            ms = native.stream_probe(rows, read_b, write_b)
            ceiling = (read_b + write_b) * ((rows + 63) // 64 * 64) / (ms * 1e-3) / 1e9
            entry["stream_ceiling_GBps"] = ceiling
            entry["frac_of_stream_ceiling"] = entry["achieved"] / ceiling
    # the dominant kernel's launches inside the timed passes themselves, per pass: never more than ms_per_step
    dominant_ms_total = sum(kernel_ms.values()) / steps if kernel_ms else None
    return dict(value=nodes * steps / elapsed, frames_per_s=len(frames) * steps / elapsed, ms_per_step=elapsed * 1e3 / steps, nodes=nodes,
                settle_passes=settle_passes, settle_ms=settle_ms, roofline=roofline, kernel_ms_per_step=dict(sorted(kernel_ms_per_step.items())),
                conv_rooflines=conv_rooflines, dominant_kernel_ms_per_step_in_timed_passes=dominant_ms_total)


def pinned_copies(cfg, mesh, lens):
    from visualmesh_amd import native
    # one page-locked allocation for all the batch's images, as a ring of camera buffers would be: images that adjoin
    # in memory go up in one copy
    sizes = [int(f["image"].nbytes) for f in cfg.frames]
    block = native.pinned_empty((sum(sizes),), np.uint8)
    held, at = [], 0
    for f, n in zip(cfg.frames, sizes):
        a = block[at:at + n].view(f["image"].dtype).reshape(f["image"].shape)
        a[...] = f["image"]
        held.append(a)
        at += n
    return held, [dict(mesh=mesh, Hoc=f["Hoc"], lens=lens, image=a, fourcc=cfg.fourcc) for f, a in zip(cfg.frames, held)]


def call_latency(index, repeats):
    """One call of the reference's interface, engine(mesh, Hoc, lens, image, fourcc) -> ClassifiedMesh by value, on the
    first frame of configuration `index`: host lookup, upload of the image, every kernel, download of the whole
    classified mesh, timed inside the C++ host library (reference example/benchmark.cpp:50-58 times this call per frame).
    From an image in ordinary (pageable) memory, as the reference's callers hold it, and from a page-locked one."""
    from visualmesh_amd import native
    cfg, engine, mesh, lens, frames = build_workload(index, 1)
    f = cfg.frames[0]
    pageable_ms, visible = engine.time_calls(mesh, f["Hoc"], lens, f["image"], cfg.fourcc, repeats)
    held = native.pinned_empty(f["image"].shape, f["image"].dtype)
    held[...] = f["image"]
    locked_ms, _ = engine.time_calls(mesh, f["Hoc"], lens, held, cfg.fourcc, repeats)
    stats = engine.graph_stats()
    return dict(pageable_image_ms=pageable_ms, page_locked_image_ms=locked_ms, visible_nodes=visible, calls=repeats,
                image_bytes=int(f["image"].nbytes), passes_as_graph_launches=stats["graph_launches"], passes_kernel_by_kernel=stats["eager_launches"],
                what="one engine(mesh, Hoc, lens, image, fourcc) call on one frame: lookup + upload + kernels + download, results by value")


def end_to_end(cfg, mesh, lens, nodes, batches):
    """What a caller pays per batch from host images to the whole classified mesh in host arrays (the reference
    benchmark's frame: example/benchmark.cpp:50-58 runs the whole operator() per frame): the host's lookups, the upload of
    images, poses and ranges, every kernel, and the download of pixels, indices, neighbourhoods and probabilities. Three
    engines in rotation, one staging, one running and one copying its results out at any time, all buffers page-locked;
    the timed region covers `batches` batches in steady state."""
    from visualmesh_amd import engine as eng
    from visualmesh_amd import native
    from visualmesh_amd import workloads as wl
    precision = {"bf16": native.BF16, "split": native.SPLIT}.get(cfg.precision, native.FP32)
    pipe = eng.Pipeline(cfg.network, cfg.model, precision)  # visualmesh::engine::hip::Pipeline<float>
    held, frames = pinned_copies(cfg, mesh, lens)

    def rotate(n):
        returned = 0
        for _ in range(n):
            returned += pipe.submit(frames, arrays=False) is not None  # stage_async + run_async; wait + fetch of the batch before; results of the one before that
        while pipe.flush(arrays=False) is not None:
            returned += 1
        assert returned == n

    rotate(6)  # buffers allocated
    # Three timed stretches of `batches` batches each; the figure is the fastest, all three are in the result: the bus
    # and the host's memory are shared with whatever else the machine is doing, and a stretch that meets other traffic
    # has been seen to read four times slower with nothing of this program's changed.
    stretches = []
    for _ in range(3):
        t0 = time.perf_counter()
        rotate(batches)
        stretches.append((time.perf_counter() - t0) / batches)
    dt = min(stretches)
    nn = wl.N_NEIGHBOURS[cfg.model]
    classes = cfg.network[-1][-1][0].shape[1]
    h2d = sum(int(f["image"].nbytes) for f in cfg.frames)
    d2h = nodes * (8 + 4) + (nodes + len(cfg.frames)) * 4 * (nn + classes)
    return dict(ms_per_batch=dt * 1e3, ms_per_batch_of_each_stretch=[x * 1e3 for x in stretches], nodes_per_s=nodes / dt, frames_per_s=len(cfg.frames) / dt, engines=3, batches=batches,
                h2d_bytes_per_batch=h2d, d2h_bytes_per_batch=d2h, pcie_GBps_each_way=[h2d / dt / 1e9, d2h / dt / 1e9],
                what="host lookup + upload from page-locked images + all kernels + download of the whole classified mesh into "
                     "page-locked arrays; three engines in rotation (one staging, one running, one copying out)")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed passes (default 1000; 50 for configurations 4 and 5, whose pass takes 20-80 ms)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed passes before them (default 100; 5 for configurations 4 and 5)")
    ap.add_argument("--settle", type=float, default=0.25, help="seconds of untimed passes before the warm-up, for the clocks to settle (0: none)")
    ap.add_argument("--config", type=int, default=2, help="workload configuration 1..6 (default 2: batched 1280x1024; 6 = configuration 4 on the split-bf16 engine)")
    ap.add_argument("--frames", type=int, default=None, help="frames per batch (default: the configuration's own)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-events", action="store_true",
                    help="no HIP events in the timed passes; no roofline is reported")
    ap.add_argument("--copy-probe", action="store_true",
                    help="accepted for older command lines: the 1 GiB plain copy kernel (the practical ceiling of the memory "
                         "system and the dispatch of known size that memory counters are scaled by) runs unless --no-copy-probe")
    ap.add_argument("--no-copy-probe", action="store_true", help="skip the plain copy kernel")
    ap.add_argument("--no-pcie", action="store_true", help="skip the PCIe-inclusive figures (serial stage + run + fetch, and the pipelined end-to-end loop)")
    ap.add_argument("--no-configs", action="store_true", help="skip the short runs of the other configurations")
    ap.add_argument("--no-calls", action="store_true", help="skip the single-call latencies (one engine(...) call per frame, configurations 1-5)")
    args = ap.parse_args()
    big = args.config in (4, 5, 6)
    args.steps = (50 if big else 1000) if args.steps is None else args.steps
    args.warmup = (5 if big else 100) if args.warmup is None else args.warmup
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (frames would shard across GPUs "
              "without any exchange); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    from visualmesh_amd import native
    from visualmesh_amd import workloads as wl

    cfg, engine, mesh, lens, frames = build_workload(args.config, args.frames)
    # PCIe-inclusive figures (never `value`). Serial: images in page-locked host memory -> stage + run + fetch of the whole
    # classified mesh into one page-locked block, one engine, the three steps one after the other. Pipelined: end_to_end()
    # above, with the serial figure's engine still alive beside the rotation's three (see GPU_MAX_HW_QUEUES at the top).
    pcie, e2e = None, None
    if not args.no_pcie:
        held, pinned_frames = pinned_copies(cfg, mesh, lens)
        for _ in range(2):
            engine.stage(pinned_frames), engine.run(), engine.fetch_packed()
        nodes = int(engine.counts().sum())
        passes = 5
        t0 = time.perf_counter()
        for _ in range(passes):
            engine.stage(pinned_frames), engine.run(), engine.fetch_packed()
        dt = (time.perf_counter() - t0) / passes
        pcie = dict(ms_per_batch=dt * 1e3, nodes_per_s=nodes / dt, frames_per_s=len(frames) / dt,
                    what="stage from page-locked images + run + fetch (all frames' arrays gathered on the device, one copy into a page-locked block), one engine, serial")
        del held, pinned_frames
        e2e = end_to_end(cfg, mesh, lens, nodes, 12 if big else 60)

    nn = wl.N_NEIGHBOURS[cfg.model]
    m = measure(cfg, engine, frames, args.steps, args.warmup, args.settle, events=not args.no_events)
    nodes = m["nodes"]
    table = layer_table(cfg, nn)

    copy_gbs = None
    if not args.no_copy_probe:
        nbytes = 1 << 30
        copy_gbs = 2 * nbytes / (native.copy_probe(nbytes, 5) * 1e-3) / 1e9

    cpu = None
    if not args.no_cpu:
        threads = min(16, os.cpu_count() or 1, len(cfg.frames))
        sample = cfg
        passes = 8  # ~1.5 s of wall clock per pass on 16 threads: about 12 s in all
        note = "all %d frames of the batch %d times, one frame per task" % (len(cfg.frames), passes)
        if args.config in (4, 5, 6):  # a frame costs ~45 s per core: time a stated subset
            sample = wl.config(args.config, n_frames=min(threads, len(cfg.frames)))
            passes = 1
            note = "the first %d frames of the batch once, one frame per task" % len(sample.frames)
        elif args.config != 2:
            passes = 1
            note = "all %d frames of the batch once, one frame per task" % len(cfg.frames)
        nps, fps, dt, kind = cpu_baseline(sample, threads, passes)
        # the reference engine is single-threaded by design: the same engine on one thread, on a few frames
        one = None
        if args.config in (1, 2, 3):
            few = wl.config(args.config, n_frames=min(3, len(cfg.frames)))
            nps1, fps1, dt1, _ = cpu_baseline(few, 1, 1)
            one = dict(value=nps1, frames_per_s=fps1, seconds=dt1, sample="the first %d frames of the batch once" % len(few.frames))
        model = ""
        try:
            with open("/proc/cpuinfo") as f:
                model = next((line.split(":", 1)[1].strip() for line in f if line.startswith("model name")), "")
        except OSError:
            pass
        cpu = dict(value=nps, unit="nodes/s", cores=threads, kind=kind, cpu_model=model, one_thread=one, frames_per_s=fps, seconds=dt, sample=note)

    # the reference's own interface: one call per frame
    calls = None
    if not args.no_calls:
        calls = {"cfg%d" % index: call_latency(index, 8 if index in (4, 5) else 50) for index in (1, 2, 3, 4, 5)}

    # the other configurations, briefly (device-resident like `value`; each one's dominant kernel against its roofline)
    others = None
    if not args.no_configs:
        others = {}
        del engine, frames
        for index in (1, 2, 3, 4, 5, 6):
            if index == args.config:
                continue
            heavy = index in (4, 5, 6)
            c, e, _, _, fr = build_workload(index)
            r = measure(c, e, fr, 10 if heavy else 300, 2 if heavy else 30, 0.1 if heavy else args.settle, events=True, stream_ceiling=not heavy)
            others[c.name] = dict(workload=workload_name(c, len(fr), layer_table(c, wl.N_NEIGHBOURS[c.model])), dtype=DTYPE[c.precision],
                                  nodes_per_s=r["value"], frames_per_s=r["frames_per_s"], ms_per_step=r["ms_per_step"], steps=10 if heavy else 300,
                                  visible_nodes_per_batch=r["nodes"], roofline=r["roofline"], conv_rooflines=r["conv_rooflines"],
                                  dominant_kernel_ms_per_step_in_timed_passes=r["dominant_kernel_ms_per_step_in_timed_passes"],
                                  kernel_ms_per_step_of_one_bracketed_pass=r["kernel_ms_per_step"])
            del e, fr, c

    out = {
        "metric": "mesh nodes classified/sec",
        "value": m["value"],
        "unit": "nodes/s",
        "frames_per_s": m["frames_per_s"],
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": m["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": DTYPE[cfg.precision],
        "data": "synthetic",
        "config": {
            "workload": workload_name(cfg, len(cfg.frames), table),
            "frames": len(cfg.frames),
            "visible_nodes_per_batch": nodes,
            "inputs": "resident in HBM before the timed region",
            "settle_passes": m["settle_passes"],   # untimed, before the warm-up passes: the clocks settle
            "untimed_passes_after_warmup": 3,      # one with events around every kernel, two in which the timed passes' graph is captured
            "settle_ms": m["settle_ms"],
            # the metric as the whole job sees it, beside `value` (which starts with the inputs resident in HBM):
            "end_to_end_ms_per_batch": e2e["ms_per_batch"] if e2e else None,      # host images -> classified mesh in host arrays, three engines in rotation
            "end_to_end_nodes_per_s": e2e["nodes_per_s"] if e2e else None,
            "end_to_end_frames_per_s": e2e["frames_per_s"] if e2e else None,
            "cpu_one_thread_nodes_per_s": cpu["one_thread"]["value"] if cpu and cpu.get("one_thread") else None,
            "cpu_nodes_per_s": cpu["value"] if cpu else None,
            "cpu_threads": cpu["cores"] if cpu else None,
            # the layers bound by memory, as fractions of the 8 TB/s HBM peak by algorithmic bytes
            "memory_bound_layers_frac_of_hbm_peak": {k: round(v["frac"], 4) for k, v in m["conv_rooflines"].items() if v["bound"] == "hbm"},
            "matrix_bound_layers_frac_of_fp32_mfma_peak": {k: round(v["frac"], 4) for k, v in m["conv_rooflines"].items() if v["bound"] == "mfma"},
            "call_ms": {k: {"pageable": round(v["pageable_image_ms"], 4), "page_locked": round(v["page_locked_image_ms"], 4)} for k, v in calls.items()} if calls else None,
            "dominant_kernel_ms_per_step_in_timed_passes": m["dominant_kernel_ms_per_step_in_timed_passes"],
        },
        "roofline": m["roofline"],
        "cpu_baseline": cpu,
        "copy_kernel_GBps": copy_gbs,
        "end_to_end": e2e,
        "pcie_inclusive": pcie,
        "call_latency": calls,
        "kernel_ms_per_step": m["kernel_ms_per_step"],   # from the one fully profiled, untimed pass (kernel by kernel, events around each: a few per cent slower than a timed pass)
        "conv_rooflines": m["conv_rooflines"],
        "configs": others,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
