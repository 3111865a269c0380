#!/usr/bin/env python3
"""Benchmark of the population-batched binary forward path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--extra 1,3,4,5] [--no-cpu]

Headline workload (configuration 2 of the five): binary linear 1024x1024, population 1024, one input row per member,
p = 0.05 flip masks sampled by threshold compare from SUPPLIED uint32 words, fused into the XOR-popcount
product.  A step is one such population forward with every operand resident in HBM.  Prints one JSON line.

value      packed binary TOPS = 2 * valid bit-MACs / s (whole job, one GPU)
roofline   the dominant kernel against MI355X's published HBM bandwidth: algorithmic bytes per launch
           (4 B per weight bit of random words + base + inputs + int32 outputs) / average launch duration
cpu_baseline  the C oracle (a port of the same arithmetic) timed on this box's host cores on a subset of
           the members of the same workload
cpu_float_formulation  the reference's own ground truth (torch.bmm on +-1 fp32) on the host cores, for information
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def measured_traffic():
    """HBM bytes per launch of the headline kernel from two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE in KiB per
    dispatch, each scaled by what the same counter reads for the 2 GiB calibration copy kernel).  Counters cannot be
    read from inside this program; the readings live in profiles/headline_traffic.json, next to the summary that
    quotes them, together with the commit they were taken at and the hash of the kernel's source file then.
    -> (bytes or None, note): None when the file is gone or the kernel's source has changed since (a stale figure
    is not reported)."""
    import hashlib
    try:
        with open(os.path.join(ROOT, "profiles", "headline_traffic.json")) as f:
            t = json.load(f)
        with open(os.path.join(ROOT, t["kernel_source"]), "rb") as f:
            same = hashlib.sha256(f.read()).hexdigest() == t["kernel_source_sha256"]
        note = "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE at commit %s; %s unchanged since: %s" % (
            t["measured_at_commit"], t["kernel_source"], same)
        if not same:
            return None, note
        return int(round((t["fetch_kib_per_dispatch"] * t["fetch_scale"]
                          + t["write_kib_per_dispatch"] * t["write_scale"]) * 1024)), note
    except (OSError, KeyError, ValueError):
        return None, "profiles/headline_traffic.json not readable"


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # a few milliseconds of work do not bring the memory clocks up: with 20 steps after 3 the headline step measures
    # 0.62 ms, from about 100 steps after 20 on it is 0.59 ms and stays there
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--extra", type=str, default="1,3,4,5",
                    help="other configurations to time as well (reported under other_configs); '' for none")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-calib", action="store_true", help="skip the measured copy / popcount ceilings")
    ap.add_argument("--cpu-members", type=int, default=256, help="members of the workload the CPU baseline runs")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="CPU time the baseline leg accumulates")
    ap.add_argument("--only-calib", action="store_true", help="run only the calibration kernels (for counter runs)")
    ap.add_argument("--only", type=int, default=0, help="time just this configuration (for profiler runs)")
    ap.add_argument("--no-graph", action="store_true", help="skip the graph-replay timings of the other configurations")
    ap.add_argument("--no-step", action="store_true", help="skip the NES step of the SmallNet-shaped network")
    ap.add_argument("--only-step", action="store_true",
                    help="time just the NES step of the SmallNet-shaped network, phase after phase (for profiler runs)")
    ap.add_argument("--kernels", action="store_true",
                    help="time the HBM-bound helper kernels (pack, unpack, samplers, max-pool, im2col) on their own")
    return ap.parse_args()


def time_steps(torch, step, steps, warmup):
    """W untimed steps, then K steps bracketed by synchronize; wall clock and HIP events on the launch stream."""
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall / steps, e0.elapsed_time(e1) * 1e-3 / steps


def time_graph(torch, step, steps, replays=5):
    """The same K steps captured once in a HIP graph and replayed: device time per step without the host's launch
    cost (a step of a few microseconds is otherwise paced by Python).  None if the capture fails."""
    try:
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(steps):
                step()
        graph.replay()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        best = None
        for _ in range(replays):
            e0.record()
            graph.replay()
            e1.record()
            torch.cuda.synchronize()
            t = e0.elapsed_time(e1) * 1e-3 / steps
            best = t if best is None or t < best else best
        del graph
        return best
    except Exception:                                      # noqa: BLE001 - capture support varies; eager figures remain
        torch.cuda.synchronize()
        return None


def time_resample(torch, w, reps=3):
    """ms to draw every member's weights of every layer again (a training step's set_noise), when the workload can."""
    fn = w.meta.get("resample")
    if fn is None:
        return
    fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        fn()
    torch.cuda.synchronize()
    w.meta["set_noise_ms"] = round((time.perf_counter() - t0) / reps * 1e3, 3)


def config_entry(cfg, w, per_wall, per_ev, per_graph=None):
    """One line of other_configs.  A compute-shaped configuration is priced against three limits: HBM (algorithmic
    bytes), the XOR-popcount issue rate of the vector ALUs and the dense int8 rate of the matrix cores (one +-1 byte
    MAC per bit-MAC); `bound` names the limit that allows the least throughput for the engine that ran, and
    `roofline_frac` is the fraction of that limit."""
    from nesgpu_amd import workloads
    from nesgpu_amd.extensions import booleanOperations as ops
    entry = {"config": cfg, "workload": w.name, "ms_per_step": round(per_wall * 1e3, 4),
             "binary_TOPS": round(2 * w.bit_macs / per_wall / 1e12, 3)}
    if "fc" in w.meta:
        entry["fc_8192_1024"] = w.meta["fc"]
    if "set_noise_ms" in w.meta:
        entry["set_noise_ms"] = w.meta["set_noise_ms"]
    if per_graph:
        # device time per step from a graph replay; the roofline fractions below use it when it is available
        entry.update(ms_per_step_graph=round(per_graph * 1e3, 4),
                     binary_TOPS_graph=round(2 * w.bit_macs / per_graph / 1e12, 3))
        per_ev = min(per_ev, per_graph)
    hbm = w.algo_bytes / per_ev / workloads.HBM_PEAK
    if w.bound == "hbm":
        entry.update(bound="hbm", roofline_frac=round(hbm, 4))
        return entry
    if "stages" in w.meta:
        # a network has no single roofline: one line per kernel instead (kernel_table), and the whole step against the
        # two compute limits
        entry.update(conv_engine="matrixcore-fp4 / window kernel",
                     frac_of_valu_popcount_peak=round(w.bit_macs / per_ev / workloads.VALU_POPC_PEAK, 4),
                     frac_of_fp4_mfma_peak=round(w.bit_macs / per_ev / workloads.MFMA_FP4_PEAK, 4))
        return entry
    valu = w.bit_macs / per_ev / workloads.VALU_POPC_PEAK
    mfma = w.bit_macs / per_ev / workloads.MFMA_INT8_PEAK
    fp4 = w.bit_macs / per_ev / workloads.MFMA_FP4_PEAK
    last = ops.conv_last_engine()                    # of the step's last conv launch
    engine = {2: "matrixcore-int8", 4: "matrixcore-fp4"}.get(last, "popcount")
    comp = {2: mfma, 4: fp4}.get(last, valu)
    entry.update(conv_engine=engine, bound="hbm" if hbm > comp else ("valu" if engine == "popcount" else "mfma"),
                 roofline_frac=round(max(hbm, comp), 4), frac_of_hbm_peak=round(hbm, 4),
                 frac_of_valu_popcount_peak=round(valu, 4), frac_of_int8_mfma_peak=round(mfma, 4),
                 frac_of_fp4_mfma_peak=round(fp4, 4))
    return entry


def extend_entry(torch, args, cfg, w, entry, steps):
    """What the conv-shaped configurations report beside their step: the same step on the XOR-popcount kernels
    (engine 1: the engine the vector-ALU roofline is about), configuration 5's launches one by one, and configuration
    5 built through the layer API."""
    from nesgpu_amd import workloads
    from nesgpu_amd.extensions import booleanOperations as ops
    if cfg in (3, 4, 5):
        prev = ops.conv_engine(1)
        try:
            n = max(3, steps // 4)
            pw, pe = time_steps(torch, w.step, n, 2)
            pg = None if args.no_graph else time_graph(torch, w.step, n)
            t = min(pe, pg) if pg else pe
            entry["engine_popcount"] = {"ms_per_step": round(t * 1e3, 4),
                                        "frac_of_valu_popcount_peak": round(w.bit_macs / t / workloads.VALU_POPC_PEAK, 4),
                                        "timing": "graph replay" if pg and pg <= pe else "eager launches",
                                        "note": "conv kernels forced to XOR + popcount (nb_conv_engine(1)); other "
                                                "kernels of the step unchanged"}
        finally:
            ops.conv_engine(prev)
    if "stages" in w.meta:
        table = []
        peaks = {"valu": workloads.VALU_POPC_PEAK, "fp4": workloads.MFMA_FP4_PEAK, "hbm": workloads.HBM_PEAK}
        for name, fn, bound, work in w.meta["stages"]():
            pw, pe = time_steps(torch, fn, max(3, steps // 2), 3)
            pg = None if args.no_graph else time_graph(torch, fn, max(3, steps // 2))
            t = min(pe, pg) if pg else pe
            table.append({"kernel": name, "us": round(t * 1e6, 2), "bound": bound,
                          "frac": round(work / t / peaks[bound], 4)})
        entry["kernel_table"] = table
        entry["kernel_table_note"] = ("each launch of the step timed alone (graph replay); frac = bit-MACs or "
                                      "algorithmic bytes per second over the peak its bound names (valu: 6.29e14 "
                                      "bit-MAC/s, fp4: 5.05e15 MAC/s, hbm: 8e12 B/s)")
    if cfg == 5:
        model, step, set_noise = workloads.cifar_net_layers()
        n = max(3, steps // 2)
        pw, pe = time_steps(torch, step, n, 3)
        pg = None if args.no_graph else time_graph(torch, step, n)
        sw, se = time_steps(torch, set_noise, 5, 2)
        fc = model.perturbed_layers[3].weight_noise
        fitness = torch.randn(model.directions, device=fc.device)

        def update():
            for layer in model.perturbed_layers:
                layer.update(fitness)
        uw, ue = time_steps(torch, update, 5, 2)
        entry["layer_api"] = {
            "workload": "the same network from BinarizedConv2d / BinarizedMaxPool2d / BinarizedLinear "
                        "(flip_probability=0.01) through PerturbedModel, fuse_packed_outputs",
            "ms_per_step": round(pw * 1e3, 4), "ms_per_step_graph": round(pg * 1e3, 4) if pg else None,
            "set_noise_ms": round(sw * 1e3, 4), "update_ms": round(uw * 1e3, 4),
            "fc_8192_1024": type(fc).__name__,
            "ratio_to_ops_level": round(pw * 1e3 / entry["ms_per_step"], 3)}
        del model, step, set_noise


def cpu_baseline(wl, members, seconds):
    """Oracle (port) on the first `members` members of the headline workload; words regenerated on the host from
    the same Philox stream the GPU words came from."""
    import numpy as np
    from oracle import oracle as O
    m = wl.meta
    out_f, in_f = m["out_f"], m["in_f"]
    members = min(members, wl.population)
    words = O.philox_words(m["seed"], m["subsequence"], 0, members * out_f * in_f).reshape(members, out_f, in_f)
    base = wl.tensors["base"].cpu().numpy()
    x = wl.tensors["x"][:members].cpu().numpy()
    times = []
    got = None
    total = 0.0
    while total < seconds or len(times) < 3:
        t0 = time.perf_counter()
        got = O.seeded_bmv_from_words(m["T"], x, words, base=base)
        dt = time.perf_counter() - t0
        times.append(dt)
        total += dt
    gpu = wl.step()[:members].cpu().numpy()
    if not np.array_equal(gpu, got):
        raise SystemExit("bench: GPU result differs from the CPU oracle on the baseline sample")
    macs = members * out_f * in_f
    med = sorted(times)[len(times) // 2]
    return {"value": round(2 * macs / med / 1e12, 6), "unit": "binary TOPS", "cores": O.max_threads(), "kind": "port",
            "sample": "first %d of %d members of the same workload, %d passes over %.1f s, median %.4f s per pass, "
                      "OpenMP over members; output checked equal to the GPU's" % (members, wl.population, len(times),
                                                                                  total, med)}


def cpu_float_formulation(wl, members, seconds):
    """The reference's own ground truth for a binary product, moved to the CPU: torch.bmm on +-1 fp32 operands
    (booloptests.py:54-55, 150-160); fp32 is exact for K <= 2**24.  The float formulation has no fused sampler, so the
    members' +-1 weight matrices are built outside the timed region; only the batched product is timed."""
    import numpy as np
    import torch
    from oracle import oracle as O
    m = wl.meta
    out_f, in_f = m["out_f"], m["in_f"]
    members = min(members, wl.population)
    words = O.philox_words(m["seed"], m["subsequence"], 0, members * out_f * in_f).reshape(members, out_f, in_f)

    def bits(t, n):                                    # packed int64 [..., Kw] -> 0/1 bytes [..., n], LSB first
        return np.unpackbits(np.ascontiguousarray(t.cpu().numpy()).view(np.uint8), axis=-1, bitorder="little")[..., :n]

    wbits = bits(wl.tensors["base"], in_f)[None] ^ (words < np.uint32(m["T"])).astype(np.uint8)
    del words
    Wf = torch.from_numpy(wbits.astype(np.float32) * 2 - 1)
    del wbits
    xf = torch.from_numpy(bits(wl.tensors["x"][:members], in_f).astype(np.float32) * 2 - 1).unsqueeze(2)
    times, total, dot = [], 0.0, None
    while total < seconds or len(times) < 3:
        t0 = time.perf_counter()
        dot = torch.bmm(Wf, xf)
        dt = time.perf_counter() - t0
        times.append(dt)
        total += dt
    popc = ((in_f - dot.squeeze(2)) / 2).to(torch.int32).numpy()
    if not np.array_equal(wl.step()[:members].cpu().numpy(), popc):
        raise SystemExit("bench: GPU result differs from the float formulation on the baseline sample")
    med = sorted(times)[len(times) // 2]
    return {"value": round(2 * members * out_f * in_f / med / 1e12, 6), "unit": "binary TOPS",
            "cores": torch.get_num_threads(), "kind": "reference formulation (torch.bmm on +-1 fp32, CPU)",
            "sample": "first %d of %d members, weights prepared outside the timed region, %d passes over %.1f s, "
                      "median %.4f s per pass; popcounts recovered as (K - dot) / 2 equal the GPU's"
                      % (members, wl.population, len(times), total, med)}


def calibrate(torch):
    """Measured ceilings reported beside the datasheet peaks: streaming copy, streaming read, xor+bcnt loop."""
    import ctypes
    path = os.path.join(ROOT, "nesgpu_amd", "libnesbin_calib.so")
    if not os.path.exists(path):
        return None
    lib = ctypes.CDLL(path)
    vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    lib.nb_calib_copy.argtypes = [vp, vp, i64, i32, vp]
    lib.nb_calib_read.argtypes = [vp, vp, i64, vp]
    lib.nb_calib_popc.argtypes = [vp, vp, i32, i32, vp]
    st = torch.cuda.current_stream().cuda_stream
    nbytes = 2 << 30
    src = torch.empty(nbytes, dtype=torch.uint8, device="cuda").fill_(1)
    dst = torch.empty_like(src)
    sink = torch.zeros(4, dtype=torch.int32, device="cuda")
    res = {}
    blocks, iters = 256 * 32, 2000
    s = torch.randint(0, 2 ** 31, (1024,), dtype=torch.int32, device="cuda")
    out = torch.empty(blocks * 256, dtype=torch.int32, device="cuda")
    per, ev = time_steps(torch, lambda: lib.nb_calib_popc(out.data_ptr(), s.data_ptr(), blocks, iters, st), 5, 1)
    lane_ops = blocks * 256 * iters * 8 * 16 * 2
    res["copy_GBps"] = res["read_GBps"] = res["read_stream_GBps"] = None   # keeps the keys' order in the printed line
    res["xor_bcnt_lane_ops_per_s"] = float("%.4g" % (lane_ops / ev))
    res["xor_bcnt_binary_TOPS"] = round(2 * (lane_ops / 4 * 64) / ev / 1e12, 1)
    # how int8 MFMAs and ordinary vector instructions share a SIMD's issue (four waves per SIMD): ns per MFMA and SIMD
    if hasattr(lib, "nb_calib_mfma_valu"):
        lib.nb_calib_mfma_valu.argtypes = [vp, i32, i32, i32, vp]
        names = ["mfma_alone", "plus_2_valu_same_wave", "plus_4_valu_same_wave", "mfma_waves_and_valu_waves_4_per_mfma",
                 "same_mfma_waves_at_priority", "same_valu_waves_at_priority"]
        mblocks, miters = 1024, 4000
        issue = {}
        for v, name in enumerate(names):
            per, ev = time_steps(torch, lambda: lib.nb_calib_mfma_valu(out.data_ptr(), mblocks, miters, v, st), 3, 1)
            mfmas_per_simd = mblocks * 4 / 1024 * miters * 8 * (1.0 if v < 3 else 0.5)
            issue[name] = round(ev * 1e9 / mfmas_per_simd, 2)
        res["ns_per_int8_mfma_per_simd"] = issue
    # the two memory-bound calibrations come last: what follows a calibration in this program is the timed region of
    # an HBM-bound kernel, and the memory clocks should not have come down behind compute-only kernels by then
    # one 16-byte chunk per thread: the workgroups in flight then cover one compact window that moves through the
    # buffer (a few thousand workgroups that each stride through all of it measured 4.3-4.6 TB/s for the same bytes)
    per, ev = time_steps(torch, lambda: lib.nb_calib_copy(dst.data_ptr(), src.data_ptr(), nbytes, nbytes // 16 // 256, st),
                         10, 2)
    res["copy_GBps"] = round(2 * nbytes / ev / 1e9, 1)
    per, ev = time_steps(torch, lambda: lib.nb_calib_read(sink.data_ptr(), src.data_ptr(), nbytes, st), 10, 2)
    res["read_GBps"] = round(nbytes / ev / 1e9, 1)
    if hasattr(lib, "nb_calib_read_stream"):
        # the loads the library's streaming kernels use (non-temporal, eight 16-byte requests per thread before the
        # first use): what a read-once stream reaches, and the figure to hold the headline kernel against
        lib.nb_calib_read_stream.argtypes = [vp, vp, i64, vp]
        per, ev = time_steps(torch, lambda: lib.nb_calib_read_stream(sink.data_ptr(), src.data_ptr(), nbytes, st), 10, 2)
        res["read_stream_GBps"] = round(nbytes / ev / 1e9, 1)
    if hasattr(lib, "nb_calib_fill"):
        # writes alone: a plain fill, and the store pattern of the conv kernels' int32 maps (configuration 3: 1024
        # members x 256 KB, a wave per 16 pixel columns of a member, 4 KB per row) alternating between two buffers
        # as successive steps do
        lib.nb_calib_fill.argtypes = [vp, i64, i32, vp]
        lib.nb_calib_store_rows.argtypes = [vp, i32, vp]
        per, ev = time_steps(torch, lambda: lib.nb_calib_fill(dst.data_ptr(), nbytes, nbytes // 16 // 256, st), 10, 2)
        res["fill_GBps"] = round(nbytes / ev / 1e9, 1)
        half = 1024 * 262144
        flip = [0]

        def rows():
            flip[0] ^= 1
            lib.nb_calib_store_rows(dst.data_ptr() + flip[0] * half, 1024, st)
        per, ev = time_steps(torch, rows, 20, 4)
        res["conv_map_store_GBps"] = round(half / ev / 1e9, 1)
    return res


def hbm_kernels(torch, steps, warmup, graph=True, core=False):
    """Each HBM-bound kernel of the path alone, at a configuration-sized shape: algorithmic bytes / event time.
    ``core``: only pack, unpack, the samplers from supplied words and max-pool (the kernels the 70 % target names)."""
    from nesgpu_amd import workloads
    from nesgpu_amd.extensions import booleanOperations as ops
    dev = "cuda"
    res = []

    def run(name, fn, nbytes):
        if core and not name.startswith(("pack", "unpack", "flip_from_words", "max_pool2d")):
            return
        pw, pe = time_steps(torch, fn, steps, warmup)
        pg = time_graph(torch, fn, steps) if graph else None   # device time without the host's launch pacing
        t = pg if pg else pe
        res.append({"kernel": name, "us": round(t * 1e6, 2), "GBps": round(nbytes / t / 1e9, 1),
                    "hbm_frac": round(nbytes / t / workloads.HBM_PEAK, 4), "algorithmic_bytes": nbytes,
                    "timing": "graph replay" if pg else "eager launches", "eager_us": round(pe * 1e6, 2)})

    g = torch.Generator(device=dev)
    g.manual_seed(0)
    # pack: config 3 activations [1024*32*32, 64] bool -> 1 word per pixel; and a wide row case
    b = torch.randint(0, 2, (1024 * 32 * 32, 64), device=dev, generator=g, dtype=torch.uint8).bool()
    run("pack [1048576,64] -> i64", lambda: ops.pack(b, torch.int64), b.numel() + b.numel() // 8)
    b2 = torch.randint(0, 2, (65536, 1024), device=dev, generator=g, dtype=torch.uint8).bool()
    run("pack [65536,1024] -> i64", lambda: ops.pack(b2, torch.int64), b2.numel() + b2.numel() // 8)
    b3 = torch.randint(0, 2, (1024 * 64 * 64, 16), device=dev, generator=g, dtype=torch.uint8).bool()
    run("pack [4194304,16] -> i64", lambda: ops.pack(b3, torch.int64), b3.numel() + b3.size(0) * 8)
    p2 = ops.pack(b2, torch.int64)
    run("unpack [65536,16] i64", lambda: ops.unpack(p2), p2.numel() * 8 + p2.numel() * 64)
    del b, b2, b3
    # samplers from supplied words: config 1 (linear 256x256, D=1024) and config 3 filters (576 x 64, D=1024)
    for (n, R, C, T) in ((1024, 256, 256, workloads.T_P01), (1024, 576, 64, workloads.T_P02), (256, 1024, 1024, workloads.T_P05)):
        words = ops.philox_words(n * R * C, 0, 7).view(n, R, C)
        base = ops.pack(torch.randint(0, 2, (R, C), device=dev, generator=g, dtype=torch.uint8).bool(), torch.int64)
        nb = words.numel() * 4 + n * R * ((C + 63) // 64) * 8
        run("flip_from_words [%d,%d,%d]" % (n, R, C), lambda: ops.flip_from_words(base, words, T), nb)
        if not core:
            thr = ops.thresholds_from_p(torch.rand(R, C, device=dev, generator=g).half())
            run("sample_bits_from_words [%d,%d,%d]" % (n, R, C),
                lambda: ops.sample_bits_from_words(thr, words, torch.int64), nb)
        del words
    # max-pool 2x2/s2 on config 4's thresholded map [1024,64,64,1] and on a 2-word map
    for shape in ((1024, 64, 64, 1), (4096, 16, 16, 2), (1024, 64, 64, 4)):
        x = torch.randint(-2 ** 62, 2 ** 62, shape, device=dev, generator=g, dtype=torch.int64)
        run("max_pool2d %s" % (list(shape),), lambda: ops.max_pool2d(x, 2, 2, 0, 0, 2, 2), x.numel() * 8 * 5 // 4)
    if core:
        return res
    x = torch.randint(-2 ** 62, 2 ** 62, (1024, 32, 32, 1), device=dev, generator=g, dtype=torch.int64)
    run("batch_im2col [1024,32,32,1] 3x3 p1", lambda: ops.batch_im2col(x, 3, 3, 1, 1, 1, 1), x.numel() * 8 * 10)
    # linear matrix-vector product streaming materialised weights (config 5's 8192 -> 1024 layer at D=1024)
    W = torch.randint(-2 ** 62, 2 ** 62, (1024, 1024, 128), device=dev, generator=g, dtype=torch.int64)
    xv = torch.randint(-2 ** 62, 2 ** 62, (1024, 128, 1), device=dev, generator=g, dtype=torch.int64)
    run("bmm N=1 [1024,1024,128]", lambda: ops.bmm(W, xv), W.numel() * 8 + xv.numel() * 8 + 1024 * 1024 * 4)
    del W, xv
    # config 1's kernel: rows of 32 bytes, one row per lane
    W1 = torch.randint(-2 ** 62, 2 ** 62, (1024, 256, 4), device=dev, generator=g, dtype=torch.int64)
    x1 = torch.randint(-2 ** 62, 2 ** 62, (1024, 4, 1), device=dev, generator=g, dtype=torch.int64)
    run("bmm N=1 [1024,256,4] (config 1)", lambda: ops.bmm(W1, x1), W1.numel() * 8 + x1.numel() * 8 + 1024 * 256 * 4)
    del W1, x1
    # sparse form of config 5's 8192 -> 1024 layer at D = 4096: flip lists drawn by the skip sampler
    b4 = torch.randint(-2 ** 62, 2 ** 62, (1024, 128), device=dev, generator=g, dtype=torch.int64)
    rows = ops.flip_rows_skip(b4, 8192, 4096, workloads.T_P01, 0, subsequence=13)
    x4 = torch.randint(-2 ** 62, 2 ** 62, (4096, 128), device=dev, generator=g, dtype=torch.int64)
    thr4 = torch.full((4096, 1024), 8192, dtype=torch.int32, device=dev)
    ex = ops.expand_rows(x4)
    G = ops.bmm_nt(ex, rows.base_expanded)
    run("expand_rows [4096,128] -> FP4 codes", lambda: ops.expand_rows(x4), x4.numel() * 8 + ex.codes.numel())
    run("bmm_nt 4096 x 1024 x 8192 bits (FP4 matrix cores; bytes: operands once + int32 out)",
        lambda: ops.bmm_nt(ex, rows.base_expanded), ex.codes.numel() + rows.base_expanded.codes.numel() + G.numel() * 4)
    run("bmv_flip_act_pack D=4096 [1024 x 8192], p=0.01 (lists + row info + G + thresholds)",
        lambda: ops.bmv_flip_act_pack(rows, x4, thr4, G=G), rows.nbytes() + G.numel() * 4 + thr4.numel() * 4 + x4.numel() * 8)
    run("flip_rows_skip D=4096 [1024 x 8192], p=0.01 (bytes written)",
        lambda: ops.flip_rows_skip(b4, 8192, 4096, workloads.T_P01, 0, subsequence=13), rows.nbytes())
    fit4 = torch.randn(4096, device=dev, generator=g).half()
    run("weighted_sum over the flip lists D=4096 [1024 x 8192], p=0.01 (lists + row info + fp16 out)",
        lambda: ops.weighted_sum(rows, fit4, 8192), rows.nbytes() + 1024 * 8192 * 2)
    del rows, x4, thr4, ex, G
    # the same layer's lists under the per-element law of latent weights whose magnitudes spread by 10 % (flip
    # probabilities of 0.8 % on average, 8 % at most): one walk at the largest probability against class by class
    sign = torch.randint(0, 2, (1024, 8192), device=dev, generator=g) * 2 - 1
    law = ops.flip_law_from_weights((sign * (1.0 + 0.1 * torch.randn((1024, 8192), device=dev, generator=g))).half())
    cap = ops.flip_capacity(8192, 0.009)
    rows = ops.flip_rows_layered(law, 4096, 0, cap)
    assert rows.overflowed() == 0
    run("flip_rows_thin D=4096 [1024 x 8192], per-element law (bytes written)",
        lambda: ops.flip_rows_thin(law, 4096, 0, cap), rows.nbytes())
    run("flip_rows_layered D=4096 [1024 x 8192], per-element law (bytes written)",
        lambda: ops.flip_rows_layered(law, 4096, 0, cap), rows.nbytes())
    del rows, law, sign
    # a conv layer's filters (128 x 3x3 taps of 64 channels) at p = 0.01 for 4096 members, both layouts: the skip
    # sampler as packed words against one draw per bit
    bc = torch.randint(-2 ** 62, 2 ** 62, (1152, 1), device=dev, generator=g, dtype=torch.int64)
    run("sample_bits_skip D=4096 x [1152 rows x 64], p=0.01, rows + conv layout (bytes written)",
        lambda: ops.sample_bits_skip(workloads.T_P01, 4096, torch.int64, 0, 11, base=bc, shape=(1152, 64), conv_taps=9),
        2 * 4096 * 1152 * 8)
    run("sample_bits_philox D=4096 x [1152 rows x 64], p=0.01, rows + conv layout (bytes written)",
        lambda: ops.sample_bits_philox(workloads.T_P01, 4096, torch.int64, 0, 11, base=bc, shape=(1152, 64), conv_taps=9),
        2 * 4096 * 1152 * 8)
    del bc
    # a layer's set_noise from the generator, per-element thresholds: conv 64 -> 256 (3x3) for 1024 members, one 32-bit
    # draw per weight bit against 16-bit draws (two per generated word)
    thr = torch.randint(0, 2 ** 31, (2304, 64), device=dev, generator=g, dtype=torch.int64).to(torch.int32).view(torch.uint32)
    for half in (False, True):
        run("sample_bits_philox D=1024 x [2304 rows x 64], per-element thresholds, %s (bytes written)"
            % ("16-bit draws" if half else "32-bit draws"),
            lambda: ops.sample_bits_philox(thr, 1024, torch.int64, 0, 12, half_draws=half), 1024 * 2304 * 8)
    del thr
    # first-layer filters of an RGB network: rows of 3 columns, one lane per row
    b1 = torch.randint(0, 8, (576, 1), device=dev, generator=g, dtype=torch.int64)
    run("sample (3-column rows) D=4096 x 576 rows, generator mode",
        lambda: ops.sample_bits_philox(workloads.T_P01, 4096, torch.int64, 0, 10, base=b1, shape=(576, 3)), 4096 * 576 * 8)
    # update step: weighted sum of the population's masks of a 1024x1024 layer (one fp32 add per member and weight
    # bit in member order: the vector ALUs, not HBM, bound it; the fraction is reported for comparison)
    m = torch.randint(-2 ** 62, 2 ** 62, (1024, 1024, 16), device=dev, generator=g, dtype=torch.int64)
    wts = torch.randn(1024, device=dev, generator=g).half()
    run("weighted_sum [1024,1024,16] -> fp16 [1024,1024]", lambda: ops.weighted_sum(m, wts, 1024),
        m.numel() * 8 + 1024 * 1024 * 2)
    # the blocked sum the layers' update uses (tables of partial sums over 8 members)
    run("weighted_sum fast [1024,1024,16] -> fp16 [1024,1024]", lambda: ops.weighted_sum(m, wts, 1024, fast=True),
        m.numel() * 8 + 1024 * 1024 * 2)
    del m
    # the same for a conv layer's masks (256 filters of 3x3 taps x 64 channels): an output of 147 456 weights, a wave or
    # two per SIMD
    m = torch.randint(-2 ** 62, 2 ** 62, (1024, 2304, 1), device=dev, generator=g, dtype=torch.int64)
    run("weighted_sum [1024,2304,1] -> fp16 [2304,64]", lambda: ops.weighted_sum(m, wts, 64), m.numel() * 8 + 2304 * 64 * 2)
    run("weighted_sum fast [1024,2304,1] -> fp16 [2304,64]", lambda: ops.weighted_sum(m, wts, 64, fast=True),
        m.numel() * 8 + 2304 * 64 * 2)
    del m
    # batch-norm conv layer: thresholds straight from the layer's input (pixel sums from counts of the image's bits, no
    # conv; bound by the latency of a workgroup's chain and by vector instructions, the fraction is for comparison)
    for (D, C, O, S) in ((1024, 64, 64, 32), (4096, 64, 128, 16)):
        x = torch.randint(-2 ** 62, 2 ** 62, (D, S, S, 1), device=dev, generator=g, dtype=torch.int64)
        f = torch.randint(-2 ** 62, 2 ** 62, (D, 9, O), device=dev, generator=g, dtype=torch.int64)
        bias = torch.randn(O, device=dev, generator=g).half()
        noise = torch.randn(D, O, device=dev, generator=g).half()
        run("conv_bn_thresholds_from_input conv %d->%d 3x3 on %dx%d, D=%d" % (C, O, S, S, D),
            lambda: ops.conv_bn_thresholds_from_input(x, f, bias, noise, 3, 3, 1, 1, 1, 1),
            x.numel() * 8 + f.numel() * 8 + D * O * 6)
    return res


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; population sharding over several GPUs is design-only "
              "(run with --gpus 1)", file=sys.stderr)
        return 2
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    from nesgpu_amd import _lib, workloads
    _lib.load()                                                   # fail loudly if the HIP library is missing
    torch.cuda.set_device(0)
    if args.only_calib:
        print(json.dumps({"measured_ceilings": calibrate(torch)}))
        return 0

    if args.kernels:
        print(json.dumps({"hbm_kernels": hbm_kernels(torch, args.steps, args.warmup, not args.no_graph)}))
        return 0
    if args.only_step:
        sn, fw, up = workloads.small_net_step()
        out = {}
        for name, fn in (("set_noise_ms", sn), ("forward_ms", fw), ("update_ms", up)):
            out[name] = round(time_steps(torch, fn, args.steps, args.warmup)[0] * 1e3, 4)
        print(json.dumps({"nes_step_smallnet": out}))
        return 0
    if args.only:
        w = workloads.BUILDERS[args.only]()
        time_resample(torch, w)
        pw, pe = time_steps(torch, w.step, args.steps, args.warmup)
        entry = config_entry(args.only, w, pw, pe, None if args.no_graph else time_graph(torch, w.step, args.steps))
        entry["event_ms_per_step"] = round(pe * 1e3, 4)
        if not args.no_graph:
            extend_entry(torch, args, args.only, w, entry, args.steps)
        print(json.dumps(entry))
        return 0

    wl = workloads.linear_flip_fused()
    # The measured ceilings (copy / read / popcount / MFMA calibration kernels, about half a second of GPU work) run
    # first: a process's first few milliseconds of kernels see memory clocks that have not come up yet, and the
    # W warm-up steps the caller asks for may be too few to get past that.
    cal = None if args.no_calib else calibrate(torch)
    per_wall, per_ev = time_steps(torch, wl.step, args.steps, args.warmup)
    tops = 2 * wl.bit_macs / per_wall / 1e12
    achieved = wl.algo_bytes / per_ev / 1e9
    traffic, traffic_note = measured_traffic()
    line = {
        "metric": "packed binary TOPS (2 x valid bit-MACs / s) per population forward",
        "value": round(tops, 4), "unit": "binary TOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(per_wall * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u64", "data": "synthetic (seed 0; inputs/base from torch CPU generator, random words from "
                                "Philox4x32-10)",
        "config": {"workload": wl.name, "population": wl.population, "word_bits": 64,
                   "bit_macs_per_step": wl.bit_macs},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": workloads.HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved * 1e9 / workloads.HBM_PEAK, 4), "traffic": traffic,
                     "traffic_source": traffic_note,
                     "kernel": "seeded_bmv_stream_kernel", "algorithmic_bytes_per_launch": wl.algo_bytes,
                     "avg_launch_ms": round(per_ev * 1e3, 4)},
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(wl, args.cpu_members, args.cpu_seconds)
        line["cpu_float_formulation"] = cpu_float_formulation(wl, 64, 4.0)
    del wl
    torch.cuda.empty_cache()

    others = []
    for tok in [t for t in args.extra.split(",") if t.strip()]:
        cfg = int(tok)
        if cfg == 2:
            continue
        w = workloads.BUILDERS[cfg]()
        time_resample(torch, w)
        steps = max(3, args.steps // 2) if cfg == 5 else args.steps
        pw, pe = time_steps(torch, w.step, steps, args.warmup)
        entry = config_entry(cfg, w, pw, pe, None if args.no_graph else time_graph(torch, w.step, steps))
        extend_entry(torch, args, cfg, w, entry, steps)
        others.append(entry)
        del w
        torch.cuda.empty_cache()
    # configuration 2 again with the words generated in the kernel (no 4 GiB operand): bound by the generator's ALU work
    wg = workloads.linear_flip_generated()
    pw, pe = time_steps(torch, wg.step, max(3, args.steps // 4), 1)
    line["generator_mode"] = {"workload": wg.name, "ms_per_step": round(pw * 1e3, 4),
                              "binary_TOPS": round(2 * wg.bit_macs / pw / 1e12, 3),
                              "random_words_per_s": float("%.4g" % (wg.bit_macs / pe)),
                              "note": "same output as the headline workload; about 14 vector ALU operations per "
                                      "generated word (a Philox round is two v_mad_u64_u32 and two v_bitop3_b32), "
                                      "so the vector ALUs are the limit, not HBM"}
    del wg
    # the same with 16 bits of the stream per weight bit (two per generated word; ties decided by a second stream)
    wh = workloads.linear_flip_generated(half_draws=True)
    ph, _ = time_steps(torch, wh.step, max(3, args.steps // 4), 1)
    line["generator_mode"]["half_draws"] = {
        "workload": wh.name, "ms_per_step": round(ph * 1e3, 4), "binary_TOPS": round(2 * wh.bit_macs / ph / 1e12, 3),
        "note": "same law (every bit flips with probability exactly T / 2^32, independently), other bits than the "
                "headline workload"}
    del wh
    if not args.no_step:
        # the layer API end to end: one NES step of a SmallNet-shaped network (population 1024), phase by phase
        sn, fw, up = workloads.small_net_step()
        reps = max(3, args.steps // 2)
        line["nes_step_smallnet"] = {
            "workload": "conv 24->64, pool, conv 64->256, pool, linear 16384->10, batch_norm everywhere, population "
                        "1024, 32x32 images of 3 x 8 bit planes, through modules.binary (eager launches)",
            "set_noise_ms": round(time_steps(torch, sn, reps, 2)[0] * 1e3, 4),
            "forward_ms": round(time_steps(torch, fw, reps, 2)[0] * 1e3, 4),
            "update_ms": round(time_steps(torch, up, reps, 2)[0] * 1e3, 4)}
        # the three phases in a loop that changes the weights every step (plain SGD on the estimated gradients), so
        # that whatever a layer keeps per version of its weights is made anew every step
        from nesgpu_amd.modules import binary as _binary
        _mods = [m for m in fw.model.modules() if isinstance(m, _binary.Binarized)]
        _opt = torch.optim.SGD(fw.model.parameters(), lr=1e-3)
        _count = [0]

        def loop_step():
            _count[0] += 1
            for j, m in enumerate(_mods):
                m.set_seed(1000 * _count[0] + j)
            sn()
            fw()
            up()
            _opt.step()
        line["nes_step_smallnet"]["training_loop_ms_per_step"] = round(time_steps(torch, loop_step, reps, 3)[0] * 1e3, 4)
        line["nes_step_smallnet"]["training_loop_note"] = ("set_seed, set_noise, forward, update and torch's SGD step, "
                                                          "new weights every step")
        del _opt, _mods
        if not args.no_graph:
            fg = time_graph(torch, fw, reps)                 # the same forward without the host's launch pacing
            if fg:
                line["nes_step_smallnet"]["forward_graph_ms"] = round(fg * 1e3, 4)
            # the same step with the forward replayed from a HIP graph (binary.capture): new noise is drawn eagerly and
            # copied to where the graph reads it
            from nesgpu_amd.modules import binary
            cap = binary.capture(fw.model, fw.input)
            line["nes_step_smallnet"]["captured"] = {
                "set_noise_ms": round(time_steps(torch, cap.set_noise, reps, 2)[0] * 1e3, 4),
                "forward_ms": round(time_steps(torch, cap, reps, 2)[0] * 1e3, 4),
                "update_ms": round(time_steps(torch, lambda: cap.update(up.fitness), reps, 2)[0] * 1e3, 4),
                "note": "binary.capture: one graph replay per forward and one per update; set_noise draws eagerly "
                        "and copies into the graph's tensors"}
            pm1, x1 = workloads.linear_layer_config1()
            eager1 = time_steps(torch, lambda: pm1.forward(x1), args.steps, 5)
            cap1 = binary.capture(pm1, x1)
            rep1 = time_steps(torch, cap1, args.steps, 5)
            # sixteen input batches per replay (a fitness evaluation over several minibatches on the same noise)
            xs = torch.stack([x1] * 16)
            cap16 = binary.capture(pm1, xs, batches=16)
            rep16 = time_steps(torch, cap16, max(5, args.steps // 4), 2)
            line["config1_layer"] = {
                "workload": "configuration 1 as BinarizedLinear(256, 256, 1024, threshold=False) through "
                            "PerturbedModel: bmm + 2*popc - K",
                "eager_us_per_step": round(eager1[0] * 1e6, 2), "captured_us_per_step": round(rep1[0] * 1e6, 2),
                "captured_16_batches_us_per_step": round(rep16[0] * 1e6 / 16, 2),
                "note": "captured: one graph replay per step, launched from Python (a replay costs about 15 us on "
                        "this stack whatever the graph holds); with sixteen input batches per replay the step is the "
                        "kernels' own time"}
            del cap, cap1, cap16, pm1
        del sn, fw, up
        # configuration 5's wide layer under the reference's own per-weight law, through the layer: base + flip lists
        # drawn class by class against the materialised form (every bit drawn)
        law = {"workload": "BinarizedLinear(8192, 1024, 4096) under P = sigmoid(5 w / mean|w|), latent weights "
                           "+-(1 + 0.1 N(0,1)): one NES step, ms (eager launches)"}
        for name, kw in (("flip_lists_class_by_class", dict(sparse=True, walk="layered")),
                         ("flip_lists_thinning", dict(sparse=True, walk="thin")),
                         ("materialised", dict(sparse=False))):
            lin, sn, fw, up = workloads.wide_linear_law_step(**kw)
            law[name] = {"set_noise_ms": round(time_steps(torch, sn, 5, 2)[0] * 1e3, 3),
                         "forward_ms": round(time_steps(torch, fw, 5, 2)[0] * 1e3, 3),
                         "update_ms": round(time_steps(torch, up, 5, 2)[0] * 1e3, 3)}
            if kw.get("sparse"):
                plan = lin._sparse_plan()
                law["mean_flip_probability"], law["largest_flip_probability"] = round(plan["mean"], 5), round(plan["peak"], 4)
                lin.sparse_walk = "auto"
                law["walk_chosen_by_the_layer"] = lin._sparse_walk_now()
            lin.free_memory()
            del lin, sn, fw, up
            torch.cuda.empty_cache()
        line["per_weight_law_layer"] = law
    # the helper kernels the 70 %-of-HBM target names, each alone, after everything above has warmed the clocks
    line["hbm_kernels"] = [{"kernel": k["kernel"], "us": k["us"], "hbm_frac": k["hbm_frac"], "timing": k["timing"]}
                           for k in hbm_kernels(torch, max(10, args.steps // 4), 5, not args.no_graph, core=True)]
    if others:
        line["other_configs"] = others
    if cal:
        line["measured_ceilings"] = cal
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
