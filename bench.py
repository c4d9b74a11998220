#!/usr/bin/env python3
"""Benchmark of the FP8 fused-MoE layer on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3_prefill] [--no-cpu] [--no-decode]

A step = one pass of the path over one batch of synthetic tokens that already sit in HBM:
router GEMM -> top-k routing -> permutation -> activation quantisation -> grouped FP8 GEMM
(W13) + SwiGLU + re-quantisation -> grouped FP8 GEMM (W2) -> shared expert -> weighted reduce.
Prints ONE JSON line.  `value` = algorithmic FP8-GEMM TFLOP/s of the whole step,
`roofline` = the dominant kernel (first grouped GEMM) against the roof that binds it,
`decode` = the same layer at T in {1, 8, 32} as weight-streaming GB/s,
`cpu_baseline` = the CPU oracle timed on this host on a bounded sample of the same workload.
"""
import argparse
import json
import os
import platform
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

PEAK_FP8_TFLOPS = 5000.0      # MI355X dense FP8 MFMA, TFLOP/s
PEAK_HBM_GBS = 8000.0         # MI355X HBM3E, GB/s

KERNEL_SOURCES = ("gemm_fp8.hip", "moe_layout.h", "moe_common.h")   # what the dominant kernel is compiled from
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "grouped_gemm_c3_prefill.txt")


def kernel_source_hash():
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "torch-tpu_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def offline_traffic(shape):
    """HBM bytes per launch of the first grouped GEMM as two `rocprofv3 --pmc` runs (FETCH_SIZE, WRITE_SIZE) counted
    them, read from the line `TRAFFIC {...}` of the committed profile summary.  That is an OFFLINE measurement: it is
    handed on only when the summary was made from the kernel sources this run was built from (same hash) and for this
    workload's shape; otherwise the figure is None and the source says why."""
    try:
        with open(TRAFFIC_FILE) as f:
            rec = next(json.loads(line.split(None, 1)[1]) for line in f if line.startswith("TRAFFIC "))
    except (OSError, StopIteration, ValueError):
        return None, "no TRAFFIC line in profiles/grouped_gemm_c3_prefill.txt"
    rel = os.path.relpath(TRAFFIC_FILE, ROOT)
    if tuple(rec.get("shape", ())) != tuple(shape):
        return None, f"{rel} covers another workload"
    if rec.get("kernel_source_sha16") != kernel_source_hash():
        return None, f"{rel} was measured on other kernel sources ({rec.get('kernel_source_sha16')}): stale, not reported"
    return rec["bytes_per_launch"], f"{rel} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, offline, kernel sources {rec['kernel_source_sha16']})"

WORKLOADS = {
    # the headline configuration: DeepSeek-V3-shaped prefill layer
    "c3_prefill": dict(H=7168, I=2048, E=256, K=8, I_sh=2048, T=4096, route="sigmoid", n_groups=8, topk_groups=4,
                       scale=2.5, desc="DeepSeek-V3-shaped FP8 MoE layer, T=4096, E=256+1 shared, top-8"),
    # Mixtral-8x7B-shaped layer at its largest T
    "c2_prefill": dict(H=4096, I=14336, E=8, K=2, I_sh=0, T=4096, route="softmax", n_groups=1, topk_groups=1,
                       scale=1.0, desc="Mixtral-8x7B-shaped FP8 MoE layer, T=4096, E=8, top-2"),
    # Qwen3-30B-A3B-shaped layer, Zipf(1.2) expert popularity, ~10% empty experts
    "c5_skewed": dict(H=2048, I=768, E=128, K=8, I_sh=0, T=16384, route="softmax", n_groups=1, topk_groups=1,
                      scale=1.0, zipf=1.2, empty=13, desc="Qwen3-30B-A3B-shaped FP8 MoE layer, T=16384, Zipf load"),
    # toy size (the one a CPU runs in seconds)
    "c1_toy": dict(H=256, I=512, E=8, K=2, I_sh=0, T=16, route="softmax", n_groups=1, topk_groups=1, scale=1.0,
                   desc="toy FP8 MoE layer, T=16"),
}


def make_weights(pkg, E, N, Kd, dev, seed):
    """[E, N, Kd] ~ N(0, 0.02) bf16 -> e4m3fn (tile-blocked) + fp32 block scales, generated on the GPU in slices."""
    return pkg.synthetic_weights(E, N, Kd, dev, seed)


def build_layer(pkg, cfg, dev):
    H, I, E, K = cfg["H"], cfg["I"], cfg["E"], cfg["K"]
    w13, w13s = make_weights(pkg, E, 2 * I, H, dev, 1)
    w2, w2s = make_weights(pkg, E, H, I, dev, 2)
    shared = None
    if cfg["I_sh"]:
        s13, s13s = make_weights(pkg, 1, 2 * cfg["I_sh"], H, dev, 3)
        s2, s2s = make_weights(pkg, 1, H, cfg["I_sh"], dev, 4)
        shared = (s13, s13s, s2, s2s)
    g = torch.Generator(device=dev).manual_seed(5)
    wr = (torch.randn(E, H, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    bias = None
    if cfg.get("zipf"):
        # popularity ~ rank^-s through a logit offset; a few experts are switched off entirely
        rank = torch.randperm(E, generator=g, device=dev).float() + 1
        bias = -cfg["zipf"] * torch.log(rank)
        bias[torch.randperm(E, generator=g, device=dev)[:cfg["empty"]]] = -1e9
    elif cfg["route"] == "sigmoid":
        bias = torch.zeros(E, device=dev)           # uniform correction bias
    moe = pkg.FusedMoE(wr, w13, w13s, w2, w2s, top_k=K, mode=cfg["route"], bias=bias, n_groups=cfg["n_groups"],
                       topk_groups=cfg["topk_groups"], renorm=True, scale=cfg["scale"], shared=shared)
    return moe


def gemm_flops(cfg, T):
    return 6.0 * cfg["H"] * cfg["I"] * T * cfg["K"] + 6.0 * cfg["H"] * cfg["I_sh"] * T


def expert_bytes(H, I):
    """fp8 weights + fp32 block scales of one expert (W13 and W2)."""
    return 3 * H * I + 4 * 3 * (H // 128) * (I // 128)


def time_steps(fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def event_time(fn, iters, warmup=2):
    """Average duration of `fn`'s launches on the current stream, by HIP events."""
    for _ in range(warmup):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    e1.synchronize()
    return e0.elapsed_time(e1) / iters * 1e-3


_MFMA_PROBE = None


def mfma_probe(workgroups, iters, out):
    """Launches the matrix-instruction yardstick of libmoe_bench_probe.so (FP8 matrix instructions on register operands
    and nothing else); returns the operations one launch performs."""
    global _MFMA_PROBE
    import ctypes
    if _MFMA_PROBE is None:
        _MFMA_PROBE = ctypes.CDLL(os.path.join(ROOT, "torch-tpu_amd", "libmoe_bench_probe.so")).bench_mfma_probe
        _MFMA_PROBE.restype = ctypes.c_int
        _MFMA_PROBE.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    assert out.numel() >= workgroups * 512 and out.dtype == torch.float32
    rc = _MFMA_PROBE(torch.cuda.current_stream(out.device).cuda_stream, workgroups, iters, out.data_ptr())
    if rc != 0:
        raise RuntimeError(f"bench_mfma_probe: code {rc}")
    return workgroups * 8 * iters * 8 * 2.0 * 16 * 16 * 128


def _sysfs_power_files():
    import glob
    base = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*"))
    if not base:
        return None
    hw = base[0]
    dev_dir = os.path.dirname(os.path.dirname(hw))
    files = dict(power=os.path.join(hw, "power1_input"), cap=os.path.join(hw, "power1_cap"),
                 sclk=os.path.join(dev_dir, "pp_dpm_sclk"))
    return files if all(os.path.exists(f) for f in files.values()) else None


def power_sample(fn, seconds=1.0):
    """Package power and shader clock while `fn` is launched back to back for `seconds`: the driver's own sysfs counters
    (hwmon power1_input / power1_cap in microwatts, the level of pp_dpm_sclk marked current), polled from a host thread.
    None when the counters cannot be read.  Why it is here: under the grouped GEMMs the package sits at its power cap
    and the shader clock falls to what the cap leaves, so a launch takes the time its energy takes at that power - a
    bound next to the memory and matrix roofs that no schedule of the same work gets around."""
    import threading
    files = _sysfs_power_files()
    if files is None:
        return None

    def read(path):
        with open(path) as f:
            return f.read()

    def sclk_now():
        for line in read(files["sclk"]).splitlines():
            if line.rstrip().endswith("*"):
                return float(line.split(":")[1].lower().replace("mhz", "").replace("*", "").strip())
        return None

    for _ in range(10):
        fn()
    torch.cuda.synchronize()
    watts, clocks, stop = [], [], [False]

    def poll():
        while not stop[0]:
            try:
                watts.append(float(read(files["power"])) / 1e6)
                c = sclk_now()
                if c is not None:
                    clocks.append(c)
            except (OSError, ValueError):
                pass
            time.sleep(0.05)

    th = threading.Thread(target=poll)
    th.start()
    t0, n = time.perf_counter(), 0
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
        n += 20
    dt = time.perf_counter() - t0
    stop[0] = True
    th.join()
    # the first readings still average over the time before the load
    w, c = watts[len(watts) // 3:], clocks[len(clocks) // 3:]
    if not w:
        return None
    try:
        cap = float(read(files["cap"])) / 1e6
    except (OSError, ValueError):
        cap = None
    return dict(watts=sum(w) / len(w), cap_watts=cap, sclk_mhz=sum(c) / len(c) if c else None, ms_per_launch=dt / n * 1e3,
                samples=len(w))


def power_roof(power, nbytes, flops, probe_bytes):
    """The roof the package power cap sets for one launch that must move `nbytes` through HBM and perform `flops` FP8
    matrix operations: energy of the two at the rates measured in this very run (watts above idle per TB/s under the
    read probe, per PFLOP/s under the matrix-instruction probe) over the power the cap leaves above idle.  A launch
    cannot take less time than that whatever its schedule; what it takes beyond is the energy of everything else it
    does (operand traffic through L2 and LDS, vector instructions) plus time it is not limited by power at all."""
    need = ("read_probe", "matrix_instructions_only", "first_gemm")
    if power is None or any(power.get(k) is None for k in need) or "idle_watts" not in power:
        return None
    idle, cap = power["idle_watts"], power["first_gemm"]["cap_watts"]
    if not cap or cap <= idle:
        return None
    probe_tbs = probe_bytes / (power["read_probe"]["ms_per_launch"] * 1e-3) / 1e12
    w_per_tbs = (power["read_probe"]["watts"] - idle) / probe_tbs
    w_per_pflops = (power["matrix_instructions_only"]["watts"] - idle) / (power["matrix_instructions_only"]["tflops"] / 1e3)
    joules = nbytes / 1e12 * w_per_tbs + flops / 1e15 * w_per_pflops
    return dict(idle_watts=idle, cap_watts=cap, watts_per_tb_per_s=w_per_tbs, watts_per_pflop_per_s=w_per_pflops,
                joules_hbm=nbytes / 1e12 * w_per_tbs, joules_matrix=flops / 1e15 * w_per_pflops,
                floor_ms=joules / (cap - idle) * 1e3,
                measured_ms=power["first_gemm"]["ms_per_launch"], measured_watts=power["first_gemm"]["watts"],
                note="first grouped GEMM: the time its HBM bytes and matrix operations alone take at the package power cap")


def bench_prefill(pkg, moe, cfg, dev, steps, warmup):
    T, H, I, E, K = cfg["T"], cfg["H"], cfg["I"], cfg["E"], cfg["K"]
    g = torch.Generator(device=dev).manual_seed(11)
    x = torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16)
    out = torch.empty(T, H, dtype=torch.bfloat16, device=dev)

    def step():
        moe(x, out=out)

    # operands of the dominant kernel on its own - the first grouped GEMM (+SwiGLU+requant) over the routed experts - and
    # of the second one, prepared BEFORE anything is timed: the stand-alone launches below then follow the timed steps
    # without a host-side pause in between
    w, ids = moe.route(x)
    xq, xs = pkg.act_quant(x)
    ss, off, s2r, ws = pkg.moe_permute(ids, E, return_workspace=True)
    hq = torch.empty(T * K, I, dtype=torch.float8_e4m3fn, device=dev)
    hs = torch.empty(T * K, pkg.scale_pitch(I // 128), dtype=torch.float32, device=dev)
    y = torch.empty(T, K, H, dtype=torch.bfloat16, device=dev)
    from torch_tpu_amd._lib import check, lib
    st = torch.cuda.current_stream().cuda_stream

    def gemm1():
        check(lib.moe_gemm1_swiglu(st, xq.data_ptr(), xs.data_ptr(), T, H, moe.w13.data_ptr(), moe.w13_scale.data_ptr(),
                                   I, E, K, ss.data_ptr(), off.data_ptr(), ws.data_ptr(), hq.data_ptr(), hs.data_ptr()),
              "gemm1")

    def gemm2():
        check(lib.moe_gemm2(st, hq.data_ptr(), hs.data_ptr(), T, H, moe.w2.data_ptr(), moe.w2_scale.data_ptr(),
                            I, E, K, ss.data_ptr(), off.data_ptr(), ws.data_ptr(), y.data_ptr()), "gemm2")

    gemm1()                                          # hq / hs hold real values before the second GEMM is timed
    torch.cuda.synchronize()

    # Coming out of a host-side pause the chip runs the first launches at a high clock, the next dozen at a low one
    # and only then settles (one fast launch, then up to 40 % slower ones over ~30 ms): a tenth of a second of the same
    # step, untimed, before the counted warm-up steps, so that the timed steps see the clocks a running service sees.
    t_end = time.perf_counter() + 0.1
    while time.perf_counter() < t_end:
        step()
        torch.cuda.synchronize()
    sec = time_steps(step, steps, warmup)
    # straight on, while the chip is in that state: the two GEMMs on their own
    k1 = event_time(gemm1, max(3, steps), warmup=5)
    k2 = event_time(gemm2, max(3, steps), warmup=5)
    # and, in the same state, what a kernel that only reads reaches: the packed W13 of the layer (far more than the
    # 256 MB of last-level cache), one workgroup per weight strip as the first GEMM has them
    probe_buf = moe.w13.view(torch.uint8).reshape(-1)
    probe_piece = 256 * H
    kp = event_time(lambda: hbm_read_probe(probe_buf, probe_piece), max(3, steps), warmup=3)
    probe_gbs = probe_buf.numel() / kp / 1e9
    # the same bytes read by short-lived workgroups of 8 KB each that sweep the buffer front to back
    kf = event_time(lambda: hbm_read_probe(probe_buf, 8192), max(3, steps), warmup=3)
    # package power and shader clock under each of them (sysfs counters, a second of back-to-back launches each)
    power = dict(first_gemm=power_sample(gemm1), second_gemm=power_sample(gemm2),
                 read_probe=power_sample(lambda: hbm_read_probe(probe_buf, probe_piece)), step=power_sample(step))
    # and under nothing but FP8 matrix instructions: the matrix roof of this GPU under its power cap
    mfma_out = torch.empty(1024 * 512, dtype=torch.float32, device=dev)
    mfma_ops = mfma_probe(1024, 2000, mfma_out)
    power["matrix_instructions_only"] = power_sample(lambda: mfma_probe(1024, 2000, mfma_out))
    if power["matrix_instructions_only"] is not None:
        power["matrix_instructions_only"]["tflops"] = mfma_ops / (power["matrix_instructions_only"]["ms_per_launch"] * 1e-3) / 1e12
    # with the GPU left alone for two seconds: what the package draws whatever runs
    torch.cuda.synchronize()
    time.sleep(2.0)
    files = _sysfs_power_files()
    if files is not None and power["read_probe"] is not None and power["matrix_instructions_only"] is not None:
        idle = []
        for _ in range(10):
            with open(files["power"]) as f:
                idle.append(float(f.read()) / 1e6)
            time.sleep(0.05)
        power["idle_watts"] = sum(idle) / len(idle)
    touched = int((off[1:] > off[:-1]).sum().item())
    # algorithmic traffic of one launch of the first GEMM: each touched expert's W13 (+scales) once,
    # quantised activations once, re-quantised SwiGLU output once
    b1 = touched * (2 * I * H + 4 * (2 * I // 128) * (H // 128)) + T * H + 4 * T * (H // 128) \
        + T * K * I + 4 * T * K * (I // 128) + 4 * T * K
    f1 = 4.0 * H * I * T * K
    b2 = touched * (I * H + 4 * (I // 128) * (H // 128)) + T * K * I + 4 * T * K * (I // 128) + 2 * T * K * H
    f2 = 2.0 * H * I * T * K
    intensity = f1 / b1
    bound = "mfma" if intensity > PEAK_FP8_TFLOPS * 1e12 / (PEAK_HBM_GBS * 1e9) else "hbm"
    if bound == "hbm":
        roof = dict(bound="hbm", achieved=b1 / k1 / 1e9, peak=PEAK_HBM_GBS, unit="GB/s")
    else:
        roof = dict(bound="mfma", achieved=f1 / k1 / 1e12, peak=PEAK_FP8_TFLOPS, unit="TFLOP/s")
    roof["frac"] = roof["achieved"] / roof["peak"]
    # HBM bytes per launch of this kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (scaled by a plain elementwise
    # kernel of known size): an offline figure, only for the profiled workload and only while the kernel is unchanged
    roof["traffic"], roof["traffic_source"] = offline_traffic((T, H, I, E, K))
    roof.update(kernel="grouped_gemm_kernel<gated> (W13 GEMM + SwiGLU + requant)", launch_ms=k1 * 1e3,
                algorithmic_bytes=b1, algorithmic_flops=f1, flop_per_byte=intensity,
                mfma_tflops=f1 / k1 / 1e12, mfma_frac=f1 / k1 / 1e12 / PEAK_FP8_TFLOPS,
                hbm_gbs=b1 / k1 / 1e9, hbm_frac=b1 / k1 / 1e9 / PEAK_HBM_GBS,
                second_gemm=dict(launch_ms=k2 * 1e3, mfma_tflops=f2 / k2 / 1e12, hbm_gbs=b2 / k2 / 1e9,
                                 hbm_frac=b2 / k2 / 1e9 / PEAK_HBM_GBS),
                experts_touched=touched, power=power, power_roof=power_roof(power, b1, f1, probe_buf.numel()),
                read_probe=dict(gbs=probe_gbs, frac_of_peak=probe_gbs / PEAK_HBM_GBS, bytes=probe_buf.numel(),
                                bytes_per_workgroup=probe_piece, gbs_short_workgroups=probe_buf.numel() / kf / 1e9,
                                note="a kernel that only reads (bench_hbm_read_probe in libmoe_bench_probe.so), same workgroup "
                                     "decomposition as the first GEMM's weight strips, timed right after it; "
                                     "gbs_short_workgroups: the same read by workgroups of 8 KB each",
                                kernel_over_probe=(b1 / k1 / 1e9) / probe_gbs))
    return sec, roof, x


def bench_decode(pkg, moe, cfg, dev, steps, warmup, batches=(1, 8, 32)):
    """The same layer at T in {1, 8, 32}: HBM-bound weight streaming.  A pool of different token
    batches is cycled so that consecutive steps touch different experts (no cache residency)."""
    H, I, E, K = cfg["H"], cfg["I"], cfg["E"], cfg["K"]
    res = []
    for T in batches:
        g = torch.Generator(device=dev).manual_seed(100 + T)
        pool = [torch.randn(T, H, generator=g, device=dev).to(torch.bfloat16) for _ in range(16)]
        out = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
        touched = []
        for x in pool:
            _, ids = moe.route(x)
            touched.append(int(torch.unique(ids).numel()))
        n_sh = 1 if cfg["I_sh"] else 0
        avg_bytes = sum((t * expert_bytes(H, I) + n_sh * expert_bytes(H, cfg["I_sh"] or I)) for t in touched) \
            / len(touched) + 2 * T * H * 2 + T * K * 8
        state = {"i": 0}

        def step():
            moe(pool[state["i"] % len(pool)], out=out)
            state["i"] += 1

        n_steps = max(steps, 32)
        sec_eager = time_steps(step, n_steps, max(warmup, 16))
        # the same steps replayed from one HIP graph (one pass over the pool per replay): removes
        # the host's launch cost, which at T=1 is of the order of the GPU work itself
        sec_graph = None
        try:
            torch.cuda.synchronize()
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for x in pool[:2]:
                    moe(x, out=out)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for x in pool:
                    moe(x, out=out)
            reps = max(2, n_steps // len(pool))
            sec_graph = time_steps(graph.replay, reps, 2) / len(pool)
            # the last replayed step must reproduce the eager result bit for bit
            check = out.clone()
            moe(pool[-1], out=out)
            torch.cuda.synchronize()
            if not torch.equal(check, out):
                sec_graph = None
        except Exception as exc:                                     # graph capture unavailable: report eager only
            print(f"graph capture failed at T={T}: {exc}", file=sys.stderr)
        # both are ways a caller can run the step; the figure quoted is the faster one, the other is kept beside it
        use_graph = sec_graph is not None and sec_graph <= sec_eager
        sec = sec_graph if use_graph else sec_eager
        res.append(dict(T=T, ms_per_step=sec * 1e3, tokens_per_s=T / sec, hbm_gbs=avg_bytes / sec / 1e9,
                        hbm_frac=avg_bytes / sec / 1e9 / PEAK_HBM_GBS, experts_touched_avg=sum(touched) / len(touched),
                        algorithmic_bytes=avg_bytes, launch_mode="hip_graph" if use_graph else "eager",
                        ms_per_step_eager=sec_eager * 1e3,
                        ms_per_step_hip_graph=None if sec_graph is None else sec_graph * 1e3,
                        power=power_sample(step, 1.0)))       # package power and shader clock under this step
    return res


def _lib():
    from torch_tpu_amd._lib import lib
    return lib


_PROBE = None


def hbm_read_probe(buf, bytes_per_workgroup=1835008):
    """Launches one pure read of `buf` (a contiguous GPU tensor whose byte size is a multiple of 16) on the current stream:
    one workgroup of eight wavefronts per contiguous piece of `bytes_per_workgroup`.  The kernel lives in
    torch-tpu_amd/libmoe_bench_probe.so, a measuring aid of this benchmark that is not part of the product library."""
    global _PROBE
    import ctypes
    if _PROBE is None:
        path = os.path.join(ROOT, "torch-tpu_amd", "libmoe_bench_probe.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: build it with `python torch-tpu_amd/build.py`")
        _PROBE = ctypes.CDLL(path).bench_hbm_read_probe
        _PROBE.restype = ctypes.c_int
        _PROBE.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_void_p]
    if not (isinstance(buf, torch.Tensor) and buf.is_cuda and buf.is_contiguous()):
        raise RuntimeError("buf must be a contiguous GPU tensor")
    nbytes = buf.numel() * buf.element_size()
    sink = torch.empty(1, dtype=torch.int32, device=buf.device)
    rc = _PROBE(torch.cuda.current_stream(buf.device).cuda_stream, buf.data_ptr(), nbytes, bytes_per_workgroup, sink.data_ptr())
    if rc != 0:
        raise RuntimeError(f"bench_hbm_read_probe: code {rc}")


def bench_dense(pkg, dev, steps, warmup):
    """The dense block-scaled layers (same kernels, one expert): DeepSeek-V3 shapes of the reference's
    dense tests at a decode and a prefill batch."""
    res = []
    g = torch.Generator(device=dev).manual_seed(7)
    for kind, M, K, N in (("mm", 32, 7168, 1536), ("mm", 256, 7168, 1536), ("mm", 4096, 7168, 1536), ("mm", 4096, 2048, 7168),
                          ("mlp", 32, 7168, 18432), ("mlp", 256, 7168, 18432), ("mlp", 4096, 7168, 18432)):
        x = torch.randn(M, K, generator=g, device=dev).to(torch.bfloat16)
        if kind == "mm":
            w, ws = make_weights(pkg, 1, N, K, dev, 31)
            w, ws = w[0], ws[0]
            out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
            wsp = torch.empty(_lib().moe_mm_fp8_workspace_bytes(M, K, N), dtype=torch.uint8, device=dev)
            fn = lambda: pkg.mm_fp8(x, w, ws, out=out, workspace=wsp)
            flops, nbytes = 2.0 * M * K * N, N * K + 2 * M * K + 2 * M * N
        else:
            I = N
            w13, w13s = make_weights(pkg, 1, 2 * I, K, dev, 32)
            w2, w2s = make_weights(pkg, 1, K, I, dev, 33)
            out = torch.empty(M, K, dtype=torch.bfloat16, device=dev)
            wsp = torch.empty(_lib().moe_mlp_fp8_workspace_bytes(M, K, I), dtype=torch.uint8, device=dev)
            fn = lambda: pkg.mlp_fp8(x, w13[0], w13s[0], w2[0], w2s[0], out=out, workspace=wsp)
            flops, nbytes = 6.0 * M * K * I, 3 * K * I + 4 * M * K
        # the small ones are tens of microseconds: more of them, so that a host hiccup does not show
        sec = time_steps(fn, max(steps, 10) * (10 if M <= 256 else 1), max(warmup, 5))
        res.append(dict(op=kind, M=M, K=K, N=N, ms=sec * 1e3, tflops=flops / sec / 1e12, hbm_gbs=nbytes / sec / 1e9))
    return res


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return platform.processor() or "unknown"


def _median(v):
    v = sorted(v)
    return v[len(v) // 2]


def device_step_with_routing(pkg, moe, cfg, x):
    """The timed step once more on the same batch, through the same entry point, asked for what its router produced:
    -> (out [T,H], scores the device selected on, weights [T,K], ids [T,K])."""
    T = x.shape[0]
    if moe._one_call(T):
        out, logits, w, ids = pkg.layer_fp8(
            x, moe.router_weight, moe.w13, moe.w13_scale, moe.w2, moe.w2_scale, cfg["K"], moe.layer_mode(), moe.bias,
            cfg["n_groups"], cfg["topk_groups"], True, cfg["scale"], shared=moe.shared, return_routing=True,
            workspace=moe._workspace(T, True))
    else:
        logits = torch.matmul(x, moe.router_weight.t())
        w, ids = moe.route(x)
        out = moe.experts(x, w, ids)
    if cfg["route"] == "sigmoid":
        w2, ids2, scores = pkg.moe_route(logits, cfg["K"], "sigmoid", moe.bias, cfg["n_groups"], cfg["topk_groups"], True,
                                         cfg["scale"], return_scores=True)
    else:
        scores = logits.float() if moe.bias is None else logits.float() + moe.bias
        w2, ids2 = pkg.moe_route(logits if moe.bias is None else logits + moe.bias, cfg["K"], "softmax")
    same = bool(torch.equal(ids, ids2) and torch.equal(w, w2))
    return out, scores, w, ids, same


def cpu_baseline(pkg, moe, cfg, x, sample_tokens, reps=3):
    """The CPU oracle (router product, routing, per-expert dequantise + fp32 matmul on the same quantised operands,
    weighted reduce) timed on `sample_tokens` tokens spread over the batch, median of `reps` runs; the device side of
    the comparison is the rows of those tokens in the output of the FULL batch - the step that is timed - and the
    comparison is made in the strict steps of oracle/parity_checks.py."""
    orc = entry.load_oracle()
    checks = entry.load_parity_checks()
    threads = torch.get_num_threads()                # the host's share of cores (OMP_NUM_THREADS) unless fewer exist
    T, K = x.shape[0], cfg["K"]
    n = min(sample_tokens, T)
    out, scores, w, ids, same_routing = device_step_with_routing(pkg, moe, cfg, x)
    torch.cuda.synchronize()
    pick = torch.unique(torch.linspace(0, T - 1, n).round().long()).to(x.device)
    n = pick.numel()
    layer = (moe.w13, moe.w13_scale, moe.w2, moe.w2_scale)
    x_s, ids_s, w_s, out_s = x[pick].contiguous(), ids[pick].contiguous(), w[pick].contiguous(), out[pick].contiguous()
    parity = {"tokens_checked": n, "rows_taken_from": f"the output of the timed step on all T={T} tokens",
              "routing_of_entry_point_equals_routing_kernel": same_routing}
    # routing of the WHOLE batch, exactly, given the scores the device selected on
    bias = None if moe.bias is None else moe.bias.cpu()
    scores_host = scores.float().cpu()
    if cfg["route"] == "sigmoid":
        w_ref, ids_ref = orc.select_sigmoid_grouped(scores_host, bias, K, cfg["n_groups"], cfg["topk_groups"], cfg["scale"])
    else:
        w_ref, ids_ref = orc.route_softmax_topk(scores_host, K)
    parity["routing_ids_equal_given_device_scores"] = bool(torch.equal(ids.cpu(), ids_ref))
    parity["routing_weights_max_abs_diff"] = (w.cpu() - w_ref).abs().max().item()
    try:
        rep = checks.check_sample(pkg, orc, x_s, ids_s, layer, w_s=w_s, shared_dev=moe.shared, out_big=out_s,
                                  what=f"sample of the T={T} step")
        parity["strict_steps"] = "passed"
        parity.update(rep)
    except AssertionError as exc:
        parity["strict_steps"] = f"FAILED: {exc}"
    # the timed CPU work: the same tokens through the oracle, only the experts they use brought to the host
    local, used = checks._localise(ids_s.cpu())
    idx = torch.tensor(used, device=x.device)
    small = checks._host_layer(pkg, tuple(t[idx] for t in layer))
    shared = None if moe.shared is None else checks._host_layer(pkg, moe.shared)
    xs = x_s.cpu()
    wr = moe.router_weight.float().cpu()
    w_host = w_s.cpu()
    torch.set_num_threads(threads)
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        logits = xs.float() @ wr.T
        if cfg["route"] == "sigmoid":
            orc.route_sigmoid_grouped(logits, bias, K, cfg["n_groups"], cfg["topk_groups"], cfg["scale"])
        else:
            orc.route_softmax_topk(logits if bias is None else logits + bias, K)
        ref = orc.moe_w8a8_fp32(xs, local, w_host, *small, shared=shared)
        times.append(time.perf_counter() - t0)
    sec = _median(times)
    got = out_s.float().cpu()
    parity["outputs_outside_rtol2e-2_atol1e-2"] = checks.outside_fraction(got, ref)
    parity["worst_violation"] = checks.worst_violation(got, ref)
    parity["cos_diff_end_to_end"] = orc.cal_diff(ref, got)[0]
    base = dict(value=gemm_flops(cfg, n) / sec / 1e12, unit="TFLOP/s", cores=threads, kind="port",
                sample=f"{n} tokens spread over the same batch through the CPU oracle (router product, routing, per-expert "
                       f"dequantise + fp32 matmul on the quantised operands, weighted reduce, shared expert), median of "
                       f"{reps} runs: {sec:.2f} s, {n / sec:.2f} tokens/s",
                tokens_per_s=n / sec, runs_s=[round(t, 3) for t in times], host_cpus=os.cpu_count() or 1,
                cpu_model=cpu_model())
    return base, parity


def literal_reference_loop(pkg, cfg, dev, T, seed):
    """The reference's own CPU ground truth, literally: one call per (token, slot), each de-quantising its expert's three
    matrices block by block in Python and running a bf16 chain (python/regression/test_llm/test_moe.py:10-50, 93-98),
    timed once on a batch of T tokens of the layer `cfg`.  Only feasible for a handful of tokens."""
    orc = entry.load_oracle()
    H, I, E, K = cfg["H"], cfg["I"], cfg["E"], cfg["K"]
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(torch.int32)
    local, used = entry.load_parity_checks()._localise(ids)
    # only the touched experts are generated: [n_used, ...] in the reference's orientation (gate, up [I,H]; down [H,I])
    w13q, w13s = (t.cpu() for t in pkg.synthetic_weights(len(used), 2 * I, H, dev, seed + 1, tile_block=False))
    w2q, w2s = (t.cpu() for t in pkg.synthetic_weights(len(used), H, I, dev, seed + 2, tile_block=False))
    nb = I // 128
    t0 = time.perf_counter()
    orc.experts_ref_bf16_literal(x, local, w13q[:, :I], w13q[:, I:], w2q, w13s[:, :nb].bfloat16(), w13s[:, nb:].bfloat16(),
                                 w2s.bfloat16())
    sec = time.perf_counter() - t0
    return dict(T=T, seconds=sec, tokens_per_s=T / sec, calls=T * K, kind="port, literal per-(token, slot) loop",
                cores=torch.get_num_threads())


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c3_prefill", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-decode", action="store_true")
    ap.add_argument("--cpu-sample", type=int, default=32)
    ap.add_argument("--decode-only", type=int, default=0, metavar="T",
                    help="run only the decode leg at this batch size and print its record (for profiling one batch size)")
    ap.add_argument("--dense-only", action="store_true",
                    help="run only the dense layers (mm / gated MLP at 32, 256 and 4096 rows) and print their records")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures ONE GPU: the path is single-device by design (sharding the experts over several "
              "GPUs is not built); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a ROCm GPU", file=sys.stderr)
        sys.exit(2)
    pkg = entry.load_package()
    dev = "cuda:0"
    if args.dense_only:
        print(json.dumps(bench_dense(pkg, dev, args.steps, args.warmup)))
        return
    cfg = WORKLOADS[args.workload]
    moe = build_layer(pkg, cfg, dev)
    if args.decode_only:
        print(json.dumps(bench_decode(pkg, moe, cfg, dev, args.steps, args.warmup, (args.decode_only,))[0]))
        return
    # a plain device copy of known size (1 GiB read + 1 GiB written): the yardstick that the
    # FETCH_SIZE / WRITE_SIZE counters of a profiled run are scaled by
    ref_src = torch.zeros(1 << 28, dtype=torch.float32, device=dev)
    ref_dst = torch.empty_like(ref_src)
    torch.neg(ref_src, out=ref_dst)              # the only negation in this program: easy to find in a trace
    del ref_src, ref_dst
    # the decode leg runs first: coming straight after seconds of the prefill load it reads 2-4 % slower (the chip is
    # still at the clocks it fell back to under that load), which says nothing about a decode step
    decode = None
    if not args.no_decode and args.workload == "c3_prefill":
        decode = bench_decode(pkg, moe, cfg, dev, args.steps, args.warmup)
    sec, roof, x = bench_prefill(pkg, moe, cfg, dev, args.steps, args.warmup)
    T = cfg["T"]
    flops = gemm_flops(cfg, T)
    result = {
        "metric": "FP8 fused-MoE layer TFLOP/s (% MFMA peak) + decode HBM GB/s (% peak), 1 GPU",
        "value": flops / sec / 1e12, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": sec * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "fp8_e4m3",
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: {cfg['desc']}", "T": T, "hidden": cfg["H"],
                   "intermediate": cfg["I"], "experts": cfg["E"], "top_k": cfg["K"], "shared_intermediate": cfg["I_sh"]},
        "tokens_per_s": T / sec, "mfma_frac_of_peak": flops / sec / 1e12 / PEAK_FP8_TFLOPS,
        "roofline": roof,
    }
    # the whole step against the HBM roof: the bytes no implementation of the layer can avoid (every touched expert's
    # weights and scales once, the shared expert's, x in, out written) over the step time
    step_bytes = roof["experts_touched"] * expert_bytes(cfg["H"], cfg["I"]) \
        + (expert_bytes(cfg["H"], cfg["I_sh"]) if cfg["I_sh"] else 0) + 4 * T * cfg["H"]
    result["step"] = dict(algorithmic_bytes=step_bytes, hbm_gbs=step_bytes / sec / 1e9,
                          step_hbm_frac=step_bytes / sec / 1e9 / PEAK_HBM_GBS,
                          first_gemm_alone_ms=roof["launch_ms"], second_gemm_alone_ms=roof["second_gemm"]["launch_ms"],
                          rest_ms=sec * 1e3 - roof["launch_ms"] - roof["second_gemm"]["launch_ms"],
                          power_floor_ms=None if not roof.get("power_roof") else
                          (step_bytes / 1e12 * roof["power_roof"]["watts_per_tb_per_s"]
                           + flops / 1e15 * roof["power_roof"]["watts_per_pflop_per_s"])
                          / (roof["power_roof"]["cap_watts"] - roof["power_roof"]["idle_watts"]) * 1e3,
                          note="the GEMM figures are the routed experts' launches on their own; inside the step the same "
                               "launches also carry the shared expert's tiles; rest = router product, routing + activation "
                               "quantisation, permutation, weighted sum and the shared expert's share; power_floor_ms = the "
                               "time the step's unavoidable bytes and matrix operations alone take at the package power cap "
                               "(coefficients of roofline.power_roof)")
    if decode is not None:
        result["decode"] = decode
        result["dense"] = bench_dense(pkg, dev, args.steps, args.warmup)
        # the same layer between decode and the headline batch: the step alone, with the bytes of the experts it touched
        sweep = []
        for Ts in (128, 512, 2048):
            g = torch.Generator(device=dev).manual_seed(200 + Ts)
            xs_ = torch.randn(Ts, cfg["H"], generator=g, device=dev).to(torch.bfloat16)
            outs_ = torch.empty(Ts, cfg["H"], dtype=torch.bfloat16, device=dev)
            ssec = time_steps(lambda: moe(xs_, out=outs_), args.steps, args.warmup)
            _, ids_ = moe.route(xs_)
            touched = int(torch.unique(ids_).numel())
            byts = touched * expert_bytes(cfg["H"], cfg["I"]) + (expert_bytes(cfg["H"], cfg["I_sh"]) if cfg["I_sh"] else 0)
            sweep.append(dict(T=Ts, ms_per_step=ssec * 1e3, tflops=gemm_flops(cfg, Ts) / ssec / 1e12,
                              weight_gbs=byts / ssec / 1e9, experts_touched=touched,
                              tile_rows=pkg.tile_rows(Ts, cfg["K"], cfg["E"])))
        result["batch_sweep"] = sweep
        # the two matrix-core-bound layer shapes of the same benchmark definition, same step, for the record
        others = []
        for name in ("c2_prefill", "c5_skewed"):
            ocfg = WORKLOADS[name]
            omoe = build_layer(pkg, ocfg, dev)
            osec, oroof, _ = bench_prefill(pkg, omoe, ocfg, dev, args.steps, args.warmup)
            oflops = gemm_flops(ocfg, ocfg["T"])
            rec = dict(workload=f"{name}: {ocfg['desc']}", ms_per_step=osec * 1e3, tflops=oflops / osec / 1e12,
                       mfma_frac_of_peak=oflops / osec / 1e12 / PEAK_FP8_TFLOPS,
                       tokens_per_s=ocfg["T"] / osec, first_gemm_ms=oroof["launch_ms"],
                       first_gemm_tflops=oroof["mfma_tflops"], second_gemm_ms=oroof["second_gemm"]["launch_ms"],
                       second_gemm_tflops=oroof["second_gemm"]["mfma_tflops"])
            if name == "c2_prefill":
                # the same few-expert layer at decode sizes: bytes of the experts a batch touches per second
                small = []
                for Ts in (1, 8, 64):
                    g = torch.Generator(device=dev).manual_seed(300 + Ts)
                    pool = [torch.randn(Ts, ocfg["H"], generator=g, device=dev).to(torch.bfloat16) for _ in range(8)]
                    outs_ = torch.empty(Ts, ocfg["H"], dtype=torch.bfloat16, device=dev)
                    state = {"i": 0}

                    def small_step():
                        omoe(pool[state["i"] % len(pool)], out=outs_)
                        state["i"] += 1

                    ssec = time_steps(small_step, max(args.steps, 32), max(args.warmup, 16))
                    touched = sum(int(torch.unique(omoe.route(xp)[1]).numel()) for xp in pool) / len(pool)
                    small.append(dict(T=Ts, ms_per_step=ssec * 1e3, experts_touched_avg=touched,
                                      weight_gbs=touched * expert_bytes(ocfg["H"], ocfg["I"]) / ssec / 1e9))
                rec["decode_sizes"] = small
            others.append(rec)
            del omoe
        result["other_shapes"] = others
    if not args.no_cpu:
        base, parity = cpu_baseline(pkg, moe, cfg, x, min(args.cpu_sample, T))
        # the reference's own ground-truth loop, literally (one de-quantisation of three matrices per token and slot),
        # on the toy layer and on one decode token of the DeepSeek-V3-shaped layer
        base["literal_reference_loop"] = [
            dict(workload="c1_toy", **literal_reference_loop(pkg, WORKLOADS["c1_toy"], dev, WORKLOADS["c1_toy"]["T"], 21)),
            dict(workload="c4_decode T=1", **literal_reference_loop(pkg, WORKLOADS["c3_prefill"], dev, 1, 22))]
        result["cpu_baseline"] = base
        result["parity_on_sample"] = parity
    print(json.dumps(result))


if __name__ == "__main__":
    main()
