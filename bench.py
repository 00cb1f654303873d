#!/usr/bin/env python3
"""Benchmark of the bit-sliced GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--quick]

One STEP is one pass of the decode hot path over the four Llama-3-8B-shaped linears
(qkv 4096->6144, o 4096->4096, gate_up 4096->28672, down 14336->4096) at batch 1,
weights sliced to 4 bits, group 128, fp16 scale and zero per group (the zero-point form).
`value` is the sliced weight bytes of a step divided by its time (GB/s): the figure the
HBM roofline is quoted on.  Inputs are resident in HBM before the timed region; every
step reads a different copy of the weights, cycling through a ring of copies larger
than 2 GiB so that the 256 MB Infinity Cache cannot serve them.

The JSON line also carries
  roofline     the dominant kernel (gate_up decode) alone: algorithmic bytes per launch /
               average launch duration measured with HIP events on the launch stream
  cpu_baseline the reference's PyTorch CPU path (slice -> dequantize -> F.linear,
               restated in oracle/torch_path.py) on the host cores, same layers, one pass
  summary      a dozen scalars of the tables below
The per-bitwidth / per-layer / small-batch / M=2048 prefill tables go to a side file (EXTRA_FILE,
named in the line's `tables` key) and to stderr, one table per line; the last stdout line stays under 4 KB.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0      # MI355X published HBM3E bandwidth
MFMA_FP16_PEAK_TFLOPS = 2500.0  # MI355X published dense fp16 matrix rate
LLAMA3_8B = {"qkv": (6144, 4096), "o": (4096, 4096), "gate_up": (28672, 4096), "down": (4096, 14336)}
LLAMA3_70B = {"qkv": (10240, 8192), "o": (8192, 8192), "gate_up": (57344, 8192), "down": (8192, 28672)}
GROUP = 128
RING_BYTES = 2.5e9
COUNTER_COPY_BYTES = 256 * 1024 * 1024
# HBM bytes per launch of the dominant kernel come from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs
# of `bench.py --counter-pass`, each counter scaled by what it reads for the 256 MiB elementwise
# copy of the same run.  The tracked summary of those runs states the kernel plan and a hash of
# the kernel sources it was taken on; the figure is reported only while both still match.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "gemv_b4_gate_up_M1_pmc.txt")
KERNEL_SOURCES = ("gemv_gfx950.hip", "device_common.h", "layout.h")


def kernel_source_hash() -> str:
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "matgptq_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(plan: str):
    """`traffic_bytes_per_launch` of the tracked counter summary if it was taken on this plan and
    on these kernel sources, else None."""
    try:
        with open(TRAFFIC_PROFILE) as f:
            fields = dict(line.strip().split("=", 1) for line in f if "=" in line and not line.startswith(" "))
    except OSError:
        return None
    if fields.get("plan") != plan or fields.get("kernel_source_hash") != kernel_source_hash():
        return None
    try:
        return int(fields["traffic_bytes_per_launch"])
    except (KeyError, ValueError):
        return None


def algorithmic_bytes(n, k, m, bits, zero_points=True):
    """Bytes a GEMV call must move: sliced codes + scales (+ zeros) + x + y."""
    aux = 2 if zero_points else 1
    return n * k * bits // 8 + 2 * n * (k // GROUP) * aux + 2 * m * k + 2 * m * n


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--quick", action="store_true", help="skip the extra sweeps and the CPU baseline")
    ap.add_argument("--counter-pass", nargs="?", const="decode", default=None, choices=("decode", "decode_b2", "decode_b3", "small", "prefill", "prefill_b6", "prefill_b8", "prefill_bf16", "midbatch", "medium"),
                    help="for rocprofv3 --pmc runs.  decode: launch only the dominant kernel over the ring of "
                         "weight copies, eagerly, then a plain elementwise copy of 256 MiB (the counter's "
                         "yardstick); decode_b2 / decode_b3: the same at 2 and 3 bits.  "
                         "prefill: launch only the M=2048 kernel of the 8192->8192 layer (prefill_bf16: on bf16 storage; "
                         "prefill_b6 / prefill_b8: 6-bit and 8-bit codes).  "
                         "midbatch: launch only the mid-batch kernel, 4096->4096 at M=64 and 14336->4096 at M=16.  "
                         "small: launch only the gemv kernel's instantiations for two and for eight batch rows, "
                         "4096->28672 at M=2 and 14336->4096 at M=8.  "
                         "medium: launch only the ring tiles that split K inside the workgroup, 8192->8192 at "
                         "M=256 (64 x 128 tiles), M=512 and M=1024")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        return 2

    import torch

    from matgptq_amd import _lib

    if not torch.cuda.is_available():
        print("bench.py needs an MI355X", file=sys.stderr)
        return 2
    L = _lib.load()  # raises if the HIP library is missing: there is no fallback
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.Stream(device=dev)  # default priority

    def launch(bits, n, k, x, packed, scales, zeros, y, flags=1):
        _lib.check(L.matgptq_gemm(bits, GROUP, n, k, x.shape[0], packed.data_ptr(), scales.data_ptr(),
                                  zeros.data_ptr() if zeros is not None else None, x.data_ptr(),
                                  y.data_ptr(), stream.cuda_stream, flags))

    g = torch.Generator(device=dev).manual_seed(0)

    def make_ring(n, k, bits, copies):
        words = L.matgptq_packed_words(bits, n, k)
        # random words are valid packed codes: every bit pattern decodes to some code
        return [torch.randint(-2 ** 31, 2 ** 31 - 1, (words,), dtype=torch.int32, device=dev, generator=g)
                for _ in range(copies)]

    def make_aux(n, k):
        groups = n * (k // GROUP)
        scales = (torch.randn(groups, device=dev, generator=g).abs() * 0.01 + 1e-3).to(torch.float16)
        zeros = torch.randint(0, 256, (groups,), device=dev, generator=g).to(torch.float16)
        return scales, zeros

    def timed_graph(build, reps=5, settle_ms=10.0):
        """Captures `build()` (launches on `stream`) into a HIP graph; returns the median
        replay time in seconds over `reps` replays, measured with events on `stream`.
        `settle_ms`: keep replaying, untimed, for that long first (the clocks take some
        milliseconds to settle after the allocation and random fill of new tensors: a boost, then
        a dip below the sustained clock; rows timed inside it read up to 20 % off either way)."""
        with torch.cuda.stream(stream):
            build()  # eager warm-up of every kernel in the graph
            stream.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                build()
            graph.replay()
            stream.synchronize()
            t_end = time.perf_counter() + settle_ms * 1e-3
            while time.perf_counter() < t_end:
                graph.replay()
                stream.synchronize()
            times = []
            for _ in range(reps):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                graph.replay()
                e1.record(stream)
                stream.synchronize()
                times.append(e0.elapsed_time(e1) * 1e-3)
        return sorted(times)[len(times) // 2]

    bits = 4
    if args.counter_pass in ("decode_b2", "decode_b3", "prefill_b6", "prefill_b8"):
        bits = int(args.counter_pass[-1])
        args.counter_pass = args.counter_pass[:-3]
    if args.counter_pass in ("prefill", "prefill_bf16"):
        n, k = LLAMA3_70B["o"]
        dt, fl = (torch.bfloat16, 3) if args.counter_pass == "prefill_bf16" else (torch.float16, 1)
        packed = make_ring(n, k, bits, 1)[0]
        sc, zr = (t.to(dt) for t in make_aux(n, k))
        x = torch.randn(2048, k, device=dev, generator=g).to(dt)
        y = torch.empty(2048, n, dtype=dt, device=dev)
        with torch.cuda.stream(stream):
            for _ in range(6):
                launch(bits, n, k, x, packed, sc, zr, y, flags=fl)
            stream.synchronize()
        print(json.dumps({"counter_pass": _lib.describe_plan(bits, GROUP, n, k, 2048, True, fl), "launches": 6}))
        return 0
    if args.counter_pass == "medium":
        n, k = LLAMA3_70B["o"]
        packed = make_ring(n, k, bits, 1)[0]
        sc, zr = make_aux(n, k)
        plans = []
        for m in (256, 512, 1024):
            x = torch.randn(m, k, device=dev, generator=g).to(torch.float16)
            y = torch.empty(m, n, dtype=torch.float16, device=dev)
            with torch.cuda.stream(stream):
                for _ in range(6):
                    launch(bits, n, k, x, packed, sc, zr, y)
                stream.synchronize()
            plans.append(f"M={m}: " + _lib.describe_plan(bits, GROUP, n, k, m, True))
        print(json.dumps({"counter_pass": plans, "launches_each": 6}))
        return 0
    if args.counter_pass in ("midbatch", "small"):
        plans = []
        for name, m in ((("o", 64), ("down", 16)) if args.counter_pass == "midbatch" else (("gate_up", 2), ("down", 8))):
            n, k = LLAMA3_8B[name]
            copies = 16
            ring = make_ring(n, k, bits, copies)
            sc, zr = make_aux(n, k)
            x = torch.randn(m, k, device=dev, generator=g).to(torch.float16)
            y = torch.empty(m, n, dtype=torch.float16, device=dev)
            with torch.cuda.stream(stream):
                for i in range(2 * copies):
                    launch(bits, n, k, x, ring[i % copies], sc, zr, y)
                stream.synchronize()
            plans.append(f"{name} M={m}: " + _lib.describe_plan(bits, GROUP, n, k, m, True))
        print(json.dumps({"counter_pass": plans, "launches_each": 32}))
        return 0
    if args.counter_pass:
        n, k = LLAMA3_8B["gate_up"]
        copies = int(RING_BYTES // (n * k * bits // 8)) + 1
        ring = make_ring(n, k, bits, copies)
        sc, zr = make_aux(n, k)
        x = torch.randn(1, k, device=dev, generator=g).to(torch.float16)
        y = torch.empty(1, n, dtype=torch.float16, device=dev)
        with torch.cuda.stream(stream):
            for i in range(2 * copies):
                launch(bits, n, k, x, ring[i % copies], sc, zr, y)
            stream.synchronize()
            src = torch.zeros(COUNTER_COPY_BYTES // 4, dtype=torch.int32, device=dev)
            dst = torch.empty_like(src)
            for _ in range(4):
                torch.add(src, 1, out=dst)  # one elementwise kernel: reads and writes COUNTER_COPY_BYTES
            stream.synchronize()
        print(json.dumps({"counter_pass": _lib.describe_plan(bits, GROUP, n, k, 1, True),
                          "kernel_source_hash": kernel_source_hash(),
                          "launches": 2 * copies, "copy_bytes_each_way": COUNTER_COPY_BYTES}))
        return 0

    # ------------------------------------------------------------------ headline
    step_bytes = sum(n * k * bits // 8 for n, k in LLAMA3_8B.values())
    copies = max(2, int(RING_BYTES // step_bytes) + 1)
    rings = {name: make_ring(n, k, bits, copies) for name, (n, k) in LLAMA3_8B.items()}
    # scales, zeros and activations rotate with the codes: no operand of a step is the one the
    # previous steps left in the caches
    aux_ring = {name: [make_aux(n, k) for _ in range(copies)] for name, (n, k) in LLAMA3_8B.items()}
    x_ring = {name: [torch.randn(1, k, device=dev, generator=g).to(torch.float16) for _ in range(copies)]
              for name, (n, k) in LLAMA3_8B.items()}
    aux = {name: aux_ring[name][0] for name in LLAMA3_8B}
    xs = {name: x_ring[name][0] for name in LLAMA3_8B}
    ys = {name: torch.empty(1, n, dtype=torch.float16, device=dev) for name, (n, k) in LLAMA3_8B.items()}

    def step(i):
        c = i % copies
        for name, (n, k) in LLAMA3_8B.items():
            launch(bits, n, k, x_ring[name][c], rings[name][c], aux_ring[name][c][0], aux_ring[name][c][1], ys[name])

    with torch.cuda.stream(stream):
        for i in range(args.warmup):
            step(i)
        stream.synchronize()
    torch.cuda.synchronize()
    t_wall0 = time.perf_counter()
    elapsed = timed_graph(lambda: [step(i) for i in range(args.steps)], reps=21, settle_ms=0.0)  # median of 21 replays
    torch.cuda.synchronize()
    t_wall = time.perf_counter() - t_wall0
    ms_per_step = elapsed / args.steps * 1e3
    value = step_bytes / (elapsed / args.steps) / 1e9

    # --------------------------------------------------------- dominant kernel
    n, k = LLAMA3_8B["gate_up"]
    launches = max(copies, 64)
    t_dom = timed_graph(lambda: [launch(bits, n, k, x_ring["gate_up"][i % copies], rings["gate_up"][i % copies],
                                        aux_ring["gate_up"][i % copies][0], aux_ring["gate_up"][i % copies][1],
                                        ys["gate_up"])
                                 for i in range(launches)], reps=21, settle_ms=0.0) / launches
    dom_bytes = algorithmic_bytes(n, k, 1, bits)
    roofline = {
        "kernel": _lib.describe_plan(bits, GROUP, n, k, 1, True),
        "bound": "hbm",
        "achieved": round(dom_bytes / t_dom / 1e9, 1),
        "peak": HBM_PEAK_GBPS,
        "unit": "GB/s",
        "frac": round(dom_bytes / t_dom / 1e9 / HBM_PEAK_GBPS, 4),
        "traffic": measured_traffic(_lib.describe_plan(bits, GROUP, n, k, 1, True)),
        "kernel_source_hash": kernel_source_hash(),
        "us_per_launch": round(t_dom * 1e6, 2),
        "algorithmic_bytes": dom_bytes,
    }

    extra = {}
    # ------------------------------------------------------------- read floor
    # What a kernel that only READ each layer's bytes takes on this GPU, measured the same way
    # (graph replays, every launch on bytes no earlier launch of the replay touched): the bare-read
    # probe of the library on the algorithmic bytes of each layer, and the four of a step in a row.
    flat = torch.empty(int(RING_BYTES * 1.25) // 4, dtype=torch.int32, device=dev)
    flat.random_(generator=g)
    flat_bytes = flat.numel() * 4
    cursor = [0]

    def probe(nbytes):
        nbytes = (nbytes + 4095) // 4096 * 4096
        if cursor[0] + nbytes > flat_bytes:
            cursor[0] = 0
        _lib.check(L.matgptq_probe_read(flat.data_ptr() + cursor[0], nbytes, stream.cuda_stream))
        cursor[0] += nbytes

    layer_bytes = {name: algorithmic_bytes(n, k, 1, bits) for name, (n, k) in LLAMA3_8B.items()}
    floor = {}
    for name, nb in layer_bytes.items():
        cnt = max(32, int(flat_bytes // nb))
        t = timed_graph(lambda: [probe(nb) for _ in range(cnt)], reps=5) / cnt
        floor[name] = {"us": round(t * 1e6, 2), "GBps": round(nb / t / 1e9, 1)}
    t = timed_graph(lambda: [[probe(nb) for nb in layer_bytes.values()] for _ in range(args.steps)], reps=5) / args.steps
    floor["step_of_four_reads_us"] = round(t * 1e6, 2)
    floor["step_measured_over_floor"] = round(ms_per_step * 1e-3 / t, 3)
    floor["dominant_kernel_over_its_read"] = round(t_dom * 1e6 / floor["gate_up"]["us"], 3)
    extra["read_floor"] = floor
    del flat
    torch.cuda.empty_cache()

    cpu_baseline = None
    if not args.quick:
        # ------------------------------------------------- per layer, per bitwidth
        table = {}
        for b in (8, 6, 4, 3, 2):
            for name, (n, k) in LLAMA3_8B.items():
                wbytes = n * k * b // 8
                cp = max(2, int(RING_BYTES // wbytes) + 1)
                ring = rings[name] if b == bits else make_ring(n, k, b, cp)
                cp = len(ring)
                reps = max(cp, 32)
                for zp in (True, False):
                    t = timed_graph(lambda: [launch(b, n, k, xs[name], ring[i % cp], aux[name][0],
                                                    aux[name][1] if zp else None, ys[name])
                                             for i in range(reps)], settle_ms=15.0) / reps
                    table[f"{name}_b{b}_{'zp' if zp else 'sym'}"] = {
                        "us": round(t * 1e6, 2),
                        "weight_GBps": round(wbytes / t / 1e9, 1),
                        "pct_hbm_peak": round(wbytes / t / 1e9 / HBM_PEAK_GBPS * 100, 1),
                    }
                del ring
        extra["gemv_M1"] = table
        # ------------- the same kernel on the Llama-3-70B layers (M = 1, 4 bits, scale + zero): larger
        # layers amortise the launch and the first-byte latency that bound the 8-60 MB layers above
        t70 = {}
        step70_us, step70_bytes = 0.0, 0
        for name, (n, k) in LLAMA3_70B.items():
            wbytes = n * k * bits // 8
            cp = max(2, int(RING_BYTES // wbytes) + 1)
            ring = make_ring(n, k, bits, cp)
            auxs = [make_aux(n, k) for _ in range(cp)]
            x70 = torch.randn(1, k, device=dev, generator=g).to(torch.float16)
            y70 = torch.empty(1, n, dtype=torch.float16, device=dev)
            reps = max(cp, 16)
            t = timed_graph(lambda: [launch(bits, n, k, x70, ring[i % cp], auxs[i % cp][0], auxs[i % cp][1], y70)
                                     for i in range(reps)]) / reps
            ab = algorithmic_bytes(n, k, 1, bits)
            t70[name] = {"us": round(t * 1e6, 2), "weight_GBps": round(wbytes / t / 1e9, 1),
                         "pct_hbm_peak": round(wbytes / t / 1e9 / HBM_PEAK_GBPS * 100, 1),
                         "algorithmic_pct_hbm_peak": round(ab / t / 1e9 / HBM_PEAK_GBPS * 100, 1),
                         "kernel": _lib.describe_plan(bits, GROUP, n, k, 1, True)}
            step70_us += t * 1e6
            step70_bytes += wbytes
            del ring, auxs
            torch.cuda.empty_cache()
        t70["step_sum_of_layers"] = {"us": round(step70_us, 2), "weight_GBps": round(step70_bytes / step70_us / 1e3, 1),
                                     "pct_hbm_peak": round(step70_bytes / step70_us / 1e3 / HBM_PEAK_GBPS * 100, 1)}
        extra["gemv_M1_llama3_70b"] = t70
        # ----------------- master-resident planes: one buffer, bitwidth chosen per call (M = 1)
        # moved bytes per weight: (b + 1) / 8 for 2, 3 and 4 bits (the top b bits and the round bit),
        # 1 for 6 and 8 bits; both rates are stated, on the sliced bytes and on the bytes moved
        mtab = {}
        for name, (n, k) in LLAMA3_8B.items():
            words = L.matgptq_master_words(n, k)
            cp = max(2, int(RING_BYTES // (n * k)) + 1)
            mring = [torch.randint(-2 ** 31, 2 ** 31 - 1, (words,), dtype=torch.int32, device=dev, generator=g)
                     for _ in range(cp)]
            reps = max(cp, 32)
            for b in (8, 6, 4, 3, 2):
                def one(i):
                    _lib.check(L.matgptq_gemm_master(b, GROUP, n, k, 1, mring[i % cp].data_ptr(), aux[name][0].data_ptr(),
                                                     aux[name][1].data_ptr(), xs[name].data_ptr(), ys[name].data_ptr(),
                                                     None, 0, stream.cuda_stream, 1))
                t = timed_graph(lambda: [one(i) for i in range(reps)]) / reps
                moved = n * k * (b + 1 if b <= 4 else 8) // 8
                mtab[f"{name}_b{b}"] = {"us": round(t * 1e6, 2),
                                        "sliced_GBps": round(n * k * b / 8 / t / 1e9, 1),
                                        "moved_GBps": round(moved / t / 1e9, 1),
                                        "pct_hbm_peak_moved": round(moved / t / 1e9 / HBM_PEAK_GBPS * 100, 1),
                                        "presliced_us": table[f"{name}_b{b}_zp"]["us"]}
            # batches of 8 and 64 rows at 4 bits from the same planes: the mid-batch kernel reads them
            # itself (no workspace, no slicing pass); beside it the same kernel on the pre-sliced tensor
            for m in (8, 64):
                xm = torch.randn(m, k, device=dev, generator=g).to(torch.float16)
                ym = torch.empty(m, n, dtype=torch.float16, device=dev)

                def planes_call(i):
                    _lib.check(L.matgptq_gemm_master(bits, GROUP, n, k, m, mring[i % cp].data_ptr(), aux[name][0].data_ptr(),
                                                     aux[name][1].data_ptr(), xm.data_ptr(), ym.data_ptr(),
                                                     None, 0, stream.cuda_stream, 1))
                assert L.matgptq_gemm_master_workspace_bytes(bits, GROUP, n, k, m, 1) == 0
                t = timed_graph(lambda: [planes_call(i) for i in range(cp)]) / cp
                ring4 = rings[name]
                tp = timed_graph(lambda: [launch(bits, n, k, xm, ring4[i % len(ring4)], aux[name][0], aux[name][1], ym)
                                          for i in range(len(ring4))]) / len(ring4)
                mtab[f"{name}_b{bits}_M{m}"] = {"us": round(t * 1e6, 2), "presliced_us": round(tp * 1e6, 2),
                                                "moved_GBps": round(n * k * (bits + 1) / 8 / t / 1e9, 1)}
            del mring
        extra["gemv_M1_master_resident"] = mtab
        # ----------------------------------------- small batch (configs[2]), all four layers
        small = {}
        for name, (n, k) in LLAMA3_8B.items():
            for b in (4, 3):
                ring = rings[name] if b == bits else make_ring(n, k, b, max(2, int(RING_BYTES // (n * k * b // 8)) + 1))
                cp = len(ring)
                for m in (2, 4, 8, 16):
                    xm = torch.randn(m, k, device=dev, generator=g).to(torch.float16)
                    ym = torch.empty(m, n, dtype=torch.float16, device=dev)
                    t = timed_graph(lambda: [launch(b, n, k, xm, ring[i % cp], aux[name][0], aux[name][1], ym)
                                             for i in range(cp)]) / cp
                    small[f"{name}_b{b}_M{m}"] = {"us": round(t * 1e6, 2),
                                                  "weight_GBps": round(n * k * b / 8 / t / 1e9, 1),
                                                  "kernel": _lib.describe_plan(b, GROUP, n, k, m, True).split()[0]}
                del ring
        # -------------------------------------------- mid batch: between decode and prefill
        mid = {}
        for name, (n, k) in LLAMA3_8B.items():
            ring = rings[name]
            cp = len(ring)
            for m in (32, 64, 128, 256):
                xm = torch.randn(m, k, device=dev, generator=g).to(torch.float16)
                ym = torch.empty(m, n, dtype=torch.float16, device=dev)
                t = timed_graph(lambda: [launch(bits, n, k, xm, ring[i % cp], aux[name][0], aux[name][1], ym)
                                         for i in range(cp)]) / cp
                mid[f"{name}_b4_M{m}"] = {"us": round(t * 1e6, 2), "TFLOPs": round(2.0 * m * n * k / t / 1e12, 1),
                                          "kernel": _lib.describe_plan(bits, GROUP, n, k, m, True).split()[0]}
        extra["mid_batch"] = mid
        extra["small_batch"] = small
        del rings
        torch.cuda.empty_cache()
        # ------------------------------------------- Mix'n'Match decode step (configs[3])
        # the 128 linears of a 32-layer Llama-3-8B-shaped decoder at batch 1, every linear at a
        # bitwidth drawn from {2,3,4,6,8} (seeded); attention, norms and the head are not part
        # of the measured path, so this is the linear share of a token, not end-to-end tokens/s
        import random
        rnd = random.Random(0)
        stack, total_bytes, hist = [], 0, {}
        for _layer in range(32):
            for name, (n, k) in LLAMA3_8B.items():
                b = rnd.choice((2, 3, 4, 6, 8))
                hist[b] = hist.get(b, 0) + 1
                stack.append((b, n, k, xs[name], make_ring(n, k, b, 1)[0], aux[name][0], aux[name][1], ys[name]))
                total_bytes += n * k * b // 8
        t = timed_graph(lambda: [launch(*item) for item in stack])
        extra["mixnmatch_decode_linears"] = {
            "linears": len(stack), "bitwidth_histogram": {str(b): c for b, c in sorted(hist.items())},
            "mean_bits": round(total_bytes * 8 / sum(n * k for _, n, k, *_ in stack), 2),
            "ms_per_token": round(t * 1e3, 4), "tokens_per_s_linears_only": round(1.0 / t, 1),
            "weight_GBps": round(total_bytes / t / 1e9, 1)}
        del stack
        torch.cuda.empty_cache()
        # ------------------------ the same decoder end to end (configs[3]): tokens/s
        # linears through the module, norms / rotary / attention over a static cache at context
        # 512 / dense head / argmax as torch operators, one token per HIP graph replay
        from matgptq_amd import decoder
        extra["mixnmatch_decoder_end_to_end"] = decoder.measure(layers=32, context=512, new_tokens=64)
        torch.cuda.empty_cache()
        # --------------------------------------------------------------- prefill
        pre = {}
        m = 2048
        for name, (n, k) in LLAMA3_70B.items():
            packed = make_ring(n, k, 4, 1)[0]
            sc, zr = make_aux(n, k)
            xm = torch.randn(m, k, device=dev, generator=g).to(torch.float16)
            ym = torch.empty(m, n, dtype=torch.float16, device=dev)
            if not pre:
                # the first launches after the light decode sections run through a clock
                # transient (boost, then a dip below the sustained clock, about 10 ms in all):
                # reach the sustained state before anything is timed
                with torch.cuda.stream(stream):
                    for _ in range(100):
                        launch(4, n, k, xm, packed, sc, zr, ym)
                    stream.synchronize()
            for zp in (True, False):
                t = timed_graph(lambda: [launch(4, n, k, xm, packed, sc, zr if zp else None, ym) for _ in range(5)],
                                settle_ms=20.0) / 5
                tf = 2.0 * m * n * k / t / 1e12
                pre[f"{name}_b4_M2048_{'zp' if zp else 'sym'}"] = {
                    "ms": round(t * 1e3, 3), "TFLOPs": round(tf, 1),
                    "pct_mfma_peak": round(tf / MFMA_FP16_PEAK_TFLOPS * 100, 1)}
            # the other bitwidths (zero-point form) and bf16 storage at 4 bits
            for b in (2, 3, 6, 8):
                pk = make_ring(n, k, b, 1)[0]
                t = timed_graph(lambda: [launch(b, n, k, xm, pk, sc, zr, ym) for _ in range(3)], reps=3, settle_ms=20.0) / 3
                tf = 2.0 * m * n * k / t / 1e12
                pre[f"{name}_b{b}_M2048_zp"] = {"ms": round(t * 1e3, 3), "TFLOPs": round(tf, 1),
                                                "pct_mfma_peak": round(tf / MFMA_FP16_PEAK_TFLOPS * 100, 1),
                                                "kernel": _lib.describe_plan(b, GROUP, n, k, m, True)}
                del pk
            xb, scb, zrb = xm.to(torch.bfloat16), sc.to(torch.bfloat16), zr.to(torch.bfloat16)
            yb = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
            t = timed_graph(lambda: [launch(4, n, k, xb, packed, scb, zrb, yb, flags=3) for _ in range(3)], reps=3,
                            settle_ms=20.0) / 3
            tf = 2.0 * m * n * k / t / 1e12
            pre[f"{name}_b4_M2048_zp_bf16"] = {"ms": round(t * 1e3, 3), "TFLOPs": round(tf, 1),
                                               "pct_mfma_peak": round(tf / MFMA_FP16_PEAK_TFLOPS * 100, 1),
                                               "kernel": _lib.describe_plan(4, GROUP, n, k, m, True, 3)}
            del packed, xm, ym, xb, yb
        extra["prefill_llama3_70b"] = pre
        torch.cuda.empty_cache()
        # ------------------- speed-up over the dense fp16 product, the reference's own methodology
        # (inference_lib/bench_matgptq_matmul.py:36-53): square layers, zero = 128 (its 8-argument
        # operator), time of F.linear(x, W_fp16) divided by the kernel's time, both as back-to-back
        # replays of one graph on ONE weight buffer (so small layers are served from the caches for
        # both sides, as in the reference's do_bench_cudagraph)
        speed = {}
        for size in (2048, 4096, 8192, 16384):
            wd = (torch.randn(size, size, device=dev, generator=g) * 0.02).to(torch.float16)
            sc1, _ = make_aux(size, size)
            for m in (1, 2, 4, 8, 16, 32, 64):
                xm = torch.randn(m, size, device=dev, generator=g).to(torch.float16)
                ym = torch.empty(m, size, dtype=torch.float16, device=dev)
                reps = 20 if size <= 8192 else 8

                def dense():
                    for _ in range(reps):
                        torch.nn.functional.linear(xm, wd)
                t_dense = timed_graph(dense, reps=3) / reps
                row = {"dense_us": round(t_dense * 1e6, 2)}
                for b in (2, 3, 4, 6, 8):
                    pk = make_ring(size, size, b, 1)[0]
                    t = timed_graph(lambda: [launch(b, size, size, xm, pk, sc1, None, ym) for _ in range(reps)], reps=3) / reps
                    row[f"b{b}"] = round(t_dense / t, 2)
                    del pk
                speed[f"{size}_M{m}"] = row
            del wd
            torch.cuda.empty_cache()
        extra["speedup_over_dense_fp16"] = speed
        # ------------------------------------------------ batches of a few hundred rows
        # (chunked prefill): the Llama-3-70B and 8B layers at 4 bits, zero-point form, beside the dense
        # fp16 product on the same GPU; graphs of five launches, median of five replays
        for table, layers, batches in (("medium_batch_llama3_70b_b4", LLAMA3_70B, (128, 256, 512, 1024)),
                                       ("medium_batch_llama3_8b_b4", LLAMA3_8B, (256, 512, 768))):
            medium = {}
            for name, (n, k) in layers.items():
                packed = make_ring(n, k, 4, 1)[0]
                sc, zr = make_aux(n, k)
                wd = (torch.randn(n, k, device=dev, generator=g) * 0.02).to(torch.float16)
                for m in batches:
                    xm = torch.randn(m, k, device=dev, generator=g).to(torch.float16)
                    ym = torch.empty(m, n, dtype=torch.float16, device=dev)
                    t = timed_graph(lambda: [launch(4, n, k, xm, packed, sc, zr, ym) for _ in range(5)]) / 5
                    t_dense = timed_graph(lambda: [torch.nn.functional.linear(xm, wd) for _ in range(5)]) / 5
                    medium[f"{name}_M{m}"] = {"us": round(t * 1e6, 1), "dense_us": round(t_dense * 1e6, 1),
                                              "speedup": round(t_dense / t, 2),
                                              "TFLOPs": round(2.0 * m * n * k / t / 1e12, 1),
                                              "kernel": _lib.describe_plan(4, GROUP, n, k, m, True)}
                del packed, wd
                torch.cuda.empty_cache()
            extra[table] = medium
        # ---------------------------------------------------------- load time
        # What process_weights_after_loading costs per layer (gate_up of Llama-3-8B, 117 M master
        # codes already in HBM): slice + pack in one kernel (reads 1 byte per code, writes b/8),
        # the master-resident planes (1 read, 1 written), the scale reorder; and the host packer
        # (the reference's route: inference_lib/matgptq_cuda/csrc/bindings.cpp:63-83) on a 4096 x 4096
        # layer with all host threads, without its two PCIe copies.
        n, k = LLAMA3_8B["gate_up"]
        master = torch.randint(0, 256, (n, k), dtype=torch.uint8, device=dev, generator=g)
        load = {}
        for b in (2, 4, 8):
            out_words = torch.empty(L.matgptq_packed_words(b, n, k), dtype=torch.int32, device=dev)
            t = timed_graph(lambda: _lib.check(L.matgptq_pack_device(master.data_ptr(), n, k, b, 1, out_words.data_ptr(),
                                                                    torch.cuda.current_stream().cuda_stream)), reps=3)
            moved = n * k * (1 + b / 8)
            load[f"slice_pack_b{b}_gate_up"] = {"us": round(t * 1e6, 1), "GBps": round(moved / t / 1e9, 1),
                                               "pct_hbm_peak": round(moved / t / 1e9 / HBM_PEAK_GBPS * 100, 1)}
            del out_words
        planes = torch.empty(L.matgptq_master_words(n, k), dtype=torch.int32, device=dev)
        t = timed_graph(lambda: _lib.check(L.matgptq_pack_master_device(master.data_ptr(), n, k, planes.data_ptr(),
                                                                       torch.cuda.current_stream().cuda_stream)), reps=3)
        load["master_planes_gate_up"] = {"us": round(t * 1e6, 1), "GBps": round(2 * n * k / t / 1e9, 1),
                                         "pct_hbm_peak": round(2 * n * k / t / 1e9 / HBM_PEAK_GBPS * 100, 1)}
        del planes, master
        import numpy as np
        hq = np.random.default_rng(0).integers(0, 256, (4096, 4096), dtype=np.uint8)
        hout = np.zeros(L.matgptq_packed_words(4, 4096, 4096), dtype=np.uint32)
        best = float("inf")
        for _ in range(3):
            t0 = time.perf_counter()
            _lib.check(L.matgptq_pack_host(hq.ctypes.data, 4096, 4096, 4, 1, hout.ctypes.data))
            best = min(best, time.perf_counter() - t0)
        load["host_slice_pack_b4_4096x4096"] = {"ms": round(best * 1e3, 2), "Mcodes_per_s": round(4096 * 4096 / best / 1e6, 1),
                                                "threads": os.cpu_count()}
        extra["load_time"] = load
        torch.cuda.empty_cache()
        # ---------------- the reference's transformers caller (inference_lib/bench_transformers_e2e.py):
        # a LlamaForCausalLM of the same shape with MatGPTQLinear modules, StaticCache,
        # torch.compile(fullgraph, reduce-overhead), timed like its time_prof
        try:
            from matgptq_amd import hf_bench
            extra["transformers_end_to_end"] = hf_bench.measure(layers=32, context=512)
        except Exception as e:  # transformers or the inductor toolchain absent: the figure is optional
            extra["transformers_end_to_end"] = {"error": f"{type(e).__name__}: {str(e)[:200]}"}
        torch.cuda.empty_cache()
        # ---------------------------------------------------------- CPU baseline
        cpu_baseline = cpu_path_baseline(step_bytes)

    headline = {"value": round(value, 1), "steps": args.steps, "warmup": args.warmup,
                "ms_per_step": round(ms_per_step, 5), "wall_s_timed_region": round(t_wall, 4)}
    extra_path = write_tables({"headline": headline, "roofline": roofline, "cpu_baseline": cpu_baseline, **extra})
    print(final_line(headline, roofline, cpu_baseline, extra, extra_path))
    return 0


EXTRA_FILE = os.path.join("gpurun_out", "bench_extra.json")
LINE_LIMIT = 4096  # bytes: the last stdout line has to fit the tail a harness keeps of the output


def write_tables(tables: dict):
    """The per-layer / per-bitwidth / per-batch tables go to a side file (and, one table per line, to
    stderr); only scalars ride in the last stdout line.  Returns the file's path relative to the
    repository root, or None when it cannot be written."""
    for name, table in tables.items():
        print(json.dumps({name: table}), file=sys.stderr)
    try:
        os.makedirs(os.path.join(ROOT, os.path.dirname(EXTRA_FILE)), exist_ok=True)
        with open(os.path.join(ROOT, EXTRA_FILE), "w") as f:
            json.dump(tables, f, indent=1)
        return EXTRA_FILE
    except OSError:
        return None


def final_line(headline: dict, roofline: dict, cpu_baseline, extra: dict, extra_path=None) -> str:
    """The ONE JSON line that ends stdout: the contract's keys, `roofline`, `cpu_baseline` and a dozen
    scalars picked from the tables.  Kept under LINE_LIMIT bytes whatever the tables hold."""
    def pick(table, row, field):
        try:
            return extra[table][row][field]
        except (KeyError, TypeError):
            return None

    floor = extra.get("read_floor") or {}
    summary = {
        "step_over_four_bare_reads": floor.get("step_measured_over_floor"),
        "dominant_kernel_over_its_bare_read": floor.get("dominant_kernel_over_its_read"),
        "four_bare_reads_us": floor.get("step_of_four_reads_us"),
    }
    for name in ("qkv", "o", "gate_up", "down"):
        summary[f"gemv_b4_{name}_us"] = pick("gemv_M1", f"{name}_b4_zp", "us")
    for b in (2, 3, 6, 8):
        summary[f"gemv_b{b}_gate_up_pct_hbm_peak"] = pick("gemv_M1", f"gate_up_b{b}_zp", "pct_hbm_peak")
    for name in ("qkv", "o", "gate_up", "down"):
        summary[f"prefill_b4_M2048_{name}_pct_mfma_peak"] = pick("prefill_llama3_70b", f"{name}_b4_M2048_zp", "pct_mfma_peak")
    wide = [v["pct_mfma_peak"] for r, v in (extra.get("prefill_llama3_70b") or {}).items()
            if ("_b6_" in r or "_b8_" in r) and "pct_mfma_peak" in v]
    summary["prefill_b6_b8_min_pct_mfma_peak"] = min(wide) if wide else None
    medium = [v["speedup"] for v in (extra.get("medium_batch_llama3_70b_b4") or {}).values() if "speedup" in v]
    summary["medium_batch_min_speedup_over_dense_fp16"] = min(medium) if medium else None
    medium = [v["speedup"] for v in (extra.get("medium_batch_llama3_8b_b4") or {}).values() if "speedup" in v]
    summary["medium_batch_8b_min_speedup_over_dense_fp16"] = min(medium) if medium else None
    summary["decoder_tokens_per_s_graph"] = (extra.get("mixnmatch_decoder_end_to_end") or {}).get("tokens_per_s_graph")
    summary["transformers_tokens_per_s_compiled"] = (extra.get("transformers_end_to_end") or {}).get("tokens_per_s_compiled")
    summary = {k: v for k, v in summary.items() if v is not None}

    roof = {k: roofline.get(k) for k in ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel",
                                         "us_per_launch", "algorithmic_bytes")}
    cpu = None
    if cpu_baseline is not None:
        cpu = {k: cpu_baseline.get(k) for k in ("value", "unit", "cores", "kind", "sample")}
    out = {
        "metric": "batch1_gemv_sliced_weight_GBps_4bit_llama3_8b_layers",
        "value": headline["value"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": headline["steps"],
        "warmup": headline["warmup"],
        "ms_per_step": headline["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "configs[1]: Llama-3-8B linears qkv/o/gate_up/down, M=1 decode, 4-bit slice, "
                               "group 128, fp16 scale+zero; ring of weight copies > 2 GiB",
                   "pct_hbm_peak": round(headline["value"] / HBM_PEAK_GBPS * 100, 1),
                   "wall_s_timed_region": headline["wall_s_timed_region"]},
        "roofline": roof,
        "cpu_baseline": cpu,
        "summary": summary,
        "tables": extra_path,
    }
    line = json.dumps(out)
    if len(line) > LINE_LIMIT:  # never let the scalars push the contract's keys out of a kept tail
        out["summary"] = {}
        line = json.dumps(out)
    return line


def cpu_path_baseline(step_bytes: int):
    """One pass of the same four layers through the reference's CPU PyTorch path."""
    import torch

    from oracle import torch_path

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    gen = torch.Generator().manual_seed(0)
    layers = []
    for name, (n, k) in LLAMA3_8B.items():
        q = torch.randint(0, 256, (n, k), dtype=torch.uint8, generator=gen)
        s = (torch.randn(n, k // GROUP, generator=gen).abs() * 0.01 + 1e-3).to(torch.float16)
        z = torch.randint(0, 256, (n, k // GROUP), generator=gen).to(torch.float16)
        x = torch.randn(1, k, generator=gen).to(torch.float16)
        layers.append((q, s, z, x))
    with torch.no_grad():
        q, s, z, x = layers[1]
        torch_path.forward(x, q, s, z, 8, 4)  # warm-up on the smallest layer
        best = float("inf")
        for _ in range(5):
            t0 = time.perf_counter()
            for q, s, z, x in layers:
                torch_path.forward(x, q, s, z, 8, 4)
            best = min(best, time.perf_counter() - t0)
        # the matrix product alone on weights dequantised beforehand, fp16 and fp32 (CPU fp16
        # GEMV can be much slower than fp32: both are stated)
        ws = [torch_path.get_weight(q, s, z, 8, 4) for q, s, z, _ in layers]
        only = {}
        for tag, cast in (("fp16", lambda t: t), ("fp32", lambda t: t.float())):
            wl = [cast(w) for w in ws]
            xl = [cast(x) for _, _, _, x in layers]
            torch.nn.functional.linear(xl[1], wl[1])
            t_best = float("inf")
            for _ in range(5):
                t0 = time.perf_counter()
                for w, x in zip(wl, xl):
                    torch.nn.functional.linear(x, w)
                t_best = min(t_best, time.perf_counter() - t0)
            only[tag] = t_best
        # configs[0] alone: one 4096 -> 4096 layer at M = 1, 4 bits (median of 5)
        q, s, z, x = layers[1]
        ts = []
        for _ in range(5):
            t0 = time.perf_counter()
            torch_path.forward(x, q, s, z, 8, 4)
            ts.append(time.perf_counter() - t0)
        cfg0 = sorted(ts)[2]
        # configs[4], the o layer (8192 -> 8192) at 4 bits: slice + dequantize once, then the
        # product on a bounded sample of the 2048 batch rows, scaled to the full batch
        n4, k4 = LLAMA3_70B["o"]
        q4 = torch.randint(0, 256, (n4, k4), dtype=torch.uint8, generator=gen)
        s4 = (torch.randn(n4, k4 // GROUP, generator=gen).abs() * 0.01 + 1e-3).to(torch.float16)
        z4 = torch.randint(0, 256, (n4, k4 // GROUP), generator=gen).to(torch.float16)
        t0 = time.perf_counter()
        w4 = torch_path.get_weight(q4, s4, z4, 8, 4)
        t_deq = time.perf_counter() - t0
        rows = 64
        x4 = torch.randn(rows, k4, generator=gen).to(torch.float16)
        t0 = time.perf_counter()
        torch.nn.functional.linear(x4, w4)
        t_rows = time.perf_counter() - t0
        if t_rows < 1.0:  # fast enough for more rows: take a larger sample
            rows = 256
            x4 = torch.randn(rows, k4, generator=gen).to(torch.float16)
            t0 = time.perf_counter()
            torch.nn.functional.linear(x4, w4)
            t_rows = time.perf_counter() - t0
        t_full = t_deq + t_rows * (2048 / rows)
        cfg4 = {"layer": "o 8192->8192, M=2048, 4-bit", "sample_rows": rows,
                "dequantize_s": round(t_deq, 3), "linear_s_sample": round(t_rows, 3),
                "s_per_call_scaled": round(t_full, 3),
                "TFLOPs": round(2.0 * 2048 * n4 * k4 / t_full / 1e12, 4)}
    return {
        "value": round(step_bytes / best / 1e9, 3),
        "unit": "GB/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"one full step (4 layers, M=1, 4-bit), best of 5, {best:.3f} s per step: "
                  "slice + dequantize + F.linear in torch on the host, fp16",
        "linear_only_s_per_step": {k: round(v, 4) for k, v in only.items()},
        "config0_4096x4096_M1_b4": {"s_per_call": round(cfg0, 4),
                                    "weight_GBps": round(4096 * 4096 * 4 / 8 / cfg0 / 1e9, 3)},
        "config4_prefill_o_layer": cfg4,
    }


if __name__ == "__main__":
    sys.exit(main())
