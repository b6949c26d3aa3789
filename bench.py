#!/usr/bin/env python3
"""Benchmark of the int4 weight-only linear hot path on one MI355X.

Workload (BASELINE.json configs[1]): GPTQ int4 decode GEMV, M=1, fp16, groupsize 128,
symmetric zeros, over the four Llama-3-8B projections (qkv 4096x6144, o 4096x4096,
gate_up 4096x28672, down 14336x4096).  One *step* = those four projections once, i.e.
the quantized-linear work of one decoder layer for one token.  Weights rotate over R
distinct copies (R * 113 MB >= 512 MB) so that every step streams from HBM and not from
the 256 MB Infinity Cache.  Inputs are resident in HBM before the timed region.

`value` = algorithmic bytes of all timed steps / wall time of the timed region (GB/s).
`roofline` = the decode kernel against the 8 TB/s HBM peak, from per-launch durations
measured with HIP events on the launch stream inside this script.
`gemm` (when the prefill kernel is built) = M=2048 TFLOP/s on the same shapes.
`cfg4` / `cfg5` = the act-order (Llama-3-70B shapes) and AWQ (Mistral-7B shapes) configurations
at their own sizes, checkpoint-layout kernels and the opt-in load-time conversions side by side.
`cpu_baseline` = the PyTorch restatement of the reference's dequantize-then-matmul path on all
host cores (torch thread pool), a bounded sample.

Prints exactly one JSON line on stdout.
"""

from __future__ import annotations

import argparse
import ctypes
import importlib
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E peak
MFMA_PEAK_TFLOPS = 2500.0    # MI355X dense fp16/bf16 MFMA peak

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE live next to the
# profile summaries they come from (the file names the commit and the summary)
TRAFFIC_FILE = ROOT / "profiles" / "hbm_traffic.json"


def measured_traffic(key, field="bytes_per_launch"):
    """Bytes per launch from the tracked counter summary (or the commit it was measured at), or
    None when there is none."""
    try:
        entry = json.loads(TRAFFIC_FILE.read_text())[key]
        return int(entry[field]) if field == "bytes_per_launch" else entry[field]
    except (OSError, KeyError, ValueError, TypeError):
        return None


PACKAGE_DIR = ROOT / "text-generation-inference_amd"
_probe_lib = None


def load_probe_lib():
    """The benchmark's own probe kernels (libq4probe.so, csrc/bench/q4_probe.hip): read-only and
    LDS-read launches.  Not part of the product library."""
    global _probe_lib
    if _probe_lib is None:
        path = PACKAGE_DIR / "libq4probe.so"
        if not path.exists():
            raise ImportError(f"{path} is missing: build it with `python {PACKAGE_DIR / 'build.py'}`")
        lib = ctypes.CDLL(str(path))
        vp, ci = ctypes.c_void_p, ctypes.c_int
        lib.q4_probe_read.restype = ci
        lib.q4_probe_read.argtypes = [vp, ctypes.c_size_t, ci, ci, ci, ci, ci, ci, vp, vp]
        lib.q4_probe_lds.restype = ci
        lib.q4_probe_lds.argtypes = [vp, ci, ci, vp, vp]
        lib.q4_probe_last_error.restype = ctypes.c_char_p
        lib.q4_probe_last_error.argtypes = []
        _probe_lib = lib
    return _probe_lib


def probe_check(rc):
    if rc < 0:
        raise RuntimeError(f"libq4probe error {rc}: {load_probe_lib().q4_probe_last_error().decode()}")

SHAPES = [  # name, K, N
    ("qkv_proj", 4096, 6144),
    ("o_proj", 4096, 4096),
    ("gate_up_proj", 4096, 28672),
    ("down_proj", 14336, 4096),
]
GROUPSIZE = 128


def gemv_bytes(M, K, N, gs=GROUPSIZE, g_idx=False):
    """Algorithmic bytes of one call: packed weights + scales + zeros (+ g_idx) + x + y."""
    G = K // gs
    return K * N // 2 + G * N * 2 + G * N // 2 + (4 * K if g_idx else 0) + 2 * M * (K + N)


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--m", type=int, default=1, help="activation rows of the decode workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-gemm", action="store_true", help="skip the prefill GEMM leg")
    ap.add_argument("--gemm-m", type=int, default=2048)
    ap.add_argument("--no-moe", action="store_true", help="skip the mixture-of-experts block leg")
    ap.add_argument("--no-batch", action="store_true",
                    help="skip the batched-decode leg (GPTQ at 4..64 rows, AWQ and act-order at 1 and 16 rows)")
    ap.add_argument("--copies", type=int, default=0, help="weight copies to rotate over (0 = auto)")
    ap.add_argument("--no-autotune", action="store_true",
                    help="skip the load-time tuning pass (ops.autotune, what the layers run in their Warmup hook): "
                         "every call then takes the library's own fitted decomposition")
    ap.add_argument("--no-dense-ref", action="store_true",
                    help="skip timing torch's dense fp16 matmul (hipBLASLt) on the GEMM shapes")
    ap.add_argument("--floor-probe", action="store_true",
                    help="time read-only kernels (q4_probe_read) on buffers of the projections' sizes and print a table")
    ap.add_argument("--lds-probe", action="store_true",
                    help="time 128-bit LDS reads (q4_probe_lds) under several lane-to-address maps and print a table")
    ap.add_argument("--awq-probe", action="store_true",
                    help="a few prefill launches (M = --gemm-m) of the AWQ-layout kernel and of the GPTQ-layout kernel on "
                         "4096 x 14336, for counter runs under rocprofv3")
    ap.add_argument("--act-probe", action="store_true",
                    help="a few launches of the act-order kernels that read the checkpoint through g_idx: decode at "
                         "M = 1 and 16 on 28672 x 8192, prefill (M = --gemm-m) on 8192 x 10240, for counter runs "
                         "under rocprofv3")
    ap.add_argument("--probe-trace", action="store_true",
                    help="eager launches of the empty and the read-only probe kernels on the decode kernels' own "
                         "grids, then of the decode kernels, for a rocprofv3 --kernel-trace run; prints no JSON line")
    ap.add_argument("--phase-breakdown", action="store_true",
                    help="run the four decode projections (M = --m) on the phase-stamp build of the library "
                         "(libq4linear_stamps.so) and print where a launch's time goes, wave by wave")
    ap.add_argument("--phase-configs", default="",
                    help="with --phase-breakdown: JSON object projection name -> explicit decode configuration "
                         "[column waves, K waves, splits, words] (as q4_gemv_tuned takes it) instead of the library's choice")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="eager launches only (a 256 MiB copy kernel, then each decode shape and one GEMM), "
                         "for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs; prints no JSON line")
    return ap.parse_args()


def make_weights(pkg, torch, device, K, N, seed):
    """Synthetic GPTQ tensors generated on the device (same distribution as the oracle's
    make_gptq: uniform nibbles, stored zero 7, scales uniform [1e-3, 2e-2])."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    qweight = torch.randint(-(2**31), 2**31 - 1, (K // 8, N), dtype=torch.int64, device=device, generator=g).to(torch.int32)
    G = K // GROUPSIZE
    qzeros = torch.full((G, N // 8), 0x77777777, dtype=torch.int32, device=device)
    scales = (torch.rand((G, N), device=device, generator=g) * (2e-2 - 1e-3) + 1e-3).to(torch.float16)
    return pkg.ops.make_packed(qweight, qzeros, scales, None, GROUPSIZE, 0)


def make_weights_variant(pkg, torch, device, K, N, seed, kind, zeros=None):
    """The same synthetic tensors in the AWQ layout ("awq": qweight [K, N/8], per-group zero
    points uniform 0..15 as BASELINE.json configs[4] states) or as GPTQ with a shuffled g_idx
    ("act_order": symmetric, one zero point, as configs[3] states; zeros="per_column" draws them
    uniformly instead)."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    G = K // GROUPSIZE
    scales = (torch.rand((G, N), device=device, generator=g) * (2e-2 - 1e-3) + 1e-3).to(torch.float16)
    if zeros is None:
        zeros = "per_column" if kind == "awq" else "one"
    if zeros == "per_column":
        qzeros = torch.randint(-(2**31), 2**31 - 1, (G, N // 8), dtype=torch.int64, device=device, generator=g).to(torch.int32)
    else:
        qzeros = torch.full((G, N // 8), 0x77777777, dtype=torch.int32, device=device)
    if kind == "awq":
        qweight = torch.randint(-(2**31), 2**31 - 1, (K, N // 8), dtype=torch.int64, device=device, generator=g).to(torch.int32)
        return pkg.ops.make_packed(qweight, qzeros, scales, None, GROUPSIZE, 1)
    qweight = torch.randint(-(2**31), 2**31 - 1, (K // 8, N), dtype=torch.int64, device=device, generator=g).to(torch.int32)
    g_idx = (torch.randperm(K, device=device, generator=g) // GROUPSIZE).to(torch.int32)
    return pkg.ops.make_packed(qweight, qzeros, scales, g_idx, GROUPSIZE, 0)


def time_kernel_launches(torch, fn_list, reps, min_replay_us=2500.0, max_reps=1024):
    """Average duration of one launch: `reps` back-to-back launches (rotating over fn_list)
    are captured into one HIP graph on a side stream and the replay is bracketed by HIP
    events recorded on that same stream.  A graph keeps the Python/ctypes launch cost
    (~10 us per call, more than these kernels run) out of the measurement, so the figure
    agrees with rocprofv3's per-kernel durations.  A replay itself carries a fixed cost of
    about 12 us (graphs of n empty kernels take 12 + 1.55 n us on MI355X): a graph whose replay
    is shorter than `min_replay_us` is captured again with proportionally more launches (at most
    `max_reps`), so that this cost stays below half a percent of every figure and is the same
    share of the decode kernels' figures as of the read-only probes' they are compared with."""
    side = torch.cuda.Stream()

    def capture(n):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            fn_list[0]()  # reserve workspace / warm on this stream before capture
            torch.cuda.synchronize()
            with torch.cuda.graph(graph, stream=side):
                for i in range(n):
                    fn_list[i % len(fn_list)]()
        torch.cuda.synchronize()
        return graph

    def replay_us(graph):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record(side)
        graph.replay()
        e1.record(side)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3

    graph = capture(reps)
    best = None
    tot = 0.0
    rounds = 3
    with torch.cuda.stream(side):
        graph.replay()
        torch.cuda.synchronize()
        first = replay_us(graph)
        if first < min_replay_us and reps < max_reps:
            more = min(max_reps, int(reps * min_replay_us / max(first, 1.0)) + 1)
            more = -(-more // len(fn_list)) * len(fn_list) if len(fn_list) <= max_reps else more  # whole turns over the copies
            if more > reps:
                del graph
                reps = more
                graph = capture(reps)
                graph.replay()
                torch.cuda.synchronize()
        for _ in range(rounds):
            t = replay_us(graph) * 1e-6 / reps
            tot += t
            best = t if best is None or t < best else best
    del graph
    return tot / rounds, best


def _blas_backend(torch):
    """Name of the BLAS library torch's CPU matmul uses, from its build configuration."""
    try:
        import re

        m = re.search(r"BLAS_INFO=([A-Za-z0-9_]+)", torch.__config__.show())
        if m:
            return m.group(1)
    except Exception:
        pass
    return "unknown"


def cpu_baseline(M):
    """The reference's dequantize-then-matmul path restated in PyTorch, on all host cores: the
    decode step (four projections, M rows), plus cfg1 (K = N = 4096, M = 16) and one prefill shape
    (o_proj at M = 2048) for context.  A bounded sample: a few repetitions each."""
    import torch

    from oracle import q4_oracle as o
    from oracle import q4_oracle_torch as ot

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)

    def tensors(K, N):
        qw, qz, sc, _ = o.make_gptq(K, N, GROUPSIZE, seed=1)
        return (torch.from_numpy(qw.view("int32")), torch.from_numpy(qz.view("int32")), torch.from_numpy(sc))

    def timed(K, N, rows, reps):
        qw, qz, sc = tensors(K, N)
        x = torch.from_numpy(o.make_x(rows, K, seed=1))
        td = tm = 0.0
        for _ in range(reps):
            t0 = time.perf_counter()
            w = ot.dequant_gptq(qw, qz, sc, None, GROUPSIZE)
            t1 = time.perf_counter()
            ot.linear_forward(x, w, None)
            t2 = time.perf_counter()
            td += t1 - t0
            tm += t2 - t1
            del w
        return td / reps, tm / reps

    detail = {}
    reps = 3
    step_t = 0.0
    step_bytes = 0
    for name, K, N in SHAPES:
        td, tm = timed(K, N, M, reps)
        detail[name] = {"dequant_ms": round(td * 1e3, 1), "matmul_ms": round(tm * 1e3, 1)}
        step_t += td + tm
        step_bytes += gemv_bytes(M, K, N)
    td, tm = timed(4096, 4096, 16, 2)
    detail["cfg1_4096x4096_m16"] = {"dequant_ms": round(td * 1e3, 1), "matmul_ms": round(tm * 1e3, 1)}
    td, tm = timed(4096, 4096, 2048, 2)
    detail["o_proj_m2048"] = {"dequant_ms": round(td * 1e3, 1), "matmul_ms": round(tm * 1e3, 1),
                              "TFLOPs": round(2.0 * 2048 * 4096 * 4096 / (td + tm) / 1e12, 3)}
    return {
        "value": round(step_bytes / step_t / 1e9, 4),
        "unit": "GB/s",
        "cores": cores,
        "kind": "port",
        "sample": f"{reps} decode steps (4 Llama-3-8B projections each, M={M}) of the PyTorch restatement of the "
                  f"reference path: unpack + dequantize to fp16, then x.float() @ W.float(); torch thread pool with "
                  f"{cores} threads, BLAS backend {_blas_backend(torch)}; "
                  f"plus cfg1 (M=16) and o_proj at M=2048, 2 repetitions each",
        "ms_per_step": round(step_t * 1e3, 1),
        "detail": detail,
    }


def read_floor_configs(K, N):
    """Grids of the read-only tile kernel for a [K/8, N] matrix of packed words: (workgroups,
    threads, unroll, column waves per workgroup) with the row steps dividing evenly, around the
    decode kernels' own grids (two column waves x four K waves x unsplit K is the gate_up launch:
    224 workgroups of 512 threads)."""
    steps_total = K // 32  # four packed rows per wave load
    out = []
    for wcol in (1, 2):
        if N % (64 * wcol):
            continue
        ntiles = N // (64 * wcol)
        for wk in (4, 8, 16):
            if wcol * wk > 16:
                continue
            for splits in (1, 2, 4, 7, 8, 14, 16):
                slots = wk * splits
                if steps_total % slots:
                    continue
                per = steps_total // slots
                wgs = ntiles * splits
                if wgs < 192 or wgs > 4096:
                    continue
                for unroll in (2, 4, 8):
                    if per % unroll == 0:
                        out.append((wgs, 64 * wk * wcol, unroll, wcol))
    return out


def time_read_floor(torch, pool, sink, nbytes, pattern, n_words, wgs, threads, unroll, hot, reps=24, wcol=1):
    """Average us of one read-only launch over `nbytes`; the launches of a graph walk through
    `pool` (larger than the last-level cache) unless `hot`."""
    lib = load_probe_lib()
    pieces = max(1, pool.numel() // nbytes)
    fns = []
    for r in range(1 if hot else min(pieces, reps)):
        ptr = pool.data_ptr() + r * nbytes

        def fn(ptr=ptr):
            probe_check(lib.q4_probe_read(ptr, nbytes, pattern, n_words, wgs, threads, unroll, wcol, sink.data_ptr(),
                                          torch.cuda.current_stream().cuda_stream))
        fns.append(fn)
    avg, best = time_kernel_launches(torch, fns, reps)
    return avg * 1e6, best * 1e6


def lds_probe(torch, dev):
    """ns per wave-level ds_read_b128 (16 waves per CU, all CUs) for lane -> 16-byte-unit maps.
    256 B per clock would be ~2.1 ns at the clock these launches run at."""
    lib = load_probe_lib()
    sink = torch.zeros(4, dtype=torch.uint8, device=dev)
    blocks = lambda order: [u for b in order for u in range(8 * b, 8 * b + 8)]  # residues per 8-lane block
    maps = [
        ("linear: lane l at unit l", [l for l in range(64)]),
        ("8-lane blocks at residues 0-7, 0-7, 8-15, 8-15 (free if lanes 0-7 pass with 24-31, 8-15 with 16-23)",
         [(l & 7) + 8 * ((l >> 4) & 1) + 16 * (l >> 3) for l in range(64)]),
        ("8-lane blocks at residues 0-7, 8-15, 8-15, 0-7 (free if lanes 0-15 pass together)",
         [(l & 7) + 8 * (((l >> 3) & 1) ^ ((l >> 4) & 1)) + 16 * (l >> 3) for l in range(64)]),
        ("32 rows x 2 units, rows of 9 units (prefill kernel of the GPTQ layout)", [(l & 31) * 9 + (l >> 5) for l in range(64)]),
        ("16 rows x 4 units, rows of 9 units", [(l & 15) * 9 + (l >> 4) for l in range(64)]),
        ("16 rows x 4 units, rows of 8 units, unit ^ (row >> 1) (prefill kernel of the AWQ layout)",
         [(l & 15) * 8 + ((l >> 4) ^ ((l & 15) >> 1)) for l in range(64)]),
        ("16 rows x 4 units, rows of 8 units, no swizzle", [(l & 15) * 8 + (l >> 4) for l in range(64)]),
        ("all lanes on the same four banks", [l * 16 for l in range(64)]),
    ]
    iters = 2000
    rows = []
    for name, m in maps:
        dm = torch.tensor(m, dtype=torch.int32, device=dev)
        stream = torch.cuda.current_stream().cuda_stream
        best = None
        for rep in range(4):
            probe_check(lib.q4_probe_lds(dm.data_ptr(), 10, 256, sink.data_ptr(), stream))
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            probe_check(lib.q4_probe_lds(dm.data_ptr(), iters, 256, sink.data_ptr(), stream))
            e1.record()
            e1.synchronize()
            ns = e0.elapsed_time(e1) * 1e6 / (16.0 * iters * 8)
            best = ns if best is None or ns < best else best
        rows.append({"map": name, "ns_per_wave_read": round(best, 2)})
        print(f"{best:6.2f} ns per wave read   {name}", flush=True)
    return rows


def floor_probe(torch, dev):
    """Table of read-only launches: empty grids, linear reads and the decode tile pattern at the
    four projections' sizes, HBM-rotating (1 GiB pool) and cache-hot."""
    pool = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 255)
    sink = torch.zeros(4, dtype=torch.uint8, device=dev)
    rows = []
    for wgs in (256, 1024, 4096):
        for threads in (256, 512):
            us, _ = time_read_floor(torch, pool, sink, 4096, 2, 0, wgs, threads, 1, True)
            rows.append({"what": "empty", "workgroups": wgs, "threads": threads, "us": round(us, 2)})
            print(f"empty kernel           wgs {wgs:5d} x {threads:4d}                       {us:7.2f} us", flush=True)
    summary = {}
    for name, K, N in SHAPES:
        nbytes = K * N // 2
        best = {}
        for wgs in (256, 512, 1024, 2048):
            for threads in (256, 512):
                for unroll in (2, 4, 8):
                    # the linear kernel reads whole rounds of threads x unroll vectors per workgroup
                    rnd = threads * unroll
                    if (nbytes // 16 // wgs // rnd * rnd) * 16 * wgs != nbytes:
                        continue
                    for hot in (False, True):
                        us, _ = time_read_floor(torch, pool, sink, nbytes, 0, 0, wgs, threads, unroll, hot)
                        key = "linear_hot" if hot else "linear"
                        if key not in best or us < best[key]["us"]:
                            best[key] = {"workgroups": wgs, "threads": threads, "unroll": unroll, "us": round(us, 2)}
                        rows.append({"what": key, "shape": name, "workgroups": wgs, "threads": threads, "unroll": unroll,
                                     "us": round(us, 2), "GBps": round(nbytes / us / 1e3, 1)})
        for wgs, threads, unroll, wcol in read_floor_configs(K, N):
            for hot in (False, True):
                us, _ = time_read_floor(torch, pool, sink, nbytes, 1, N, wgs, threads, unroll, hot, wcol=wcol)
                key = "tile_hot" if hot else "tile"
                if key not in best or us < best[key]["us"]:
                    best[key] = {"workgroups": wgs, "threads": threads, "unroll": unroll, "column_waves": wcol, "us": round(us, 2)}
                rows.append({"what": key, "shape": name, "workgroups": wgs, "threads": threads, "unroll": unroll,
                             "column_waves": wcol, "bytes_in_flight_per_wave": unroll * 1024, "us": round(us, 2),
                             "GBps": round(nbytes / us / 1e3, 1)})
                print(f"{name:13s} {key:9s} wgs {wgs:5d} x {threads:4d} ({wcol} column waves) unroll {unroll}  "
                      f"{nbytes / 1e6:6.1f} MB  {us:7.2f} us  {nbytes / us / 1e3:7.1f} GB/s", flush=True)
        for key, b in best.items():
            b["GBps"] = round(nbytes / b["us"] / 1e3, 1)
        summary[name] = {"bytes": nbytes, **best}
        print(f"== {name}: " + "  ".join(f"{k} {v['us']} us ({v['GBps']} GB/s, {v['workgroups']}x{v['threads']} u{v['unroll']})"
                                          for k, v in best.items()), flush=True)
    print(json.dumps({"read_floor": summary}))


# launch geometries at M = 1 on the four projections: (workgroups, threads, column waves per
# workgroup) for the probe launches that are compared with the decode kernels.  First the
# short-launch kernel's own grid (column tiles x K splits workgroups of four K waves), then, where
# it differs, the grid of the kernels that stage an activation slab per workgroup (gate_up: 224
# workgroups of two column waves x four K waves, unsplit).
DECODE_GRIDS = {"qkv_proj": [(768, 256, 1)], "o_proj": [(512, 256, 1)],
                "gate_up_proj": [(3584, 256, 1), (224, 512, 2)], "down_proj": [(896, 256, 1), (256, 512, 1)]}


def probe_trace(pkg, torch, dev, weights, xs, ys, reps=40):
    """Eager launches for a rocprofv3 --kernel-trace run: per projection an empty kernel and the
    read-only tile kernel on the decode kernel's grid (weights-sized ranges of a 1 GiB pool, so
    every launch reads from HBM), then the decode kernel itself on rotating weights.  The trace
    gives all three in the same unit (begin -> end of a dispatch)."""
    lib = load_probe_lib()
    pool = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 255)
    sink = torch.zeros(4, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    for i, (name, K, N) in enumerate(SHAPES):
        nbytes = K * N // 2
        pieces = pool.numel() // nbytes
        for wgs, threads, wcol in DECODE_GRIDS[name]:
            steps = (K // 32) // ((wgs // (N // (64 * wcol))) * (threads // 64 // wcol))
            unroll = 8 if steps % 8 == 0 else (4 if steps % 4 == 0 else (2 if steps % 2 == 0 else 1))
            for r in range(reps):
                probe_check(lib.q4_probe_read(pool.data_ptr(), 4096, 2, 0, wgs, threads, 1, 1, sink.data_ptr(), stream))
            torch.cuda.synchronize()
            for r in range(reps):
                probe_check(lib.q4_probe_read(pool.data_ptr() + (r % pieces) * nbytes, nbytes, 1, N, wgs, threads, unroll, wcol,
                                              sink.data_ptr(), stream))
            torch.cuda.synchronize()
            print(f"probe trace: {name} {K}x{N}: {reps} empty launches ({wgs} x {threads}), {reps} read-only launches of "
                  f"{nbytes} B (unroll {unroll}, {wcol} column waves)", file=sys.stderr)
        for r in range(reps):
            pkg.ops.linear(weights[r % len(weights)][i], xs[i], None, out=ys[i])
        torch.cuda.synchronize()
        print(f"probe trace: {name} {K}x{N}: {reps} decode launches", file=sys.stderr)


PHASES = ["entry", "activations staged", "first chunk consumed", "K loop done",
          "K waves combined (LDS)", "split-K combine returned", "first weight loads issued", "exit"]
PHASE_ORDER = [0, 6, 1, 2, 3, 4, 5, 7]


def phase_breakdown(pkg, torch, dev, M, copies, launches=24, configs=None):
    """Where a decode launch's time goes.  Runs the phase-stamp build of the library: every wave
    reads the 100 MHz clock at its phase boundaries (PhaseStamps, csrc/q4_gemv_kernels.cuh) and
    stores the readings when it ends.  Launches run as a HIP graph over rotating weights, like the
    timed legs.  Per stamp: the earliest / median / latest wave, in us since the first wave of the
    launch entered, averaged over the launches."""
    import numpy as np

    lib = pkg._lib.load()
    targets = [lib.q4_phase_stamps_target, lib.q4_phase_stamps_target_direct]
    for fn in targets:
        fn.restype = None
        fn.argtypes = [ctypes.c_void_p]

    def set_target(ptr):
        for fn in targets:
            fn(ptr)

    configs = configs or {}
    out = {}
    lib.q4_phase_stamps_slots.restype = ctypes.c_int
    lib.q4_phase_stamps_slots.argtypes = []
    slots = int(lib.q4_phase_stamps_slots())  # waves per launch the library stamps at most (a larger launch leaves none)
    for i, (name, K, N) in enumerate(SHAPES):
        ws = [make_weights(pkg, torch, dev, K, N, seed=17 * c + i) for c in range(copies)]
        x = torch.randn((M, K), device=dev, dtype=torch.float16)
        y = torch.empty((M, N), device=dev, dtype=torch.float16)
        stamps = torch.zeros((launches, slots, 8), dtype=torch.int64, device=dev)
        pkg.ops.reserve_workspace(dev, pkg.ops.workspace_bytes(M, K, N))
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            cfg = tuple(configs[name]) if name in configs else None
            set_target(None)
            pkg.ops.linear(ws[0], x, None, out=y, gemv_config=cfg)
            torch.cuda.synchronize()
            with torch.cuda.graph(graph, stream=side):
                for r in range(launches):
                    set_target(stamps[r].data_ptr())
                    pkg.ops.linear(ws[r % copies], x, None, out=y, gemv_config=cfg)
            set_target(None)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            stamps.zero_()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(side)
            graph.replay()
            e1.record(side)
            torch.cuda.synchronize()
            us_per_launch = e0.elapsed_time(e1) * 1e3 / launches
        t = stamps.cpu().numpy().astype(np.int64)
        rows = {ph: [] for ph in range(8)}
        spans, waves = [], 0
        for r in range(launches):
            live = t[r][t[r][:, 0] != 0]
            if live.shape[0] == 0:
                continue
            waves = live.shape[0]
            t0 = live[:, 0].min()
            spans.append((live[:, 7].max() - t0) * 0.01)
            for ph in range(8):
                v = live[:, ph]
                v = v[v != 0]
                if v.size:
                    rel = (v - t0) * 0.01  # 100 MHz counter -> us
                    rows[ph].append((rel.min(), np.median(rel), rel.max(), v.size))
        entry = {"K": K, "N": N, "waves": int(waves), "us_per_launch_with_stamps": round(us_per_launch, 2),
                 "first_entry_to_last_exit_us": round(float(np.mean(spans)), 2) if spans else None, "phases": {}}
        print(f"== {name} {K}x{N} M={M}{' config ' + str(cfg) if cfg else ''}: {waves} waves, {us_per_launch:.2f} us per launch (graph replay, stamps on), "
              f"first wave in -> last wave out {entry['first_entry_to_last_exit_us']} us", flush=True)
        for ph in PHASE_ORDER:
            if rows[ph]:
                a = np.array([r[:3] for r in rows[ph]], dtype=np.float64).mean(axis=0)
                n = int(np.mean([r[3] for r in rows[ph]]))
                entry["phases"][PHASES[ph]] = {"first_wave_us": round(a[0], 2), "median_wave_us": round(a[1], 2),
                                               "last_wave_us": round(a[2], 2), "waves": n}
                print(f"   {PHASES[ph]:42s} first {a[0]:6.2f}  median {a[1]:6.2f}  last {a[2]:6.2f}  ({n} waves)", flush=True)
        out[name] = entry
        del ws, stamps, graph
        torch.cuda.empty_cache()
    print(json.dumps({"phase_breakdown": out}))


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on one GPU; --gpus {args.gpus} is not supported "
              "(no collectives or sharding are part of the hot path)", file=sys.stderr)
        sys.exit(2)
    import torch

    pkg = importlib.import_module("text-generation-inference_amd")
    if args.phase_breakdown:
        # this process runs the measurement build of the library (same sources, -DQ4_PHASE_STAMPS)
        pkg._lib.LIB_PATH = PACKAGE_DIR / "libq4linear_stamps.so"
    pkg._lib.load()
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    M = args.m
    step_weight_bytes = sum(gemv_bytes(0, K, N) for _, K, N in SHAPES)
    step_bytes = sum(gemv_bytes(M, K, N) for _, K, N in SHAPES)
    copies = args.copies or max(2, -(-512 * 1024 * 1024 // step_weight_bytes) + 1)

    if args.phase_breakdown:
        phase_breakdown(pkg, torch, dev, M, copies, configs=json.loads(args.phase_configs) if args.phase_configs else None)
        return
    weights = [[make_weights(pkg, torch, dev, K, N, seed=17 * c + i) for i, (_, K, N) in enumerate(SHAPES)]
               for c in range(copies)]
    xs = [torch.randn((M, K), device=dev, dtype=torch.float16) for _, K, N in SHAPES]
    ys = [torch.empty((M, N), device=dev, dtype=torch.float16) for _, K, N in SHAPES]
    for _, K, N in SHAPES:
        pkg.ops.reserve_workspace(dev, pkg.ops.workspace_bytes(M, K, N))

    # Per-projection legs rotate over enough copies of that one shape to exceed the 256 MB
    # last-level cache as well (the whole-step legs get there with `copies` of all four)
    COLD_BYTES = 512 * 1024 * 1024
    probe_mode = (args.lds_probe or args.awq_probe or args.act_probe or args.floor_probe)
    shape_ws = []
    for i, (_, K, N) in enumerate(SHAPES):
        n = copies if probe_mode else max(copies, -(-COLD_BYTES // gemv_bytes(0, K, N)))
        shape_ws.append([weights[c][i] for c in range(copies)] +
                        [make_weights(pkg, torch, dev, K, N, seed=1000 + 17 * c + i) for c in range(copies, n)])

    # Load-time step, as the layers do it in their Warmup hook: measured decode plans for the row
    # counts this run times
    tuning = None
    if not args.no_autotune and not probe_mode:
        t0 = time.perf_counter()
        rows = sorted({M, 1, 2, 4, 8, 16} if M <= 16 else {1, 2, 4, 8, 16})
        report = pkg.ops.autotune([w for ws in shape_ws for w in ws], rows=rows)
        tuning = {"seconds": round(time.perf_counter() - t0, 2),
                  "plans": {f"{K}x{N}_m{Mr}": {"config": list(cfg) if cfg else None, "library_choice_us": base, "chosen_us": best}
                            for (K, N, _, Mr), (cfg, base, best) in report.items()}}

    def step(c):
        for i in range(len(SHAPES)):
            pkg.ops.linear(weights[c % copies][i], xs[i], None, out=ys[i])

    if args.lds_probe:
        print(json.dumps({"lds_probe": lds_probe(torch, dev)}))
        return
    if args.awq_probe:
        K, N, Mg = 4096, 14336, args.gemm_m
        wa = make_weights_variant(pkg, torch, dev, K, N, 5, "awq")
        wg = make_weights(pkg, torch, dev, K, N, 6)
        xg = torch.randn((Mg, K), device=dev, dtype=torch.float16)
        yg = torch.empty((Mg, N), device=dev, dtype=torch.float16)
        for _ in range(6):
            pkg.ops.linear(wa, xg, None, out=yg)
            pkg.ops.linear(wg, xg, None, out=yg)
        torch.cuda.synchronize()
        print("awq probe done: 6 launches each of the AWQ-layout and the GPTQ-layout prefill kernel, %d x %d, M=%d"
              % (K, N, Mg), file=sys.stderr)
        return
    if args.act_probe:
        Kd, Nd = 28672, 8192
        wd = [make_weights_variant(pkg, torch, dev, Kd, Nd, 5 + c, "act_order") for c in range(3)]
        for Md in (1, 16):
            xd = torch.randn((Md, Kd), device=dev, dtype=torch.float16)
            yd = torch.empty((Md, Nd), device=dev, dtype=torch.float16)
            for _ in range(4):
                for w in wd:
                    pkg.ops.linear(w, xd, None, out=yd)
        torch.cuda.synchronize()
        del wd
        Kp, Np, Mg = 8192, 10240, args.gemm_m
        wp = [make_weights_variant(pkg, torch, dev, Kp, Np, 9 + c, "act_order") for c in range(2)]
        xg = torch.randn((Mg, Kp), device=dev, dtype=torch.float16)
        yg = torch.empty((Mg, Np), device=dev, dtype=torch.float16)
        for _ in range(3):
            for w in wp:
                pkg.ops.linear(w, xg, None, out=yg)
        torch.cuda.synchronize()
        print("act probe done: 12 decode launches each at M=1 and M=16 on %d x %d, 6 prefill launches at M=%d on %d x %d"
              % (Kd, Nd, Mg, Kp, Np), file=sys.stderr)
        return
    if args.floor_probe:
        floor_probe(torch, dev)
        return
    if args.probe_trace:
        probe_trace(pkg, torch, dev, weights, xs, ys)
        return

    if args.traffic_probe:
        # calibration: a plain device-to-device copy of known size (reads and writes 256 MiB)
        src = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        for c in range(3 * copies):
            step(c)
        torch.cuda.synchronize()
        Mg = args.gemm_m
        for i, (name, K, N) in enumerate(SHAPES):
            if args.no_gemm:
                break
            xg = torch.randn((Mg, K), device=dev, dtype=torch.float16)
            yg = torch.empty((Mg, N), device=dev, dtype=torch.float16)
            for c in range(copies):
                pkg.ops.linear(weights[c][i], xg, None, out=yg)
            torch.cuda.synchronize()
            del xg, yg
        print("traffic probe done: copy 268435456 B x5, decode steps (M=%d) x%d%s"
              % (M, 3 * copies, "" if args.no_gemm else ", gemm M=%d x%d per shape" % (Mg, copies)), file=sys.stderr)
        return

    # ---- whole-job throughput: W warmup steps, then exactly K steps in one HIP graph
    for c in range(args.warmup):
        step(c)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        for _, K, N in SHAPES:
            pkg.ops.reserve_workspace(dev, pkg.ops.workspace_bytes(M, K, N))
        step(0)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            for c in range(args.steps):
                step(c)
    torch.cuda.synchronize()
    graph.replay()  # untimed replay: instantiation and first-launch costs
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    graph.replay()
    e1.record()
    torch.cuda.synchronize()
    total_s = e0.elapsed_time(e1) * 1e-3
    ms_per_step = total_s / args.steps * 1e3
    value = step_bytes * args.steps / total_s / 1e9

    # ---- per-kernel durations of the decode kernel (graph of back-to-back launches)
    per_shape = {}
    all_durs = []
    all_bytes = 0
    reps = max(200, copies * 8)
    for i, (name, K, N) in enumerate(SHAPES):
        fns = [(lambda w=w, i=i: pkg.ops.linear(w, xs[i], None, out=ys[i])) for w in shape_ws[i]]
        avg, best = time_kernel_launches(torch, fns, max(reps, 2 * len(fns)))
        b = gemv_bytes(M, K, N)
        hot_avg, _ = time_kernel_launches(torch, fns[:1], reps)
        per_shape[name] = {
            "K": K, "N": N, "bytes": b,
            "us_avg": round(avg * 1e6, 2), "us_best_round": round(best * 1e6, 2),
            "GBps": round(b / avg / 1e9, 1), "frac_of_hbm_peak": round(b / avg / 1e9 / HBM_PEAK_GBS, 4),
            "cache_hot_us": round(hot_avg * 1e6, 2), "cache_hot_GBps": round(b / hot_avg / 1e9, 1),
            "path": pkg.ops.select_path(weights[0][i], M),
            "tuned_config": pkg.ops.PackedWeight.plan(weights[0][i], M, 0)[2],
            "weight_copies_rotated": len(shape_ws[i]),
        }
        all_durs.append(avg)
        all_bytes += b
    # read-only launches over the same weight bytes (decode tile pattern, rotating through
    # HBM like the weights): the time such a launch takes when it computes nothing
    if M == 1:
        pool = torch.empty(1 << 29, dtype=torch.uint8, device=dev).random_(0, 255)
        sink = torch.zeros(4, dtype=torch.uint8, device=dev)
        for name, K, N in SHAPES:
            floor = min(time_read_floor(torch, pool, sink, K * N // 2, 1, N, wgs, threads, unroll, False, wcol=wcol)[0]
                        for wgs, threads, unroll, wcol in read_floor_configs(K, N) if unroll == 4)
            per_shape[name]["read_only_floor_us"] = round(floor, 2)
        del pool
    # the same call outside a graph: Python + ctypes + launch per call (o_proj, M rows)
    for _ in range(50):
        pkg.ops.linear(weights[0][1], xs[1], None, out=ys[1])
    torch.cuda.synchronize()
    n_eager = 2000
    t0 = time.perf_counter()
    for c in range(n_eager):
        pkg.ops.linear(weights[c % copies][1], xs[1], None, out=ys[1])
    torch.cuda.synchronize()
    per_shape["o_proj"]["eager_us_per_call"] = round((time.perf_counter() - t0) / n_eager * 1e6, 2)
    achieved = all_bytes / sum(all_durs) / 1e9
    roofline = {
        "bound": "hbm",
        "kernel": "q4::gemv_gptq_direct_kernel",
        "achieved": round(achieved, 1),
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBS, 4),
        # HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on this
        # workload (mean over the four projections, calibrated with a 256 MiB copy kernel);
        # only valid for the default M=1 workload, null otherwise
        "traffic": measured_traffic("decode_m1") if M == 1 else None,
        "traffic_measured_at_commit": measured_traffic("decode_m1", "measured_at_commit") if M == 1 else None,
        "bytes_per_launch": all_bytes // len(SHAPES),
        "us_per_launch": round(sum(all_durs) / len(SHAPES) * 1e6, 2),
    }

    out = {
        "metric": "int4 GEMV HBM GB/s (M=1) + GEMM TFLOP/s (M=2048), Llama-3-8B shapes, % roofline",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": f"GPTQ int4 decode GEMV M={M}, Llama-3-8B projections (qkv/o/gate_up/down), fp16, "
                        f"groupsize 128, sym; one step = the four projections once",
            "weight_copies_rotated": copies,
            "per_projection_legs": "rotate over enough copies of the one shape to exceed 512 MB",
            "bytes_per_step": step_bytes,
            "timing": "one HIP graph of all timed steps, bracketed by HIP events + synchronize",
        },
        "roofline": roofline,
        "per_shape": per_shape,
        "load_time_tuning": tuning,
    }

    # ---- prefill GEMM leg (M=2048) when the kernel is available
    if not args.no_gemm:
        gm = {}
        Mg = args.gemm_m
        tot_f = 0.0
        tot_t = 0.0
        for i, (name, K, N) in enumerate(SHAPES):
            if pkg.ops.select_path(weights[0][i], Mg) != "gemm":
                continue
            xg = torch.randn((Mg, K), device=dev, dtype=torch.float16)
            yg = torch.empty((Mg, N), device=dev, dtype=torch.float16)
            fns = [(lambda c=c, i=i: pkg.ops.linear(weights[c][i], xg, None, out=yg)) for c in range(copies)]
            avg, _ = time_kernel_launches(torch, fns, 20)
            fl = 2.0 * Mg * N * K
            gm[name] = {"us_avg": round(avg * 1e6, 1), "TFLOPs": round(fl / avg / 1e12, 1),
                        "frac_of_mfma_peak": round(fl / avg / 1e12 / MFMA_PEAK_TFLOPS, 4)}
            tot_f += fl
            tot_t += avg
            # the same kernel on bf16 activations (bf16 weights rounded once from the fp32 product)
            xb = torch.randn((Mg, K), device=dev, dtype=torch.bfloat16)
            yb = torch.empty((Mg, N), device=dev, dtype=torch.bfloat16)
            bfns = [(lambda c=c, i=i: pkg.ops.linear(weights[c][i], xb, None, out=yb)) for c in range(copies)]
            bavg, _ = time_kernel_launches(torch, bfns, 20)
            gm[name]["bf16_TFLOPs"] = round(fl / bavg / 1e12, 1)
            del xb, yb
            if not args.no_dense_ref:
                # context, not the product: the vendor library's dense fp16 GEMM on the same
                # shape and box (weights already dequantized, 4x the weight bytes), timed the same way
                dense = [torch.randn((K, N), device=dev, dtype=torch.float16) * 0.02 for _ in range(2)]
                dfns = [(lambda c=c: torch.matmul(xg, dense[c], out=yg)) for c in range(2)]
                davg, _ = time_kernel_launches(torch, dfns, 20)
                gm[name]["dense_fp16_matmul_TFLOPs"] = round(fl / davg / 1e12, 1)
                del dense
            del xg, yg
        # gated MLP first half (gate_up projection + act(gate) * up): one fused launch against
        # the GEMM followed by the elementwise kernel, fp16
        gated = None
        if "gate_up_proj" in gm:
            name, K, N = SHAPES[2]
            xg = torch.randn((Mg, K), device=dev, dtype=torch.float16)
            yh = torch.empty((Mg, N // 2), device=dev, dtype=torch.float16)
            gated = {"shape": f"{K}x{N}", "M": Mg}
            for key, fused in (("fused_us", True), ("gemm_plus_act_mul_us", False)):
                try:
                    fns = [(lambda c=c: pkg.ops.linear_gate_up(weights[c][2], xg, "silu", None, out=yh, fused=fused))
                           for c in range(copies)]
                    avg, _ = time_kernel_launches(torch, fns, 20)
                    gated[key] = round(avg * 1e6, 1)
                except pkg._lib.Q4Error:
                    gated[key] = None
            del xg, yh
        power = None
        if gm and not args.no_dense_ref:
            # What bounds the GEMM: the same kernel (and the vendor library's dense GEMM) on all-zero
            # operands, which toggle no data lines and draw far less power (gate_up, fp16)
            name, K, N = SHAPES[2]
            wz = [make_weights(pkg, torch, dev, K, N, seed=900 + c) for c in range(2)]
            for w in wz:
                w.qweight.zero_()
            xz = torch.zeros((Mg, K), device=dev, dtype=torch.float16)
            yz = torch.empty((Mg, N), device=dev, dtype=torch.float16)
            zavg, _ = time_kernel_launches(torch, [(lambda c=c: pkg.ops.linear(wz[c], xz, None, out=yz)) for c in range(2)], 20)
            dz = [torch.zeros((K, N), device=dev, dtype=torch.float16) for _ in range(2)]
            dzavg, _ = time_kernel_launches(torch, [(lambda c=c: torch.matmul(xz, dz[c], out=yz)) for c in range(2)], 20)
            # in between: real activations, weights whose dequantized values are small integers
            # (all scales 1.0: few mantissa bits switch in the B operand)
            wi = [make_weights(pkg, torch, dev, K, N, seed=950 + c) for c in range(2)]
            for w in wi:
                w.scales.fill_(1.0)
            xr = torch.randn((Mg, K), device=dev, dtype=torch.float16)
            iavg, _ = time_kernel_launches(torch, [(lambda c=c: pkg.ops.linear(wi[c], xr, None, out=yz)) for c in range(2)], 20)
            del wi, xr
            fl = 2.0 * Mg * N * K
            power = {"shape": name, "zero_operands_TFLOPs": round(fl / zavg / 1e12, 1),
                     "unit_scale_weights_random_activations_TFLOPs": round(fl / iavg / 1e12, 1),
                     "random_operands_TFLOPs": gm[name]["TFLOPs"],
                     "dense_fp16_matmul_zero_operands_TFLOPs": round(fl / dzavg / 1e12, 1),
                     "dense_fp16_matmul_random_operands_TFLOPs": gm[name].get("dense_fp16_matmul_TFLOPs")}
            del wz, xz, yz, dz
        if gm:
            out["gemm"] = {
                "M": Mg, "per_shape": gm,
                "roofline": {"bound": "mfma", "kernel": "q4::gemm_gptq_kernel / q4::gemm_gptq_wide_kernel (qkv)", "achieved": round(tot_f / tot_t / 1e12, 1),
                             "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                             "frac": round(tot_f / tot_t / 1e12 / MFMA_PEAK_TFLOPS, 4),
                             "traffic": measured_traffic(f"gemm_m{Mg}"),
                             "traffic_measured_at_commit": measured_traffic(f"gemm_m{Mg}", "measured_at_commit")},
                "power_probe": power,
                "gated_mlp": gated,
            }

    # ---- batched decode: the same four projections with more activation rows (the serving
    # batch), and the other two weight formats; us per step = sum over the four projections
    if not args.no_batch:
        batch = {}

        def step_us(wlist, Mb, per_shape=None):
            tot = 0.0
            paths = []
            for i, (name, K, N) in enumerate(SHAPES):
                xb = torch.randn((Mb, K), device=dev, dtype=torch.float16)
                yb = torch.empty((Mb, N), device=dev, dtype=torch.float16)
                rot = per_shape[i] if per_shape is not None else [row[i] for row in wlist]
                fns = [(lambda w=w: pkg.ops.linear(w, xb, None, out=yb)) for w in rot]
                avg, _ = time_kernel_launches(torch, fns, max(48, 2 * len(fns)))
                tot += avg
                paths.append(pkg.ops.select_path(wlist[0][i], Mb))
                del xb, yb
            return {"us_per_step": round(tot * 1e6, 1), "weight_GBps": round(step_weight_bytes / tot / 1e9, 1),
                    "paths": "/".join(paths)}

        for Mb in (4, 16, 18, 32, 64):
            batch[f"gptq_m{Mb}"] = step_us(weights, Mb, per_shape=shape_ws)

        # ---- BASELINE.json configs[1] beyond one row, projection by projection, and configs[0]
        # (K = N = 4096, M = 16: the o_proj shape at 16 rows)
        rows_leg = {}
        for Mb in (2, 4, 8, 16):
            entry = {}
            tot_t = 0.0
            tot_b = 0
            for i, (name, K, N) in enumerate(SHAPES):
                xb = torch.randn((Mb, K), device=dev, dtype=torch.float16)
                yb = torch.empty((Mb, N), device=dev, dtype=torch.float16)
                fns = [(lambda w=w: pkg.ops.linear(w, xb, None, out=yb)) for w in shape_ws[i]]
                avg, _ = time_kernel_launches(torch, fns, max(96, 2 * len(fns)))
                b = gemv_bytes(Mb, K, N)
                entry[name] = {"us": round(avg * 1e6, 2), "GBps": round(b / avg / 1e9, 1),
                               "frac_of_hbm_peak": round(b / avg / 1e9 / HBM_PEAK_GBS, 4)}
                tot_t += avg
                tot_b += b
                del xb, yb
            entry["all_four"] = {"us": round(tot_t * 1e6, 2), "GBps": round(tot_b / tot_t / 1e9, 1),
                                 "frac_of_hbm_peak": round(tot_b / tot_t / 1e9 / HBM_PEAK_GBS, 4)}
            rows_leg[f"m{Mb}"] = entry
        out["cfg2_decode_rows"] = rows_leg
        out["cfg1_4096x4096_m16"] = dict(rows_leg["m16"]["o_proj"], path=pkg.ops.select_path(weights[0][1], 16))
        # awq / act_order: the kernels that read the checkpoint layout (what the layers run);
        # *_converted / *_repacked: the opt-in load-time conversions (AWQ -> GPTQ layout, rows
        # into group order with x read through the permutation)
        for kind in ("awq", "act_order", "act_order_repacked"):
            wl = [[make_weights_variant(pkg, torch, dev, K, N, 31 * c + i, "awq" if kind == "awq" else "act_order")
                   for i, (_, K, N) in enumerate(SHAPES)] for c in range(min(copies, 3))]
            if kind == "act_order_repacked":
                wl = [[pkg.ops.make_sequential(w) for w in row] for row in wl]
                torch.cuda.empty_cache()
            for Mb in (1, 16):
                batch[f"{kind}_m{Mb}"] = step_us(wl, Mb)
            del wl
            torch.cuda.empty_cache()
        out["batched_decode"] = batch

        # ---- BASELINE.json configs[2]: bf16 prefill away from the headline M
        cfg3 = {}
        for Mb in (512, 4096):
            tot_f = 0.0
            tot_t = 0.0
            entry = {}
            for i, (name, K, N) in enumerate(SHAPES):
                xb = torch.randn((Mb, K), device=dev, dtype=torch.bfloat16)
                yb = torch.empty((Mb, N), device=dev, dtype=torch.bfloat16)
                fns = [(lambda c=c, i=i: pkg.ops.linear(weights[c][i], xb, None, out=yb)) for c in range(copies)]
                avg, _ = time_kernel_launches(torch, fns, 12)
                fl = 2.0 * Mb * N * K
                entry[name] = {"us": round(avg * 1e6, 1), "TFLOPs": round(fl / avg / 1e12, 1)}
                tot_f += fl
                tot_t += avg
                del xb, yb
            entry["TFLOPs_aggregate"] = round(tot_f / tot_t / 1e12, 1)
            cfg3[f"m{Mb}"] = entry
        out["cfg3_bf16_prefill"] = cfg3

        # ---- BASELINE.json configs[3] and [4] at their own shapes
        def shape_us(make, K, N, Mb, ncopies):
            ws_ = [make(c) for c in range(ncopies)]
            xb = torch.randn((Mb, K), device=dev, dtype=torch.float16)
            yb = torch.empty((Mb, N), device=dev, dtype=torch.float16)
            fns = [(lambda c=c: pkg.ops.linear(ws_[c], xb, None, out=yb)) for c in range(ncopies)]
            avg, _ = time_kernel_launches(torch, fns, 48 if Mb <= 64 else 12)
            path = pkg.ops.select_path(ws_[0], Mb)
            del ws_, xb, yb
            torch.cuda.empty_cache()
            return avg, path

        cfg4 = {}
        for K, N in ((8192, 10240), (28672, 8192)):
            nc = max(2, -(-600 * 1024 * 1024 // (K * N // 2)))
            for Mb in (1, 16, 1024):
                entry = {}
                # symmetric weights (one zero point: what configs[3] states) and, for the kernels that
                # look zero points up per weight, the same with a zero point per group and column
                variants = [("g_idx_kernels", False, "one"), ("g_idx_kernels_per_column_zeros", False, "per_column"),
                            ("rows_in_group_order", True, "one")]
                for label, seq, zeros in variants:
                    def make(c, seq=seq, zeros=zeros):
                        w = make_weights_variant(pkg, torch, dev, K, N, 71 * c + Mb, "act_order", zeros=zeros)
                        return pkg.ops.make_sequential(w) if seq else w
                    avg, path = shape_us(make, K, N, Mb, nc)
                    entry[label] = {"us": round(avg * 1e6, 1), "path": path}
                    if Mb <= 16:
                        entry[label]["GBps"] = round(gemv_bytes(Mb, K, N, g_idx=True) / avg / 1e9, 1)
                    else:
                        entry[label]["TFLOPs"] = round(2.0 * Mb * N * K / avg / 1e12, 1)
                cfg4[f"{K}x{N}_m{Mb}"] = entry
        out["cfg4_act_order_llama70b"] = cfg4
        cfg5 = {}
        for K, N in ((4096, 14336), (14336, 4096)):
            nc = max(2, -(-600 * 1024 * 1024 // (K * N // 2)))
            conv = importlib.import_module(f"{pkg.__name__}.layers.awq.conversion_utils")
            for Mb in (1, 16, 256, 2048):
                entry = {}
                for label, convert in (("awq_layout_kernels", False), ("converted_to_gptq_layout", True)):
                    def make(c, convert=convert):
                        w = make_weights_variant(pkg, torch, dev, K, N, 53 * c + Mb, "awq")
                        if not convert:
                            return w
                        gq, gz = conv.fast_awq_to_gptq(w.qweight, w.qzeros)
                        return pkg.ops.make_packed(gq.contiguous(), gz.contiguous(), w.scales, None, GROUPSIZE, 0)
                    avg, path = shape_us(make, K, N, Mb, nc)
                    e = {"us": round(avg * 1e6, 1), "path": path}
                    if Mb <= 16:
                        e["GBps"] = round(gemv_bytes(Mb, K, N) / avg / 1e9, 1)
                    else:
                        e["TFLOPs"] = round(2.0 * Mb * N * K / avg / 1e12, 1)
                    entry[label] = e
                cfg5[f"{K}x{N}_m{Mb}"] = entry
        out["cfg5_awq_mistral7b"] = cfg5

    # ---- mixture-of-experts block (Mixtral-8x7B shapes: 8 experts, top-2, 4096 -> 2 x 14336 -> 4096):
    # routing, both grouped projections, activation and weighted sum, per block call
    if not args.no_moe:
        del weights
        torch.cuda.empty_cache()
        E, topk, H, I = 8, 2, 4096, 14336
        gen = torch.Generator(device=dev).manual_seed(7)

        def experts(K, N):
            qw = torch.randint(-2**31, 2**31 - 1, (E, K // 8, N), dtype=torch.int32, device=dev, generator=gen)
            qz = torch.full((E, K // GROUPSIZE, N // 8), 0x77777777, dtype=torch.int32, device=dev)
            sc = (torch.rand((E, K // GROUPSIZE, N), device=dev, generator=gen) * 0.019 + 0.001).half()
            return pkg.ops.make_packed_moe(qw, qz, sc, GROUPSIZE)

        gate_up, down = experts(H, 2 * I), experts(I, H)
        moe = {}
        for T in (1, 16, 1024):
            xm = torch.randn((T, H), device=dev, dtype=torch.float16)
            logits = torch.randn((T, E), device=dev, dtype=torch.float32, generator=gen)
            active = int(torch.unique(torch.topk(logits, topk, dim=1).indices).numel())
            fn = lambda: pkg.ops.moe_forward(gate_up, down, xm, logits, topk, True, "silu")
            avg, _ = time_kernel_launches(torch, [fn], 10)
            wbytes = active * 3 * H * I / 2
            fl = 2.0 * T * topk * 3 * H * I
            moe[f"tokens_{T}"] = {"us_avg": round(avg * 1e6, 1), "experts_active": active,
                                  "weight_GBps": round(wbytes / avg / 1e9, 1), "TFLOPs": round(fl / avg / 1e12, 1)}
        out["moe_block"] = {"experts": E, "topk": topk, "hidden": H, "intermediate": I, "per_tokens": moe}
        # the same block with act-order experts (the reference's Mixtral test checkpoint is one):
        # rows put into group order when the layer is built, activations gathered per sorted row for
        # the first projection
        del gate_up, down
        torch.cuda.empty_cache()

        def act_order_experts(K, N):
            w = experts(K, N)
            g_idx = torch.stack([(torch.randperm(K, device=dev, generator=gen) // GROUPSIZE).to(torch.int32)
                                 for _ in range(E)])
            w = pkg.ops.make_packed_moe(w.qweight, w.qzeros, w.scales, GROUPSIZE, g_idx)
            return pkg.ops.make_sequential_moe(w)

        gate_up, down = act_order_experts(H, 2 * I), act_order_experts(I, H)
        # as the layer does: the down projections' input order goes into the gate_up columns
        gate_up, down = pkg.ops.fold_moe_down_permutation(gate_up, down)
        torch.cuda.empty_cache()
        moe_act = {}
        for T in (1, 16, 1024):
            xm = torch.randn((T, H), device=dev, dtype=torch.float16)
            logits = torch.randn((T, E), device=dev, dtype=torch.float32, generator=gen)
            fn = lambda: pkg.ops.moe_forward(gate_up, down, xm, logits, topk, True, "silu")
            avg, _ = time_kernel_launches(torch, [fn], 10)
            moe_act[f"tokens_{T}"] = {"us_avg": round(avg * 1e6, 1)}
        out["moe_block"]["act_order_experts"] = moe_act

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(M)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
