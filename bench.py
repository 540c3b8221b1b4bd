#!/usr/bin/env python3
"""Benchmark of the quantized linear-layer hot path on one MI355X.

One JSON line. The headline is the decode multiply the metric is quoted on:
Q4_K weights, M = 1, K = 4096, N = 14336 (Llama-3-8B FFN-up shape). A step is
one dispatch of matvec_q4_k through the command stream over one copy of the
weights; steps rotate over enough distinct copies to exceed L2 plus the
256 MB Infinity Cache, so the rate is HBM's. Inputs are resident in device
memory before the timed region, which is K back-to-back dispatches in one
submit bracketed by blocking submits on both sides.

  value      algorithmic bytes per step x steps / wall time of the timed region
  roofline   algorithmic bytes per launch / mean launch time from HIP events
             recorded on the host's stream around the same K launches
  cpu_baseline  the CPU oracle (a C restatement of the reference's src/ref
             multiply) on the same weights, all physical cores, bounded sample

The other shapes of the path (Q8_0 decode, fused gate/up at M = 1, 4, 8, the
Q8_0 prefill multiply on bf16 MFMA, the bf16 lm_head) are reported under
"also" with their own roofline fractions.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published
MFMA_INT8_PEAK_TOPS = 5000.0    # MI355X dense int8, published
ROTATE_BYTES = 640 << 20    # distinct weight bytes a rotation must exceed (L2 + Infinity Cache, with margin)
# HBM bytes one launch of the headline kernel moves, from rocprofv3 FETCH_SIZE and
# WRITE_SIZE counter runs scaled by a plain copy of known size (profiles/matvec_quant_kernel_q4k_c2.txt).
C2_TRAFFIC_BYTES = 33_395_507


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--only", default="", help="comma-separated subset of: c1,c3,c4,c4_int8,long,c5,formats,down,replay,floor for the 'also' section; 'none' skips it")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-replay", action="store_true",
                    help="launch every dispatch of a repeated submit instead of replaying it from a HIP graph (for runs under a kernel tracer, "
                         "which has crashed on replayed graphs of several hundred kernel nodes)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="first run 4 plain elementwise copies (256 MiB read + 256 MiB written each) so a counter run has a kernel of known traffic to scale by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path is built and measured on one GPU; --gpus above 1 is not supported "
              "(more GPUs would each take a share of the output rows)", file=sys.stderr)
        return 2

    if args.calibrate_copy:
        import torch

        a = torch.ones(64 << 20, dtype=torch.float32, device="cuda:0")
        o = torch.empty_like(a)
        for _ in range(4):
            torch.add(a, 1.0, out=o)  # one elementwise kernel: reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del a, o

    only_early = [w for w in args.only.split(",") if w]
    vendor_c4 = vendor_c4_context() if ("none" not in only_early and (not only_early or "c4" in only_early)) else None

    from zllm_amd import Device, Host, cmd, synth
    from zllm_amd import kernels as K
    from zllm_amd.kernels import Kernel, TensorType, params as P

    dev = Device.open(0, Device.NO_REPLAY if args.no_replay else 0)
    host = Host(dev)
    rec = cmd.Recorder()
    kset = K.Set.create(rec)
    token = [0]

    def flush():
        token[0] += 1
        rec.submit(token[0])
        done = []
        host.execute(rec.batch(), done)
        rec.clear()
        return done

    flush()
    storage = cmd.Usage.storage | cmd.Usage.copy_dst | cmd.Usage.copy_src

    def upload(arr) -> K.Arg:
        arr = np.ascontiguousarray(arr)
        raw = arr.reshape(-1).view(np.uint8)
        size = (raw.size + 15) & ~15
        buf = rec.create_buffer(size, storage)
        rec.write_buffer(buf, 0, raw if raw.size % 4 == 0 else np.concatenate([raw, np.zeros(size - raw.size, np.uint8)]))
        flush()
        return K.Arg(buf, size)

    def output(n_bytes: int) -> K.Arg:
        buf = rec.create_buffer(n_bytes, storage)
        return K.Arg(buf, n_bytes)

    def read(arg: K.Arg, dtype=np.float32) -> np.ndarray:
        dst = np.zeros(arg.size, dtype=np.uint8)
        rec.read_buffer(0xFFFF0000, arg.buffer, 0, dst)
        flush()
        return dst.view(dtype)

    def timed(launches, steps: int, warmup: int, per_step: int = 1):
        """Runs `warmup` then `steps` steps cycling over `launches` (each records
        `per_step` dispatches); returns (wall seconds, GPU seconds from the
        host's stream events)."""
        for n, is_timed in ((warmup, False), (steps, True)):
            if n == 0:
                continue
            for i in range(n):
                launches[i % len(launches)].record(rec, K.Extent(rows=launches[i % len(launches)].rows))
            token[0] += 1
            rec.submit(token[0])
            words = rec.batch()
            done = []
            t0 = time.perf_counter()
            host.execute(words, done)
            wall = time.perf_counter() - t0
            rec.clear()
            ns, count = host.last_submit()
            assert count == n * per_step
        return wall, ns * 1e-9

    def protocol(launches, per_step: int = 1):
        """The tuner's timing protocol (src/tune/tune.zig:8-11,24-27) whatever --steps says:
        batches of at least 200 back-to-back steps in one blocking submit (a whole number of
        rotations over `launches`), 3 warm-up batches, then 7 timed ones; returns the median
        batch as (wall seconds, GPU seconds from the host's stream events, steps in a batch).
        Identical batches are replayed from a HIP graph from their second submit on, as the
        host does for any repeated submit."""
        n = -(-200 // len(launches)) * len(launches)
        walls, gpus = [], []
        for rep in range(3 + 7):
            for i in range(n):
                launches[i % len(launches)].record(rec, K.Extent(rows=launches[i % len(launches)].rows))
            token[0] += 1
            rec.submit(token[0])
            words = rec.batch()
            t0 = time.perf_counter()
            host.execute(words, [])
            wall = time.perf_counter() - t0
            rec.clear()
            ns, count = host.last_submit()
            assert count == n * per_step
            if rep >= 3:
                walls.append(wall)
                gpus.append(ns * 1e-9)
        return float(np.median(walls)), float(np.median(gpus)), n

    class L:
        """A prebuilt launch and the token rows its grid resolves with."""

        def __init__(self, launch, rows):
            self.launch, self.rows = launch, rows

        def record(self, r, e):
            self.launch.record(r, e)

    class Chain:
        """Several prebuilt launches recorded as one step."""

        def __init__(self, launches, rows):
            self.launches, self.rows = launches, rows

        def record(self, r, e):
            for l in self.launches:
                l.record(r, e)

    b = K.Builder(rec, kset)

    def rotation(w_bytes: int) -> int:
        return max(2, -(-ROTATE_BYTES // w_bytes))

    def matvec_workload(t: TensorType, raw_rows: np.ndarray, n_out: int, k: int, m: int, pair: bool, x: np.ndarray, variant=None, norm_w=None, eps=1e-6):
        """Uploads a rotation of weight copies and builds one launch per copy."""
        kernel = K.weight_kernel("matvec", t)
        rb = K.row_bytes(t, k)
        w_rows = 2 * n_out if pair else n_out
        copies = rotation(w_rows * rb)
        src = upload(raw_rows)
        xa = upload(x)
        out = output(4 * m * n_out)
        launches = []
        first = None
        for _ in range(copies):
            if K.needs_layout(t):
                wa = output(w_rows * rb)
                K.Launcher(rec, kset).layout(t, src, wa, w_rows, k)
            else:
                buf = rec.create_buffer(src.size, storage)
                rec.copy_buffer(src.buffer, 0, buf, 0, src.size)
                wa = K.Arg(buf, src.size)
            first = first or wa
            v = variant or K.MatvecVariant()
            p = P.MatvecBf16(n=n_out, k=k, col0=0, out_stride=n_out, eps=eps if norm_w is not None else 0.0, norm=norm_w is not None, silu_pair=pair, half=n_out if pair else 0)
            na = upload(norm_w) if norm_w is not None else wa
            if K.is_half(t):
                launches.append(L(b.add(kernel, p, [xa, wa, out, na], K.Grid.rows_y(K.div_ceil(n_out, K.matvec_rows))), m))
            else:
                launches.append(L(b.add_matvec(kernel, v, p, [xa, wa, out, na], K.Grid.rows_y(K.div_ceil(n_out, v.group_rows()))), m))
        b.finish()
        flush()
        return launches, out

    def hbm_entry(name, bytes_per_step, wall, gpu_s, steps, extra=None):
        e = {
            "workload": name,
            "bytes_per_step": bytes_per_step,
            "us_per_step_wall": round(wall / steps * 1e6, 3),
            "us_per_launch_gpu": round(gpu_s / steps * 1e6, 3),
            "GBps_wall": round(bytes_per_step * steps / wall / 1e9, 1),
            "GBps_gpu": round(bytes_per_step * steps / gpu_s / 1e9, 1),
            "hbm_frac": round(bytes_per_step * steps / gpu_s / 1e9 / HBM_PEAK_GBPS, 4),
        }
        e.update(extra or {})
        return e

    def check_matvec(got, want_f64, w_rows_f32, x):
        """(max |err| / (||row|| ||x||), max |err| / max |want|)."""
        got = got.astype(np.float64)
        wn = np.linalg.norm(w_rows_f32.astype(np.float64), axis=1)
        xn = np.linalg.norm(x.astype(np.float64).reshape(got.shape[0], -1), axis=1)
        err = np.abs(got - want_f64)
        return float(np.max(err / np.maximum(xn[:, None] * wn[None, :], 1e-30))), float(np.max(err) / max(np.max(np.abs(want_f64)), 1e-30))

    # ---- headline: C2, Q4_K decode multiply M = 1, K = 4096, N = 14336 ----------------------
    n, k = 14336, 4096
    g = synth.rng(0xC2)
    raw = synth.q4_k_rows(g, n, k)
    x = synth.activations(g, 1, k)
    launches, out = matvec_workload(TensorType.q4_k, raw, n, k, 1, False, x)
    c2_bytes = n * K.row_bytes(TensorType.q4_k, k) + 4 * k + 4 * n  # 33,103,872
    wall, _ = timed(launches, args.steps, args.warmup)
    _, p_gpu, p_steps = protocol(launches)
    got = read(out)[:n].reshape(1, n)

    import oracle  # the checker and the CPU baseline; never the measured path

    w_f32 = oracle.dequantize(oracle.Q4_K, raw, n * k).reshape(n, k)
    want = oracle.matmul_f64(x, w_f32)
    bound, rel = check_matvec(got, want, w_f32, x)
    if not bound <= 1e-3:
        print(f"bench.py: parity failed on the headline workload: |err| / (||row|| ||x||) = {bound}", file=sys.stderr)
        return 1

    cpu = None
    if not args.no_cpu:
        threads = oracle.default_threads()
        m = oracle.Matrix(oracle.Q4_K, raw, n, k, threads)
        oracle.matmul(x, m, threads)  # warm-up
        times = []
        t_end = time.perf_counter() + 12.0
        while len(times) < 5 or (time.perf_counter() < t_end and len(times) < 400):
            t0 = time.perf_counter()
            oracle.matmul(x, m, threads)
            times.append(time.perf_counter() - t0)
        med = float(np.median(times))
        cpu = {
            "value": round(c2_bytes / med / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"C restatement of the reference's src/ref multiply (no Zig toolchain), the same C2 weights and input, "
                      f"median of {len(times)} full multiplies ({med * 1e3:.2f} ms each) after 1 warm-up",
        }

    result = {
        "metric": "Q4_K decode matvec GB/s (% HBM peak); Q8_0 prefill matmul TFLOP/s (% MFMA)",
        "value": round(c2_bytes * args.steps / wall / 1e9, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall / args.steps * 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "C2: Q4_K decode matvec, M=1, K=4096, N=14336 (Llama-3-8B FFN-up), f32 activations, "
                        f"rotating over {len(launches)} weight copies ({len(launches) * n * K.row_bytes(TensorType.q4_k, k) >> 20} MiB)",
            "kernel": "matvec_q4_k",
            "bytes_per_step": c2_bytes,
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(c2_bytes * p_steps / p_gpu / 1e9, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(c2_bytes * p_steps / p_gpu / 1e9 / HBM_PEAK_GBPS, 4),
            "traffic": C2_TRAFFIC_BYTES,
            "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command, profiles/matvec_quant_kernel_q4k_c2.txt",
            "us_per_launch": round(p_gpu / p_steps * 1e6, 3),
            "protocol": f"median of 7 batches of {p_steps} back-to-back launches after 3 warm-up batches, HIP events on the host's stream",
        },
        "cpu_baseline": cpu,
        "parity": {"max_err_over_row_x_norms": bound, "max_err_over_max_want": rel, "bound": 1e-3},
    }

    only = [s for s in args.only.split(",") if s]
    also = {}
    if "none" not in only:
        for name, fn in (("c1", bench_c1), ("c3", bench_c3), ("c4", bench_c4), ("c4_int8", bench_c4_int8), ("long", bench_long), ("c5", bench_c5), ("formats", bench_formats), ("down", bench_down), ("replay", bench_replay), ("floor", bench_floor)):
            if not only or name in only:
                try:
                    also[name] = fn(locals())
                except Exception as e:  # a secondary workload must not lose the headline
                    also[name] = {"error": f"{type(e).__name__}: {e}"}
    if also:
        result["also"] = also
    print(json.dumps(result))
    return 0


def vendor_c4_context():
    """Context only: the vendor library's bf16 multiply of C4's shape over weights dequantised
    beforehand (bf16 in, bf16 out; not this path's contract), same protocol. Runs before this
    library opens the device (torch brings its own copy of the HIP runtime)."""
    rows, k, n = 512, 4096, 4096
    try:
        import torch

        tx = torch.randn(rows, k, device="cuda:0", dtype=torch.bfloat16)
        tws = [torch.randn(n, k, device="cuda:0", dtype=torch.bfloat16) * 0.02 for _ in range(4)]
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ts = []
        for rep in range(3 + 7):
            ev0.record()
            for i in range(200):
                torch.matmul(tx, tws[i % 4].t())
            ev1.record()
            torch.cuda.synchronize()
            if rep >= 3:
                ts.append(ev0.elapsed_time(ev1) * 1e-3 / 200)
        tt = float(np.median(ts))
        del tx, tws
        torch.cuda.empty_cache()
        return {"what": "torch.matmul (hipBLASLt), bf16 x bf16 -> bf16, weights dequantised beforehand", "us_per_launch_gpu": round(tt * 1e6, 3),
                "TFLOPs_gpu": round(2 * rows * n * k / tt / 1e12, 1), "mfma_frac": round(2 * rows * n * k / tt / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)}
    except Exception as e:  # context only
        return {"error": f"{type(e).__name__}: {e}"}


def bench_c1(env):
    """Q8_0 decode multiply M = 1, K = 1024, N = 3072."""
    synth, oracle, K, TensorType = env["synth"], env["oracle"], env["K"], env["TensorType"]
    n, k = 3072, 1024
    g = synth.rng(0xC1)
    raw = synth.q8_0_rows(g, n, k)
    x = synth.activations(g, 1, k)
    launches, out = env["matvec_workload"](TensorType.q8_0, raw, n, k, 1, False, x)
    wall, gpu_s, steps = env["protocol"](launches)
    got = env["read"](out)[:n].reshape(1, n)
    w = oracle.dequantize(oracle.Q8_0, raw, n * k).reshape(n, k)
    bound, rel = env["check_matvec"](got, oracle.matmul_f64(x, w), w, x)
    nbytes = n * k // 32 * 34 + 4 * k + 4 * n  # GGUF bytes: 3,358,720
    e = env["hbm_entry"]("C1: Q8_0 decode matvec M=1 K=1024 N=3072, rotating over weight copies", nbytes, wall, gpu_s, steps,
                         {"copies": len(launches), "max_err_over_row_x_norms": bound, "max_err_over_max_want": rel})
    # The same launch over one copy: the weights stay in L2 (3.3 MB), what a benchmark that
    # reuses its buffers sees.
    hwall, hgpu, hsteps = env["protocol"](launches[:1])
    e["hot"] = {"us_per_step_wall": round(hwall / hsteps * 1e6, 3), "us_per_launch_gpu": round(hgpu / hsteps * 1e6, 3),
                "GBps_gpu": round(nbytes * hsteps / hgpu / 1e9, 1), "copies": 1}
    return e


def bench_floor(env):
    """What the machine gives a plain copy through the same command stream: copy_buffer of
    33 MB (the headline's weight bytes) and 311 MB (the lm_head's), rotating over distinct
    sources beyond the Infinity Cache, batches of back-to-back copies in one blocking submit,
    median of 7 batches after 3 warm-ups. A copy reads and writes its size."""
    rec, host, token, cmd = env["rec"], env["host"], env["token"], env["cmd"]

    res = {}
    for name, size in (("33MB", 14336 * 2304), ("311MB", 151936 * 1024 * 2)):
        copies = env["rotation"](size)
        srcs = [env["output"](size) for _ in range(copies)]
        dst = env["output"](size)
        for sbuf in srcs:
            rec.clear_buffer(sbuf.buffer, 0, size)
        env["flush"]()
        n = -(-200 // copies) * copies if size < (100 << 20) else 10 * copies
        gpus = []
        for rep in range(3 + 7):
            for i in range(n):
                rec.copy_buffer(srcs[i % copies].buffer, 0, dst.buffer, 0, size)
            token[0] += 1
            rec.submit(token[0])
            host.execute(rec.batch(), [])
            rec.clear()
            if rep >= 3:
                gpus.append(host.last_submit()[0] * 1e-9)
        t = float(np.median(gpus)) / n
        res[name] = {"bytes_copied": size, "us_per_copy": round(t * 1e6, 3), "GBps_read_plus_write": round(2 * size / t / 1e9, 1),
                     "GBps_read": round(size / t / 1e9, 1), "sources": copies, "copies_per_batch": n}
        for sbuf in srcs + [dst]:
            rec.destroy(cmd.Kind.buffer, sbuf.buffer)
        env["flush"]()
    # A read-only stream of the headline's size through the lightest decode multiply the path
    # has: matvec_bf16 over a 33 MB bf16 matrix (two bytes and one FMA a weight, rows as long as
    # C2's), one launch a step like C2. What this takes is what a single launch reading 33 MB
    # takes here, whatever the format.
    synth, oracle, TensorType = env["synth"], env["oracle"], env["TensorType"]
    n, k = 4040, 4096
    g = synth.rng(0xF100)
    wbits = synth.bf16_matrix(g, n, k, 0.02)
    x = synth.activations(g, 1, k, bf16=True)
    launches, out = env["matvec_workload"](TensorType.bf16, wbits, n, k, 1, False, x)
    wall, gpu_s, steps = env["protocol"](launches)
    got = env["read"](out)[:n].reshape(1, n)
    w = synth.bf16_bits_to_f32(wbits)
    rel = float(np.max(np.abs(got - oracle.matmul_f64(x, w))) / np.max(np.abs(oracle.matmul_f64(x, w))))
    res["read_33MB_bf16_matvec"] = env["hbm_entry"](f"matvec_bf16 M=1 K={k} N={n}: a read of 33 MB in one launch", 2 * n * k + 4 * k + 4 * n, wall, gpu_s, steps,
                                                    {"copies": len(launches), "max_err_over_max_want": rel})
    return res


def bench_replay(env):
    """A decode step's worth of small dependent-looking launches (224 one-row Q8_0 multiplies,
    K = 1024, N = 3072, the same batch submitted again and again as a decoder does per
    token): wall time per submit when the host replays the batch from a HIP graph and when
    it launches it kernel by kernel, each on a context of its own."""
    import time

    from zllm_amd import Device, Host, cmd
    synth, K, TensorType, P = env["synth"], env["K"], env["TensorType"], env["P"]
    n, k, count, submits = 3072, 1024, 224, 12
    g = synth.rng(0xC1)
    raw, x = synth.q8_0_rows(g, n, k), synth.activations(g, 1, k)
    storage = cmd.Usage.storage | cmd.Usage.copy_dst | cmd.Usage.copy_src
    out = {}
    for name, flags in (("replayed", 0), ("launched", Device.NO_REPLAY)):
        dev = Device.open(0, flags)
        host, rec = Host(dev), cmd.Recorder()
        kset = K.Set.create(rec)
        token = [0]

        def flush():
            token[0] += 1
            rec.submit(token[0])
            t0 = time.perf_counter()
            host.execute(rec.batch(), [])
            wall = time.perf_counter() - t0
            rec.clear()
            return wall

        def upload(arr):
            a8 = np.ascontiguousarray(arr).reshape(-1).view(np.uint8)
            buf = rec.create_buffer(a8.size, storage)
            rec.write_buffer(buf, 0, a8)
            return K.Arg(buf, a8.size)

        src, xa = upload(raw), upload(x)
        wa = K.Arg(rec.create_buffer(n * K.row_bytes(TensorType.q8_0, k), storage), n * K.row_bytes(TensorType.q8_0, k))
        K.Launcher(rec, kset).layout(TensorType.q8_0, src, wa, n, k)
        oa = K.Arg(rec.create_buffer(4 * n, storage), 4 * n)
        b = K.Builder(rec, kset)
        launch = b.add(K.weight_kernel("matvec", TensorType.q8_0), P.MatvecBf16(n=n, k=k, col0=0, out_stride=n), [xa, wa, oa, wa],
                       K.Grid.rows_y(K.div_ceil(n, K.MatvecVariant().group_rows())))
        b.finish()
        flush()
        walls, gpus = [], []
        for _ in range(submits):
            for _ in range(count):
                launch.record(rec, K.Extent(rows=1))
            walls.append(flush())
            gpus.append(host.last_submit()[0])
        out[name] = {"us_per_submit_wall": round(float(np.median(walls[3:])) * 1e6, 1), "us_per_submit_gpu": round(float(np.median(gpus[3:])) * 1e-3, 1),
                     "replayed_submits": host.replayed_submits()}
        dev.deinit()
    out["workload"] = f"{count} x matvec_q8_0 M=1 K={k} N={n} per submit, {submits} submits, medians after the third"
    return out


def bench_formats(env):
    """The decode multiply at C2's shape (M = 1, K = 4096, N = 14336) for the other
    GGUF formats the kernel reads: algorithmic bytes are the file's bytes per row."""
    synth, oracle, K, TensorType = env["synth"], env["oracle"], env["K"], env["TensorType"]
    n, k = 14336, 4096
    x = synth.activations(synth.rng(0xF0), 1, k)
    res = {}
    for name, ot in (("q8_0", oracle.Q8_0), ("q6_k", oracle.Q6_K), ("q5_k", oracle.Q5_K), ("q3_k", oracle.Q3_K)):
        t = TensorType[name]
        raw = synth.random_blocks(synth.rng(0xF1), name, n, k)
        launches, out = env["matvec_workload"](t, raw, n, k, 1, False, x)
        wall, gpu_s, steps = env["protocol"](launches)
        got = env["read"](out)[:n].reshape(1, n)
        w = oracle.dequantize(ot, raw, n * k).reshape(n, k)
        bound, rel = env["check_matvec"](got, oracle.matmul_f64(x, w), w, x)
        e, bb = K.LAYOUT[t]
        nbytes = n * (k // e) * bb + 4 * k + 4 * n
        res[name] = env["hbm_entry"](f"{name} decode matvec M=1 K={k} N={n}", nbytes, wall, gpu_s, steps,
                                     {"copies": len(launches), "max_err_over_row_x_norms": bound, "max_err_over_max_want": rel})
    # Steps of several tokens on Q8_0 (a speculative verify step): the default variant, and the
    # matrix-core variant (MatvecVariant wg 512, lanes 64, rows 16) a tuner would pick for them.
    mc = K.MatvecVariant(wg=512, lanes=64, rows=16)
    raw = synth.random_blocks(synth.rng(0xF1), "q8_0", n, k)
    w = oracle.dequantize(oracle.Q8_0, raw, n * k).reshape(n, k)
    e, bb = K.LAYOUT[TensorType.q8_0]
    for m, variant, tag in ((4, None, "q8_0_m4"), (2, mc, "q8_0_m2_matrix_cores"), (4, mc, "q8_0_m4_matrix_cores"), (8, mc, "q8_0_m8_matrix_cores")):
        xm = synth.activations(synth.rng(0xF8 + m), m, k)
        launches, out = env["matvec_workload"](TensorType.q8_0, raw, n, k, m, False, xm, variant)
        wall, gpu_s, steps = env["protocol"](launches)
        got = env["read"](out)[: m * n].reshape(m, n).astype(np.float64)
        want = xm.astype(np.float64) @ w.astype(np.float64).T
        rel = float(np.max(np.abs(got - want)) / np.max(np.abs(want)))
        nbytes = n * (k // e) * bb + m * 4 * k + m * 4 * n
        res[tag] = env["hbm_entry"](f"q8_0 decode matvec M={m} K={k} N={n}" + (", matrix-core variant" if variant else ""), nbytes, wall, gpu_s, steps,
                                    {"copies": len(launches), "max_err_over_max_want": rel})
    # The K formats at eight tokens: default variant and matrix-core variant.
    for name, ot in (("q6_k", oracle.Q6_K), ("q5_k", oracle.Q5_K), ("q3_k", oracle.Q3_K)):
        t = TensorType[name]
        raw = synth.random_blocks(synth.rng(0xF1), name, n, k)
        w = oracle.dequantize(ot, raw, n * k).reshape(n, k)
        e, bb = K.LAYOUT[t]
        m = 8
        xm = synth.activations(synth.rng(0xF8 + m), m, k)
        want = xm.astype(np.float64) @ w.astype(np.float64).T
        for variant, tag in ((None, f"{name}_m8"), (mc, f"{name}_m8_matrix_cores")):
            launches, out = env["matvec_workload"](t, raw, n, k, m, False, xm, variant)
            wall, gpu_s, steps = env["protocol"](launches)
            got = env["read"](out)[: m * n].reshape(m, n).astype(np.float64)
            rel = float(np.max(np.abs(got - want)) / np.max(np.abs(want)))
            nbytes = n * (k // e) * bb + m * 4 * k + m * 4 * n
            res[tag] = env["hbm_entry"](f"{name} decode matvec M={m} K={k} N={n}" + (", matrix-core variant" if variant else ""), nbytes, wall, gpu_s, steps,
                                        {"copies": len(launches), "max_err_over_max_want": rel})
    return res


def bench_down(env):
    """The FFN-down multiply of the same model (K = 14336, N = 4096: rows longer than a step's
    tokens can share workgroup memory for) at one, two and four tokens, Q4_K and Q8_0."""
    synth, oracle, K, TensorType = env["synth"], env["oracle"], env["K"], env["TensorType"]
    n, k = 4096, 14336
    res = {}
    for name, ot in (("q4_k", oracle.Q4_K), ("q8_0", oracle.Q8_0)):
        t = TensorType[name]
        raw = synth.random_blocks(synth.rng(0xD0), name, n, k)
        w = oracle.dequantize(ot, raw, n * k).reshape(n, k)
        e, bb = K.LAYOUT[t]
        for m in (1, 2, 4):
            xm = synth.activations(synth.rng(0xD8 + m), m, k)
            launches, out = env["matvec_workload"](t, raw, n, k, m, False, xm)
            wall, gpu_s, steps = env["protocol"](launches)
            got = env["read"](out)[: m * n].reshape(m, n).astype(np.float64)
            want = xm.astype(np.float64) @ w.astype(np.float64).T
            rel = float(np.max(np.abs(got - want)) / np.max(np.abs(want)))
            nbytes = n * (k // e) * bb + m * 4 * k + m * 4 * n
            res[f"{name}_m{m}"] = env["hbm_entry"](f"{name} decode matvec M={m} K={k} N={n}", nbytes, wall, gpu_s, steps,
                                                    {"copies": len(launches), "max_err_over_max_want": rel})
    return res


def bench_c3(env):
    """Fused gate+up Q4_K decode multiply with the SiLU pair epilogue, M in 1, 4, 8."""
    synth, oracle, K, TensorType = env["synth"], env["oracle"], env["K"], env["TensorType"]
    n, k = 14336, 4096
    gate = synth.q4_k_rows(synth.rng(0xC3A), n, k)
    up = synth.q4_k_rows(synth.rng(0xC3B), n, k)
    raw = np.concatenate([gate, up])
    w = oracle.dequantize(oracle.Q4_K, raw, 2 * n * k).reshape(2 * n, k)
    res = {}
    # The default variant, and for the multi-token steps the matrix-core variant
    # (MatvecVariant wg 512, lanes 64, rows 16) a tuner would pick for them.
    mc = K.MatvecVariant(wg=512, lanes=64, rows=16)
    nw = synth.activations(synth.rng(0xC3F), 1, k).reshape(-1)
    for m, variant, tag, norm in ((1, None, "m1", False), (4, None, "m4", False), (8, None, "m8", False),
                                  (4, mc, "m4_matrix_cores", False), (8, mc, "m8_matrix_cores", False),
                                  (1, None, "m1_norm", True), (4, mc, "m4_matrix_cores_norm", True), (8, mc, "m8_matrix_cores_norm", True)):
        x = synth.activations(synth.rng(0xC30 + m), m, k)
        launches, out = env["matvec_workload"](TensorType.q4_k, raw, n, k, m, True, x, variant, nw if norm else None)
        wall, gpu_s, steps = env["protocol"](launches)
        got = env["read"](out)[: m * n].reshape(m, n).astype(np.float64)
        xin = x.astype(np.float64)
        if norm:
            xin = xin / np.sqrt(np.mean(xin * xin, axis=1, keepdims=True) + 1e-6) * nw.astype(np.float64)
        both = xin @ w.astype(np.float64).T
        gt, u = both[:, :n], both[:, n:]
        want = gt / (1 + np.exp(-gt)) * u
        rel = float(np.max(np.abs(got - want)) / np.max(np.abs(want)))
        nbytes = 2 * n * K.row_bytes(TensorType.q4_k, k) + m * 4 * k + m * 4 * n
        name = f"C3: fused gate+up Q4_K + SiLU*mul, M={m}, K=4096, N=2x14336" + (", matrix-core variant" if variant else "") + (", RMSNorm prologue as the planner's FFN launch has" if norm else "")
        res[tag] = env["hbm_entry"](name, nbytes, wall, gpu_s, steps, {"copies": len(launches), "max_err_over_max_want": rel})
    return res


def bench_c4(env):
    """Q8_0 prefill multiply M = 512, K = 4096, N = 4096 on the bf16 MFMA rung."""
    synth, oracle, K, TensorType, P = env["synth"], env["oracle"], env["K"], env["TensorType"], env["P"]
    rec, kset, b = env["rec"], env["kset"], env["b"]
    rows, k, n = 512, 4096, 4096
    g = synth.rng(0xC4)
    raw = synth.q8_0_rows(g, n, k)
    x = synth.activations(g, rows, k, bf16=True)
    kset.select_prefill(rec, K.Prefill.bf16_mfma_xbf16)
    src = env["upload"](raw)
    xa = env["upload"](synth.to_bf16_bits(x))
    rb = K.row_bytes(TensorType.q8_0, k)
    out = env["output"](4 * rows * n)
    launches, weight_copies = [], []
    for _ in range(4):
        wa = env["output"](n * rb)
        weight_copies.append(wa)
        K.Launcher(rec, kset).layout(TensorType.q8_0, src, wa, n, k)
        p = P.MatmulQuant(rows=rows, n=n, k=k, col0=0, out_stride=n, k_slice=k)
        launches.append(env["L"](b.add(K.Kernel.matmul_q8_0_float, p, [xa, wa, out], K.Grid.tiles_y(K.div_ceil(n, 64), 16)), rows))
    b.finish()
    env["flush"]()
    wall, gpu_s, steps = env["protocol"](launches)
    got = env["read"](out)[: rows * n].reshape(rows, n).astype(np.float64)
    w = oracle.dequantize(oracle.Q8_0, raw, n * k).reshape(n, k)
    want = x.astype(np.float64) @ w.astype(np.float64).T
    # The reference's own ladder on the same shape, activations bound as f32 as its contract
    # says: the exact f32 rung and the two f16 matrix-core rungs.
    xf = env["upload"](x)
    ladder = {}
    for rung, share in ((K.Prefill.fp16_single, 4), (K.Prefill.fp16_compensated, 4), (K.Prefill.scalar_f32, 40)):
        kset.select_prefill(rec, rung)
        rl = []
        for wa in weight_copies:
            rl.append(env["L"](b.add(K.Kernel.matmul_q8_0_float, P.MatmulQuant(rows=rows, n=n, k=k, col0=0, out_stride=n, k_slice=k), [xf, wa, out], K.Grid.tiles_y(K.div_ceil(n, 64), 16)), rows))
        b.finish()
        env["flush"]()
        _, rgpu, rsteps = env["protocol"](rl)
        rgot = env["read"](out)[: rows * n].reshape(rows, n).astype(np.float64)
        ladder[rung.name] = {"us_per_launch_gpu": round(rgpu / rsteps * 1e6, 3), "TFLOPs_gpu": round(2 * rows * n * k * rsteps / rgpu / 1e12, 1),
                             "max_err_over_max_want": float(np.max(np.abs(rgot - want)) / np.max(np.abs(want)))}
    kset.select_prefill(rec, K.Prefill.scalar_f32)
    vendor = env.get("vendor_c4")
    wn = np.linalg.norm(w.astype(np.float64), axis=1)
    xn = np.linalg.norm(x.astype(np.float64), axis=1)
    bound = float(np.max(np.abs(got - want) / (xn[:, None] * wn[None, :])))
    flops = 2 * rows * n * k
    return {
        "workload": "C4: Q8_0 prefill matmul M=512 K=4096 N=4096, bf16 activations (bound as packed bf16), bf16 MFMA, fp32 accumulate; "
                    "rotating over 4 weight copies (71 MB: within the 256 MB Infinity Cache, the kernel is bound by the path into the CUs, not by HBM)",
        "flops_per_step": flops,
        "us_per_step_wall": round(wall / steps * 1e6, 3),
        "us_per_launch_gpu": round(gpu_s / steps * 1e6, 3),
        "TFLOPs_wall": round(flops * steps / wall / 1e12, 1),
        "TFLOPs_gpu": round(flops * steps / gpu_s / 1e12, 1),
        "mfma_frac": round(flops * steps / gpu_s / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
        "max_err_over_row_x_norms": bound,
        "max_err_over_max_want": float(np.max(np.abs(got - want)) / np.max(np.abs(want))),
        "reference_ladder_f32_activations": ladder,
        "vendor_library_context": vendor,
    }


def bench_long(env):
    """Longer prefill steps of the same multiply (2048 tokens): the 256 x 128 tiling."""
    synth, oracle, K, TensorType, P = env["synth"], env["oracle"], env["K"], env["TensorType"], env["P"]
    rec, kset, b = env["rec"], env["kset"], env["b"]
    res = {}
    for rows, k, n in ((2048, 4096, 4096), (2048, 4096, 14336)):
        g = synth.rng(0x10 + n)
        raw = synth.q8_0_rows(g, n, k)
        x = synth.activations(g, rows, k, bf16=True)
        kset.select_prefill(rec, K.Prefill.bf16_mfma_xbf16)
        src = env["upload"](raw)
        xa = env["upload"](synth.to_bf16_bits(x))
        rb = K.row_bytes(TensorType.q8_0, k)
        out = env["output"](4 * rows * n)
        launches = []
        for _ in range(3):
            wa = env["output"](n * rb)
            K.Launcher(rec, kset).layout(TensorType.q8_0, src, wa, n, k)
            p = P.MatmulQuant(rows=rows, n=n, k=k, col0=0, out_stride=n, k_slice=k)
            launches.append(env["L"](b.add(K.Kernel.matmul_q8_0_float, p, [xa, wa, out], K.Grid.tiles_y(K.div_ceil(n, 64), 16)), rows))
        b.finish()
        env["flush"]()
        wall, gpu_s, steps = env["protocol"](launches)
        kset.select_prefill(rec, K.Prefill.scalar_f32)
        # Checked on every 16th token (the whole product in float64 would take the CPU longer than the bench).
        got = env["read"](out)[: rows * n].reshape(rows, n)[::16].astype(np.float64)
        w = oracle.dequantize(oracle.Q8_0, raw, n * k).reshape(n, k)
        want = x[::16].astype(np.float64) @ w.astype(np.float64).T
        flops = 2 * rows * n * k
        res[f"m{rows}_k{k}_n{n}"] = {
            "workload": f"Q8_0 prefill matmul M={rows} K={k} N={n}, packed bf16 activations, bf16 MFMA, fp32 accumulate; 3 weight copies",
            "flops_per_step": flops,
            "us_per_launch_gpu": round(gpu_s / steps * 1e6, 3),
            "TFLOPs_gpu": round(flops * steps / gpu_s / 1e12, 1),
            "mfma_frac": round(flops * steps / gpu_s / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
            "max_err_over_max_want": float(np.max(np.abs(got - want)) / np.max(np.abs(want))),
        }
    return res


def bench_c4_int8(env):
    """The same product as C4 the way the reference's default prefill computes it:
    quantize_q8 rounds the f32 activations to Q8_0 blocks, matmul_q8_0 multiplies
    integers on the int8 matrix cores and scales every 32-weight unit. The K
    formats' multiplies (Q8_K activations) on the same shape ride along."""
    synth, oracle, K, TensorType, P = env["synth"], env["oracle"], env["K"], env["TensorType"], env["P"]
    rec, kset, b = env["rec"], env["kset"], env["b"]
    rows, k, n = 512, 4096, 4096
    g = synth.rng(0xC4)
    x = synth.activations(g, rows, k)
    xa = env["upload"](x)
    out = env["output"](4 * rows * n)
    ops = 2 * rows * n * k

    def one(t, raw, otype, what):
        block = K.act_block(t)
        src = env["upload"](raw)
        rb = K.row_bytes(t, k)
        qx, dx = env["output"](rows * k), env["output"](4 * rows * k // block)
        launches = []
        for _ in range(4):
            wa = env["output"](n * rb)
            if K.needs_layout(t):
                K.Launcher(rec, kset).layout(t, src, wa, n, k)
            else:
                rec.copy_buffer(src.buffer, src.offset, wa.buffer, wa.offset, raw.size)
            quant = b.add(K.Kernel.quantize_q8, P.QuantizeQ8(k=k, block=block), [xa, qx, dx, xa], K.Grid.tiles_y(K.div_ceil(k, 256), 1))
            p = P.MatmulQuant(rows=rows, n=n, k=k, col0=0, out_stride=n, k_slice=k)
            mul = b.add(K.weight_kernel("matmul", t), p, [qx, wa, out, dx], K.Grid.tiles_y(K.div_ceil(n, K.matmul_quant_tile_n), K.matmul_quant_tile_t))
            launches.append(env["Chain"]([quant, mul], rows))
        b.finish()
        env["flush"]()
        wall, gpu_s, steps = env["protocol"](launches, per_step=2)
        got = env["read"](out)[: rows * n].reshape(rows, n).astype(np.float64)
        w = oracle.dequantize(otype, raw, n * k).reshape(n, k)
        xs = oracle.round_like_llama(otype, x)
        want = xs.astype(np.float64) @ w.astype(np.float64).T
        return {
            "workload": what,
            "ops_per_step": ops,
            "us_per_step_wall": round(wall / steps * 1e6, 3),
            "us_per_step_gpu": round(gpu_s / steps * 1e6, 3),
            "TOPs_gpu": round(ops * steps / gpu_s / 1e12, 1),
            "int8_mfma_frac": round(ops * steps / gpu_s / 1e12 / MFMA_INT8_PEAK_TOPS, 4),
            "max_err_over_max_want": float(np.max(np.abs(got - want)) / np.max(np.abs(want))),
        }

    res = one(TensorType.q8_0, synth.q8_0_rows(g, n, k), oracle.Q8_0,
              "C4 shape through quantize_q8 + matmul_q8_0: f32 activations rounded to Q8_0 blocks, int8 MFMA, f32 scaling per 32-weight unit")
    res["k_formats"] = {}
    for t, otype in ((TensorType.q4_k, oracle.Q4_K), (TensorType.q5_k, oracle.Q5_K), (TensorType.q6_k, oracle.Q6_K), (TensorType.q3_k, oracle.Q3_K)):
        r = one(t, synth.random_blocks(g, t.name, n, k), otype, f"the same shape through quantize_q8 (Q8_K blocks) + matmul_{t.name}")
        res["k_formats"][t.name] = {key: r[key] for key in ("us_per_step_gpu", "TOPs_gpu", "max_err_over_max_want")}
    return res


def bench_c5(env):
    """bf16 lm_head K = 1024, N = 151936 at M = 1 (decode) and M = 128 (prefill chunk)."""
    synth, oracle, K, TensorType, P = env["synth"], env["oracle"], env["K"], env["TensorType"], env["P"]
    rec, kset, b = env["rec"], env["kset"], env["b"]
    n, k = 151936, 1024
    g = synth.rng(0xC5)
    wbits = synth.bf16_matrix(g, n, k, 0.02)
    w = synth.bf16_bits_to_f32(wbits)
    res = {}
    # M = 1: the decode multiply.
    x = synth.activations(g, 1, k, bf16=True)
    launches, out = env["matvec_workload"](TensorType.bf16, wbits, n, k, 1, False, x)
    wall, gpu_s, steps = env["protocol"](launches)
    got = env["read"](out)[:n].reshape(1, n)
    want = oracle.matmul_f64(x, w)
    bound, rel = env["check_matvec"](got, want, w, x)
    nbytes = 2 * n * k + 2 * k + 4 * n
    res["m1"] = env["hbm_entry"]("C5: bf16 lm_head matvec M=1 K=1024 N=151936", nbytes, wall, gpu_s, steps,
                                 {"copies": len(launches), "max_err_over_row_x_norms": bound, "max_err_over_max_want": rel,
                                  "argmax_equal": bool(int(np.argmax(got[0])) == oracle.argmax(want[0].astype(np.float32)))})
    # M = 4 and 8: the widths of a speculative verify step, still the decode multiply.
    for m in (4, 8):
        xm = synth.activations(g, m, k, bf16=True)
        launches, out = env["matvec_workload"](TensorType.bf16, wbits, n, k, m, False, xm)
        wall, gpu_s, steps = env["protocol"](launches)
        got = env["read"](out)[: m * n].reshape(m, n)
        wantm = oracle.matmul_f64(xm, w)
        res[f"m{m}"] = env["hbm_entry"](f"C5: bf16 lm_head matvec M={m} K=1024 N=151936", 2 * n * k + 4 * m * k + 4 * m * n, wall, gpu_s, steps,
                                        {"copies": len(launches), "max_err_over_max_want": float(np.max(np.abs(got - wantm)) / np.max(np.abs(wantm)))})
    # The same projection with Q8_0 weights (rows of 1024 weights with their scales: 1088 bytes,
    # 8.5 cache lines): the default variant, and the matrix-core variant at verify widths.
    mc = K.MatvecVariant(wg=512, lanes=64, rows=16)
    raw = synth.random_blocks(synth.rng(0xC8), "q8_0", n, k)
    wq = oracle.dequantize(oracle.Q8_0, raw, n * k).reshape(n, k)
    e, bb = K.LAYOUT[TensorType.q8_0]
    for m, variant in ((1, None), (4, None), (4, mc), (8, mc)):
        xm = synth.activations(synth.rng(0xC8 + m), m, k)
        launches, out = env["matvec_workload"](TensorType.q8_0, raw, n, k, m, False, xm, variant)
        wall, gpu_s, steps = env["protocol"](launches)
        got = env["read"](out)[: m * n].reshape(m, n)
        wantm = oracle.matmul_f64(xm, wq)
        res[f"q8_0_m{m}" + ("_matrix_cores" if variant else "")] = env["hbm_entry"](
            f"q8_0 lm_head matvec M={m} K=1024 N=151936" + (", matrix-core variant" if variant else ""),
            n * (k // e) * bb + 4 * m * k + 4 * m * n, wall, gpu_s, steps,
            {"copies": len(launches), "max_err_over_max_want": float(np.max(np.abs(got - wantm)) / np.max(np.abs(wantm)))})
    del wq
    # M = 128: the prefill multiply on the bf16 MFMA rung.
    rows = 128
    x = synth.activations(g, rows, k, bf16=True)
    kset.select_prefill(rec, K.Prefill.bf16_mfma_xbf16)
    xa = env["upload"](synth.to_bf16_bits(x))
    out = env["output"](4 * rows * n)
    p = P.MatmulBf16(rows=rows, n=n, k=k, col0=0, out_stride=n)
    copies = env["rotation"](2 * n * k)  # three copies: 934 MB, beyond the Infinity Cache
    launches = []
    for _ in range(copies):
        wa = env["upload"](wbits)
        launches.append(env["L"](b.add(K.Kernel.matmul_bf16, p, [xa, wa, out], K.Grid.tiles_y(K.div_ceil(n, 64), 16)), rows))
    b.finish()
    env["flush"]()
    wall, gpu_s, steps = env["protocol"](launches)
    got = env["read"](out)[: rows * n].reshape(rows, n)
    kset.select_prefill(rec, K.Prefill.scalar_f32)
    want = oracle.matmul_f64(x, w)
    rel = float(np.max(np.abs(got - want)) / np.max(np.abs(want)))
    nbytes = 2 * n * k + 2 * rows * k + 4 * rows * n
    res["m128"] = env["hbm_entry"]("C5: bf16 lm_head matmul M=128 K=1024 N=151936 (bf16 MFMA)", nbytes, wall, gpu_s, steps,
                                   {"copies": copies, "max_err_over_max_want": rel,
                                    "argmax_rows_equal": int(np.count_nonzero(np.argmax(got, axis=1) == np.argmax(want, axis=1))), "rows": rows})
    return res


if __name__ == "__main__":
    sys.exit(main())
