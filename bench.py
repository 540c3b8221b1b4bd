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

The other configurations the metric names ride in the same object: roofline.c4
(the Q8_0 prefill multiply on the bf16 matrix cores: TFLOP/s and its fraction of
the 2.5 PFLOP/s peak), roofline.c3 (fused gate / up at 1, 4 and 8 tokens),
roofline.c1 and roofline.c5. "also" holds the rest (other formats, the FFN-down
shape, the int8 prefill, the scheduler's step sizes, floors), every entry as
{"us": GPU microseconds a step, "frac": fraction of the roofline that bounds it,
"err": max |error| / max |expected|, "err_bound": max |error| / (||row|| ||x||)};
every figure but `value` is timed by the reference tuner's protocol (protocol()
below), and `value` is the wall time of one blocking submit of --steps launches,
host overhead included.
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
# WRITE_SIZE counter runs scaled by a plain copy of known size (profiles/matvec_quant_row_kernel_q4k_c2.txt).
C2_TRAFFIC_BYTES = 33_427_456


def sig2(v: float) -> float:
    """v to two significant digits (errors in the record)."""
    return float(f"{v:.1e}")


SECTIONS = ("c1", "c3", "c4", "c5", "formats", "down", "c4_int8", "prefill_grid", "replay", "floor")  # and, on request: long


def make_env(flags: int = 0) -> dict:
    """A context of its own on GPU 0 (zhip_options flags as given) with the helpers the
    workloads share; env["close"]() ends it."""
    from zllm_amd import Device, Host, cmd, synth
    from zllm_amd import kernels as K
    from zllm_amd.kernels import Kernel, TensorType, params as P

    dev = Device.open(0, flags)
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

    def release(*args_) -> None:
        for a in args_:
            rec.destroy(cmd.Kind.buffer, a.buffer)
        flush()

    def read(arg: K.Arg, dtype=np.float32) -> np.ndarray:
        dst = np.zeros(arg.size, dtype=np.uint8)
        rec.read_buffer(0xFFFF0000, arg.buffer, 0, dst)
        flush()
        return dst.view(dtype)

    def timed(launches, steps: int, warmup: int, per_step: int = 1):
        """Runs `warmup` then `steps` steps cycling over `launches` (each records
        `per_step` dispatches), each count as one blocking submit; returns (wall
        seconds, GPU seconds from the host's stream events) of the second."""
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

    def protocol(launches, per_step: int = 1, least: int = 200):
        """The tuner's timing protocol (src/tune/tune.zig:8-11,24-27) whatever --steps says:
        batches of at least `least` back-to-back steps in one blocking submit (a whole number
        of rotations over `launches`), 3 warm-up batches, then 7 timed ones; returns the median
        batch as (wall seconds, GPU seconds from the host's stream events, steps in a batch).
        Identical batches are replayed from a HIP graph from their second submit on, as the
        host does for any repeated submit."""
        n = -(-least // len(launches)) * len(launches)
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
        """Uploads a rotation of weight copies and builds one launch per copy; returns the
        launches, the output and the buffers to release afterwards."""
        kernel = K.weight_kernel("matvec", t)
        rb = K.row_bytes(t, k)
        w_rows = 2 * n_out if pair else n_out
        copies = rotation(w_rows * rb)
        src = upload(raw_rows)
        xa = upload(x)
        out = output(4 * m * n_out)
        held = [src, xa, out]
        launches = []
        for _ in range(copies):
            if K.needs_layout(t):
                wa = output(w_rows * rb)
                K.Launcher(rec, kset).layout(t, src, wa, w_rows, k)
            else:
                buf = rec.create_buffer(src.size, storage)
                rec.copy_buffer(src.buffer, 0, buf, 0, src.size)
                wa = K.Arg(buf, src.size)
            held.append(wa)
            v = variant or K.MatvecVariant()
            p = P.MatvecBf16(n=n_out, k=k, col0=0, out_stride=n_out, eps=eps if norm_w is not None else 0.0, norm=norm_w is not None, silu_pair=pair, half=n_out if pair else 0)
            na = wa
            if norm_w is not None:
                na = upload(norm_w)
                held.append(na)
            if K.is_half(t):
                launches.append(L(b.add(kernel, p, [xa, wa, out, na], K.Grid.rows_y(K.div_ceil(n_out, K.matvec_rows))), m))
            else:
                launches.append(L(b.add_matvec(kernel, v, p, [xa, wa, out, na], K.Grid.rows_y(K.div_ceil(n_out, v.group_rows()))), m))
        b.finish()
        flush()
        return launches, out, held

    def hbm_entry(bytes_per_step, gpu_s, steps, extra=None):
        """One compact record: GPU microseconds a step, the fraction of the HBM peak its
        algorithmic bytes reach, and what `extra` adds (errors to two digits)."""
        e = {"us": round(gpu_s / steps * 1e6, 2), "frac": round(bytes_per_step * steps / gpu_s / 1e9 / HBM_PEAK_GBPS, 3)}
        for key, v in (extra or {}).items():
            e[key] = sig2(v) if isinstance(v, float) else v
        return e

    def check_matvec(got, want_f64, w_rows_f32, x):
        """(max |err| / (||row|| ||x||), max |err| / max |want|)."""
        got = got.astype(np.float64)
        wn = np.linalg.norm(w_rows_f32.astype(np.float64), axis=1)
        xn = np.linalg.norm(x.astype(np.float64).reshape(got.shape[0], -1), axis=1)
        err = np.abs(got - want_f64)
        return float(np.max(err / np.maximum(xn[:, None] * wn[None, :], 1e-30))), float(np.max(err) / max(np.max(np.abs(want_f64)), 1e-30))

    def close():
        dev.deinit()

    return locals()


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--only", default="", help="comma-separated subset of: " + ",".join(SECTIONS) + ",long for the sections beside the headline; 'none' skips them")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-replay", action="store_true",
                    help="launch every dispatch of a repeated submit instead of replaying it from a HIP graph")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="first run 4 plain elementwise copies (256 MiB read + 256 MiB written each) so a counter run has a kernel of known traffic to scale by")
    ap.add_argument("--grid", default="", help="with prefill_grid: only these keys (comma-separated, e.g. m512_k4096_n14336), for a profile of one shape")
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

    only = [w for w in args.only.split(",") if w]
    wanted = [] if "none" in only else [name for name in SECTIONS + ("long",) if (name in only if only else name != "long")]
    # What needs torch runs before this library opens the device (torch brings its own copy of the HIP runtime).
    vendor_c4 = vendor_c4_context() if "c4" in wanted else None
    torch_read = torch_read_floor() if "floor" in wanted else None

    from zllm_amd import Device

    env = make_env(Device.NO_REPLAY if args.no_replay else 0)
    env.update(vendor_c4=vendor_c4, torch_read=torch_read, make_env=make_env, Device=Device, grid=[w for w in args.grid.split(",") if w])
    synth, K, TensorType = env["synth"], env["K"], env["TensorType"]

    # ---- headline: C2, Q4_K decode multiply M = 1, K = 4096, N = 14336 ----------------------
    n, k = 14336, 4096
    g = synth.rng(0xC2)
    raw = synth.q4_k_rows(g, n, k)
    x = synth.activations(g, 1, k)
    launches, out, held = env["matvec_workload"](TensorType.q4_k, raw, n, k, 1, False, x)
    c2_bytes = n * K.row_bytes(TensorType.q4_k, k) + 4 * k + 4 * n  # 33,103,872
    # The protocol's batches first: the timed steps below then run on a machine in the state a
    # decode loop keeps it in (clocks up, code and host paths warm), not on one just opened.
    _, p_gpu, p_steps = env["protocol"](launches)
    wall, _ = env["timed"](launches, args.steps, args.warmup)
    got = env["read"](out)[:n].reshape(1, n)
    n_copies = len(launches)
    env["release"](*held)

    import oracle  # the checker and the CPU baseline; never the measured path

    env["oracle"] = oracle
    w_f32 = oracle.dequantize(oracle.Q4_K, raw, n * k).reshape(n, k)
    want = oracle.matmul_f64(x, w_f32)
    bound, rel = env["check_matvec"](got, want, w_f32, x)
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
    del w_f32

    roofline = {
        "bound": "hbm",
        "achieved": round(c2_bytes * p_steps / p_gpu / 1e9, 1),
        "peak": HBM_PEAK_GBPS,
        "unit": "GB/s",
        "frac": round(c2_bytes * p_steps / p_gpu / 1e9 / HBM_PEAK_GBPS, 4),
        "traffic": C2_TRAFFIC_BYTES,
        "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command, profiles/matvec_quant_row_kernel_q4k_c2.txt",
        "us_per_launch": round(p_gpu / p_steps * 1e6, 3),
        "protocol": f"median of 7 batches of {p_steps} back-to-back launches after 3 warm-up batches, HIP events on the host's stream",
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
                        f"rotating over {n_copies} weight copies ({n_copies * n * K.row_bytes(TensorType.q4_k, k) >> 20} MiB)",
            "kernel": "matvec_q4_k",
            "bytes_per_step": c2_bytes,
            "value_is": "wall time of one blocking submit of --steps launches (host decode, launch and wake-up included); the kernel's own period is roofline.us_per_launch",
        },
        "roofline": roofline,
        "cpu_baseline": cpu,
        "parity": {"max_err_over_row_x_norms": sig2(bound), "max_err_over_max_want": sig2(rel), "bound": 1e-3},
    }

    fns = {"c1": bench_c1, "c3": bench_c3, "c4": bench_c4, "c5": bench_c5, "formats": bench_formats, "down": bench_down, "c4_int8": bench_c4_int8,
           "prefill_grid": bench_prefill_grid, "long": bench_long, "replay": bench_replay, "floor": bench_floor}
    also = {}
    for name in wanted:
        try:
            r = fns[name](env)
        except Exception as e:  # a secondary workload must not lose the headline
            r = {"error": f"{type(e).__name__}: {e}"}
        # The other configurations the metric is quoted on go into `roofline`, beside the headline's.
        if name in ("c1", "c3", "c4", "c5") and "error" not in r:
            roofline[name] = r.pop("headline", None)
            if r:
                also[name] = r
        else:
            also[name] = r
    if also:
        result["also"] = also
    env["close"]()
    print(json.dumps(result, separators=(",", ":")))
    return 0


def vendor_c4_context():
    """Context only: the vendor library's bf16 multiply of C4's shape over weights dequantised
    beforehand (bf16 in, bf16 out; not this path's contract), same protocol."""
    rows, k, n = 512, 4096, 4096
    try:
        import torch

        tx = torch.randn(rows, k, device="cuda:0", dtype=torch.bfloat16)
        copies = -(-ROTATE_BYTES // (2 * n * k))  # (weights from HBM, like the kernel beside it)
        tws = [torch.randn(n, k, device="cuda:0", dtype=torch.bfloat16) * 0.02 for _ in range(copies)]
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ts = []
        for rep in range(3 + 7):
            ev0.record()
            for i in range(200):
                torch.matmul(tx, tws[i % copies].t())
            ev1.record()
            torch.cuda.synchronize()
            if rep >= 3:
                ts.append(ev0.elapsed_time(ev1) * 1e-3 / 200)
        tt = float(np.median(ts))
        del tx, tws
        torch.cuda.empty_cache()
        return {"what": "torch.matmul (hipBLASLt) bf16 x bf16 -> bf16, weights dequantised beforehand", "us": round(tt * 1e6, 2),
                "frac": round(2 * rows * n * k / tt / 1e12 / MFMA_BF16_PEAK_TFLOPS, 3)}
    except Exception as e:  # context only
        return {"error": f"{type(e).__name__}: {e}"}


def torch_read_floor():
    """Context only: what a kernel that does nothing but read the headline's bytes takes on this
    machine, launched back to back like the headline: torch.sum over 33 MB tensors rotating
    beyond the Infinity Cache (a vendor reduction kernel; one launch reads one tensor)."""
    try:
        import torch

        size = 14336 * 2304
        copies = max(2, -(-ROTATE_BYTES // size))
        ts_ = [torch.ones(size // 4, device="cuda:0", dtype=torch.float32) for _ in range(copies)]
        outs = torch.empty(copies, device="cuda:0", dtype=torch.float32)
        n = -(-200 // copies) * copies
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ts = []
        for rep in range(3 + 7):
            ev0.record()
            for i in range(n):
                torch.sum(ts_[i % copies], dim=0, out=outs[i % copies])
            ev1.record()
            torch.cuda.synchronize()
            if rep >= 3:
                ts.append(ev0.elapsed_time(ev1) * 1e-3 / n)
        tt = float(np.median(ts))
        del ts_, outs
        torch.cuda.empty_cache()
        return {"what": "torch.sum of 33 MB of f32, one launch a tensor, rotating over 661 MiB", "us": round(tt * 1e6, 2), "frac": round(size / tt / 1e9 / HBM_PEAK_GBPS, 3)}
    except Exception as e:  # context only
        return {"error": f"{type(e).__name__}: {e}"}


def bench_c1(env):
    """Q8_0 decode multiply M = 1, K = 1024, N = 3072: rotating over weight copies, and
    `hot_us` over one copy that stays in L2 (what a benchmark that reuses its buffers sees)."""
    synth, oracle, TensorType = env["synth"], env["oracle"], env["TensorType"]
    n, k = 3072, 1024
    g = synth.rng(0xC1)
    raw = synth.q8_0_rows(g, n, k)
    x = synth.activations(g, 1, k)
    launches, out, held = env["matvec_workload"](TensorType.q8_0, raw, n, k, 1, False, x)
    _, gpu_s, steps = env["protocol"](launches)
    got = env["read"](out)[:n].reshape(1, n)
    w = oracle.dequantize(oracle.Q8_0, raw, n * k).reshape(n, k)
    bound, rel = env["check_matvec"](got, oracle.matmul_f64(x, w), w, x)
    nbytes = n * k // 32 * 34 + 4 * k + 4 * n  # GGUF bytes: 3,358,720
    e = env["hbm_entry"](nbytes, gpu_s, steps, {"err_bound": bound, "err": rel})
    _, hgpu, hsteps = env["protocol"](launches[:1])
    e["hot_us"] = round(hgpu / hsteps * 1e6, 2)
    env["release"](*held)
    return {"headline": e}


def bench_floor(env):
    """What the machine gives plain transfers: copy_buffer of 33 MB (the headline's weight
    bytes) and 311 MB (the lm_head's) through the same command stream, rotating over distinct
    sources beyond the Infinity Cache (a copy reads and writes its size: `frac` counts both);
    the vendor's read-only reduction over 33 MB; and matvec_bf16 over a 33 MB matrix with rows
    as long as the headline's (a multiply, not a floor)."""
    rec, host, token, cmd = env["rec"], env["host"], env["token"], env["cmd"]
    res = {}
    for name, size in (("copy_33MB", 14336 * 2304), ("copy_311MB", 151936 * 1024 * 2)):
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
        res[name] = {"us": round(t * 1e6, 2), "frac": round(2 * size / t / 1e9 / HBM_PEAK_GBPS, 3)}
        env["release"](*srcs, dst)
    res["torch_sum_33MB"] = env.get("torch_read")
    synth, oracle, TensorType = env["synth"], env["oracle"], env["TensorType"]
    n, k = 4040, 4096
    g = synth.rng(0xF100)
    wbits = synth.bf16_matrix(g, n, k, 0.02)
    x = synth.activations(g, 1, k, bf16=True)
    launches, out, held = env["matvec_workload"](TensorType.bf16, wbits, n, k, 1, False, x)
    _, gpu_s, steps = env["protocol"](launches)
    got = env["read"](out)[:n].reshape(1, n)
    want = oracle.matmul_f64(x, synth.bf16_bits_to_f32(wbits))
    res["matvec_bf16_33MB"] = env["hbm_entry"](2 * n * k + 4 * k + 4 * n, gpu_s, steps, {"err": float(np.max(np.abs(got - want)) / np.max(np.abs(want)))})
    env["release"](*held)
    return res


def bench_replay(env):
    """A decode step's worth of small launches (224 one-row Q8_0 multiplies, K = 1024,
    N = 3072, the same batch submitted again and again as a decoder does per token): wall
    microseconds per submit when the host replays the batch from a HIP graph and when it
    launches it kernel by kernel, each on a context of its own."""
    out = {}
    for name, flags in (("replayed", 0), ("launched", env["Device"].NO_REPLAY)):
        e2 = env["make_env"](flags)
        synth, K, TensorType, P, rec, host = e2["synth"], e2["K"], e2["TensorType"], e2["P"], e2["rec"], e2["host"]
        n, k, count, submits = 3072, 1024, 224, 12
        g = synth.rng(0xC1)
        raw, x = synth.q8_0_rows(g, n, k), synth.activations(g, 1, k)
        src, xa = e2["upload"](raw), e2["upload"](x)
        wa = e2["output"](n * K.row_bytes(TensorType.q8_0, k))
        K.Launcher(rec, e2["kset"]).layout(TensorType.q8_0, src, wa, n, k)
        oa = e2["output"](4 * n)
        b = e2["b"]
        launch = b.add(K.weight_kernel("matvec", TensorType.q8_0), P.MatvecBf16(n=n, k=k, col0=0, out_stride=n), [xa, wa, oa, wa],
                       K.Grid.rows_y(K.div_ceil(n, K.MatvecVariant().group_rows())))
        b.finish()
        e2["flush"]()
        walls = []
        for _ in range(submits):
            for _ in range(count):
                launch.record(rec, K.Extent(rows=1))
            e2["token"][0] += 1
            rec.submit(e2["token"][0])
            t0 = time.perf_counter()
            host.execute(rec.batch(), [])
            walls.append(time.perf_counter() - t0)
            rec.clear()
        out[name] = {"us_per_submit_wall": round(float(np.median(walls[3:])) * 1e6, 1), "replayed_submits": host.replayed_submits()}
        e2["close"]()
    return out


def _multi_token(env, t, otype, raw, n, k, m, variant, pair=False, norm_w=None):
    """One decode-multiply entry at m tokens (checked against float64 on the decoded weights)."""
    synth, oracle, K = env["synth"], env["oracle"], env["K"]
    xm = synth.activations(synth.rng(0xF8 + m), m, k)
    launches, out, held = env["matvec_workload"](t, raw, n, k, m, pair, xm, variant, norm_w)
    _, gpu_s, steps = env["protocol"](launches)
    got = env["read"](out)[: m * n].reshape(m, n).astype(np.float64)
    env["release"](*held)
    rows = 2 * n if pair else n
    w = oracle.dequantize(otype, raw, rows * k).reshape(rows, k).astype(np.float64)
    xin = xm.astype(np.float64)
    if norm_w is not None:
        xin = xin / np.sqrt(np.mean(xin * xin, axis=1, keepdims=True) + 1e-6) * norm_w.astype(np.float64)
    want = xin @ w.T
    if pair:
        gt, u = want[:, :n], want[:, n:]
        want = gt / (1 + np.exp(-gt)) * u
    e, bb = K.LAYOUT[t]
    nbytes = rows * (k // e) * bb + m * 4 * k + m * 4 * n
    return env["hbm_entry"](nbytes, gpu_s, steps, {"err": float(np.max(np.abs(got - want)) / np.max(np.abs(want)))})


def bench_formats(env):
    """The decode multiply at C2's shape (K = 4096, N = 14336) for the other GGUF formats, one
    token; then eight tokens (Q8_0 also four) on the default variant and on the matrix-core
    variant id (`_mc`: MatvecVariant wg 512, lanes 64, rows 16). Algorithmic bytes are the
    file's bytes per row."""
    synth, oracle, K, TensorType = env["synth"], env["oracle"], env["K"], env["TensorType"]
    n, k = 14336, 4096
    mc = K.MatvecVariant(wg=512, lanes=64, rows=16)
    res = {}
    for name, ot in (("q8_0", oracle.Q8_0), ("q6_k", oracle.Q6_K), ("q5_k", oracle.Q5_K), ("q3_k", oracle.Q3_K)):
        t = TensorType[name]
        raw = synth.random_blocks(synth.rng(0xF1), name, n, k)
        res[name] = _multi_token(env, t, ot, raw, n, k, 1, None)
        for m, variant in ((4, None), (4, mc)) if name == "q8_0" else ():
            res[f"{name}_m{m}" + ("_mc" if variant else "")] = _multi_token(env, t, ot, raw, n, k, m, variant)
        for variant in (None, mc):
            res[f"{name}_m8" + ("_mc" if variant else "")] = _multi_token(env, t, ot, raw, n, k, 8, variant)
    return res


def bench_down(env):
    """The FFN-down multiply of the same model (K = 14336, N = 4096: rows longer than a step's
    tokens can share workgroup memory for) at one, two, four and eight tokens, Q4_K and Q8_0, on
    the default variant and (`_mc`, four and eight tokens) on the matrix-core variant id, where
    the workgroups that share a tile take 2048 columns each."""
    synth, oracle, K, TensorType = env["synth"], env["oracle"], env["K"], env["TensorType"]
    n, k = 4096, 14336
    mc = K.MatvecVariant(wg=512, lanes=64, rows=16)
    res = {}
    for name, ot in (("q4_k", oracle.Q4_K), ("q8_0", oracle.Q8_0)):
        raw = synth.random_blocks(synth.rng(0xD0), name, n, k)
        for m, variant in ((1, None), (2, None), (4, None), (8, None), (4, mc), (8, mc)):
            res[f"{name}_m{m}" + ("_mc" if variant else "")] = _multi_token(env, TensorType[name], ot, raw, n, k, m, variant)
    return res


def bench_c3(env):
    """Fused gate+up Q4_K decode multiply with the SiLU pair epilogue, K = 4096, N = 2 x 14336,
    at 1, 4 and 8 tokens: the default variant (m1, m4, m8), the matrix-core variant id a tuner
    given it as a candidate picks for verify steps (`_mc`), and both with the RMSNorm prologue
    the planner's FFN launch carries (`_norm`)."""
    synth, oracle, K, TensorType = env["synth"], env["oracle"], env["K"], env["TensorType"]
    n, k = 14336, 4096
    raw = np.concatenate([synth.q4_k_rows(synth.rng(0xC3A), n, k), synth.q4_k_rows(synth.rng(0xC3B), n, k)])
    mc = K.MatvecVariant(wg=512, lanes=64, rows=16)
    nw = synth.activations(synth.rng(0xC3F), 1, k).reshape(-1)
    head, rest = {}, {}
    for m, variant, tag, norm in ((1, None, "m1", False), (4, None, "m4", False), (8, None, "m8", False),
                                  (4, mc, "m4_mc", False), (8, mc, "m8_mc", False),
                                  (1, None, "m1_norm", True), (4, mc, "m4_mc_norm", True), (8, mc, "m8_mc_norm", True)):
        e = _multi_token(env, TensorType.q4_k, oracle.Q4_K, raw, n, k, m, variant, pair=True, norm_w=nw if norm else None)
        (rest if norm else head)[tag] = e
    return {"headline": head, **rest}


def _prefill_q8(env, rows, k, n, rung, copies=None, f32_x=False, check_stride=1):
    """matmul_q8_0_float at rows x k x n on a prefill rung: (GPU seconds a step, err, err_bound).
    The launches rotate over weight copies that together exceed L2 and the Infinity Cache (a
    prefill step finds a layer's weights in HBM), unless `copies` says otherwise."""
    synth, oracle, K, TensorType, P = env["synth"], env["oracle"], env["K"], env["TensorType"], env["P"]
    rec, kset, b = env["rec"], env["kset"], env["b"]
    g = synth.rng(0xC4 if (rows, k, n) == (512, 4096, 4096) else 0x10 + n + rows)
    raw = synth.q8_0_rows(g, n, k)
    x = synth.activations(g, rows, k, bf16=True)
    kset.select_prefill(rec, rung)
    src = env["upload"](raw)
    xa = env["upload"](x if f32_x else synth.to_bf16_bits(x))
    rb = K.row_bytes(TensorType.q8_0, k)
    out = env["output"](4 * rows * n)
    held, launches = [src, xa, out], []
    for _ in range(copies or env["rotation"](n * rb)):
        wa = env["output"](n * rb)
        held.append(wa)
        K.Launcher(rec, kset).layout(TensorType.q8_0, src, wa, n, k)
        p = P.MatmulQuant(rows=rows, n=n, k=k, col0=0, out_stride=n, k_slice=k)
        launches.append(env["L"](b.add(K.Kernel.matmul_q8_0_float, p, [xa, wa, out], K.Grid.tiles_y(K.div_ceil(n, 64), 16)), rows))
    b.finish()
    env["flush"]()
    _, gpu_s, steps = env["protocol"](launches, least=200 if rows * n * k <= (1 << 34) else 40)
    got = env["read"](out)[: rows * n].reshape(rows, n)[::check_stride].astype(np.float64)
    kset.select_prefill(rec, K.Prefill.scalar_f32)
    env["release"](*held)
    w = oracle.dequantize(oracle.Q8_0, raw, n * k).reshape(n, k).astype(np.float64)
    xs = x[::check_stride].astype(np.float64)
    want = xs @ w.T
    err = np.abs(got - want)
    bound = float(np.max(err / (np.linalg.norm(xs, axis=1)[:, None] * np.linalg.norm(w, axis=1)[None, :])))
    return gpu_s / steps, float(np.max(err) / np.max(np.abs(want))), bound


def _mfma_entry(t, flops, err=None, bound=None):
    e = {"us": round(t * 1e6, 2), "TFLOPs": round(flops / t / 1e12, 1), "frac": round(flops / t / 1e12 / MFMA_BF16_PEAK_TFLOPS, 3)}
    if err is not None:
        e["err"] = sig2(err)
    if bound is not None:
        e["err_bound"] = sig2(bound)
    return e


def bench_c4(env):
    """Q8_0 prefill multiply M = 512, K = 4096, N = 4096 on the bf16 MFMA rung with the
    activations bound as packed bf16, the weights from HBM (launches rotate over 36 copies,
    641 MB) - `weights_in_cache` is the same with 4 copies, 71 MB, which the Infinity Cache
    holds; then the reference's own ladder on the same shape with f32-bound activations (its
    two f16 matrix-core rungs and the exact f32 rung), and the vendor library's bf16 multiply
    for context, its weights rotating the same way."""
    K = env["K"]
    rows, k, n = 512, 4096, 4096
    flops = 2 * rows * n * k
    t, err, bound = _prefill_q8(env, rows, k, n, K.Prefill.bf16_mfma_xbf16)
    head = _mfma_entry(t, flops, err, bound)
    head.update(bound="mfma", peak=MFMA_BF16_PEAK_TFLOPS, unit="TFLOP/s", flops=flops)
    ladder = {}
    for rung in (K.Prefill.fp16_single, K.Prefill.fp16_compensated, K.Prefill.scalar_f32):
        rt, rerr, _ = _prefill_q8(env, rows, k, n, rung, f32_x=True)
        ladder[rung.name] = _mfma_entry(rt, flops, rerr)
    tw, errw, _ = _prefill_q8(env, rows, k, n, K.Prefill.bf16_mfma_xbf16, copies=4)
    return {"headline": head, "weights_in_cache": _mfma_entry(tw, flops, errw), "ladder_f32_activations": ladder, "vendor_library": env.get("vendor_c4")}


def bench_long(env):
    """Longer prefill steps of the same multiply (2048 tokens; beyond what the reference's
    planner records, src/plan/plan.zig:129): context only, on request (--only long)."""
    K = env["K"]
    res = {}
    for rows, k, n in ((2048, 4096, 4096), (2048, 4096, 14336)):
        t, err, _ = _prefill_q8(env, rows, k, n, K.Prefill.bf16_mfma_xbf16, copies=3, check_stride=16)
        res[f"m{rows}_k{k}_n{n}"] = _mfma_entry(t, 2 * rows * n * k, err)
    return res


def _prefill_int8(env, t, otype, raw, rows, k, n, check_stride=1):
    """quantize_q8 + matmul_<t> as one step: (GPU seconds a step, err against the float64
    product of the rounded activations with the decoded weights)."""
    synth, oracle, K, P = env["synth"], env["oracle"], env["K"], env["P"]
    rec, kset, b = env["rec"], env["kset"], env["b"]
    x = synth.activations(synth.rng(0xC4 + rows), rows, k)
    xa = env["upload"](x)
    out = env["output"](4 * rows * n)
    block = K.act_block(t)
    src = env["upload"](raw)
    rb = K.row_bytes(t, k)
    qx, dx = env["output"](rows * k), env["output"](4 * rows * k // block)
    held, launches = [xa, out, src, qx, dx], []
    for _ in range(env["rotation"](n * rb)):
        wa = env["output"](n * rb)
        held.append(wa)
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
    _, gpu_s, steps = env["protocol"](launches, per_step=2)
    got = env["read"](out)[: rows * n].reshape(rows, n)[::check_stride].astype(np.float64)
    env["release"](*held)
    w = oracle.dequantize(otype, raw, n * k).reshape(n, k).astype(np.float64)
    want = oracle.round_like_llama(otype, x)[::check_stride].astype(np.float64) @ w.T
    return gpu_s / steps, float(np.max(np.abs(got - want)) / np.max(np.abs(want)))


def _int8_entry(t, ops, err):
    return {"us": round(t * 1e6, 2), "TOPs": round(ops / t / 1e12, 1), "frac": round(ops / t / 1e12 / MFMA_INT8_PEAK_TOPS, 3), "err": sig2(err)}


def bench_c4_int8(env):
    """C4's shape the way the reference's default prefill computes it: quantize_q8 rounds the f32
    activations to Q8_0 (for the K formats: Q8_K) blocks, matmul_<format> multiplies integers
    on the int8 matrix cores and scales every unit; the pair of launches is a step, `frac` is
    of the 5 POP/s int8 peak."""
    synth, oracle, TensorType = env["synth"], env["oracle"], env["TensorType"]
    rows, k, n = 512, 4096, 4096
    g = synth.rng(0xC4)
    res = {}
    for t, otype in ((TensorType.q8_0, oracle.Q8_0), (TensorType.q4_k, oracle.Q4_K), (TensorType.q5_k, oracle.Q5_K), (TensorType.q6_k, oracle.Q6_K), (TensorType.q3_k, oracle.Q3_K)):
        raw = synth.q8_0_rows(g, n, k) if t == TensorType.q8_0 else synth.random_blocks(g, t.name, n, k)
        tt, err = _prefill_int8(env, t, otype, raw, rows, k, n)
        res[t.name] = _int8_entry(tt, 2 * rows * n * k, err)
    return res


def bench_prefill_grid(env):
    """The Q8_0 prefill multiply at the step sizes the reference's scheduler issues (chunks cut
    at multiples of 8 with a first chunk of 64, a step capped at 512 tokens:
    src/sched/sched.zig:77-91, src/plan/plan.zig:129) on the three shapes of a layer: keys
    `m<tokens>_k<k>_n<n>`, each with the bf16 matrix-core rung on packed bf16 activations
    ("bf16": us, fraction of the 2.5 PFLOP/s peak) and the reference's default path, quantize_q8
    + matmul_q8_0 on the int8 matrix cores ("int8": us, fraction of the 5 POP/s peak), and the
    same default path over Q4_K weights of the shape, the format of most of a Q4_K_M file
    ("q4_k": us). Checked on every 8th token."""
    synth, oracle, K, TensorType = env["synth"], env["oracle"], env["K"], env["TensorType"]
    res = {}
    for k, n in ((4096, 14336), (14336, 4096), (4096, 4096)):
        raw = synth.q8_0_rows(synth.rng(0x9D + n), n, k)
        raw4 = synth.q4_k_rows(synth.rng(0x9E + n), n, k)
        for rows in (64, 128, 256, 512):
            if env.get("grid") and f"m{rows}_k{k}_n{n}" not in env["grid"]:
                continue
            flops = 2 * rows * n * k
            t, err, _ = _prefill_q8(env, rows, k, n, K.Prefill.bf16_mfma_xbf16, check_stride=8)
            ti, erri = _prefill_int8(env, TensorType.q8_0, oracle.Q8_0, raw, rows, k, n, check_stride=8)
            t4, err4 = _prefill_int8(env, TensorType.q4_k, oracle.Q4_K, raw4, rows, k, n, check_stride=8)
            res[f"m{rows}_k{k}_n{n}"] = {"bf16": [round(t * 1e6, 2), round(flops / t / 1e12 / MFMA_BF16_PEAK_TFLOPS, 3)],
                                         "int8": [round(ti * 1e6, 2), round(flops / ti / 1e12 / MFMA_INT8_PEAK_TOPS, 3)],
                                         "q4_k": round(t4 * 1e6, 2), "err": [sig2(err), sig2(erri), sig2(err4)]}
    return res


def bench_c5(env):
    """bf16 lm_head K = 1024, N = 151936: M = 1 (decode) and M = 128 (prefill chunk, bf16 MFMA
    rung, three weight copies = 934 MB) are the configuration's own; beside them the widths of a
    speculative verify step through the decode multiply (m4, m8), the same in a context opened
    with ZHIP_OPTION_WIDE_DECODE (`wide_m1`, `wide_m4`, `wide_m8`: the weights read once for all
    tokens, at every width), and the projection with Q8_0 weights (default variant and the
    matrix-core variant id, `_mc`)."""
    synth, oracle, K, TensorType, P = env["synth"], env["oracle"], env["K"], env["TensorType"], env["P"]
    rec, kset, b = env["rec"], env["kset"], env["b"]
    n, k = 151936, 1024
    g = synth.rng(0xC5)
    wbits = synth.bf16_matrix(g, n, k, 0.02)
    w = synth.bf16_bits_to_f32(wbits)
    head, rest = {}, {}

    def decode(e_, m):
        xm = synth.activations(synth.rng(0xC50 + m), m, k, bf16=True)
        launches, out, held = e_["matvec_workload"](TensorType.bf16, wbits, n, k, m, False, xm)
        _, gpu_s, steps = e_["protocol"](launches)
        got = e_["read"](out)[: m * n].reshape(m, n)
        e_["release"](*held)
        want = oracle.matmul_f64(xm, w)
        bound, rel = env["check_matvec"](got, want, w, xm)
        extra = {"err": rel, "err_bound": bound, "argmax_equal": bool(np.array_equal(np.argmax(got, axis=1), [oracle.argmax(r.astype(np.float32)) for r in want]))}
        return env["hbm_entry"](2 * n * k + 2 * m * k + 4 * m * n, gpu_s, steps, extra)

    head["m1"] = decode(env, 1)
    for m in (4, 8):
        rest[f"m{m}"] = decode(env, m)
    wide = env["make_env"](env["Device"].WIDE_DECODE)
    for m in (1, 4, 8):
        rest[f"wide_m{m}"] = decode(wide, m)
    wide["close"]()
    mc = K.MatvecVariant(wg=512, lanes=64, rows=16)
    raw = synth.random_blocks(synth.rng(0xC8), "q8_0", n, k)
    for m, variant in ((1, None), (4, None), (4, mc), (8, mc)):
        rest[f"q8_0_m{m}" + ("_mc" if variant else "")] = _multi_token(env, TensorType.q8_0, oracle.Q8_0, raw, n, k, m, variant)
    # M = 128: the prefill multiply on the bf16 MFMA rung.
    rows = 128
    x = synth.activations(g, rows, k, bf16=True)
    kset.select_prefill(rec, K.Prefill.bf16_mfma_xbf16)
    xa = env["upload"](synth.to_bf16_bits(x))
    out = env["output"](4 * rows * n)
    p = P.MatmulBf16(rows=rows, n=n, k=k, col0=0, out_stride=n)
    copies = env["rotation"](2 * n * k)
    held, launches = [xa, out], []
    for _ in range(copies):
        wa = env["upload"](wbits)
        held.append(wa)
        launches.append(env["L"](b.add(K.Kernel.matmul_bf16, p, [xa, wa, out], K.Grid.tiles_y(K.div_ceil(n, 64), 16)), rows))
    b.finish()
    env["flush"]()
    _, gpu_s, steps = env["protocol"](launches)
    got = env["read"](out)[: rows * n].reshape(rows, n)
    kset.select_prefill(rec, K.Prefill.scalar_f32)
    env["release"](*held)
    want = oracle.matmul_f64(x, w)
    head["m128"] = env["hbm_entry"](2 * n * k + 2 * rows * k + 4 * rows * n, gpu_s, steps,
                                    {"err": float(np.max(np.abs(got - want)) / np.max(np.abs(want))),
                                     "argmax_rows_equal": int(np.count_nonzero(np.argmax(got, axis=1) == np.argmax(want, axis=1))), "rows": rows})
    return {"headline": head, **rest}


if __name__ == "__main__":
    sys.exit(main())
