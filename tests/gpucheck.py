"""A kernel-check context in the shape of the reference's own
(src/kernels/check.zig:98-203): seeded inputs, uploads, outputs, launches
through the recorder and reads back through the host."""
from __future__ import annotations

import numpy as np

from zllm_amd import Host, cmd
from zllm_amd import kernels as K


def rel_err(got: np.ndarray, want: np.ndarray) -> float:
    """max |got - want| / max |want|; infinite if any output is not finite
    (src/kernels/check.zig:205-222)."""
    got = np.asarray(got, dtype=np.float64).reshape(-1)
    want = np.asarray(want, dtype=np.float64).reshape(-1)
    assert got.shape == want.shape
    if not np.all(np.isfinite(got)):
        return float("inf")
    return float(np.max(np.abs(got - want)) / max(np.max(np.abs(want)), 1e-30))


def bound_err(got, want, w_rows: np.ndarray, x: np.ndarray) -> float:
    """max over outputs of |err| / (||row||2 * ||x||2): the acceptance bound is
    1e-3 of it. got/want are tokens x outputs, w_rows outputs x k, x tokens x k."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    if not np.all(np.isfinite(got)):
        return float("inf")
    wn = np.linalg.norm(np.asarray(w_rows, dtype=np.float64), axis=1)
    xn = np.linalg.norm(np.asarray(x, dtype=np.float64).reshape(got.shape[0], -1), axis=1)
    scale = np.maximum(xn[:, None] * wn[None, :], 1e-30)
    return float(np.max(np.abs(got - want) / scale))


class Ctx:
    def __init__(self, device, seed: int = 0x5EED):
        self.device = device
        self.host = Host(device)
        self.rec = cmd.Recorder()
        self.rand = np.random.Generator(np.random.PCG64(seed))
        self.token = 0
        self.set = K.Set.create(self.rec)
        self.flush()

    def flush(self) -> list:
        """Submits what is recorded and returns the completions."""
        self.token += 1
        self.rec.submit(self.token)
        done: list = []
        try:
            self.host.execute(self.rec.batch(), done)
        finally:
            self.rec.clear()
        return done

    def launcher(self) -> K.Launcher:
        return K.Launcher(self.rec, self.set)

    def random(self, n: int, scale: float) -> np.ndarray:
        """n floats uniform in [-scale, scale)."""
        return ((self.rand.random(n, dtype=np.float32) * 2 - 1) * np.float32(scale)).astype(np.float32)

    def upload(self, data) -> K.Arg:
        arr = np.ascontiguousarray(data)
        size = (arr.nbytes + 3) & ~3
        buf = self.rec.create_buffer(max(size, 4), cmd.Usage.storage | cmd.Usage.copy_dst | cmd.Usage.copy_src)
        if arr.nbytes:
            raw = arr.reshape(-1).view(np.uint8)
            if raw.size != size:
                raw = np.concatenate([raw, np.zeros(size - raw.size, dtype=np.uint8)])
            self.rec.write_buffer(buf, 0, raw)
        return K.Arg(buf, max(size, 4))

    def output(self, n_floats: int) -> K.Arg:
        buf = self.rec.create_buffer(max(4 * n_floats, 4), cmd.Usage.storage | cmd.Usage.copy_dst | cmd.Usage.copy_src)
        return K.Arg(buf, max(4 * n_floats, 4))

    def read_bytes(self, arg: K.Arg) -> np.ndarray:
        dst = np.zeros(arg.size, dtype=np.uint8)
        self.token += 1
        tok = self.token
        self.rec.read_buffer(tok, arg.buffer, arg.offset, dst)
        done = self.flush()
        assert any(c.token == tok and c.status == 0 for c in done)
        return dst

    def read(self, arg: K.Arg) -> np.ndarray:
        return self.read_bytes(arg).view(np.float32)

    def read_words(self, arg: K.Arg) -> np.ndarray:
        return self.read_bytes(arg).view(np.uint32)

    def gpu_weights(self, t: K.TensorType, raw: np.ndarray, k: int) -> K.Arg:
        """Uploads raw GGUF rows in the layout the quantized kernels read, laid
        out on the GPU as the model loader does (src/kernels/check.zig:483-497)."""
        raw = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
        e, b = K.LAYOUT[t]
        rows = raw.size // (k // e * b)
        padded = np.zeros((raw.size + 15) & ~15, dtype=np.uint8)
        padded[: raw.size] = raw
        src = self.upload(padded)
        if not K.needs_layout(t):
            return src
        out = self.output(((rows * K.row_bytes(t, k) + 15) & ~15) // 4)
        self.launcher().layout(t, src, out, rows, k)
        return out
