"""Load-time tuning of the quantized decode multiplies, as the reference does it
(src/tune/tune.zig): for each (type, n, k) shape every MatvecVariant candidate the
device fits runs on the shape's real weights; each is checked against the default
variant first (relative L2 error above 1e-5: dropped), then timed, 3 warm-up
batches (the first is the correctness run) and the median of 7; the fastest per
shape is kept unless it is the default.

The same non-blocking state machine: the host runs each batch `next` returns and
passes its time to `done`, until `next` returns None. Times are of whole batches,
submission to completion; a batch repeats its dispatch clamp(256 MB / bytes, 2, 64)
times (tune.zig:94).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field

import numpy as np

from . import cmd
from . import kernels as K

TIMED = 7        # tune.zig:26
WARMUP = 3       # tune.zig:27
TOLERANCE = 1e-5  # tune.zig:30
READ_TOKEN = 0xFFFFFFFD  # tune.zig:218


@dataclass
class Shape:
    """One shape to tune: the first chunk of a matrix of its (type, n, k)."""

    type: K.TensorType
    n: int
    k: int
    chunk: K.Arg
    rows: int
    reps: int = 0

    def __post_init__(self):
        self.reps = int(min(max((256 << 20) // max(self.chunk.size, 1), 2), 64))


@dataclass
class Entry:
    type: K.TensorType
    n: int
    k: int
    variant: K.MatvecVariant


def rel_err(got: np.ndarray, want: np.ndarray) -> float:
    """tune.zig:220-231: relative L2 error; infinite on NaN."""
    d = got.astype(np.float64) - want.astype(np.float64)
    num, den = float(np.sum(d * d)), float(np.sum(want.astype(np.float64) ** 2))
    if math.isnan(num):
        return math.inf
    return math.sqrt(num) if den == 0 else math.sqrt(num / den)


@dataclass
class Sweep:
    rec: cmd.Recorder
    set: K.Set
    shapes: list
    limits: K.DeviceLimits
    tokens: int
    candidates: tuple = K.MatvecVariant.candidates
    max_rows: int = K.decode_max_rows
    entries: list = field(default_factory=list)
    dropped: int = 0
    log: list = field(default_factory=list)  # (shape index, variant, median ns) of every candidate timed

    def __post_init__(self):
        assert 1 <= self.tokens <= self.max_rows  # tune.zig:78
        self.candidates = tuple(v for v in self.candidates if v.fits(self.limits))
        assert self.candidates and self.candidates[0] == K.MatvecVariant()  # the default first: the reference the others must match
        self.shape = self.candidate = self.batch = 0
        self.times = [0] * TIMED
        self.diverged = False
        self.best = None
        if not self.shapes:
            return
        k_max, n_max = max(s.k for s in self.shapes), max(s.rows for s in self.shapes)
        usage = cmd.Usage.storage | cmd.Usage.copy_dst | cmd.Usage.copy_src
        self.x = K.Arg(self.rec.create_buffer(self.tokens * k_max * 4, usage), self.tokens * k_max * 4)
        self.out = K.Arg(self.rec.create_buffer(self.tokens * n_max * 4, usage), self.tokens * n_max * 4)
        self.params = K.Arg(self.rec.create_buffer(32, cmd.Usage.uniform | cmd.Usage.copy_dst), 32)
        # Deterministic inputs of RMS about 1, as normed activations are (tune.zig:134-136).
        self.rec.write_buffer(self.x.buffer, 0, np.sin(np.arange(self.tokens * k_max, dtype=np.float32) * np.float32(0.7)).astype(np.float32))
        self.reference = np.zeros(self.tokens * n_max, dtype=np.float32)
        self.got = np.zeros(self.tokens * n_max, dtype=np.float32)

    def next(self):
        """The next batch to run, or None when the sweep is done (tune.zig:141-172)."""
        if self.shape == len(self.shapes):
            return None
        sh, v = self.shapes[self.shape], self.candidates[self.candidate]
        if self.batch == 0:
            kernel = K.weight_kernel("matvec", sh.type)
            self.pipeline = self.set.matvec(self.rec, kernel, v)
            self.rec.write_buffer(self.params.buffer, 0, np.frombuffer(K.params.MatvecBf16(n=sh.rows, k=sh.k, col0=0, out_stride=sh.rows, eps=1e-6).pack(), dtype=np.uint8))
            x_bytes = self.tokens * sh.k * 4
            self.bind_group = K.bind_group(self.rec, self.pipeline, self.params,
                                           [K.Arg(self.x.buffer, x_bytes), sh.chunk, K.Arg(self.out.buffer, self.tokens * sh.rows * 4), K.Arg(self.x.buffer, x_bytes)])
        groups = (K.div_ceil(sh.rows, v.group_rows()), self.tokens, 1)
        for _ in range(1 if self.batch == 0 else sh.reps):
            self.rec.dispatch(self.pipeline, groups, [self.bind_group])
        if self.batch == 0:
            dst = self.reference if self.candidate == 0 else self.got
            self.rec.read_buffer(READ_TOKEN, self.out.buffer, 0, dst[: self.tokens * sh.rows])
        self.rec.submit(0)
        return self.rec.batch()

    def done(self, elapsed_ns: int) -> None:
        """The batch `next` returned ran in `elapsed_ns`, its readback done (tune.zig:175-208)."""
        self.rec.clear()
        sh = self.shapes[self.shape]
        n = self.tokens * sh.rows
        if self.batch == 0 and self.candidate > 0:
            self.diverged = rel_err(self.got[:n], self.reference[:n]) > TOLERANCE
        if self.batch >= WARMUP:
            self.times[self.batch - WARMUP] = elapsed_ns
        self.batch += 1
        if not self.diverged and self.batch < WARMUP + TIMED:
            return
        if self.diverged:
            self.dropped += 1
        else:
            ns = sorted(self.times)[TIMED // 2]
            self.log.append((self.shape, self.candidates[self.candidate], ns))
            if self.best is None or ns < self.best[1]:
                self.best = (self.candidates[self.candidate], ns)
        self.batch, self.diverged = 0, False
        self.candidate += 1
        while self.candidate < len(self.candidates) and not (self.candidates[self.candidate].suits(sh.type) and self.candidates[self.candidate].fits_rows(sh.rows)):
            self.candidate += 1
        if self.candidate < len(self.candidates):
            return
        best = self.best[0]
        if best != K.MatvecVariant():
            self.entries.append(Entry(sh.type, sh.n, sh.k, best))
        self.best, self.candidate = None, 0
        self.shape += 1

    def variant(self, t: K.TensorType, n: int, k: int) -> K.MatvecVariant:
        """plan.Tuning.matvec: the shape's winner, or the default."""
        for e in self.entries:
            if (e.type, e.n, e.k) == (t, n, k):
                return e.variant
        return K.MatvecVariant()
