"""The reference's load-time sweep (src/tune/tune.zig) run over this backend: the sixteen
candidates of src/kernels/kernels.zig:372-381 and the matrix-core id the HIP backend adds to
them, under the device limits it reports."""
import time

import numpy as np
import pytest

from zllm_amd import cmd, synth, tune
from zllm_amd import kernels as K
from zllm_amd.kernels import MatvecVariant, TensorType

MC = MatvecVariant(wg=512, lanes=64, rows=16)


def test_candidates_under_the_limits():
    """Under WebGPU's default limits (src/kernels/kernels.zig:390-393) the reference's sixteen
    fit and the matrix-core id does not (512 threads); under the HIP backend's it does."""
    assert len(MatvecVariant.candidates) == 16 and MatvecVariant.candidates[0] == MatvecVariant()
    assert MatvecVariant.hip_candidates[:16] == MatvecVariant.candidates and MatvecVariant.hip_candidates[16] == MC
    web, hip = K.DeviceLimits(), K.DeviceLimits.hip()
    assert all(v.fits(web) for v in MatvecVariant.candidates) and not MC.fits(web)
    assert all(v.fits(hip) for v in MatvecVariant.hip_candidates)
    assert MC.id() == 0x00104010 and MC.group_rows() == 128
    # lanes = 64 suits Q8_0 alone in the reference; the matrix-core id every type its kernels take.
    assert MatvecVariant(lanes=64).suits(TensorType.q8_0) and not MatvecVariant(lanes=64).suits(TensorType.q4_k)
    assert all(MC.suits(t) for t in (TensorType.q8_0, TensorType.q3_k, TensorType.q4_k, TensorType.q5_k, TensorType.q6_k)) and not MC.suits(TensorType.bf16)


def test_rel_err_is_the_tuners():
    a = np.array([3.0, 4.0], dtype=np.float32)
    assert tune.rel_err(a, a) == 0.0
    assert abs(tune.rel_err(a + np.float32(0.5), a) - np.sqrt(0.5) / 5.0) < 1e-7
    assert tune.rel_err(np.array([np.nan], dtype=np.float32), a[:1]) == float("inf")
    assert tune.rel_err(a, np.zeros(2, dtype=np.float32)) == 5.0


def run_sweep(c, shapes, tokens, candidates, limits):
    sweep = tune.Sweep(c.rec, c.set, shapes, limits, tokens, candidates=candidates, max_rows=K.hip_decode_max_rows)
    while True:
        words = sweep.next()
        if words is None:
            return sweep
        t0 = time.perf_counter_ns()
        c.host.execute(words, [])
        sweep.done(time.perf_counter_ns() - t0)


@pytest.mark.gpu
def test_sweep_picks_the_matrix_cores_for_verify_steps(ctx):
    """The sweep at the widths the reference runs it (1 token, 2 where decoding speculates,
    src/generate.zig:360) and at a verify width of 4, over the stacked gate / up matrix of C3
    (Q4_K 28672 x 4096) and a Q8_0 14336 x 4096 matrix: no candidate is dropped (every id is
    within the tuner's 1e-5 of the default), at one token the matrix-core id loses, and at four
    tokens it wins both shapes."""
    c = ctx
    g = synth.rng(0x7E)
    shapes = []
    for t, n, k in ((TensorType.q4_k, 28672, 4096), (TensorType.q8_0, 14336, 4096)):
        raw = synth.random_blocks(g, t.name, n, k)
        shapes.append(tune.Shape(t, n, k, c.gpu_weights(t, raw, k), n))
    c.flush()
    winners = {}
    for tokens in (1, 2, 4):
        sweep = run_sweep(c, shapes, tokens, MatvecVariant.hip_candidates, K.DeviceLimits.hip())
        assert sweep.dropped == 0
        timed = {(s, v.id()) for s, v, _ in sweep.log}
        assert (0, MC.id()) in timed and (1, MC.id()) in timed
        # lanes = 64 candidates of the reference run on Q8_0 only: 12 + the id for Q4_K, 16 + the id for Q8_0.
        assert sum(1 for s, _, _ in sweep.log if s == 0) == 13 and sum(1 for s, _, _ in sweep.log if s == 1) == 17
        winners[tokens] = [sweep.variant(sh.type, sh.n, sh.k) for sh in shapes]
    assert all(not v.is_matrix_cores() for v in winners[1]), winners[1]
    assert all(v.is_matrix_cores() for v in winners[4]), winners[4]
    # Under the reference's own limits the id is never run: an unchanged tuner keeps the default kernels.
    sweep = run_sweep(c, shapes[:1], 2, MatvecVariant.hip_candidates, K.DeviceLimits())
    assert all(not v.is_matrix_cores() for _, v, _ in sweep.log) and len(sweep.log) == 12
