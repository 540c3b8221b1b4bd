"""The entry point that allocates nothing (zhip_matmul_q8_0_float_no_alloc)
against the dispatch it is a variant of: matmul_q8_0_float in the bf16 rung with
f32-bound activations through zhip_execute. Same inputs, bit for bit the same
outputs, on two calls in a row of which the second is smaller, so that the
fixed scratch array still holds the first call's activations when the second
runs. The caller's own buffers come from the HIP runtime the library itself is
linked against (found among the process's mappings once the library is loaded);
the call must not allocate: the device's free memory is read before and after
every call, the first one in the context included, and each call runs before the
dispatch it is compared with, so nothing has warmed its kernels up.
"""
import ctypes as C

import numpy as np
import pytest

from gpucheck import Ctx, rel_err
from zllm_amd import Device, _lib, host, synth
from zllm_amd import kernels as K
from zllm_amd.kernels import Kernel, TensorType, params as P

pytestmark = pytest.mark.gpu


class Runtime:
    """hipMalloc / hipMemcpy / hipFree for the test's own operands."""

    def __init__(self):
        # The runtime libzllm_hip.so brought in, whatever its soname.
        with open("/proc/self/maps") as maps:
            paths = sorted({line.split()[-1] for line in maps if "libamdhip64.so" in line})
        assert paths, "libzllm_hip.so is loaded, so its HIP runtime must be mapped"
        self.hip = C.CDLL(paths[0])
        self.hip.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        self.hip.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
        self.hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        self.hip.hipFree.argtypes = [C.c_void_p]
        self.live = []

    def upload(self, arr) -> C.c_void_p:
        raw = np.ascontiguousarray(arr).reshape(-1).view(np.uint8)
        p = C.c_void_p()
        assert self.hip.hipMalloc(C.byref(p), max(raw.size, 16)) == 0
        self.live.append(p)
        assert self.hip.hipMemcpy(p, raw.ctypes.data, raw.size, 1) == 0
        return p

    def download(self, p, count: int) -> np.ndarray:
        out = np.empty(count, dtype=np.float32)
        assert self.hip.hipDeviceSynchronize() == 0
        assert self.hip.hipMemcpy(out.ctypes.data, p, out.nbytes, 2) == 0
        return out

    def free_bytes(self) -> int:
        """The device's free memory once everything launched has finished."""
        free, total = C.c_size_t(), C.c_size_t()
        assert self.hip.hipDeviceSynchronize() == 0
        assert self.hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
        return free.value

    def free(self):
        for p in self.live:
            self.hip.hipFree(p)
        self.live = []


def through_execute(c: Ctx, x, raw, init, rows, n, k, col0, stride, accumulate):
    """The existing entry point: one matmul_q8_0_float dispatch of variant 0xfffb0000; also
    returns the weights as repack_q8_0 laid them out on the GPU."""
    c.set.select_prefill(c.rec, K.Prefill.bf16_mfma)
    wa = c.gpu_weights(TensorType.q8_0, raw, k)
    out = c.upload(init)
    c.launcher().launch(Kernel.matmul_q8_0_float, P.MatmulQuant(rows=rows, n=n, k=k, col0=col0, out_stride=stride, accumulate=accumulate, k_slice=k),
                        [c.upload(x), wa, out], (K.div_ceil(n, 64), K.div_ceil(rows, 16), 1))
    got = c.read(out).copy()
    split_rows = c.read_bytes(wa)[: n * K.row_bytes(TensorType.q8_0, k)].copy()
    return got, split_rows


CASES = [
    # rows, n, k, col0, stride, accumulate: the first fills 3.2 MiB of the scratch array, the second 23 KiB of it
    (400, 200, 4096, 3, 211, 1),
    (37, 70, 320, 0, 70, 0),
]


def test_no_alloc_entry_matches_the_dispatch_twice_in_a_row():
    import oracle

    dev = Device.open(0)
    rt = Runtime()
    try:
        c = Ctx(dev)
        g = synth.rng(0xA110C)
        for rows, n, k, col0, stride, accumulate in CASES:
            x = synth.activations(g, rows, k)
            raw = synth.q8_0_rows(g, n, k)
            init = synth.activations(g, rows, stride)
            # The weights in split rows, laid out on the CPU: the new entry point runs first.
            split_rows = oracle.repack_q8_0(raw, n, k)
            dx, dw, do = rt.upload(x), rt.upload(split_rows), rt.upload(init)
            free_before = rt.free_bytes()
            r = _lib.lib.zhip_matmul_q8_0_float_no_alloc(dev.ctx, None, dx, dw, do, rows, n, k, col0, stride, accumulate)
            dev.check(r)
            assert rt.free_bytes() == free_before, "the call changed the device's free memory"
            got = rt.download(do, rows * stride)
            want, gpu_rows = through_execute(c, x, raw, init, rows, n, k, col0, stride, accumulate)
            assert gpu_rows.tobytes() == np.ascontiguousarray(split_rows).view(np.uint8).reshape(-1)[: gpu_rows.size].tobytes()
            assert got.tobytes() == want.tobytes(), (rows, n, k)
            # And the dispatch itself is the rung's arithmetic: both operands rounded to bf16.
            values = oracle.dequantize(oracle.Q8_0, raw, n * k).reshape(n, k)
            prod = synth.bf16_round(x).astype(np.float64) @ synth.bf16_round(values).astype(np.float64).T
            ref = prod + (init[:, col0 : col0 + n] if accumulate else 0)
            assert rel_err(got.reshape(rows, stride)[:, col0 : col0 + n], ref) <= 1e-5
        # More tokens than the fixed array holds: a clear error, nothing launched.
        cap = _lib.lib.zhip_no_alloc_capacity()
        assert cap == 8 << 20
        rows = cap // (2 * 4096) + 1
        r = _lib.lib.zhip_matmul_q8_0_float_no_alloc(dev.ctx, None, dx, dw, do, rows, 64, 4096, 0, 64, 0)
        assert r == -3
        with pytest.raises(host.BadCommand, match="scratch"):
            dev.check(r)
    finally:
        rt.free()
        dev.deinit()
