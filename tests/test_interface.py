"""The op interface and the C ABI without a GPU: kernel ordinals, contracts,
parameter blocks, layouts, variant ids and grids as the reference defines them
(src/kernels/kernels.zig), and the shared library exporting every symbol its
header declares."""
import ctypes
import os
import re
import struct

import numpy as np
import pytest

from zllm_amd import _lib, cmd
from zllm_amd import kernels as K
from zllm_amd.kernels import Kernel, TensorType, params as P

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "zllm_hip.h")).read()
    declared = set(re.findall(r"\b(zhip_[a-z0-9_]+)\s*\(", header))
    assert declared == set(_lib.EXPORTS)
    for name in declared:
        assert getattr(_lib.lib, name) is not None


def test_abi_struct_sizes_match_the_header():
    # zhip_caps: 4 u32, 4 u64, char[128], char[32]; zhip_timing: 4 u32, 2 u64.
    assert ctypes.sizeof(_lib.Caps) == 16 + 32 + 160
    assert ctypes.sizeof(_lib.CTiming) == 32 and ctypes.sizeof(_lib.CCompletion) == 8 and ctypes.sizeof(_lib.Options) == 8


def test_kernel_ordinals_follow_the_reference_enum():
    # src/kernels/kernels.zig:24-92 in declaration order.
    assert len(Kernel) == 57
    for name, ordinal in (("rmsnorm", 0), ("matmul_bf16", 1), ("matmul_reduce", 3), ("matvec_bf16", 4), ("silu_mul", 6), ("repad", 36),
                          ("repack_q8_0", 38), ("matvec_q8_0", 40), ("matvec_q4_k", 42), ("matmul_q8_0_float", 46), ("embed_q4_k", 53), ("embed_iq4_xs", 56)):
        assert int(Kernel[name]) == ordinal
        assert _lib.kernel_ordinal(name) == ordinal
    assert _lib.kernel_ordinal("no_such_kernel") == -1


def test_contracts():
    # src/kernels/kernels.zig:209-221.
    assert K.contract(Kernel.matmul_q8_0_float) == K.Contract(4, 0b1000)
    assert K.contract(Kernel.matvec_q8_0).reads(1) and not K.contract(Kernel.matvec_q8_0).reads(3)
    for k in Kernel:
        assert K.contract(k).writes != 0


def test_artifacts_name_the_kernel_and_missing_kernels_are_empty():
    assert K.artifact(Kernel.matvec_q4_k) == b"zhip:v1:matvec_q4_k:00000000"
    v = K.MatvecVariant(128, 16, 2)
    assert K.artifact(Kernel.matvec_q8_0, v) == b"zhip:v1:matvec_q8_0:%08x" % v.id()
    assert K.artifact(Kernel.rmsnorm) == b"" and K.artifact(Kernel.attn_split) == b""
    assert K.backend_source(Kernel.matvec_q4_k).startswith(b"zhip:src:matvec_q4_k:r")
    assert K.backend_source(Kernel.sample) == b""
    rec = cmd.Recorder()
    s = K.Set.create(rec)
    implemented = {Kernel.matvec_q8_0, Kernel.matvec_q4_k, Kernel.matvec_bf16, Kernel.matmul_bf16, Kernel.matmul_q8_0_float, Kernel.matmul_reduce,
                   Kernel.silu_mul, Kernel.repack_q8_0, Kernel.repad, Kernel.embed_q8_0, Kernel.embed_q4_k, Kernel.embed_bf16,
                   Kernel.matvec_q3_k, Kernel.matvec_q5_k, Kernel.matvec_q6_k, Kernel.embed_q3_k, Kernel.embed_q5_k, Kernel.embed_q6_k,
                   Kernel.repack_q3_k, Kernel.quantize_q8, Kernel.matmul_q8_0, Kernel.matmul_q3_k, Kernel.matmul_q4_k, Kernel.matmul_q5_k, Kernel.matmul_q6_k,
                   Kernel.matvec_f16, Kernel.matmul_f16, Kernel.embed_f16, Kernel.embed_iq4_xs}
    assert set(Kernel) - s.missing == implemented
    with pytest.raises(K.UnsupportedKernel):
        s.require_all()
    # One create_kernel per identity, variant 0, in enum order (src/kernels/kernels.zig:773-787).
    created = [c for c in cmd.iterate(rec.batch()) if c.op == cmd.Op.create_kernel]
    assert [c.args[1] for c in created] == list(range(57)) and all(c.args[2] == 0 for c in created)
    assert all(c.args[3] == K.contract(Kernel(c.args[1])).writes for c in created)


def test_params_blocks_are_the_reference_extern_structs():
    # src/kernels/kernels.zig:432-505: field order, little endian, multiples of 16.
    p = P.MatvecBf16(n=7, k=1024, col0=3, out_stride=100, eps=1e-6, norm=True, silu_pair=True, half=50, x_stride=66).pack()
    assert len(p) == 32
    assert struct.unpack("<IIIIfIII", p) == (7, 1024, 3, 100, pytest.approx(1e-6), 0b101, 50, 66)
    assert struct.unpack("<8I", P.MatmulQuant(rows=5, n=6, k=64, col0=1, out_stride=9, accumulate=1, k_slice=32, slice_stride=30).pack()) == (5, 6, 64, 1, 9, 1, 32, 30)
    assert struct.unpack("<8I", P.MatmulBf16(rows=5, n=6, k=64, col0=1, out_stride=9).pack()) == (5, 6, 64, 1, 9, 0, 0, 0)
    assert struct.unpack("<8I", P.MatmulReduce(rows=5, n=6, slices=2, col0=1, out_stride=9, accumulate=1, slice_stride=30).pack()) == (5, 6, 2, 1, 9, 1, 30, 0)
    assert len(P.SiluMul(10, 5).pack()) == 16 and len(P.RepackQ80(3, 64).pack()) == 16 and len(P.Repad(1, 110, 128).pack()) == 16


def test_layouts_and_split_policy():
    assert K.row_bytes(TensorType.q8_0, 4096) == 4352 and K.row_bytes(TensorType.q8_0, 96) == 112  # src/kernels/kernels.zig:157-160
    assert K.row_bytes(TensorType.q4_k, 4096) == 2304 and K.row_bytes(TensorType.bf16, 1024) == 2048
    assert K.needs_layout(TensorType.q8_0) and not K.needs_layout(TensorType.q4_k) and not K.needs_layout(TensorType.bf16)
    assert K.matmul_slices(4096, 4096) == K.Slices(8, 512)       # src/kernels/kernels.zig:289-295
    assert K.matmul_slices(28672, 4096) == K.Slices(2, 2048)
    assert K.matmul_slices(151936, 1024) == K.Slices(1, 1024)


def test_matvec_variant_ids_and_candidates():
    # src/kernels/kernels.zig:328-373.
    assert K.MatvecVariant().id() == 0 and K.MatvecVariant().group_rows() == 8
    v = K.MatvecVariant(128, 16, 2, 4)
    assert v.id() == (4 | 16 << 8 | 2 << 16 | 4 << 24) and v.group_rows() == 16
    assert K.MatvecVariant(act_div=300).id() >> 24 == 255
    assert len(K.MatvecVariant.candidates) == 16
    assert K.MatvecVariant(256, 64, 1).suits(TensorType.q8_0) and not K.MatvecVariant(256, 64, 1).suits(TensorType.q4_k)
    assert not K.MatvecVariant(256, 8, 1).fits_rows(8 * 65536 * 4)


def test_grids():
    # src/kernels/kernels.zig:985-1027.
    assert K.elementwise(256) == (1, 1, 1) and K.elementwise(257) == (2, 1, 1)
    assert K.elementwise(65535 * 256 + 1) == (65535, 2, 1)
    e = K.Extent(rows=37)
    assert K.Grid.rows_y(1792).resolve(e) == (1792, 37, 1)
    assert K.Grid.tiles_y(64, 16, 8).resolve(e) == (64, 3, 8)
    assert K.Grid.elems(100).resolve(e) == K.elementwise(3700)
    assert K.Grid.fixed_((3, 2, 1)).resolve(e) == (3, 2, 1)


def test_builder_packs_parameter_pages():
    """Parameter blocks go into 64 KiB uniform pages at 256-byte slots, uploaded
    by finish (src/kernels/kernels.zig:1046-1106)."""
    rec = cmd.Recorder()
    s = K.Set.create(rec)
    rec.clear()
    b = K.Builder(rec, s)
    a = K.Arg(99, 1024)
    l1 = b.add(Kernel.silu_mul, P.SiluMul(10, 5), [a, a], K.Grid.elems(5))
    l2 = b.add(Kernel.silu_mul, P.SiluMul(20, 5), [a, a], K.Grid.elems(5))
    b.finish()
    cs = list(cmd.iterate(rec.batch()))
    assert [c.op for c in cs] == [cmd.Op.create_buffer, cmd.Op.create_bind_group, cmd.Op.create_bind_group, cmd.Op.write_buffer]
    assert cs[0].u64_at(1) == 65536 and cs[0].args[3] == int(cmd.Usage.uniform | cmd.Usage.copy_dst)
    # Binding 0 of the two groups: the same page at offsets 0 and 256, 16 bytes each.
    assert (cs[1].args[4], cmd.join(*cs[1].args[6:8]), cmd.join(*cs[1].args[8:10])) == (0, 0, 16)
    assert (cs[2].args[4], cmd.join(*cs[2].args[6:8]), cmd.join(*cs[2].args[8:10])) == (0, 256, 16)
    assert cs[3].u64_at(5) == 512
    rec.clear()
    l2.record(rec, K.Extent(rows=300))
    l1.record(rec, K.Extent(rows=0))  # an empty grid records nothing
    d = list(cmd.iterate(rec.batch()))
    assert len(d) == 1 and d[0].args[:5] == [s.pipelines[Kernel.silu_mul], 6, 1, 1, 1]


def test_no_device_is_a_typed_error():
    """Without a gfx950 device the library still loads; opening a device fails
    with NoDevice rather than falling back to anything."""
    from zllm_amd import Device, host

    if os.path.exists("/dev/kfd"):
        pytest.skip("a GPU is present")
    with pytest.raises(host.NoDevice):
        Device.open(0)
