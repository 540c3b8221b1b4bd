"""Kernel identities, parameter blocks, contracts and launch builders.

A twin of the reference's op interface (src/kernels/kernels.zig) for the
quantized linear-layer path: the same kernel tag names and ordinals, the same
parameter blocks field for field, the same weight layouts, split-k policy,
MatvecVariant ids, and the same Launcher / Builder calls that turn a kernel,
its parameters, its buffers and a workgroup grid into command-stream words.
"""
from __future__ import annotations

import enum
import struct
from dataclasses import dataclass, field

import numpy as np

from . import cmd
from . import _lib

# kernels.Kernel in declaration order (src/kernels/kernels.zig:24-92).
KERNEL_NAMES = (
    "rmsnorm matmul_bf16 matmul_f16 matmul_reduce matvec_bf16 matvec_f16 silu_mul embed_bf16 embed_f16 "
    "rope_append attn_split attn_split_wide attn_split_sparse attn_combine qsa_keys qsa_pool qsa_score "
    "qsa_select delta_prep delta_rule gated_norm mark_tokens sample draft gyro_matvec gyro_matmul moe_group "
    "moe_logits moe_route rotate128 moe_combine hc_act hc_mix hc_combine ple_mix ple_conv repad repack_q3_k "
    "repack_q8_0 quantize_q8 matvec_q8_0 matvec_q3_k matvec_q4_k matvec_q5_k matvec_q6_k matmul_q8_0 "
    "matmul_q8_0_float matmul_q3_k matmul_q4_k matmul_q5_k matmul_q6_k embed_q8_0 embed_q3_k embed_q4_k "
    "embed_q5_k embed_q6_k embed_iq4_xs"
).split()

Kernel = enum.IntEnum("Kernel", {name: i for i, name in enumerate(KERNEL_NAMES)})


class TensorType(enum.IntEnum):
    """GGML storage types on this path (src/gguf/gguf.zig:17-46)."""

    f32 = 0
    f16 = 1
    q8_0 = 8
    q3_k = 11
    q4_k = 12
    q5_k = 13
    q6_k = 14
    iq4_xs = 23
    bf16 = 30


# (block_elems, block_bytes): src/gguf/gguf.zig:69-109.
LAYOUT = {TensorType.f32: (1, 4), TensorType.f16: (1, 2), TensorType.bf16: (1, 2), TensorType.q8_0: (32, 34), TensorType.q3_k: (256, 110), TensorType.q4_k: (256, 144),
          TensorType.q5_k: (256, 176), TensorType.q6_k: (256, 210), TensorType.iq4_xs: (256, 136)}


@dataclass(frozen=True)
class Contract:
    """A kernel's bindings (src/kernels/kernels.zig:181-188): 0 .. count - 1,
    binding 0 the params block; bit i of ``writes``: binding i is read_write."""

    count: int
    writes: int

    def reads(self, binding: int) -> bool:
        return binding < self.count and not (self.writes >> binding) & 1


# The contracts the reference parses out of its WGSL binding declarations, for
# the kernels of this path (src/kernels/*.wgsl; tests: kernels.zig:209-221).
CONTRACTS = {
    Kernel.matvec_q8_0: Contract(5, 0b01000),
    Kernel.matvec_q3_k: Contract(5, 0b01000),
    Kernel.matvec_q4_k: Contract(5, 0b01000),
    Kernel.matvec_q5_k: Contract(5, 0b01000),
    Kernel.matvec_q6_k: Contract(5, 0b01000),
    Kernel.matvec_bf16: Contract(5, 0b01000),
    Kernel.matvec_f16: Contract(5, 0b01000),
    Kernel.matmul_bf16: Contract(4, 0b1000),
    Kernel.matmul_f16: Contract(4, 0b1000),
    Kernel.matmul_q8_0_float: Contract(4, 0b1000),
    Kernel.matmul_q8_0: Contract(5, 0b01000),
    Kernel.matmul_q3_k: Contract(5, 0b01000),
    Kernel.matmul_q4_k: Contract(5, 0b01000),
    Kernel.matmul_q5_k: Contract(5, 0b01000),
    Kernel.matmul_q6_k: Contract(5, 0b01000),
    Kernel.quantize_q8: Contract(5, 0b01100),
    Kernel.matmul_reduce: Contract(3, 0b100),
    Kernel.silu_mul: Contract(3, 0b100),
    Kernel.repack_q8_0: Contract(3, 0b100),
    Kernel.repack_q3_k: Contract(3, 0b100),
    Kernel.repad: Contract(3, 0b100),
    Kernel.embed_q8_0: Contract(4, 0b1000),
    Kernel.embed_q3_k: Contract(4, 0b1000),
    Kernel.embed_q4_k: Contract(4, 0b1000),
    Kernel.embed_q5_k: Contract(4, 0b1000),
    Kernel.embed_q6_k: Contract(4, 0b1000),
    Kernel.embed_bf16: Contract(4, 0b1000),
    Kernel.embed_f16: Contract(4, 0b1000),
    Kernel.embed_iq4_xs: Contract(4, 0b1000),
}


def contract(k: Kernel) -> Contract:
    # Kernels outside this path keep a nonzero write set so a recorder can
    # still create their (missing) pipelines.
    return CONTRACTS.get(k, Contract(2, 0b10))


def is_template(k: Kernel) -> bool:
    """Whether the kernel takes a MatvecVariant (src/kernels/kernels.zig:111-116)."""
    return k in (Kernel.matvec_q8_0, Kernel.matvec_q3_k, Kernel.matvec_q4_k, Kernel.matvec_q5_k, Kernel.matvec_q6_k)


def weight_kernel(op: str, t: TensorType) -> Kernel:
    """Kernel.weight (src/kernels/kernels.zig:118-134): op in matvec/matmul/embed."""
    return Kernel[f"{op}_{t.name}"]


def block_stride(t: TensorType) -> int:
    """src/kernels/kernels.zig:144-151: the GGUF block size, padded to a multiple
    of 16 where it is not one (Q6_K: 210 -> 224, IQ4_XS: 136 -> 144, laid out by
    repad); Q3_K is repacked into eight 16-byte units (repack_q3_k)."""
    return {TensorType.q6_k: 224, TensorType.q3_k: 128, TensorType.iq4_xs: 144}.get(t, LAYOUT[t][1])


def row_bytes(t: TensorType, k: int) -> int:
    """Bytes per row of k weights as the kernels read it (src/kernels/kernels.zig:157-160)."""
    if t == TensorType.q8_0:
        return (k + k // 16 + 15) & ~15
    return k // LAYOUT[t][0] * block_stride(t)


def needs_layout(t: TensorType) -> bool:
    """src/kernels/kernels.zig:164-166."""
    return t == TensorType.q8_0 or block_stride(t) != LAYOUT[t][1]


def act_block(t: TensorType) -> int:
    """Activations per rounding block of the int8 prefill multiply for weights
    of type t (src/kernels/kernels.zig:301-303)."""
    return 32 if t == TensorType.q8_0 else 256


def is_half(t: TensorType) -> bool:
    return t in (TensorType.bf16, TensorType.f16)


matmul_tile_n, matmul_tile_t, matmul_tile_k = 64, 16, 32
matmul_quant_tile_n, matmul_quant_tile_t = 128, 32
matmul_target_groups, matmul_min_slice = 256, 512
decode_max_rows = 4
matvec_rows = 8
# Rows the HIP backend's decode multiplies accept (an extension of decode_max_rows).
hip_decode_max_rows = 8


def div_ceil(a: int, b: int) -> int:
    return -(-a // b)


@dataclass(frozen=True)
class Slices:
    count: int
    k_slice: int


def matmul_slices(n: int, k: int) -> Slices:
    """src/kernels/kernels.zig:289-295."""
    tiles = div_ceil(n, matmul_quant_tile_n)
    want = div_ceil(matmul_target_groups, tiles)
    count = min(max(want, 1), max(1, k // matmul_min_slice))
    k_slice = div_ceil(div_ceil(k, count), 32) * 32
    return Slices(div_ceil(k, k_slice), k_slice)


@dataclass(frozen=True)
class MatvecVariant:
    """A quantized decode multiply's tunables (src/kernels/kernels.zig:319-388)."""

    wg: int = 256
    lanes: int = 32
    rows: int = 1
    act_div: int = 0

    def id(self) -> int:
        if self == MatvecVariant():
            return 0
        return (self.wg // 32) | (self.lanes << 8) | (self.rows << 16) | (min(self.act_div, 255) << 24)

    def group_rows(self) -> int:
        return self.wg // self.lanes * self.rows

    def fits_rows(self, n: int) -> bool:
        return div_ceil(n, self.group_rows()) <= 65535

    def fits(self, d: "DeviceLimits") -> bool:
        """Whether the device runs it: threads per workgroup, and the WGSL kernel's workgroup
        memory (src/kernels/kernels.zig:343-345)."""
        return self.wg <= d.invocations and 2048 * 4 + 2 * self.wg * self.rows * 4 <= d.workgroup_storage

    def is_matrix_cores(self) -> bool:
        """The id that names this backend's matrix-core decode kernels (wg 512, lanes 64,
        rows 16: a geometry no WGSL variant has)."""
        return (self.wg, self.lanes, self.rows) == (512, 64, 16)

    def suits(self, t: TensorType) -> bool:
        """src/kernels/kernels.zig:355-357, and with the edit the HIP backend asks for: the
        matrix-core id suits every type its kernels take."""
        return self.lanes <= 32 or (t == TensorType.q8_0 and self.lanes == 64) or \
            (self.is_matrix_cores() and t in (TensorType.q8_0, TensorType.q3_k, TensorType.q4_k, TensorType.q5_k, TensorType.q6_k))


@dataclass(frozen=True)
class DeviceLimits:
    """Device limits kernel variants are checked against (src/kernels/kernels.zig:390-393:
    WebGPU's defaults); `hip()` is what the HIP backend reports (1024 threads a workgroup,
    160 KB of workgroup memory a CU), under which the matrix-core id fits."""

    invocations: int = 256
    workgroup_storage: int = 16384

    @classmethod
    def hip(cls) -> "DeviceLimits":
        return cls(invocations=1024, workgroup_storage=160 * 1024)


# The reference's sweep (src/kernels/kernels.zig:372-381), and the HIP backend's: the same
# sixteen and the matrix-core id.
MatvecVariant.candidates = tuple(
    MatvecVariant(wg=wg, lanes=lanes, rows=rows) for wg in (256, 128) for lanes in (32, 16, 8, 64) for rows in (1, 2)
)
MatvecVariant.hip_candidates = MatvecVariant.candidates + (MatvecVariant(wg=512, lanes=64, rows=16),)


# Reserved create_kernel variants of the prefill identities
# (src/agility/kernels.zig:114-131) and the HIP backend's bf16 MFMA rung.
class Prefill(enum.IntEnum):
    scalar_f32 = 0
    fp16_single = 1
    fp16_compensated = 2
    bf16_mfma = 3
    bf16_mfma_xbf16 = 4  # the same with activations bound as packed bf16


PREFILL_VARIANT = {Prefill.scalar_f32: 0, Prefill.fp16_single: 0xFFFC0000, Prefill.fp16_compensated: 0xFFFF0000, Prefill.bf16_mfma: 0xFFFB0000, Prefill.bf16_mfma_xbf16: 0xFFFA0000}
# The identities a prefill rung switches (src/agility/kernels.zig:111-112, without gyro_matmul).
# The bf16 rungs are this backend's own and leave matmul_f16 on the exact f32 kernel.
prefill_kernels = (Kernel.matmul_q8_0_float, Kernel.matmul_bf16, Kernel.matmul_f16)


def prefill_kernels_of(rung: "Prefill") -> tuple:
    if rung in (Prefill.bf16_mfma, Prefill.bf16_mfma_xbf16):
        return (Kernel.matmul_q8_0_float, Kernel.matmul_bf16)
    return prefill_kernels


class params:
    """The parameter blocks (src/kernels/kernels.zig:432-505): extern structs,
    little-endian, sizes multiples of 16."""

    @dataclass
    class MatvecBf16:
        n: int
        k: int
        col0: int
        out_stride: int
        eps: float = 0.0
        norm: bool = False
        accumulate: bool = False
        silu_pair: bool = False
        half: int = 0
        x_stride: int = 0

        def pack(self) -> bytes:
            flags = int(self.norm) | int(self.accumulate) << 1 | int(self.silu_pair) << 2
            return struct.pack("<IIIIfIII", self.n, self.k, self.col0, self.out_stride, self.eps, flags, self.half, self.x_stride)

    @dataclass
    class MatmulBf16:
        rows: int
        n: int
        k: int
        col0: int
        out_stride: int
        accumulate: int = 0

        def pack(self) -> bytes:
            return struct.pack("<8I", self.rows, self.n, self.k, self.col0, self.out_stride, self.accumulate, 0, 0)

    @dataclass
    class MatmulQuant:
        rows: int
        n: int
        k: int
        col0: int
        out_stride: int
        accumulate: int = 0
        k_slice: int = 0
        slice_stride: int = 0

        def pack(self) -> bytes:
            return struct.pack("<8I", self.rows, self.n, self.k, self.col0, self.out_stride, self.accumulate, self.k_slice, self.slice_stride)

    @dataclass
    class QuantizeQ8:
        """src/kernels/kernels.zig:495-501. mode: 0 x, 1 RMSNorm(x) * w, 2 silu(gate) * up."""
        k: int
        block: int
        mode: int = 0
        eps: float = 0.0

        def pack(self) -> bytes:
            return struct.pack("<3If", self.k, self.block, self.mode, self.eps)

    @dataclass
    class MatmulReduce:
        rows: int
        n: int
        slices: int
        col0: int
        out_stride: int
        accumulate: int = 0
        slice_stride: int = 0

        def pack(self) -> bytes:
            return struct.pack("<8I", self.rows, self.n, self.slices, self.col0, self.out_stride, self.accumulate, self.slice_stride, 0)

    @dataclass
    class SiluMul:
        count: int
        width: int

        def pack(self) -> bytes:
            return struct.pack("<4I", self.count, self.width, 0, 0)

    @dataclass
    class RepackQ80:
        rows: int
        k: int

        def pack(self) -> bytes:
            return struct.pack("<4I", self.rows, self.k, 0, 0)

    @dataclass
    class RepackQ3K:
        blocks: int

        def pack(self) -> bytes:
            return struct.pack("<4I", self.blocks, 0, 0, 0)

    @dataclass
    class Repad:
        blocks: int
        src_bytes: int
        dst_bytes: int

        def pack(self) -> bytes:
            return struct.pack("<4I", self.blocks, self.src_bytes, self.dst_bytes, 0)

    @dataclass
    class EmbedBf16:
        dim: int
        row0: int
        chunk_rows: int
        stride: int = 0

        def pack(self) -> bytes:
            return struct.pack("<4I", self.dim, self.row0, self.chunk_rows, self.stride)


def artifact(k: Kernel, v: MatvecVariant | int = 0) -> bytes:
    """The HIP backend's artifact for kernel ``k`` (the backend arm of
    kernels.artifact, src/kernels/kernels.zig:904-912): empty when the backend
    does not implement it."""
    variant = v.id() if isinstance(v, MatvecVariant) else int(v)
    return _lib.kernel_artifact(k.name, variant)


def backend_source(k: Kernel) -> bytes:
    """What the plan cache's key hashes (src/kernels/kernels.zig:914-922)."""
    return _lib.backend_source(k.name)


class UnsupportedKernel(Exception):
    pass


class Set:
    """One pipeline per kernel, plus the decode-multiply variants and prefill
    rungs asked for (src/kernels/kernels.zig:748-839)."""

    def __init__(self) -> None:
        self.pipelines: dict[Kernel, int] = {}
        self.missing: set[Kernel] = set()
        self.variants: dict[tuple[Kernel, MatvecVariant], int] = {}
        self.scalar_prefill: dict[Kernel, int] = {}
        self.prefill_variants: dict[tuple[Prefill, Kernel], int] = {}

    @classmethod
    def create(cls, rec: cmd.Recorder) -> "Set":
        s = cls()
        for k in Kernel:
            code = artifact(k)
            if not code:
                s.missing.add(k)
            s.pipelines[k] = rec.create_kernel(int(k), 0, contract(k).writes, code)
        for k in prefill_kernels:
            s.scalar_prefill[k] = s.pipelines[k]
        return s

    def require_all(self) -> None:
        if self.missing:
            raise UnsupportedKernel(", ".join(sorted(k.name for k in self.missing)))

    def select_prefill(self, rec: cmd.Recorder, rung: Prefill) -> None:
        """Switches the prefill identities' pipelines without changing their
        contracts or grids (src/kernels/kernels.zig:798-822)."""
        if rung == Prefill.scalar_f32:
            for k in prefill_kernels:
                self.pipelines[k] = self.scalar_prefill[k]
            return
        for k in prefill_kernels:
            self.pipelines[k] = self.scalar_prefill[k]
        for k in prefill_kernels_of(rung):
            if (rung, k) not in self.prefill_variants:
                self.prefill_variants[(rung, k)] = rec.create_kernel(int(k), PREFILL_VARIANT[rung], contract(k).writes, artifact(k, PREFILL_VARIANT[rung]))
        for k in prefill_kernels_of(rung):
            self.pipelines[k] = self.prefill_variants[(rung, k)]

    def matvec(self, rec: cmd.Recorder, k: Kernel, v: MatvecVariant) -> int:
        if v == MatvecVariant():
            return self.pipelines[k]
        if (k, v) not in self.variants:
            self.variants[(k, v)] = rec.create_kernel(int(k), v.id(), contract(k).writes, artifact(k, v))
        return self.variants[(k, v)]


@dataclass(frozen=True)
class Arg:
    """A buffer range bound at binding 1, 2, ... in kernel order."""

    buffer: int
    size: int
    offset: int = 0


def bind_group(rec: cmd.Recorder, pipeline: int, uniform: Arg, args: list[Arg]) -> int:
    entries = [cmd.Binding(0, uniform.buffer, uniform.size, uniform.offset)]
    entries += [cmd.Binding(i, a.buffer, a.size, a.offset) for i, a in enumerate(args, 1)]
    return rec.create_bind_group(pipeline, 0, entries)


def elementwise(count: int) -> tuple[int, int, int]:
    """Workgroup grid for ``count`` threads at 256 per group, folded into y
    past 65535 (src/kernels/kernels.zig:985-991)."""
    groups = div_ceil(count, 256)
    if groups <= 65535:
        return (groups, 1, 1)
    return (65535, div_ceil(groups, 65535), 1)


class Launcher:
    """Records kernel launches (src/kernels/kernels.zig:941-992)."""

    def __init__(self, rec: cmd.Recorder, kset: Set) -> None:
        self.rec = rec
        self.set = kset

    def launch(self, kernel: Kernel, p, args: list[Arg], groups) -> None:
        self.launch_pipeline(self.set.pipelines[kernel], p, args, groups)

    def launch_pipeline(self, pipeline: int, p, args: list[Arg], groups) -> None:
        data = np.frombuffer(p.pack(), dtype=np.uint8)
        assert data.size % 16 == 0
        ub = self.rec.create_buffer(data.size, cmd.Usage.uniform | cmd.Usage.copy_dst)
        self.rec.write_buffer(ub, 0, data)
        bg = bind_group(self.rec, pipeline, Arg(ub, data.size), args)
        self.rec.dispatch(pipeline, groups, [bg])

    def layout(self, t: TensorType, src: Arg, dst: Arg, rows: int, k: int) -> None:
        """Lays out raw GGUF rows as the quantized kernels read them
        (src/kernels/kernels.zig:972-983)."""
        e, b = LAYOUT[t]
        blocks = rows * k // e
        if t == TensorType.q8_0:
            self.launch(Kernel.repack_q8_0, params.RepackQ80(rows, k), [src, dst], elementwise(rows * row_bytes(t, k) // 4))
        elif t == TensorType.q3_k:
            self.launch(Kernel.repack_q3_k, params.RepackQ3K(blocks), [src, dst], elementwise(blocks * 8))
        else:
            stride = block_stride(t)
            self.launch(Kernel.repad, params.Repad(blocks, b, stride), [src, dst], elementwise(blocks * stride // 4))


@dataclass(frozen=True)
class Extent:
    rows: int
    keys: int = 0


@dataclass(frozen=True)
class Grid:
    """How a prebuilt launch's grid follows the step's extent
    (src/kernels/kernels.zig:999-1027)."""

    kind: str
    x: int = 0
    tile: int = 1
    z: int = 1
    fixed: tuple[int, int, int] = (0, 0, 0)

    @staticmethod
    def fixed_(g) -> "Grid":
        return Grid("fixed", fixed=tuple(g))

    @staticmethod
    def rows_y(x: int) -> "Grid":
        return Grid("rows_y", x=x)

    @staticmethod
    def tiles_y(x: int, tile: int, z: int = 1) -> "Grid":
        return Grid("tiles_y", x=x, tile=tile, z=z)

    @staticmethod
    def elems(width: int) -> "Grid":
        return Grid("elems", x=width)

    def resolve(self, e: Extent) -> tuple[int, int, int]:
        if self.kind == "fixed":
            return self.fixed
        if self.kind == "rows_x":
            return (e.rows, 1, 1)
        if self.kind == "rows_y":
            return (self.x, e.rows, 1)
        if self.kind == "tiles_y":
            return (self.x, div_ceil(e.rows, self.tile), self.z)
        if self.kind == "elems":
            return elementwise(e.rows * self.x)
        raise ValueError(self.kind)


@dataclass
class Launch:
    """A launch whose bind group is built once; each step only dispatches it
    (src/kernels/kernels.zig:1031-1044)."""

    kernel: Kernel
    pipeline: int
    bind_group: int
    grid: Grid

    def record(self, rec: cmd.Recorder, e: Extent) -> None:
        g = self.grid.resolve(e)
        if 0 in g:
            return
        rec.dispatch(self.pipeline, g, [self.bind_group])


class Builder:
    """Builds Launches; parameter blocks are packed into 64 KiB uniform buffers
    at 256-byte slots, uploaded by ``finish`` (src/kernels/kernels.zig:1046-1106)."""

    page_size = 64 * 1024
    slot = 256

    def __init__(self, rec: cmd.Recorder, kset: Set) -> None:
        self.rec = rec
        self.set = kset
        self.pages: list[list] = []  # [buffer, bytearray, used]

    def _param(self, p) -> Arg:
        data = p.pack()
        assert len(data) % 16 == 0 and len(data) <= self.slot
        if not self.pages or self.pages[-1][2] == self.page_size:
            buf = self.rec.create_buffer(self.page_size, cmd.Usage.uniform | cmd.Usage.copy_dst)
            self.pages.append([buf, bytearray(self.page_size), 0])
        page = self.pages[-1]
        page[1][page[2] : page[2] + len(data)] = data
        arg = Arg(page[0], len(data), page[2])
        page[2] += self.slot
        return arg

    def add(self, kernel: Kernel, p, args: list[Arg], grid: Grid) -> Launch:
        return self.add_with(kernel, self._param(p), args, grid)

    def add_with(self, kernel: Kernel, uniform: Arg, args: list[Arg], grid: Grid) -> Launch:
        return self._add_pipeline(kernel, self.set.pipelines[kernel], uniform, args, grid)

    def add_matvec(self, kernel: Kernel, v: MatvecVariant, p, args: list[Arg], grid: Grid) -> Launch:
        return self._add_pipeline(kernel, self.set.matvec(self.rec, kernel, v), self._param(p), args, grid)

    def _add_pipeline(self, kernel: Kernel, pipeline: int, uniform: Arg, args: list[Arg], grid: Grid) -> Launch:
        return Launch(kernel, pipeline, bind_group(self.rec, pipeline, uniform, args), grid)

    def finish(self) -> None:
        for buf, data, used in self.pages:
            self.rec.write_buffer(buf, 0, np.frombuffer(bytes(data[:used]), dtype=np.uint8))
