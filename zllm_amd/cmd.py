"""The command stream: how the zllm core drives a GPU host.

A twin of the reference's recorder (src/gpu/cmd.zig): little-endian u32 words,
each command headed by ``opcode | (words << 8)`` where ``words`` counts the
header; objects named by ids assigned densely from 0 per kind; addresses as two
words. Tests and the benchmark drive the HIP host with exactly the words zllm
would record.
"""
from __future__ import annotations

import enum
from dataclasses import dataclass

import numpy as np


class Op(enum.IntEnum):
    """src/gpu/cmd.zig:21-59."""

    create_buffer = 1
    write_buffer = 2
    create_kernel = 3
    create_bind_group = 5
    dispatch = 6
    copy_buffer = 7
    read_buffer = 8
    submit = 9
    destroy = 10
    clear_buffer = 11
    write_file = 12


class Usage(enum.IntFlag):
    """WebGPU GPUBufferUsage bits (src/gpu/cmd.zig:62-74)."""

    map_read = 1
    map_write = 2
    copy_src = 4
    copy_dst = 8
    index = 16
    vertex = 32
    uniform = 64
    storage = 128
    indirect = 256
    query_resolve = 512


class Kind(enum.IntEnum):
    buffer = 0
    pipeline = 1
    bind_group = 2


@dataclass(frozen=True)
class Binding:
    binding: int
    buffer: int
    size: int
    offset: int = 0


@dataclass(frozen=True)
class Completion:
    token: int
    status: int  # 0 ok, 1 failed


def split(v: int) -> list[int]:
    return [v & 0xFFFFFFFF, (v >> 32) & 0xFFFFFFFF]


def join(lo: int, hi: int) -> int:
    return (hi << 32) | lo


def header(op: int, words: int) -> int:
    return int(op) | (words << 8)


class DecodeError(Exception):
    pass


class Truncated(DecodeError):
    pass


class BadLength(DecodeError):
    pass


@dataclass
class Command:
    op: int
    args: list[int]

    def u64_at(self, i: int) -> int:
        return join(self.args[i], self.args[i + 1])


def iterate(words):
    """Walks a batch command by command, checking every header
    (src/gpu/cmd.zig:229-246)."""
    words = [int(w) for w in words]
    pos = 0
    while pos < len(words):
        n = words[pos] >> 8
        if n == 0:
            raise BadLength()
        if n > len(words) - pos:
            raise Truncated()
        yield Command(words[pos] & 0xFF, words[pos + 1 : pos + n])
        pos += n


class Recorder:
    """Appends commands (src/gpu/cmd.zig:98-203). Data handed to write_buffer,
    create_kernel and read_buffer must stay valid until the batch has executed;
    the recorder keeps a reference to each array until ``clear``."""

    def __init__(self) -> None:
        self.words: list[int] = []
        self.next = [0, 0, 0]
        self._keep: list[object] = []

    def batch(self) -> np.ndarray:
        return np.asarray(self.words, dtype=np.uint32)

    def clear(self) -> None:
        self.words = []
        self._keep = []

    def created(self, kind: Kind) -> int:
        return self.next[kind]

    def destroy_since(self, kind: Kind, first: int) -> None:
        for i in range(first, self.created(kind)):
            self.destroy(kind, i)

    def _alloc(self, kind: Kind) -> int:
        i = self.next[kind]
        self.next[kind] += 1
        return i

    def _put(self, op: Op, args: list[int]) -> None:
        self.words.append(header(op, len(args) + 1))
        self.words.extend(int(a) & 0xFFFFFFFF for a in args)

    def create_buffer(self, size: int, usage: Usage) -> int:
        i = self._alloc(Kind.buffer)
        self._put(Op.create_buffer, [i, *split(size), int(usage)])
        return i

    def write_buffer(self, buffer: int, offset: int, data) -> None:
        arr = np.ascontiguousarray(data)
        self._keep.append(arr)
        self._put(Op.write_buffer, [buffer, *split(offset), *split(arr.ctypes.data), *split(arr.nbytes)])

    def write_file(self, buffer: int, offset: int, file_offset: int, size: int) -> None:
        self._put(Op.write_file, [buffer, *split(offset), *split(file_offset), *split(size)])

    def create_kernel(self, kernel: int, variant: int, writes: int, artifact: bytes) -> int:
        i = self._alloc(Kind.pipeline)
        arr = np.frombuffer(bytes(artifact), dtype=np.uint8) if len(artifact) else np.zeros(1, dtype=np.uint8)
        self._keep.append(arr)
        self._put(Op.create_kernel, [i, kernel, variant, writes, *split(arr.ctypes.data), len(artifact)])
        return i

    def create_bind_group(self, pipeline: int, group: int, entries: list[Binding]) -> int:
        i = self._alloc(Kind.bind_group)
        args = [i, pipeline, group, len(entries)]
        for e in entries:
            args += [e.binding, e.buffer, *split(e.offset), *split(e.size)]
        self._put(Op.create_bind_group, args)
        return i

    def dispatch(self, pipeline: int, groups, bind_groups: list[int]) -> None:
        self._put(Op.dispatch, [pipeline, groups[0], groups[1], groups[2], len(bind_groups), *bind_groups])

    def copy_buffer(self, src: int, src_offset: int, dst: int, dst_offset: int, size: int) -> None:
        self._put(Op.copy_buffer, [src, *split(src_offset), dst, *split(dst_offset), *split(size)])

    def clear_buffer(self, buffer: int, offset: int, size: int) -> None:
        self._put(Op.clear_buffer, [buffer, *split(offset), *split(size)])

    def read_buffer(self, token: int, buffer: int, offset: int, dst: np.ndarray) -> None:
        assert dst.flags.c_contiguous and dst.flags.writeable
        self._keep.append(dst)
        self._put(Op.read_buffer, [token, buffer, *split(offset), *split(dst.nbytes), *split(dst.ctypes.data)])

    def submit(self, token: int) -> None:
        self._put(Op.submit, [token])

    def destroy(self, kind: Kind, obj: int) -> None:
        self._put(Op.destroy, [int(kind), obj])


def buffer_bytes(words, alignment: int) -> int:
    """Bytes of buffers created in this batch and still resident at its end
    (src/gpu/cmd.zig:248-283)."""
    assert alignment & (alignment - 1) == 0
    sizes: dict[int, int] = {}
    total = 0
    for c in iterate(words):
        if c.op == Op.create_buffer:
            if len(c.args) != 4 or c.args[0] in sizes:
                raise BadLength()
            size = c.u64_at(1) + alignment - 1
            if size >= 1 << 64:
                raise OverflowError()
            rounded = size & ~(alignment - 1)
            sizes[c.args[0]] = rounded
            total += rounded
            if total >= 1 << 64:
                raise OverflowError()
        elif c.op == Op.destroy:
            if len(c.args) != 2:
                raise BadLength()
            if c.args[0] == Kind.buffer and c.args[1] in sizes:
                total -= sizes.pop(c.args[1])
    return total
