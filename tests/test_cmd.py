"""The command-stream encoding, as the reference's own tests pin it
(src/gpu/cmd.zig:285-392): recorded words decode back to the same commands,
the iterator rejects malformed batches, and the buffer footprint counts what
stays resident."""
import numpy as np
import pytest

from zllm_amd import cmd
from zllm_amd.cmd import Op, Usage


def test_recorder_output_decodes_back_to_the_same_commands():
    r = cmd.Recorder()
    data = np.array([1, 2, 3, 4], dtype=np.uint8)
    dst = np.zeros(8, dtype=np.uint8)
    buf = r.create_buffer(1 << 33, Usage.storage | Usage.copy_dst)
    r.write_buffer(buf, 16, data)
    pl = r.create_kernel(5, 2, 0b1000, b"wgsl")
    bg = r.create_bind_group(pl, 0, [cmd.Binding(0, buf, 64), cmd.Binding(3, buf, 1 << 32, offset=256)])
    r.dispatch(pl, (4, 2, 1), [bg])
    r.read_buffer(7, buf, 8, dst)
    r.clear_buffer(buf, 4, 1 << 32)
    r.write_file(buf, 1 << 32, (5 << 32) + 12, 3 << 31)
    r.submit(9)
    second = r.create_buffer(4, Usage.uniform)
    assert second == 1

    it = cmd.iterate(r.batch())
    c = next(it)
    assert c.op == Op.create_buffer and c.u64_at(1) == 1 << 33 and c.args[3] == 0x88  # copy_dst | storage
    c = next(it)
    assert c.op == Op.write_buffer and c.u64_at(1) == 16 and c.u64_at(5) == 4
    assert c.u64_at(3) == r._keep[0].ctypes.data
    c = next(it)
    assert c.op == Op.create_kernel and c.args[:4] == [0, 5, 2, 0b1000] and c.args[6] == 4
    c = next(it)
    assert c.op == Op.create_bind_group and c.args[3] == 2 and c.args[4 + 6] == 3
    assert cmd.join(c.args[4 + 6 + 4], c.args[4 + 6 + 5]) == 1 << 32
    c = next(it)
    assert c.op == Op.dispatch and c.args == [0, 4, 2, 1, 1, 0]
    c = next(it)
    assert c.op == Op.read_buffer and c.u64_at(6) == dst.ctypes.data
    c = next(it)
    assert c.op == Op.clear_buffer and c.u64_at(1) == 4 and c.u64_at(3) == 1 << 32
    c = next(it)
    assert c.op == Op.write_file and c.args[0] == 0 and c.u64_at(1) == 1 << 32 and c.u64_at(3) == (5 << 32) + 12 and c.u64_at(5) == 3 << 31
    c = next(it)
    assert c.op == Op.submit and c.args[0] == 9
    assert next(it).op == Op.create_buffer
    assert next(it, None) is None


def test_header_layout():
    # opcode | (words << 8), words counting the header (src/gpu/cmd.zig:8-16).
    r = cmd.Recorder()
    r.submit(3)
    assert r.batch().tolist() == [9 | (2 << 8), 3]
    r.clear()
    r.destroy(cmd.Kind.pipeline, 7)
    assert r.batch().tolist() == [10 | (3 << 8), 1, 7]


def test_iterator_rejects_zero_length_and_truncated_commands():
    with pytest.raises(cmd.BadLength):
        list(cmd.iterate([int(Op.submit)]))
    with pytest.raises(cmd.Truncated):
        list(cmd.iterate([cmd.header(Op.submit, 3), 1]))


def test_buffer_footprint_counts_resident_allocations_across_submits():
    r = cmd.Recorder()
    older = r.create_buffer(8, Usage.storage)
    r.clear()
    weights = r.create_buffer((1 << 32) + 4, Usage.storage)
    staging = r.create_buffer(65537, Usage.copy_dst)
    r.submit(0)
    r.destroy(cmd.Kind.buffer, staging)
    r.destroy(cmd.Kind.buffer, older)
    r.destroy(cmd.Kind.pipeline, weights)
    r.create_buffer(16, Usage.uniform)
    assert cmd.buffer_bytes(r.batch(), 1) == (1 << 32) + 20
    assert cmd.buffer_bytes(r.batch(), 65536) == (1 << 32) + 2 * 65536
    assert cmd.buffer_bytes([], 65536) == 0


def test_buffer_footprint_rejects_malformed_allocations_and_overflow():
    with pytest.raises(cmd.BadLength):
        cmd.buffer_bytes([cmd.header(Op.create_buffer, 2), 0], 1)
    with pytest.raises(cmd.BadLength):
        cmd.buffer_bytes([cmd.header(Op.destroy, 2), 0], 1)
    r = cmd.Recorder()
    r.create_buffer((1 << 64) - 1, Usage.storage)
    with pytest.raises(OverflowError):
        cmd.buffer_bytes(r.batch(), 65536)
    r.create_buffer(1, Usage.storage)
    with pytest.raises(OverflowError):
        cmd.buffer_bytes(r.batch(), 1)


def test_ids_are_dense_per_kind_and_survive_clear():
    r = cmd.Recorder()
    assert [r.create_buffer(4, Usage.storage) for _ in range(3)] == [0, 1, 2]
    assert r.create_kernel(1, 0, 8, b"") == 0
    r.clear()
    assert r.create_buffer(4, Usage.storage) == 3 and r.created(cmd.Kind.buffer) == 4
    r.destroy_since(cmd.Kind.buffer, 2)
    ops = [(c.op, c.args) for c in cmd.iterate(r.batch())]
    assert ops[-2:] == [(Op.destroy, [0, 2]), (Op.destroy, [0, 3])]
