"""Conversation checkpoints through the C ABI (sd_checkpoint_buffer / sd_checkpoint_copy / sd_checkpoint_clone /
sd_state_copy, reference gpu/kernels.cpp:3905-4041): what is saved comes back bit for bit, states are packed in the order
given, a strided part of a state is the numpy slice of it, and what does not fit or is not this device's is refused."""
import ctypes

import numpy as np
import pytest

from gpu_util import backend
from straydog_amd.backend import StraydogError

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    with backend() as handle:
        yield handle


def _host_bytes(pointer, count):
    return np.ctypeslib.as_array(ctypes.cast(pointer, ctypes.POINTER(ctypes.c_uint8)), shape=(count,))


def test_states_are_saved_packed_and_restored(gpu):
    rng = np.random.default_rng(5)
    sizes = [4096, 272 * 37, 4 * 1000]
    contents = [rng.integers(0, 256, size=n, dtype=np.uint8) for n in sizes]
    states = [gpu.upload(c) for c in contents]
    total = sum(sizes)
    checkpoint = gpu.checkpoint_buffer(total + 100)
    gpu.checkpoint_copy(True, [s.base() for s in states], checkpoint)
    assert np.array_equal(_host_bytes(checkpoint, total), np.concatenate(contents))       # packed, in the order given
    # another order packs another way
    gpu.checkpoint_copy(True, [states[2].base(), states[0].base()], checkpoint)
    assert np.array_equal(_host_bytes(checkpoint, sizes[2] + sizes[0]), np.concatenate([contents[2], contents[0]]))
    # a clone holds the same bytes; the states are overwritten and come back from the clone
    gpu.checkpoint_copy(True, [s.base() for s in states], checkpoint)
    clone = gpu.checkpoint_buffer(total + 100)
    gpu.checkpoint_clone(checkpoint, clone)
    for s, n in zip(states, sizes):
        gpu.write_buffer(s, 0, np.zeros(n, dtype=np.uint8))
    gpu.checkpoint_copy(False, [s.base() for s in states], clone)
    for s, c in zip(states, contents):
        assert np.array_equal(gpu.read_buffer(s, 0, np.uint8, c.size), c)
    gpu.checkpoint_release(clone)
    gpu.checkpoint_release(checkpoint)
    for s in states:
        gpu.release(s)


def test_refusals(gpu):
    state = gpu.upload(np.arange(1024, dtype=np.float32))
    small = gpu.checkpoint_buffer(1000)
    other = gpu.checkpoint_buffer(2000)
    with pytest.raises(StraydogError):
        gpu.checkpoint_copy(True, [state.base()], small)                    # 4096 bytes do not fit 1000
    with pytest.raises(StraydogError):
        gpu.checkpoint_copy(True, [state.base() + 16], other)               # not the base of an allocation
    with pytest.raises(StraydogError):
        gpu.checkpoint_copy(True, [state.base()], state.base())             # not a checkpoint buffer
    with pytest.raises(StraydogError):
        gpu.checkpoint_clone(small, other)                                  # sizes differ
    with pytest.raises(StraydogError):
        gpu.checkpoint_clone(small, small)
    with pytest.raises(StraydogError):
        gpu.checkpoint_release(state.base())
    host = np.zeros((4, 8), dtype=np.float32)
    with pytest.raises(StraydogError):
        gpu.state_copy(state.base(), 0, 4, 8, 4, host, 0, True)             # runs that overlap (pitch < width)
    with pytest.raises(StraydogError):
        gpu.state_copy(state.base(), 1000, 8, 8, 4, host, 0, True)          # past the state's end
    gpu.checkpoint_release(small)
    gpu.checkpoint_release(other)
    gpu.release(state)


def test_a_part_of_a_state_is_its_slice(gpu):
    # a K/V plane of 64 positions x 68 floats (272 bytes a row), two planes: positions 10..29 of the second plane; and an
    # indexer's pooled blocks, one run per column
    rng = np.random.default_rng(9)
    planes, positions, row = 2, 64, 68
    content = rng.standard_normal((planes, positions, row)).astype(np.float32)
    state = gpu.upload(content)
    part = np.empty((1, 20 * row), dtype=np.float32)
    gpu.state_copy(state.base(), (positions + 10) * row, 20 * row, 20 * row, 1, part, 10, True)
    assert np.array_equal(part.reshape(20, row), content[1, 10:30])
    columns, blocks = 16, 40
    pooled = rng.standard_normal((columns, blocks)).astype(np.float32)
    index_state = gpu.upload(pooled)
    some = np.empty((columns, 7), dtype=np.float32)
    gpu.state_copy(index_state.base(), 5, blocks, 7, columns, some, 0, True)
    assert np.array_equal(some, pooled[:, 5:12])
    # restoring writes the runs back and leaves the rest alone
    patch = rng.standard_normal((columns, 7)).astype(np.float32)
    gpu.state_copy(index_state.base(), 5, blocks, 7, columns, patch, 0, False)
    want = pooled.copy()
    want[:, 5:12] = patch
    assert np.array_equal(gpu.read_buffer(index_state, 0, np.float32, columns * blocks).reshape(columns, blocks), want)
    gpu.release(state)
    gpu.release(index_state)
