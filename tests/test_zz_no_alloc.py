"""GPU check of nh_argmax_static, the greedy choice that allocates nothing: through the C ABI, against nh_argmax on the
same values, bit for bit (indices), on two calls in a row, the second over a smaller input (the array keeps the first
call's partials), then at the vocabulary of the benchmark, on ties, and past the limit it states."""
import ctypes

import numpy as np
import pytest

from neura_amd import NeuraError, _check

pytestmark = pytest.mark.gpu


def both(device, values):
    values = np.ascontiguousarray(values, dtype=np.float32)
    rows, n = values.shape
    held = device.upload(values)
    plain, static = device.alloc(rows * 4), device.alloc(rows * 4)
    _check(device.lib.nh_argmax(device.handle, held.pointer, rows, n, plain.pointer))
    _check(device.lib.nh_argmax_static(device.handle, held.pointer, rows, n, static.pointer))
    got = plain.numpy(np.uint32), static.numpy(np.uint32)
    for buffer in (held, plain, static):
        buffer.release()
    return got


def test_the_static_choice_answers_as_the_allocating_one(device):
    rng = np.random.default_rng(77)
    first = rng.standard_normal((8, 152064)).astype(np.float32)
    plain, static = both(device, first)
    assert np.array_equal(static, plain) and np.array_equal(static, first.argmax(axis=1))
    second = rng.standard_normal((3, 5000)).astype(np.float32)  # smaller: fewer rows, fewer sections, stale partials behind them
    plain, static = both(device, second)
    assert np.array_equal(static, plain) and np.array_equal(static, second.argmax(axis=1))
    ties = np.zeros((2, 4097), dtype=np.float32)
    ties[0, [9, 4096]] = 3.0
    ties[1, :] = -np.inf
    plain, static = both(device, ties)
    assert list(static) == list(plain) == [9, 0]  # the lowest index wins a tie
    widest = rng.standard_normal((64, 3000)).astype(np.float32)
    plain, static = both(device, widest)
    assert np.array_equal(static, plain)


def test_the_static_choice_refuses_what_its_array_cannot_hold(device):
    values = device.upload(np.zeros((65, 16), dtype=np.float32))
    out = device.alloc(65 * 4)
    with pytest.raises(NeuraError) as refused:
        _check(device.lib.nh_argmax_static(device.handle, values.pointer, 65, 16, out.pointer))
    assert "static scratch" in str(refused.value)
    values.release(), out.release()
