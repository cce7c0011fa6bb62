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


def test_the_static_choice_allocates_nothing_on_a_device_that_has_chosen_nothing_yet():
    """A handle opened here has no scratch yet and never calls nh_argmax: nh_argmax_static must answer from the static array
    alone.  The device's free memory (hipMemGetInfo) is the same before and after the calls, and the second call's values
    differ from the first's, so that partials left in the array cannot pass for fresh ones."""
    import neura_amd

    fresh = neura_amd.Device(0)
    hip = ctypes.CDLL("libamdhip64.so")

    def free_bytes():
        free, total = ctypes.c_size_t(), ctypes.c_size_t()
        assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
        return free.value

    rng = np.random.default_rng(78)
    first = rng.standard_normal((8, 152064)).astype(np.float32)
    second = rng.standard_normal((8, 152064)).astype(np.float32)
    held_first, held_second, out = fresh.upload(first), fresh.upload(second), fresh.alloc(8 * 4)
    fresh.sync()
    before = free_bytes()
    _check(fresh.lib.nh_argmax_static(fresh.handle, held_first.pointer, 8, 152064, out.pointer))
    assert np.array_equal(out.numpy(np.uint32), first.argmax(axis=1))
    _check(fresh.lib.nh_argmax_static(fresh.handle, held_second.pointer, 8, 152064, out.pointer))
    assert np.array_equal(out.numpy(np.uint32), second.argmax(axis=1))
    fresh.sync()
    assert free_bytes() == before
    for buffer in (held_first, held_second, out):
        buffer.release()
    fresh.close()


def test_the_static_choice_refuses_what_its_array_cannot_hold(device):
    values = device.upload(np.zeros((65, 16), dtype=np.float32))
    out = device.alloc(65 * 4)
    with pytest.raises(NeuraError) as refused:
        _check(device.lib.nh_argmax_static(device.handle, values.pointer, 65, 16, out.pointer))
    assert "static scratch" in str(refused.value)
    values.release(), out.release()
