"""neura_amd: Python binding of libneura_hip.so, the MI355X implementation of Neura's
quantized-GGUF decoder path.  Everything here goes through the C ABI of include/neura_hip.h;
numpy arrays are host buffers only.  A failed call raises NeuraError with the library's
message, where the reference panics with prose."""
import ctypes

import numpy as np

from . import _abi
from ._abi import NH_F16, NH_F32, NH_Q3_K, NH_Q4_K, NH_Q5_K, NH_Q6_K, NH_Q8_0, UINT64_MAX, Epilogue, ModelConfig, TensorTable

BLOCK = {NH_Q8_0: (32, 34), NH_Q3_K: (256, 110), NH_Q4_K: (256, 144), NH_Q5_K: (256, 176), NH_Q6_K: (256, 210), NH_F16: (1, 2), NH_F32: (1, 4)}  # elements, bytes


class NeuraError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(message)
        self.code = code


def payload_bytes(element, elements):
    """Element::payload_bytes (crates/neura-abi/src/element.rs:231-240)."""
    per, size = BLOCK[element]
    return -(-elements // per) * size


def _check(status):
    if status != 0:
        raise NeuraError(status, _abi.library().nh_last_error().decode())


class Buffer:
    """Device memory owned by a Device (freed with the device or by release())."""

    def __init__(self, device, pointer, nbytes):
        self.device, self.pointer, self.nbytes = device, pointer, nbytes

    def release(self):
        if self.pointer:
            _check(self.device.lib.nh_free(self.device.handle, self.pointer))
            self.pointer = None

    def numpy(self, dtype, shape=None):
        out = np.empty(self.nbytes // np.dtype(dtype).itemsize, dtype=dtype)
        _check(self.device.lib.nh_download(self.device.handle, out.ctypes.data, self.pointer, out.nbytes))
        return out.reshape(shape) if shape is not None else out


class Device:
    """Runtime::open (crates/neura-runtime/src/runtime.rs:183)."""

    def __init__(self, index=0):
        self.lib = _abi.library()
        self.handle = self.lib.nh_open(index)
        if not self.handle:
            raise NeuraError(_abi.NH_E_DEVICE, self.lib.nh_last_error().decode())
        self._buffers = []

    def close(self):
        if self.handle:
            for held in self._buffers:
                if held.pointer:
                    self.lib.nh_free(self.handle, held.pointer)
                    held.pointer = None
            self.lib.nh_close(self.handle)
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    # ---- memory
    def alloc(self, nbytes):
        pointer = self.lib.nh_alloc(self.handle, nbytes)
        if not pointer:
            raise NeuraError(_abi.NH_E_MEMORY, self.lib.nh_last_error().decode())
        held = Buffer(self, pointer, nbytes)
        self._buffers.append(held)
        return held

    def upload(self, array):
        array = np.ascontiguousarray(array)
        held = self.alloc(max(array.nbytes, 4))
        if array.nbytes:
            _check(self.lib.nh_upload(self.handle, held.pointer, array.ctypes.data, array.nbytes))
        held.nbytes = array.nbytes
        return held

    def sync(self):
        _check(self.lib.nh_sync(self.handle))

    def timer_start(self):
        _check(self.lib.nh_timer_start(self.handle))

    def timer_stop(self):
        seconds = ctypes.c_double()
        _check(self.lib.nh_timer_stop(self.handle, ctypes.byref(seconds)))
        return seconds.value

    def profile_begin(self):
        _check(self.lib.nh_profile_begin(self.handle))

    def profile_end(self):
        """(device seconds, launches, weight bytes) of the narrow products since profile_begin"""
        seconds, launches, nbytes = ctypes.c_double(), ctypes.c_uint64(), ctypes.c_uint64()
        _check(self.lib.nh_profile_end(self.handle, ctypes.byref(seconds), ctypes.byref(launches), ctypes.byref(nbytes)))
        return seconds.value, launches.value, nbytes.value

    # ---- operators (numpy in, numpy out unless a Buffer is passed)
    def _dev(self, value):
        return value if isinstance(value, Buffer) else self.upload(value)

    def dequant(self, element, raw, elements):
        src = self._dev(raw)
        out = self.alloc(elements * 4)
        _check(self.lib.nh_dequant(self.handle, element, src.pointer, elements, out.pointer))
        return out.numpy(np.float32)

    def convert_half(self, values):
        src = self._dev(np.asarray(values, dtype=np.float32))
        n = src.nbytes // 4
        out = self.alloc(n * 2)
        _check(self.lib.nh_convert_half(self.handle, src.pointer, n, out.pointer))
        return out.numpy(np.uint16)

    def pack_q8_0(self, values):
        """fp32 numbers into Q8_0 blocks on the device; the bytes end on a four-byte word"""
        src = self._dev(np.asarray(values, dtype=np.float32))
        n = src.nbytes // 4
        out = self.alloc(((n + 31) // 32 * 34 + 3) // 4 * 4)
        _check(self.lib.nh_pack_q8_0(self.handle, src.pointer, n, out.pointer))
        return out.numpy(np.uint8)

    def gemv(self, element, W, N, K, x, residual=None, swiglu=False, out=None):
        W, x = self._dev(W), self._dev(np.asarray(x, dtype=np.float32))
        rows = x.nbytes // 4 // K
        outputs = N // 2 if swiglu else N
        y = out if out is not None else self.alloc(rows * outputs * 4)
        epilogue = None
        if residual is not None or swiglu:
            held = self._dev(np.asarray(residual, dtype=np.float32)) if residual is not None else None
            epilogue = Epilogue(held.pointer if held else None, 1 if swiglu else 0)
        _check(self.lib.nh_gemv(self.handle, element, W.pointer, N, K, x.pointer, rows, y.pointer,
                                ctypes.byref(epilogue) if epilogue else None))
        return y.numpy(np.float32, (rows, outputs)) if out is None else y

    def gemm(self, element, W, N, K, X, residual=None, out=None):
        X = X if isinstance(X, Buffer) else np.ascontiguousarray(X)
        if isinstance(X, Buffer):
            raise TypeError("gemm takes a numpy activation matrix")
        x_element = NH_F16 if X.dtype == np.float16 else NH_F32
        if x_element == NH_F32:
            X = X.astype(np.float32, copy=False)
        M = X.size // K
        W, Xd = self._dev(W), self.upload(X)
        y = out if out is not None else self.alloc(M * N * 4)
        epilogue = None
        if residual is not None:
            held = self._dev(np.asarray(residual, dtype=np.float32))
            epilogue = Epilogue(held.pointer, 0)
        _check(self.lib.nh_gemm(self.handle, element, W.pointer, N, K, Xd.pointer, x_element, M, y.pointer,
                                ctypes.byref(epilogue) if epilogue else None))
        return y.numpy(np.float32, (M, N)) if out is None else y

    def rmsnorm(self, x, w, eps, residual=None, want_sum=False):
        x = np.ascontiguousarray(x, dtype=np.float32)
        rows, C = x.shape
        xd, wd = self.upload(x), (self.upload(np.asarray(w, dtype=np.float32)) if w is not None else None)
        rd = self.upload(np.asarray(residual, dtype=np.float32)) if residual is not None else None
        out = self.alloc(x.nbytes)
        total = self.alloc(x.nbytes) if want_sum else None
        _check(self.lib.nh_rmsnorm(self.handle, xd.pointer, rd.pointer if rd else None, wd.pointer if wd else None, eps, rows, C,
                                   out.pointer, total.pointer if total else None))
        result = out.numpy(np.float32, (rows, C))
        return (result, total.numpy(np.float32, (rows, C))) if want_sum else result

    def rope(self, x, cursor, base):
        x = np.ascontiguousarray(x, dtype=np.float32)
        planes, batch, rows, width = x.shape
        xd = self.upload(x)
        cd = self.upload(np.asarray(cursor, dtype=np.uint32)) if cursor is not None else None
        out = self.alloc(x.nbytes)
        _check(self.lib.nh_rope(self.handle, xd.pointer, planes, batch, rows, width, cd.pointer if cd else None, base, out.pointer))
        return out.numpy(np.float32, x.shape)

    def cache_write(self, k, v, cache_k, cache_v, capacity, window, cursor, mask=None, ring=False, element=NH_F16):
        k = np.ascontiguousarray(k, dtype=np.float32)
        v = np.ascontiguousarray(v, dtype=np.float32)
        kv_heads, batch, rows, width = k.shape
        kd, vd = self.upload(k), self.upload(v)
        cd = self.upload(np.asarray(cursor, dtype=np.uint32))
        md = self.upload(np.asarray(mask, dtype=np.uint8)) if mask is not None else None
        if element == NH_F16:
            _check(self.lib.nh_cache_write(self.handle, kd.pointer, vd.pointer, cache_k.pointer, cache_v.pointer, kv_heads, batch, rows, width,
                                           capacity, window, cd.pointer, md.pointer if md else None, 1 if ring else 0))
        else:
            _check(self.lib.nh_cache_write_element(self.handle, kd.pointer, vd.pointer, cache_k.pointer, cache_v.pointer, kv_heads, batch, rows,
                                                   width, capacity, window, cd.pointer, md.pointer if md else None, 1 if ring else 0, element))

    def attention(self, q, cache_k, cache_v, kv_heads, capacity, keys, cursor, scale, reach=0, element=NH_F16):
        q = np.ascontiguousarray(q, dtype=np.float32)
        heads, batch, rows, width = q.shape
        qd = self.upload(q)
        kd, vd = self._dev(cache_k), self._dev(cache_v)
        cd = self.upload(np.asarray(cursor, dtype=np.uint32))
        out = self.alloc(q.nbytes)
        if element == NH_F16:
            _check(self.lib.nh_attention(self.handle, qd.pointer, kd.pointer, vd.pointer, heads, kv_heads, batch, rows, width, capacity, keys, reach,
                                         cd.pointer, scale, out.pointer))
        else:
            _check(self.lib.nh_attention_element(self.handle, qd.pointer, kd.pointer, vd.pointer, heads, kv_heads, batch, rows, width, capacity, keys,
                                                 reach, cd.pointer, scale, out.pointer, element))
        return out.numpy(np.float32, q.shape)

    def gather(self, element, table, vocab, width, tokens, batch=1, mask=None):
        td = self._dev(table)
        tokens = np.ascontiguousarray(tokens, dtype=np.uint32)
        kd = self.upload(tokens)
        md = self.upload(np.asarray(mask, dtype=np.uint8)) if mask is not None else None
        out = self.alloc(tokens.size * width * 4)
        _check(self.lib.nh_gather(self.handle, element, td.pointer, vocab, width, kd.pointer, tokens.size, batch,
                                  md.pointer if md else None, out.pointer))
        return out.numpy(np.float32, (tokens.size, width))

    def argmax(self, values):
        values = np.ascontiguousarray(values, dtype=np.float32)
        rows, n = values.shape
        vd = self.upload(values)
        out = self.alloc(rows * 4)
        _check(self.lib.nh_argmax(self.handle, vd.pointer, rows, n, out.pointer))
        return out.numpy(np.uint32)

    def sample(self, values, draws):
        """one column per row of `values`, drawn with the records of `draws` (dtype DRAW)"""
        values = np.ascontiguousarray(values, dtype=np.float32)
        draws = np.ascontiguousarray(draws, dtype=DRAW)
        rows, n = values.shape
        assert draws.size == rows
        vd = self.upload(values)
        out = self.alloc(max(rows, 1) * 4)
        _check(self.lib.nh_sample(self.handle, vd.pointer, rows, n, draws.ctypes.data, out.pointer))
        return out.numpy(np.uint32)[:rows]


# one row's draw, laid out as nh_draw: seed bits, temperature, candidates kept, cumulative mass
DRAW = np.dtype([("seed", np.uint32), ("temperature", np.float32), ("keep", np.uint32), ("cumulative", np.float32)])

__all__ = ["Device", "DRAW", "Buffer", "NeuraError", "payload_bytes", "NH_F32", "NH_F16", "NH_Q8_0", "NH_Q3_K", "NH_Q4_K", "NH_Q5_K", "NH_Q6_K", "UINT64_MAX", "Epilogue",
           "ModelConfig", "TensorTable"]
