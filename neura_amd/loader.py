"""Host-side loading of a decoder into the weight arena and the Python face of nh_model.

Mirrors what the reference's Runtime::load does with a Source
(crates/neura-runtime/src/runtime.rs:356-367, crates/neura-plan/src/layout.rs:29-36): every
tensor goes verbatim to a 256-byte aligned offset of one arena."""
import ctypes

import numpy as np

from . import _abi
from ._abi import ModelConfig, TensorTable, UINT64_MAX

ALIGNMENT = 256
LAYER_TENSORS = ("attn_norm", "attn_q", "attn_k", "attn_v", "attn_output", "ffn_norm", "ffn_gate", "ffn_up", "ffn_down")
MATRICES = ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down")


def _check(status):
    if status != 0:
        from . import NeuraError
        raise NeuraError(status, _abi.library().nh_last_error().decode())


class Weights:
    """One arena filled from an iterable of (name, element, dims, raw bytes)."""

    def __init__(self, device, tensors, total_bytes=None):
        self.device, self.lib = device, device.lib
        self.offsets, self.elements = {}, {}
        tensors = iter(tensors)
        pending = []
        if total_bytes is None:  # two passes over a materialised list
            pending = list(tensors)
            total_bytes = sum(-(-len(raw) // ALIGNMENT) * ALIGNMENT for _, _, _, raw in pending)
            tensors = iter(pending)
        self.handle = self.lib.nh_weights_create(device.handle, total_bytes)
        if not self.handle:
            from . import NeuraError
            raise NeuraError(_abi.NH_E_MEMORY, self.lib.nh_last_error().decode())
        at = 0
        for name, element, dims, raw in tensors:
            raw = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
            _check(self.lib.nh_weights_put(self.handle, at, raw.ctypes.data, raw.nbytes))
            self.offsets[name], self.elements[name] = at, element
            at += -(-raw.nbytes // ALIGNMENT) * ALIGNMENT
        self.used = at

    def pointer(self, name):
        return self.lib.nh_weights_at(self.handle, self.offsets[name])

    def release(self):
        if self.handle:
            self.lib.nh_weights_destroy(self.handle)
            self.handle = None


class Model:
    """nh_model over a Weights arena; tokens / cursors / mask are host arrays."""

    def __init__(self, device, weights, shape, element, batch, context, max_rows=1, rope_base=1e6, eps=1e-6, layers=None, window=None,
                 cache_element=1):
        self.device, self.lib, self.weights = device, device.lib, weights
        L = shape["layers"] if layers is None else layers
        self.config = ModelConfig(L, shape["hidden"], shape["heads"], shape["kv_heads"], shape["head_dim"], shape["ffn"], shape["vocab"],
                                  context, batch, max_rows, window or 0, rope_base, eps, cache_element)
        # what the key and value states hold: NH_F16 (1, two bytes read as uint16), NH_BF16 (30, the same) or NH_F32 (0, float32)
        self.cache_dtype = np.float32 if cache_element == 0 else np.uint16
        table = TensorTable()
        table.matrix_element = element
        table.token_embd = weights.offsets["token_embd.weight"]
        table.output = weights.offsets.get("output.weight", UINT64_MAX)
        table.output_norm = weights.offsets["output_norm.weight"]
        self._arrays = []
        for name in LAYER_TENSORS:
            array = (ctypes.c_uint64 * L)(*[weights.offsets["blk.%d.%s.weight" % (i, name)] for i in range(L)])
            self._arrays.append(array)
            setattr(table, name, ctypes.cast(array, ctypes.POINTER(ctypes.c_uint64)))
        # every matrix keeps the element it was stored with (a Q4_K_M file mixes Q4_K and Q6_K); Qwen2's q/k/v biases ride along
        names = ["token_embd.weight", "output.weight"] + ["blk.%d.%s.weight" % (i, n) for i in range(L) for n in MATRICES]
        held = [weights.elements.get(n, element) for n in names]
        if any(e != element for e in held):
            array = (ctypes.c_int32 * len(held))(*held)
            self._arrays.append(array)
            table.matrix_elements = ctypes.cast(array, ctypes.POINTER(ctypes.c_int32))
        for which in ("q", "k", "v"):
            offsets = [weights.offsets.get("blk.%d.attn_%s.bias" % (i, which), UINT64_MAX) for i in range(L)]
            if any(o != UINT64_MAX for o in offsets):
                array = (ctypes.c_uint64 * L)(*offsets)
                self._arrays.append(array)
                setattr(table, "attn_%s_bias" % which, ctypes.cast(array, ctypes.POINTER(ctypes.c_uint64)))
        self.handle = self.lib.nh_model_create(device.handle, ctypes.byref(self.config), weights.handle, ctypes.byref(table))
        if not self.handle:
            from . import NeuraError
            raise NeuraError(_abi.NH_E_ARGUMENT, self.lib.nh_last_error().decode())
        self.batch, self.vocab, self.layers = batch, shape["vocab"], L
        self.capacity = self.lib.nh_model_capacity(self.handle)
        self.cache_shape = (shape["kv_heads"], batch, self.capacity, shape["head_dim"])

    def release(self):
        if self.handle:
            self.lib.nh_model_destroy(self.handle)
            self.handle = None

    def seam_fallbacks(self):
        """decode steps that were run again, one launch a product, because a seam of a chained launch gave up"""
        return int(self.lib.nh_model_seam_fallbacks(self.handle))

    @staticmethod
    def _u32(values):
        return np.ascontiguousarray(values, dtype=np.uint32)

    def decode_step(self, tokens, cursors, mask=None):
        tokens, cursors = self._u32(tokens), self._u32(cursors)
        mask = np.ones(self.batch, dtype=np.uint8) if mask is None else np.ascontiguousarray(mask, dtype=np.uint8)
        chosen = np.empty(self.batch, dtype=np.uint32)
        u32, u8 = ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(ctypes.c_uint8)
        _check(self.lib.nh_decode_step(self.handle, tokens.ctypes.data_as(u32), cursors.ctypes.data_as(u32), mask.ctypes.data_as(u8),
                                       self.batch, chosen.ctypes.data_as(u32)))
        return chosen

    def decode_step_sampled(self, tokens, cursors, draws, mask=None):
        """a decode step whose chosen tokens are drawn: `draws` holds one record (dtype neura_amd.DRAW) a plane"""
        from . import DRAW

        tokens, cursors = self._u32(tokens), self._u32(cursors)
        draws = np.ascontiguousarray(draws, dtype=DRAW)
        assert draws.size == self.batch
        mask = np.ones(self.batch, dtype=np.uint8) if mask is None else np.ascontiguousarray(mask, dtype=np.uint8)
        chosen = np.empty(self.batch, dtype=np.uint32)
        u32, u8 = ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(ctypes.c_uint8)
        _check(self.lib.nh_decode_step_sampled(self.handle, tokens.ctypes.data_as(u32), cursors.ctypes.data_as(u32), mask.ctypes.data_as(u8),
                                               self.batch, draws.ctypes.data, chosen.ctypes.data_as(u32)))
        return chosen

    def prefill(self, tokens, rows, cursors, mask=None):
        tokens, cursors = self._u32(tokens), self._u32(cursors)
        mask = np.ones(self.batch, dtype=np.uint8) if mask is None else np.ascontiguousarray(mask, dtype=np.uint8)
        u32, u8 = ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(ctypes.c_uint8)
        _check(self.lib.nh_prefill(self.handle, tokens.ctypes.data_as(u32), rows, cursors.ctypes.data_as(u32), mask.ctypes.data_as(u8),
                                   self.batch))

    def time_products(self, steps):
        """(device seconds, launches, weight bytes) of `steps` back-to-back passes over the narrow products of a decode step"""
        seconds, launches, nbytes = ctypes.c_double(), ctypes.c_uint64(), ctypes.c_uint64()
        _check(self.lib.nh_model_time_products(self.handle, steps, ctypes.byref(seconds), ctypes.byref(launches), ctypes.byref(nbytes)))
        return seconds.value, launches.value, nbytes.value

    def reset(self, flags):
        flags = np.ascontiguousarray(flags, dtype=np.uint8)
        _check(self.lib.nh_model_reset(self.handle, flags.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)), self.batch))

    def logits(self):
        out = np.empty((self.batch, self.vocab), dtype=np.float32)
        _check(self.lib.nh_model_logits(self.handle, out.ctypes.data))
        return out

    def cache_write(self, layer, value_not_key, halves):
        halves = np.ascontiguousarray(halves, dtype=self.cache_dtype)
        assert halves.size == int(np.prod(self.cache_shape))
        _check(self.lib.nh_model_cache_write(self.handle, layer, int(value_not_key), halves.ctypes.data))

    def cache_read(self, layer, value_not_key):
        out = np.empty(self.cache_shape, dtype=self.cache_dtype)
        _check(self.lib.nh_model_cache_read(self.handle, layer, int(value_not_key), out.ctypes.data))
        return out
