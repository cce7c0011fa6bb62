"""ctypes binding of oracle/libneura_oracle.so for the tests (the checker, never the product)."""
import ctypes
import os
import subprocess
from ctypes import POINTER, c_float, c_int, c_uint8, c_uint16, c_uint32, c_uint64, c_void_p

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
LIBRARY = os.path.join(ORACLE_DIR, "libneura_oracle.so")

EL_F32, EL_F16, EL_Q8_0, EL_Q4_K, EL_Q6_K = 0, 1, 8, 12, 14
EL_Q3_K, EL_Q5_K = 11, 13
EL_BF16 = 30


class OracleModel(ctypes.Structure):
    _fields_ = [(n, c_uint32) for n in ("layers", "hidden", "heads", "kv_heads", "head_dim", "ffn", "vocab", "capacity", "window", "batch", "ring")] + [
        ("rope_base", c_float), ("eps", c_float), ("matrix_element", c_int),
        ("token_embd", c_void_p), ("output", c_void_p), ("output_norm", c_void_p),
        ("attn_norm", POINTER(c_void_p)), ("attn_q", POINTER(c_void_p)), ("attn_k", POINTER(c_void_p)), ("attn_v", POINTER(c_void_p)),
        ("attn_o", POINTER(c_void_p)), ("ffn_norm", POINTER(c_void_p)), ("ffn_gate", POINTER(c_void_p)), ("ffn_up", POINTER(c_void_p)),
        ("ffn_down", POINTER(c_void_p)), ("cache_k", POINTER(c_void_p)), ("cache_v", POINTER(c_void_p)),
        ("matrix_elements", POINTER(c_int)), ("attn_q_bias", POINTER(c_void_p)), ("attn_k_bias", POINTER(c_void_p)),
        ("attn_v_bias", POINTER(c_void_p)), ("cache_element", c_int),
    ]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIBRARY):
            subprocess.run(["make", "-C", ORACLE_DIR], check=True, capture_output=True)
        # the benchmark's CPU-baseline leg may name another build of the same source (one compiled for the machine it times)
        held = ctypes.CDLL(os.environ.get("NEURA_ORACLE_LIBRARY") or LIBRARY)
        held.oracle_f32_to_f16.restype = c_uint16
        held.oracle_f32_to_f16.argtypes = [c_float]
        held.oracle_f16_to_f32.restype = c_float
        held.oracle_f16_to_f32.argtypes = [c_uint16]
        held.oracle_unit.restype = c_float
        held.oracle_unit.argtypes = [POINTER(c_uint32)]
        held.oracle_rope_angle.restype = c_float
        held.oracle_rope_angle.argtypes = [c_uint32, c_uint32, c_uint32, c_float]
        held.oracle_payload_bytes.restype = c_uint64
        held.oracle_payload_bytes.argtypes = [c_int, c_uint64]
        held.oracle_argmax.restype = c_uint32
        held.oracle_argmax.argtypes = [c_void_p, c_uint32]
        held.oracle_gumbel_noise.restype = c_float
        held.oracle_gumbel_noise.argtypes = [c_uint32, c_uint32]
        held.oracle_plane_seed.restype = c_uint32
        held.oracle_plane_seed.argtypes = [c_uint32, c_uint32]
        held.oracle_seed_bits.restype = c_uint32
        held.oracle_seed_bits.argtypes = [c_uint32]
        _lib = held
    return _lib


def _p(array):
    return array.ctypes.data_as(c_void_p)


def f32_to_f16(values):
    values = np.ascontiguousarray(values, dtype=np.float32)
    out = np.empty(values.size, dtype=np.uint16)
    lib().oracle_f32_to_f16_many(_p(values), c_uint64(values.size), _p(out))
    return out.reshape(values.shape)


def f16_to_f32(bits):
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    out = np.empty(bits.size, dtype=np.float32)
    lib().oracle_f16_to_f32_many(_p(bits), c_uint64(bits.size), _p(out))
    return out.reshape(bits.shape)


def random(count, seed):
    out = np.empty(count, dtype=np.float32)
    lib().oracle_random(c_uint32(count), c_uint32(seed), _p(out))
    return out


def unpack(element, raw, elements):
    raw = np.ascontiguousarray(raw, dtype=np.uint8)
    out = np.empty(elements, dtype=np.float32)
    status = lib().oracle_unpack(c_int(element), _p(raw), c_uint64(elements), _p(out))
    assert status == 0, status
    return out


def pack(element, values):
    values = np.ascontiguousarray(values, dtype=np.float32)
    out = np.zeros(lib().oracle_payload_bytes(element, values.size), dtype=np.uint8)
    status = lib().oracle_pack(c_int(element), _p(values), c_uint64(values.size), _p(out))
    assert status == 0, status
    return out


def scale_min_k4(scales, at):
    scales = np.ascontiguousarray(scales, dtype=np.uint8)
    sc, mn = c_uint32(), c_uint32()
    lib().oracle_scale_min_k4(_p(scales), c_uint32(at), ctypes.byref(sc), ctypes.byref(mn))
    return sc.value, mn.value


def put_scale_min_k4(scales, at, scale, minimum):
    lib().oracle_put_scale_min_k4(_p(scales), c_uint32(at), c_uint32(scale), c_uint32(minimum))


def gemv(element, W, N, K, x, threads=1):
    W = np.ascontiguousarray(W, dtype=np.uint8)
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, K)
    y = np.empty((x.shape[0], N), dtype=np.float32)
    status = lib().oracle_gemv(c_int(element), _p(W), c_uint32(N), c_uint32(K), _p(x), c_uint32(x.shape[0]), _p(y), c_int(threads))
    assert status == 0, status
    return y


def gemm(element, W, N, K, X, threads=1):
    W = np.ascontiguousarray(W, dtype=np.uint8)
    X = np.ascontiguousarray(X, dtype=np.float32).reshape(-1, K)
    Y = np.empty((X.shape[0], N), dtype=np.float32)
    status = lib().oracle_gemm(c_int(element), _p(W), c_uint32(N), c_uint32(K), _p(X), c_uint32(X.shape[0]), _p(Y), c_int(threads))
    assert status == 0, status
    return Y


def rmsnorm(x, w, eps, residual=None):
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, C = x.shape
    out = np.empty_like(x)
    total = np.empty_like(x)
    w = np.ascontiguousarray(w, dtype=np.float32) if w is not None else None
    r = np.ascontiguousarray(residual, dtype=np.float32) if residual is not None else None
    lib().oracle_rmsnorm(_p(x), _p(r) if r is not None else None, _p(w) if w is not None else None, c_float(eps), c_uint32(rows),
                         c_uint32(C), _p(out), _p(total))
    return out, total


def rope(x, origin, base):
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, width = x.shape
    out = np.empty_like(x)
    lib().oracle_rope(_p(x), c_uint32(rows), c_uint32(width), c_uint32(origin), c_float(base), _p(out))
    return out


def cache_cast(values, element):
    """float32 numbers as a cache of `element` holds them (halves and bfloat16 as uint16 bits, single as it is)"""
    values = np.ascontiguousarray(values, dtype=np.float32)
    if element == EL_F32:
        return values.copy()
    out = np.empty(values.size, dtype=np.uint16)
    lib().oracle_cache_put_many(_p(out), c_int(element), c_uint64(0), _p(values.reshape(-1)), c_uint64(values.size))
    return out.reshape(values.shape)


def attention(q, K, V, kv_heads, capacity, keys, cursor, scale, reach=0, element=None):
    q = np.ascontiguousarray(q, dtype=np.float32)
    heads, batch, rows, width = q.shape
    if element is not None and element != EL_F32:
        el = element
    elif K.dtype == np.uint16:
        el = EL_F16
    else:
        el = EL_F32
        K, V = np.ascontiguousarray(K, dtype=np.float32), np.ascontiguousarray(V, dtype=np.float32)
    K, V = np.ascontiguousarray(K), np.ascontiguousarray(V)
    cursor = np.ascontiguousarray(cursor, dtype=np.uint32)
    out = np.empty_like(q)
    status = lib().oracle_attention(_p(q), _p(K), _p(V), c_int(el), c_uint32(heads), c_uint32(kv_heads), c_uint32(batch), c_uint32(rows),
                                    c_uint32(width), c_uint32(capacity), c_uint32(keys), c_uint32(reach), _p(cursor), c_float(scale), _p(out))
    assert status == 0, status
    return out


def attention_f64(q, K, V, kv_heads, origin, causal, scale):
    q = np.ascontiguousarray(q, dtype=np.float32)
    K, V = np.ascontiguousarray(K, dtype=np.float32), np.ascontiguousarray(V, dtype=np.float32)
    heads, batch, rows, width = q.shape
    keys = K.shape[2]
    out = np.empty_like(q)
    lib().oracle_attention_f64(_p(q), _p(K), _p(V), c_uint32(heads), c_uint32(kv_heads), c_uint32(batch), c_uint32(rows), c_uint32(width),
                               c_uint32(keys), c_uint32(origin), c_int(1 if causal else 0), c_float(scale), _p(out))
    return out


def argmax(values):
    values = np.ascontiguousarray(values, dtype=np.float32)
    return lib().oracle_argmax(_p(values), c_uint32(values.size))


DRAW = np.dtype([("seed", np.uint32), ("temperature", np.float32), ("keep", np.uint32), ("cumulative", np.float32)])


def draws(entries):
    """[(seed, temperature, keep, cumulative), ...] as the records both libraries take"""
    return np.array([tuple(entry) for entry in entries], dtype=DRAW)


def sample(logits, drawn):
    """one column per row of `logits`, drawn as graph.sample draws it (oracle_sample)"""
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    logits = logits.reshape(-1, logits.shape[-1])
    drawn = np.ascontiguousarray(drawn, dtype=DRAW)
    assert drawn.size == logits.shape[0]
    out = np.empty(logits.shape[0], dtype=np.uint32)
    status = lib().oracle_sample(_p(logits), c_uint32(logits.shape[0]), c_uint32(logits.shape[1]), _p(drawn), _p(out))
    assert status == 0, status
    return out


class Model:
    """The oracle's decoder over host copies of the same GGUF tensors the device gets."""

    def __init__(self, shape, element, tensors, batch, context, max_rows=1, rope_base=1e6, eps=1e-6, layers=None, elements=None,
                 window=None, cache_element=EL_F16):
        """`elements`: name -> element of the matrices that differ from `element`; tensors named blk.N.attn_{q,k,v}.bias
        are added to the projections before the rotation.  `window`: the caches are rings of that many positions
        (BatchSpec::window, crates/neura-generate/src/batch.rs:148-152, :313-325)."""
        self.keep = []
        L = shape["layers"] if layers is None else layers
        self.window = context if window is None else window
        self.capacity = self.window + max_rows
        m = OracleModel()
        m.ring = 0 if window is None else 1
        m.layers, m.hidden, m.heads, m.kv_heads = L, shape["hidden"], shape["heads"], shape["kv_heads"]
        m.head_dim, m.ffn, m.vocab = shape["head_dim"], shape["ffn"], shape["vocab"]
        m.capacity, m.window, m.batch = self.capacity, self.window, batch
        m.rope_base, m.eps, m.matrix_element = rope_base, eps, element

        def hold(array):
            array = np.ascontiguousarray(array)
            self.keep.append(array)
            return array.ctypes.data

        def table(suffix):
            pointers = (c_void_p * L)(*[hold(tensors["blk.%d.%s.weight" % (i, suffix)]) for i in range(L)])
            self.keep.append(pointers)
            return ctypes.cast(pointers, POINTER(c_void_p))

        m.token_embd = hold(tensors["token_embd.weight"])
        m.output = hold(tensors["output.weight"]) if "output.weight" in tensors else None
        m.output_norm = hold(tensors["output_norm.weight"])
        m.attn_norm, m.attn_q, m.attn_k, m.attn_v = table("attn_norm"), table("attn_q"), table("attn_k"), table("attn_v")
        m.attn_o, m.ffn_norm = table("attn_output"), table("ffn_norm")
        m.ffn_gate, m.ffn_up, m.ffn_down = table("ffn_gate"), table("ffn_up"), table("ffn_down")
        if elements:
            names = ["token_embd.weight", "output.weight"] + ["blk.%d.%s.weight" % (i, n) for i in range(L) for n in
                                                              ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up", "ffn_down")]
            held = (c_int * len(names))(*[elements.get(n, element) for n in names])
            self.keep.append(held)
            m.matrix_elements = ctypes.cast(held, POINTER(c_int))
        for which in ("q", "k", "v"):
            if any("blk.%d.attn_%s.bias" % (i, which) in tensors for i in range(L)):
                pointers = (c_void_p * L)(*[hold(np.asarray(tensors["blk.%d.attn_%s.bias" % (i, which)], dtype=np.float32))
                                            if "blk.%d.attn_%s.bias" % (i, which) in tensors else None for i in range(L)])
                self.keep.append(pointers)
                setattr(m, "attn_%s_bias" % which, ctypes.cast(pointers, POINTER(c_void_p)))
        cache_elements = shape["kv_heads"] * batch * self.capacity * shape["head_dim"]
        m.cache_element = cache_element
        held_as = np.float32 if cache_element == EL_F32 else np.uint16
        self.cache_k = [np.zeros(cache_elements, dtype=held_as) for _ in range(L)]
        self.cache_v = [np.zeros(cache_elements, dtype=held_as) for _ in range(L)]
        ks = (c_void_p * L)(*[a.ctypes.data for a in self.cache_k])
        vs = (c_void_p * L)(*[a.ctypes.data for a in self.cache_v])
        self.keep += [ks, vs]
        m.cache_k, m.cache_v = ctypes.cast(ks, POINTER(c_void_p)), ctypes.cast(vs, POINTER(c_void_p))
        self.m, self.batch, self.vocab = m, batch, shape["vocab"]

    def forward(self, tokens, rows, cursor, mask=None, want_logits=True, threads=8):
        tokens = np.ascontiguousarray(tokens, dtype=np.uint32)
        cursor = np.ascontiguousarray(cursor, dtype=np.uint32)
        mask = np.ones(self.batch, dtype=np.uint8) if mask is None else np.ascontiguousarray(mask, dtype=np.uint8)
        logits = np.empty((self.batch, self.vocab), dtype=np.float32) if want_logits else None
        chosen = np.empty(self.batch, dtype=np.uint32) if want_logits else None
        status = lib().oracle_model_forward(ctypes.byref(self.m), _p(tokens), c_uint32(rows), _p(cursor), _p(mask),
                                            _p(logits) if want_logits else None, _p(chosen) if want_logits else None, c_int(threads))
        assert status == 0, status
        return logits, chosen
