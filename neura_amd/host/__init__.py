"""ctypes face of libneura_host.so: the C++ host layer (neura.hpp) behind a flat C surface.

The classes here read like the reference's own (Gguf, GgufFile, Batch); a refusal of the
C++ layer -- a panic of the reference -- surfaces as `Panic` carrying the same sentence.
Loading touches no GPU; only Runtime() does.
"""
import ctypes
import os
from ctypes import POINTER, byref, c_char_p, c_double, c_float, c_int32, c_int64, c_size_t, c_uint32, c_uint64, c_void_p

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY = os.path.join(os.path.dirname(HERE), "libneura_host.so")


class Panic(RuntimeError):
    pass


class TensorInfo(ctypes.Structure):
    _fields_ = [("element", c_int32), ("rank", c_uint32), ("elements", c_uint64), ("shape", c_uint64 * 4), ("at", c_uint64), ("bytes", c_uint64)]


SIGNATURES = {
    "nhost_last_error": (c_char_p, []),
    "nhost_gguf_decode": (c_void_p, [c_void_p, c_size_t]),
    "nhost_gguf_open": (c_void_p, [c_char_p]),
    "nhost_gguf_close": (None, [c_void_p]),
    "nhost_gguf_tensors": (c_uint64, [c_void_p]),
    "nhost_gguf_reads": (c_uint64, [c_void_p]),
    "nhost_gguf_tensor": (c_int32, [c_void_p, c_char_p, POINTER(TensorInfo)]),
    "nhost_gguf_has": (c_int32, [c_void_p, c_char_p]),
    "nhost_gguf_word": (c_int32, [c_void_p, c_char_p, POINTER(c_uint32)]),
    "nhost_gguf_single": (c_int32, [c_void_p, c_char_p, POINTER(c_float)]),
    "nhost_gguf_flag": (c_int32, [c_void_p, c_char_p, POINTER(c_int32)]),
    "nhost_gguf_text": (c_int64, [c_void_p, c_char_p, c_void_p, c_size_t]),
    "nhost_gguf_integer": (c_int32, [c_void_p, c_char_p, POINTER(c_uint64)]),
    "nhost_gguf_array_len": (c_int64, [c_void_p, c_char_p]),
    "nhost_gguf_array_text": (c_int64, [c_void_p, c_char_p, c_uint64, c_void_p, c_size_t]),
    "nhost_gguf_array_number": (c_int64, [c_void_p, c_char_p, c_uint64, POINTER(c_double)]),
    "nhost_gguf_payload": (c_int64, [c_void_p, c_char_p, c_void_p, c_size_t]),
    "nhost_gguf_placed": (c_int32, [c_void_p, c_char_p, POINTER(c_int32), POINTER(c_uint64), POINTER(c_float), POINTER(c_uint64), POINTER(c_uint64)]),
    "nhost_writer_new": (c_void_p, [c_uint64]),
    "nhost_writer_free": (None, [c_void_p]),
    "nhost_writer_u32": (None, [c_void_p, c_char_p, c_uint32]),
    "nhost_writer_f32": (None, [c_void_p, c_char_p, c_float]),
    "nhost_writer_text": (None, [c_void_p, c_char_p, c_char_p]),
    "nhost_writer_tensor": (None, [c_void_p, c_char_p, c_int32, POINTER(c_uint64), c_uint32, c_void_p, c_size_t]),
    "nhost_writer_save": (c_int32, [c_void_p, c_char_p]),
    "nhost_matrix": (c_int32, [c_void_p, c_char_p, c_uint32, c_uint32, POINTER(c_int32)]),
    "nhost_vector": (c_int32, [c_void_p, c_char_p, c_uint32, POINTER(c_int32)]),
    "nhost_cache_validate": (c_int32, [c_char_p] + [c_uint32] * 6 + [c_int32]),
    "nhost_payload_bytes": (c_uint64, [c_int32, c_uint64]),
    "nhost_template_render": (c_int64, [c_char_p, c_char_p, c_char_p, c_void_p, c_size_t]),
    "nhost_template_render_gguf": (c_int64, [c_void_p, c_char_p, c_char_p, c_void_p, c_size_t]),
    "nhost_pack": (c_int64, [c_int32, c_float, c_void_p, c_size_t, c_void_p, c_size_t]),
    "nhost_unpack": (c_int32, [c_int32, c_size_t, c_void_p, c_size_t, c_void_p]),
    "nhost_half_bits": (c_uint32, [c_float]),
    "nhost_half_value": (c_float, [c_uint32]),
    "nhost_runtime_open": (c_void_p, [c_int32]),
    "nhost_runtime_close": (None, [c_void_p]),
    "nhost_batch_open": (c_void_p, [c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, POINTER(c_uint32), c_uint32, c_uint32, c_int32]),
    "nhost_batch_open_element": (c_void_p, [c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, POINTER(c_uint32), c_uint32, c_uint32, c_int32, c_int32]),
    "nhost_batch_open_sampled": (c_void_p, [c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, POINTER(c_uint32), c_uint32, c_float, c_uint32, c_float,
                                            c_uint32, c_int32]),
    "nhost_batch_prefix": (c_int32, [c_void_p, POINTER(c_uint32), c_uint32]),
    "nhost_batch_forget_prefix": (c_int32, [c_void_p]),
    "nhost_batch_window_check": (c_int32, [c_uint32]),
    "nhost_batch_window": (c_int64, [c_void_p]),
    "nhost_sampling_check": (c_int32, [c_float, c_uint32, c_float]),
    "nhost_plane_seed": (c_uint32, [c_uint32, c_uint32]),
    "nhost_seed_bits": (c_uint32, [c_uint32]),
    "nhost_batch_set_seed": (c_int32, [c_void_p, c_int32, c_uint32]),
    "nhost_batch_seed_of": (c_int64, [c_void_p, c_uint32]),
    "nhost_batch_set_temperature": (c_int32, [c_void_p, c_int32, c_float]),
    "nhost_batch_set_keep": (c_int32, [c_void_p, c_int32, c_uint32]),
    "nhost_batch_set_cumulative": (c_int32, [c_void_p, c_int32, c_float]),
    "nhost_batch_spec_check": (c_int32, [c_uint32, c_uint32, POINTER(c_uint32), c_uint32, c_uint32]),
    "nhost_snapshot_round_trip": (c_int64, [c_char_p, c_size_t, c_void_p, c_size_t]),
    "nhost_batch_snapshot": (c_int64, [c_void_p, c_void_p, c_size_t]),
    "nhost_batch_restore": (c_int32, [c_void_p, c_char_p, c_size_t]),
    "nhost_batch_save_state": (c_int32, [c_void_p, c_char_p]),
    "nhost_batch_restore_state": (c_int32, [c_void_p, c_char_p, c_char_p, c_size_t]),
    "nhost_tokenizer_open": (c_void_p, [c_void_p, c_char_p]),
    "nhost_tokenizer_close": (None, [c_void_p]),
    "nhost_tokenizer_vocabulary": (c_uint64, [c_void_p]),
    "nhost_tokenizer_id": (c_int64, [c_void_p, c_char_p]),
    "nhost_tokenizer_encode": (c_int64, [c_void_p, c_char_p, c_size_t, POINTER(c_uint32), c_size_t]),
    "nhost_tokenizer_piece": (c_int64, [c_void_p, c_uint32, c_void_p, c_size_t]),
    "nhost_rule_pieces": (c_int64, [c_char_p, c_char_p, c_size_t, POINTER(c_uint64), c_size_t]),
    "nhost_text_open": (c_void_p, []),
    "nhost_text_close": (None, [c_void_p]),
    "nhost_text_push": (c_int64, [c_void_p, c_void_p, c_size_t, c_int32, c_void_p, c_size_t]),
    "nhost_batch_close": (None, [c_void_p]),
    "nhost_batch_admit": (c_int32, [c_void_p, POINTER(c_uint32), c_uint32]),
    "nhost_batch_restart": (c_int32, [c_void_p, c_uint32, POINTER(c_uint32), c_uint32]),
    "nhost_batch_resume": (c_int32, [c_void_p, c_uint32, POINTER(c_uint32), c_uint32]),
    "nhost_batch_suspend": (c_int32, [c_void_p, c_uint32]),
    "nhost_batch_finish": (c_int32, [c_void_p, c_uint32]),
    "nhost_batch_step": (c_int32, [c_void_p, POINTER(c_uint32), c_uint32]),
    "nhost_batch_cursor": (c_int64, [c_void_p, c_uint32]),
    "nhost_batch_remaining": (c_int64, [c_void_p, c_uint32]),
    "nhost_batch_planes": (c_uint64, [c_void_p]),
    "nhost_batch_logits": (c_int32, [c_void_p, c_void_p]),
}

_lib = None


def library():
    global _lib
    if _lib is None:
        if not os.path.exists(LIBRARY):
            raise RuntimeError("%s is not built: run `python -m neura_amd.build`" % LIBRARY)
        lib = ctypes.CDLL(LIBRARY)
        for name, (restype, argtypes) in SIGNATURES.items():
            entry = getattr(lib, name)
            entry.restype, entry.argtypes = restype, argtypes
        _lib = lib
    return _lib


def _refused():
    return Panic(library().nhost_last_error().decode("utf-8", "replace"))


def _words(values):
    held = (c_uint32 * max(len(values), 1))(*[int(v) for v in values])
    return held, len(values)


class _Archive:
    """What Gguf and GgufFile share: metadata accessors, the tensor table, Source."""

    handle = None

    def close(self):
        if self.handle:
            library().nhost_gguf_close(self.handle)
            self.handle = None

    def __del__(self):
        self.close()

    def tensors(self):
        return int(library().nhost_gguf_tensors(self.handle))

    def tensor(self, name):
        info = TensorInfo()
        if not library().nhost_gguf_tensor(self.handle, name.encode(), byref(info)):
            return None
        return {"element": info.element, "elements": info.elements, "shape": list(info.shape), "rank": info.rank, "at": info.at, "bytes": info.bytes}

    def has(self, key):
        return bool(library().nhost_gguf_has(self.handle, key.encode()))

    def word(self, key):
        out = c_uint32()
        if library().nhost_gguf_word(self.handle, key.encode(), byref(out)) != 0:
            raise _refused()
        return out.value

    def optional_word(self, key):
        return self.word(key) if self.has(key) else None

    def single(self, key):
        out = c_float()
        if library().nhost_gguf_single(self.handle, key.encode(), byref(out)) != 0:
            raise _refused()
        return out.value

    def flag(self, key):
        out = c_int32()
        if library().nhost_gguf_flag(self.handle, key.encode(), byref(out)) != 0:
            raise _refused()
        return bool(out.value)

    def text(self, key):
        room = ctypes.create_string_buffer(1 << 16)
        length = library().nhost_gguf_text(self.handle, key.encode(), room, len(room))
        if length < 0:
            raise _refused()
        return room.raw[:length].decode()

    def integer(self, key):
        out = c_uint64()
        status = library().nhost_gguf_integer(self.handle, key.encode(), byref(out))
        if status < 0:
            raise _refused()
        return out.value if status else None

    def array_len(self, key):
        length = library().nhost_gguf_array_len(self.handle, key.encode())
        if length < 0:
            raise _refused()
        return length

    def texts(self, key):
        out = []
        room = ctypes.create_string_buffer(1 << 12)
        for index in range(self.array_len(key)):
            length = library().nhost_gguf_array_text(self.handle, key.encode(), index, room, len(room))
            if length < 0:
                raise _refused()
            out.append(room.raw[:length].decode())
        return out

    def numbers(self, key):
        out = []
        for index in range(self.array_len(key)):
            held = c_double()
            status = library().nhost_gguf_array_number(self.handle, key.encode(), index, byref(held))
            if status < 0:
                raise _refused()
            out.append(held.value if status else None)
        return out

    def placed(self, name):
        element, elements, scale, payload, table = c_int32(), c_uint64(), c_float(), c_uint64(), c_uint64()
        if not library().nhost_gguf_placed(self.handle, name.encode(), byref(element), byref(elements), byref(scale), byref(payload), byref(table)):
            return None
        return {"element": element.value, "elements": elements.value, "scale": scale.value, "payload_bytes": payload.value, "table_bytes": table.value}

    def payload(self, name):
        placed = self.placed(name)
        room = np.empty(placed["payload_bytes"] if placed else 0, dtype=np.uint8)
        length = library().nhost_gguf_payload(self.handle, name.encode(), room.ctypes.data, room.size)
        if length < 0:
            raise _refused()
        return room.tobytes()

    def matrix(self, name, rows, columns):
        element = c_int32()
        if library().nhost_matrix(self.handle, name.encode(), rows, columns, byref(element)) != 0:
            raise _refused()
        return element.value

    def vector(self, name, width):
        element = c_int32()
        if library().nhost_vector(self.handle, name.encode(), width, byref(element)) != 0:
            raise _refused()
        return element.value


class Gguf(_Archive):
    @classmethod
    def decode(cls, data):
        held = np.frombuffer(bytes(data), dtype=np.uint8)
        out = cls()
        out.handle = library().nhost_gguf_decode(held.ctypes.data if held.size else None, held.size)
        if not out.handle:
            raise _refused()
        return out


class GgufFile(_Archive):
    @classmethod
    def open(cls, path):
        out = cls()
        out.handle = library().nhost_gguf_open(os.fspath(path).encode())
        if not out.handle:
            raise _refused()
        return out

    def reads(self):
        return int(library().nhost_gguf_reads(self.handle))


class Writer:
    def __init__(self, alignment=32):
        self.handle = library().nhost_writer_new(alignment)

    def u32(self, key, value):
        library().nhost_writer_u32(self.handle, key.encode(), value)

    def f32(self, key, value):
        library().nhost_writer_f32(self.handle, key.encode(), value)

    def text(self, key, value):
        library().nhost_writer_text(self.handle, key.encode(), value.encode())

    def tensor(self, name, element, shape, payload):
        held = np.frombuffer(bytes(payload), dtype=np.uint8)
        dims = (c_uint64 * len(shape))(*shape)
        library().nhost_writer_tensor(self.handle, name.encode(), element, dims, len(shape), held.ctypes.data if held.size else None, held.size)

    def save(self, path):
        if library().nhost_writer_save(self.handle, os.fspath(path).encode()) != 0:
            raise _refused()

    def __del__(self):
        if self.handle:
            library().nhost_writer_free(self.handle)
            self.handle = None


def cache_validate(name, heads, width, capacity, window, batch, rows, element=1):
    if library().nhost_cache_validate(name.encode(), heads, width, capacity, window, batch, rows, element) != 0:
        raise _refused()


def batch_spec_check(context, batch, chunks, window=None):
    """BatchSpec::new(context, batch, chunks)[.window(window)] as Batch::new checks it, with no device"""
    held, count = _words(chunks)
    if window is not None and library().nhost_batch_window_check(window) != 0:
        raise _refused()
    if library().nhost_batch_spec_check(context, batch, held, count, window or 0) != 0:
        raise _refused()


class Tokenizer:
    """crates/neura-tokenizer: the byte level bpe a gpt2 GGUF holds under a split rule ("qwen", or "per_character",
    "per_space", "whole" as the reference's own tests define them)."""

    def __init__(self, archive, rule="qwen"):
        self.handle = library().nhost_tokenizer_open(archive.handle, rule.encode())
        if not self.handle:
            raise _refused()

    def close(self):
        if self.handle:
            library().nhost_tokenizer_close(self.handle)
            self.handle = None

    def vocabulary(self):
        return int(library().nhost_tokenizer_vocabulary(self.handle))

    def id(self, token):
        held = library().nhost_tokenizer_id(self.handle, token.encode())
        return None if held < 0 else int(held)

    def encode(self, text):
        raw = text.encode() if isinstance(text, str) else bytes(text)
        room = (c_uint32 * max(1, len(raw)))()  # a token spells at least one byte
        count = library().nhost_tokenizer_encode(self.handle, raw, len(raw), room, len(room))
        if count < 0:
            raise _refused()
        return list(room[:count])

    def piece(self, id):
        room = ctypes.create_string_buffer(1024)
        length = library().nhost_tokenizer_piece(self.handle, id, room, len(room))
        if length < 0:
            raise _refused()
        return room.raw[:length]

    def decode(self, ids):
        """the text the pieces of `ids` spell (through Text: ill-formed bytes read as U+FFFD)"""
        text = Text()
        out = "".join(text.push(self.piece(id)) for id in ids) + text.flush()
        text.close()
        return out


def rule_pieces(rule, text):
    """the pieces a split rule cuts a text into"""
    raw = text.encode()
    ends = (c_uint64 * max(1, len(raw)))()
    count = library().nhost_rule_pieces(rule.encode(), raw, len(raw), ends, len(ends))
    if count < 0:
        raise _refused()
    out, at = [], 0
    for end in ends[:count]:
        out.append(raw[at:end].decode())
        at = end
    return out


class Text:
    """crates/neura-tokenizer/src/text.rs: pieces in, whole characters out"""

    def __init__(self):
        self.handle = library().nhost_text_open()

    def close(self):
        if self.handle:
            library().nhost_text_close(self.handle)
            self.handle = None

    def _call(self, raw, flush):
        room = ctypes.create_string_buffer(4 * len(raw) + 64)
        length = library().nhost_text_push(self.handle, raw, len(raw), flush, room, len(room))
        return room.raw[:length].decode()

    def push(self, piece):
        return self._call(bytes(piece), 0)

    def flush(self):
        return self._call(b"", 1)


def snapshot_round_trip(raw):
    """BatchSnapshot::from_bytes then to_bytes (crates/neura-generate/src/snapshot.rs), with no device"""
    room = ctypes.create_string_buffer(len(raw) + 64)
    length = library().nhost_snapshot_round_trip(bytes(raw), len(raw), room, len(room))
    if length < 0:
        raise _refused()
    return room.raw[:length]


def sampling_check(temperature, keep, cumulative):
    """Sampling::sampled's refusals (crates/neura-generate/src/sampling.rs:16-29), with no device"""
    if library().nhost_sampling_check(temperature, keep, cumulative) != 0:
        raise _refused()


def plane_seed(seed, slot):
    return int(library().nhost_plane_seed(seed, slot))


def seed_bits(seed):
    return int(library().nhost_seed_bits(seed))


def payload_bytes(element, elements):
    return int(library().nhost_payload_bytes(element, elements))


def render_template(source, messages, values=None):
    """neura_template::Template::parse(source).render(messages, values) (crates/neura-template/src/template.rs): `source` is the
    template text, or an opened GGUF whose tokenizer.chat_template is read; messages are mappings with a role and a content"""
    import json

    listed = json.dumps(list(messages), ensure_ascii=False).encode("utf-8")
    named = json.dumps(dict(values or {}), ensure_ascii=False).encode("utf-8")
    room = ctypes.create_string_buffer(1 << 16)
    for _ in range(2):
        if isinstance(source, (str, bytes)):
            text = source.encode("utf-8") if isinstance(source, str) else source
            length = library().nhost_template_render(text, listed, named, room, len(room))
        else:
            length = library().nhost_template_render_gguf(source.handle, listed, named, room, len(room))
        if length < 0:
            raise _refused()
        if length <= len(room):
            return room.raw[:length].decode("utf-8")
        room = ctypes.create_string_buffer(length)
    raise RuntimeError("a rendered template outgrew its room twice")


def pack(element, values, quantum=0.0):
    """neura_precision::pack (crates/neura-precision/src/lib.rs:5-24): float32 numbers into the format's bytes"""
    values = np.ascontiguousarray(values, dtype=np.float32).reshape(-1)
    room = np.zeros(payload_bytes(element, max(values.size, 1)) + 8, dtype=np.uint8)
    length = library().nhost_pack(element, quantum, values.ctypes.data, values.size, room.ctypes.data, room.size)
    if length < 0:
        raise _refused()
    return room[:length].copy()


def unpack(element, elements, raw):
    """neura_precision::unpack (crates/neura-precision/src/lib.rs:26-68): the numbers `raw` holds"""
    raw = np.ascontiguousarray(np.frombuffer(bytes(raw), dtype=np.uint8) if not isinstance(raw, np.ndarray) else raw, dtype=np.uint8)
    out = np.zeros(max(elements, 1), dtype=np.float32)
    if library().nhost_unpack(element, elements, raw.ctypes.data, raw.size, out.ctypes.data) != 0:
        raise _refused()
    return out[:elements]


class Runtime:
    def __init__(self, index=0):
        self.handle = library().nhost_runtime_open(index)
        if not self.handle:
            raise _refused()

    def close(self):
        if self.handle:
            library().nhost_runtime_close(self.handle)
            self.handle = None


class Batch:
    """A Qwen2 GGUF loaded onto a runtime with a generation batch above it: greedy, or drawing with
    `sampling` = (temperature, keep, cumulative) as BatchSpec::sampled(Sampling::sampled(..)) does."""

    def __init__(self, runtime, archive, vocabulary, context, batch, chunks=(), sampling=None, window=None, shared=False, cache=None):
        """`window`: BatchSpec::window -- the caches are rings of that many tokens and a sequence attends to its last `window`;
        `shared`: BatchSpec::shared -- the batch can keep one prefix (`prefix`) every prompt then starts from;
        `cache`: the element of the key and value states (0 single, 1 half -- the default --, 30 bfloat16), greedy batches"""
        held, count = _words(chunks)
        self.planes = batch
        self.vocabulary = vocabulary
        if window is not None and library().nhost_batch_window_check(window) != 0:
            raise _refused()
        if sampling is None and cache is not None:
            self.handle = library().nhost_batch_open_element(runtime.handle, archive.handle, vocabulary, context, batch, held, count, window or 0,
                                                             1 if shared else 0, cache)
        elif sampling is None:
            self.handle = library().nhost_batch_open(runtime.handle, archive.handle, vocabulary, context, batch, held, count, window or 0,
                                                     1 if shared else 0)
        else:
            temperature, keep, cumulative = sampling
            self.handle = library().nhost_batch_open_sampled(runtime.handle, archive.handle, vocabulary, context, batch, held, count,
                                                             temperature, keep, cumulative, window or 0, 1 if shared else 0)
        if not self.handle:
            raise _refused()

    # what a sampled batch draws with (crates/neura-generate/src/batch.rs:643-732, :829-864); slot None names every plane
    def set_seed(self, seed, slot=None):
        self._status(library().nhost_batch_set_seed(self.handle, -1 if slot is None else slot, seed))

    def seed_of(self, slot):
        return self._status(library().nhost_batch_seed_of(self.handle, slot))

    def set_temperature(self, value, slot=None):
        self._status(library().nhost_batch_set_temperature(self.handle, -1 if slot is None else slot, value))

    def set_keep(self, keep, slot=None):
        self._status(library().nhost_batch_set_keep(self.handle, -1 if slot is None else slot, keep))

    def set_cumulative(self, value, slot=None):
        self._status(library().nhost_batch_set_cumulative(self.handle, -1 if slot is None else slot, value))

    def close(self):
        if self.handle:
            library().nhost_batch_close(self.handle)
            self.handle = None

    def _status(self, status):
        if status < 0:
            raise _refused()
        return status

    def admit(self, tokens):
        held, count = _words(tokens)
        return self._status(library().nhost_batch_admit(self.handle, held, count))

    def restart(self, slot, tokens):
        held, count = _words(tokens)
        self._status(library().nhost_batch_restart(self.handle, slot, held, count))

    def resume(self, slot, tokens):
        held, count = _words(tokens)
        self._status(library().nhost_batch_resume(self.handle, slot, held, count))

    def suspend(self, slot):
        self._status(library().nhost_batch_suspend(self.handle, slot))

    def finish(self, slot):
        self._status(library().nhost_batch_finish(self.handle, slot))

    # what the batch holds between steps (crates/neura-generate/src/batch.rs:484-628): the host side as "NBS1" bytes,
    # the key and value states of the device as a container file
    def snapshot(self):
        room = ctypes.create_string_buffer(1 << 20)
        length = library().nhost_batch_snapshot(self.handle, room, len(room))
        if length < 0 or length > len(room):
            raise _refused()
        return room.raw[:length]

    def restore(self, snapshot):
        self._status(library().nhost_batch_restore(self.handle, bytes(snapshot), len(snapshot)))

    def save_state(self, path):
        self._status(library().nhost_batch_save_state(self.handle, str(path).encode()))

    def restore_state(self, path, snapshot):
        self._status(library().nhost_batch_restore_state(self.handle, str(path).encode(), bytes(snapshot), len(snapshot)))

    def step(self):
        room = (c_uint32 * (2 * self.planes))()
        count = self._status(library().nhost_batch_step(self.handle, room, self.planes))
        return [(room[2 * i], room[2 * i + 1]) for i in range(count)]

    def cursor(self, slot):
        at = library().nhost_batch_cursor(self.handle, slot)
        if at == -2:
            raise _refused()
        return None if at < 0 else at

    def window(self):
        return self._status(library().nhost_batch_window(self.handle))

    def prefix(self, tokens):
        """Batch::prefix (crates/neura-generate/src/batch.rs:885-994)"""
        held, count = _words(tokens)
        self._status(library().nhost_batch_prefix(self.handle, held, count))

    def forget_prefix(self):
        self._status(library().nhost_batch_forget_prefix(self.handle))

    def remaining(self, slot):
        left = library().nhost_batch_remaining(self.handle, slot)
        if left == -2:
            raise _refused()
        return None if left < 0 else left

    def active(self):
        planes = library().nhost_batch_planes(self.handle)
        return [slot for slot in range(self.planes) if planes >> slot & 1]

    def occupied(self):
        planes = library().nhost_batch_planes(self.handle)
        return [slot for slot in range(self.planes) if planes >> (32 + slot) & 1]

    def logits(self):
        out = np.empty((self.planes, self.vocabulary), dtype=np.float32)
        self._status(library().nhost_batch_logits(self.handle, out.ctypes.data))
        return out
