"""The C++ host layer's GGUF reader, tensor declarations and construction refusals, on the CPU.

The cases follow the reference's own GGUF tests (crates/neura-gguf/tests/gguf.rs:28-272) on
fixtures built by tests/gguf_fixture.py; a panic of the reference is a Panic here, and the
sentence it carries is checked where the reference's source fixes it."""
import numpy as np
import pytest

from gguf_fixture import build
from neura_amd import host

ALIGN = [("general.alignment", "u32", 32)]
ELEMENT_KIND = {0: 0, 1: 1, 8: 8, 11: 11, 12: 12, 13: 13, 14: 14, 30: 30}  # element code == ggml type


def refuses(action, *needles):
    with pytest.raises(host.Panic) as caught:
        action()
    for needle in needles:
        assert needle in str(caught.value), str(caught.value)


def test_a_gguf_hands_back_the_metadata_it_holds():
    data, _, _ = build(32, ALIGN + [
        ("example.architecture", "string", "nothing in particular"),
        ("example.count", "u64", 9),
        ("example.ratio", "f32", 0.125),
        ("example.precise", "f64", 0.5),
        ("example.flag", "bool", 1),
        ("example.byte", "u8", 200),
        ("example.signed", "i8", -5),
        ("example.tags", "array", ("string", ["one", "two"])),
        ("example.counts", "array", ("u32", [3, 4])),
        ("example.short", "i16", -300),
        ("example.wide", "i64", -(1 << 40)),
        ("example.nested", "array", ("array", [("u16", [1, 2]), ("u16", [3])])),
    ], [])
    gguf = host.Gguf.decode(data)
    assert gguf.tensors() == 0
    assert gguf.text("example.architecture") == "nothing in particular"
    assert gguf.integer("example.count") == 9
    assert gguf.single("example.ratio") == 0.125
    assert gguf.single("example.precise") == 0.5
    assert gguf.flag("example.flag") is True
    assert gguf.integer("example.byte") == 200
    assert gguf.integer("example.signed") == (-5) % (1 << 64)  # two's complement, as `-5i64 as u64`
    assert gguf.integer("example.short") == (-300) % (1 << 64)
    assert gguf.integer("example.wide") == (-(1 << 40)) % (1 << 64)
    assert gguf.numbers("example.counts") == [3.0, 4.0]
    assert gguf.texts("example.tags") == ["one", "two"]
    assert gguf.array_len("example.nested") == 2
    assert not gguf.has("example.absent")
    assert gguf.integer("example.ratio") is None  # a number that is no whole number
    assert gguf.word("example.count") == 9
    assert gguf.optional_word("example.absent") is None
    # the accessors name the key and the type they found (crates/neura-gguf/src/metadata.rs:21-103)
    refuses(lambda: gguf.word("example.absent"), "this gguf holds no example.absent")
    refuses(lambda: gguf.text("example.count"), "example.count", "u64", "where a string stands")
    refuses(lambda: gguf.word("example.signed"), "example.signed", "where a word holds")
    refuses(lambda: gguf.flag("example.byte"), "where a flag stands")
    refuses(lambda: gguf.texts("example.counts"), "where a string stands")
    refuses(lambda: gguf.array_len("example.flag"), "where an array stands")


def test_a_gguf_names_the_element_every_tensor_packs():
    held = [(0, "single", 8), (1, "half", 16), (8, "q8_0", 32), (11, "q3_k", 256), (12, "q4_k", 256), (13, "q5_k", 256), (14, "q6_k", 256),
            (30, "bfloat16", 4)]
    expected_bytes = {"single": 32, "half": 32, "q8_0": 34, "q3_k": 110, "q4_k": 144, "q5_k": 176, "q6_k": 210, "bfloat16": 8}
    rng = np.random.default_rng(3)
    payloads = {name: rng.integers(0, 256, expected_bytes[name], dtype=np.uint8).tobytes() for _, name, _ in held}
    data, start, at = build(32, ALIGN, [(name, ELEMENT_KIND[element], [elements], payloads[name]) for element, name, elements in held])
    gguf = host.Gguf.decode(data)
    assert gguf.tensors() == len(held)
    for element, name, elements in held:
        tensor = gguf.tensor(name)
        assert tensor is not None
        assert tensor["element"] == element and tensor["elements"] == elements
        assert tensor["shape"] == [elements, 1, 1, 1] and tensor["rank"] == 1
        assert tensor["bytes"] == expected_bytes[name] == host.payload_bytes(element, elements)
        assert tensor["at"] == at[name]
        placed = gguf.placed(name)
        assert placed == {"element": element, "elements": elements, "scale": 1.0, "payload_bytes": tensor["bytes"], "table_bytes": 0}
        handed = gguf.payload(name)
        assert handed == data[start + tensor["at"]: start + tensor["at"] + tensor["bytes"]] == payloads[name]
    assert gguf.tensor("absent") is None and gguf.placed("absent") is None
    refuses(lambda: gguf.payload("absent"), "this gguf holds no tensor named absent")


def test_a_gguf_refuses_a_tensor_this_framework_cannot_read():
    data, _, _ = build(32, ALIGN, [("packed", 23, [256], bytes(136))])
    refuses(lambda: host.Gguf.decode(data), "packed", "ggml type 23", "IQ4_XS", "does not read")


def test_a_gguf_refuses_a_file_that_does_not_follow_its_layout():
    good, _, _ = build(32, ALIGN, [("weights", 12, [256], bytes(144))])
    host.Gguf.decode(good)
    refuses(lambda: host.Gguf.decode(b"GGFU" + good[4:]), "where a gguf opens with GGUF")
    refuses(lambda: host.Gguf.decode(good[:4] + (9).to_bytes(4, "little") + good[8:]), "declares version 9")
    refuses(lambda: host.Gguf.decode(good[:8]), "a gguf header runs past the bytes this file holds")
    refuses(lambda: host.Gguf.decode(b""), "a gguf header runs past the bytes this file holds")
    half, _, _ = build(32, ALIGN, [("weights", 12, [128], bytes(144))])
    refuses(lambda: host.Gguf.decode(half), "weights", "128 numbers of q4_k storage", "packs 256")
    cut, start, _ = build(32, ALIGN, [("weights", 8, [32], bytes(34))])
    refuses(lambda: host.Gguf.decode(cut[:start]), "where the tensor weights runs to byte %d" % (start + 34))
    off, _, _ = build(8, ALIGN, [("first", 12, [256], bytes(144)), ("second", 12, [256], bytes(144))])
    refuses(lambda: host.Gguf.decode(off), "the tensor second begins at byte 144", "aligns it by 32")
    # further refusals the header parser states (crates/neura-gguf/src/header.rs:43-148)
    twice, _, _ = build(32, ALIGN, [("same", 0, [8], bytes(32)), ("same", 0, [8], bytes(32))])
    refuses(lambda: host.Gguf.decode(twice), "two tensors of one gguf carry the name same")
    keys, _, _ = build(32, ALIGN + [("k", "u8", 1), ("k", "u8", 2)], [])
    refuses(lambda: host.Gguf.decode(keys), "two entries of this gguf carry the metadata key k")
    odd, _, _ = build(32, [("general.alignment", "u32", 12)], [])
    refuses(lambda: host.Gguf.decode(odd), "aligns its tensors by 12")
    deep, _, _ = build(32, ALIGN, [("deep", 0, [1, 1, 1, 1, 1], bytes(4))])
    refuses(lambda: host.Gguf.decode(deep), "declares 5 dimensions")
    flagged, _, _ = build(32, ALIGN + [("f", "bool", 2)], [])
    refuses(lambda: host.Gguf.decode(flagged), "where a flag holds zero or one")


def test_a_gguf_refuses_offsets_and_sizes_that_wrap_around():
    """A crafted table whose offset sits just below 2^64, or whose tensor spans more bytes than 2^64 counts, must not wrap
    to an end inside the file: the reader copies payloads with memcpy, where the reference's slices would panic."""
    good, _, _ = build(32, ALIGN, [("weights", 8, [32], bytes(34))])
    at = good.index(b"weights") + len(b"weights") + 4 + 8 + 4  # rank, one dimension, ggml type: then the offset
    assert good[at:at + 8] == bytes(8)
    far = good[:at] + (2 ** 64 - 32).to_bytes(8, "little") + good[at + 8:]
    refuses(lambda: host.Gguf.decode(far), "where the tensor weights runs to byte")
    huge, _, _ = build(32, ALIGN, [("wide", 0, [2 ** 62, 2], bytes(32))])  # 2^63 floats: 2^65 bytes
    refuses(lambda: host.Gguf.decode(huge), "wide", "more bytes than a gguf counts")
    big, _, _ = build(32, ALIGN, [("wide", 0, [2 ** 58], bytes(32))])  # 2^60 bytes: counted, but far past the file
    refuses(lambda: host.Gguf.decode(big), "where the tensor wide runs to byte")


def test_a_gguf_without_an_alignment_key_aligns_by_thirty_two_and_reads_version_two():
    data, start, at = build(32, [("general.name", "string", "x")], [("a", 0, [3], bytes(12)), ("b", 0, [2, 2], bytes(range(16)))], version=2)
    gguf = host.Gguf.decode(data)
    assert start % 32 == 0 and gguf.tensor("b")["at"] == at["b"] == 32
    assert gguf.tensor("b")["shape"] == [2, 2, 1, 1] and gguf.tensor("b")["rank"] == 2
    assert gguf.payload("b") == bytes(range(16))


def test_a_gguf_file_hands_a_store_the_same_bytes_as_the_whole_file(tmp_path):
    data, _, _ = build(32, [("general.alignment", "u32", 16)], [("weights", 12, [256], bytes([7]) * 144)])
    path = tmp_path / "weights.gguf"
    path.write_bytes(data)
    file = host.GgufFile.open(path)
    whole = host.Gguf.decode(data)
    assert file.tensors() == 1
    assert file.tensor("weights") == whole.tensor("weights")
    assert file.payload("weights") == whole.payload("weights") == bytes([7]) * 144
    assert file.reads() > 0
    refuses(lambda: host.GgufFile.open(tmp_path / "absent.gguf"), "could not be opened")
    (tmp_path / "short.gguf").write_bytes(data[:40])
    refuses(lambda: host.GgufFile.open(tmp_path / "short.gguf"), "holds 40 bytes where its metadata and its tensor table run past them")
    (tmp_path / "cut.gguf").write_bytes(data[:-24])  # 16 bytes of padding and 8 of the tensor
    refuses(lambda: host.GgufFile.open(tmp_path / "cut.gguf"), "where the tensor weights runs to byte")


def test_a_gguf_file_reads_a_header_wider_than_its_first_window(tmp_path):
    # 40000 vocabulary strings push the header past the first 1 MiB the reader takes
    # (crates/neura-gguf/src/lib.rs:21, :117-148), and a 200 KiB tensor streams in 64 KiB reads
    tags = ["token-%028d" % i for i in range(40000)]
    payload = np.random.default_rng(5).integers(0, 256, 200 * 1024, dtype=np.uint8).tobytes()
    data, start, _ = build(32, ALIGN + [("tokenizer.ggml.tokens", "array", ("string", tags))], [("blob", 0, [50 * 1024], payload)])
    assert start > (1 << 20)
    path = tmp_path / "wide.gguf"
    path.write_bytes(data)
    file = host.GgufFile.open(path)
    assert file.array_len("tokenizer.ggml.tokens") == 40000
    assert file.payload("blob") == payload
    assert file.reads() == 4  # 3 full chunks of 64 KiB and the 8 KiB that is left


def test_the_writer_lays_a_gguf_out_as_the_fixture_builder_does(tmp_path):
    rng = np.random.default_rng(9)
    first, second = rng.integers(0, 256, 144, dtype=np.uint8).tobytes(), rng.integers(0, 256, 68, dtype=np.uint8).tobytes()
    writer = host.Writer(32)
    writer.u32("general.alignment", 32)
    writer.text("general.architecture", "qwen2")
    writer.f32("qwen2.rope.freq_base", 1e6)
    writer.tensor("first", 12, [256], first)
    writer.tensor("second", 8, [32, 2], second)
    path = tmp_path / "written.gguf"
    writer.save(path)
    expected, _, _ = build(32, ALIGN + [("general.architecture", "string", "qwen2"), ("qwen2.rope.freq_base", "f32", 1e6)],
                           [("first", 12, [256], first), ("second", 8, [32, 2], second)])
    assert path.read_bytes() == expected


def test_a_declaration_walks_the_gguf_it_names():
    # crates/neura-decoder/src/parameter.rs:5-27: a matrix of `rows` rows of `columns` numbers is
    # the GGUF tensor [columns, rows]; a vector of `width` numbers is [width]
    data, _, _ = build(32, ALIGN, [("w", 8, [64, 3], bytes(34 * 6)), ("v", 0, [64], bytes(256))])
    gguf = host.Gguf.decode(data)
    assert gguf.matrix("w", 3, 64) == 8
    assert gguf.vector("v", 64) == 0
    refuses(lambda: gguf.matrix("w", 64, 3), "the tensor w of this gguf walks 2 dimensions of [64, 3, 1, 1]", "64 rows of 3 numbers walk [1, 1, 64, 3]")
    refuses(lambda: gguf.matrix("v", 1, 64), "the tensor v of this gguf walks 1 dimensions")
    refuses(lambda: gguf.vector("v", 32), "where 32 numbers walk [1, 1, 1, 32]")
    refuses(lambda: gguf.vector("w", 64), "walks 2 dimensions")
    refuses(lambda: gguf.matrix("absent", 1, 1), "this gguf holds no tensor named absent")


def test_a_cache_refuses_a_shape_it_cannot_keep():
    # crates/neura-decoder/src/cache.rs:92-134
    host.cache_validate("blk.0.cache", 2, 64, 1088, 1024, 4, 64)
    refuses(lambda: host.cache_validate("", 2, 64, 16, 16, 1, 1), "a cache names the state it keeps")
    refuses(lambda: host.cache_validate("c", 0, 64, 16, 16, 1, 1), "holds no key")
    refuses(lambda: host.cache_validate("c", 2, 64, 0, 0, 1, 1), "a cache of 0 positions holds no key")
    refuses(lambda: host.cache_validate("c", 2, 64, 16, 17, 1, 1), "a cache of 16 positions keeps a window of 17 positions")
    refuses(lambda: host.cache_validate("c", 2, 64, 16, 0, 1, 1), "keeps a window of 0 positions")
    refuses(lambda: host.cache_validate("c", 2, 64, 32, 16, 1, 17), "a cache of a 16 position window takes 17 rows at a time")
    refuses(lambda: host.cache_validate("c", 2, 64, 16, 16, 1, 1, element=12), "q4_k storage carries another grid")


def test_a_batch_refuses_a_spec_it_cannot_fill():
    # crates/neura-generate/src/batch.rs:279-330
    host.batch_spec_check(1088, 8, [64, 8])
    host.batch_spec_check(16, 1, [])
    refuses(lambda: host.batch_spec_check(16, 0, []), "a batch of no plane answers nothing")
    refuses(lambda: host.batch_spec_check(0, 1, []), "a context of no token holds no batch")
    refuses(lambda: host.batch_spec_check(128, 1, [8, 64]), "fills the largest chunk first, and fills 8 then 64")
    refuses(lambda: host.batch_spec_check(128, 1, [8, 8]), "fills 8 then 8")
    refuses(lambda: host.batch_spec_check(128, 1, [8, 1]), "a batch fills 1 rows of a context of 128")
    refuses(lambda: host.batch_spec_check(64, 1, [64]), "a batch fills 64 rows of a context of 64")


def test_a_sampling_refuses_what_spreads_or_keeps_nothing():
    # crates/neura-generate/src/sampling.rs:16-29
    host.sampling_check(1.0, 1, 1.0)
    host.sampling_check(0.01, 64, 0.05)
    refuses(lambda: host.sampling_check(0.0, 4, 1.0), "a sampling temperature of 0 spreads no logits")
    refuses(lambda: host.sampling_check(float("inf"), 4, 1.0), "a sampling temperature of inf spreads no logits")
    refuses(lambda: host.sampling_check(1.0, 0, 1.0), "a sample keeps 0 candidates where a row holds between one and 64")
    refuses(lambda: host.sampling_check(1.0, 65, 1.0), "a sample keeps 65 candidates where a row holds between one and 64")
    refuses(lambda: host.sampling_check(1.0, 4, 0.0), "a cumulative mass of 0 keeps no candidate or names more than every candidate")
    refuses(lambda: host.sampling_check(1.0, 4, 1.5), "a cumulative mass of 1.5 keeps no candidate")


def test_plane_seeds_and_the_bits_a_batch_writes():
    # crates/neura-generate/src/batch.rs:1841-1847, against the oracle's restatement and by hand
    import oracle

    assert host.plane_seed(0, 0) == 0x9E3779B9 and host.plane_seed(0, 1) == (2 * 0x9E3779B9) & 0xFFFFFFFF
    for seed in (0, 1, 77, 0x9E3779B9, 0xFFFFFFFF):
        for slot in (0, 1, 7):
            assert host.plane_seed(seed, slot) == oracle.lib().oracle_plane_seed(seed, slot)
        assert host.seed_bits(seed) == oracle.lib().oracle_seed_bits(seed) == 0x3F800000 | ((seed ^ (seed >> 23)) & 0x7FFFFF)


def test_a_batch_snapshot_reads_and_writes_the_nbs1_wire_format():
    # crates/neura-generate/src/snapshot.rs:47-236, the bytes laid out here by hand: little-endian words, counted lists
    import struct

    def words(*values):
        return struct.pack("<%dI" % len(values), *values)

    def floats(*values):
        return struct.pack("<I", len(values)) + struct.pack("<%df" % len(values), *values)

    raw = (b"NBS1" + words(3, 96, 96) + words(1)            # batch, context, window; sampled
           + words(0)                                        # no shared prefix
           + words(3)                                        # three slots
           + words(1, 7) + words(2, 41, 42)                  # prompting at cursor 7 with two tokens left
           + words(0)                                        # an empty plane
           + words(2, 19, 555)                               # generating at cursor 19, feeding token 555
           + words(3, 11, 22, 33)                            # seeds
           + floats(0.5, 1.0, 1.5) + floats(40.0, 1.0, 64.0) + floats(0.9, 1.0, 0.25)
           + words(1) + words(4) + b"gate"                   # one named state ...
           + words(1) + floats(0.0, 1.0, 0.0))               # ... of a value a plane
    assert host.snapshot_round_trip(raw) == raw
    suspended = raw.replace(words(2, 19, 555), words(3, 19))
    assert host.snapshot_round_trip(suspended) == suspended
    prefixed = raw.replace(b"NBS1" + words(3, 96, 96) + words(1) + words(0), b"NBS1" + words(3, 96, 96) + words(1) + words(1) + words(2, 5, 6))
    assert host.snapshot_round_trip(prefixed) == prefixed
    refuses(lambda: host.snapshot_round_trip(b"NBS2" + raw[4:]), "a batch snapshot opens with the four bytes NBS1")
    refuses(lambda: host.snapshot_round_trip(raw[:-2]), "bytes where its reader asks for")
    refuses(lambda: host.snapshot_round_trip(raw + b"\0\0\0\0"), "bytes where its reader stops at")
    refuses(lambda: host.snapshot_round_trip(raw.replace(words(3, 96, 96) + words(1), words(3, 96, 96) + words(2))), "a batch snapshot samples by 2")
    refuses(lambda: host.snapshot_round_trip(raw.replace(words(3, 96, 96), words(2, 96, 96))), "a snapshot of 2 planes names 3 slots")
    refuses(lambda: host.snapshot_round_trip(raw.replace(words(2, 19, 555), words(4, 19, 555))), "a slot snapshot holds phase 4")
    refuses(lambda: host.snapshot_round_trip(raw.replace(words(3, 11, 22, 33), words(2, 11, 22))), "a snapshot of 3 planes carries 2 seeds")
