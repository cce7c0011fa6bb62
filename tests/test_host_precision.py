"""The host encoders and decoders (neura::precision in neura_amd/host/neura.hpp) against the CPU
oracle: byte-equal packing and bit-equal unpacking of every format a GGUF decoder meets, on the
data the reference's own packing tests draw (crates/neura-runtime/tests/runtime.rs:717-736: seed 7,
shapes 5x96, 3x33 and 7; runtime.rs:24: seed 23)."""
import numpy as np
import pytest

import oracle
from neura_amd import host

BLOCKS = {8: (32, 34), 11: (256, 110), 12: (256, 144), 13: (256, 176), 14: (256, 210)}


def oracle_pack_ragged(element, values):
    """oracle.pack takes whole blocks; the reference packs a ragged tail with zeros behind it and ends on a word"""
    per, size = BLOCKS[element]
    blocks = -(-values.size // per)
    padded = np.zeros(blocks * per, dtype=np.float32)
    padded[: values.size] = values
    raw = oracle.pack(element, padded)
    assert raw.size == blocks * size
    return np.concatenate([raw, np.zeros(-raw.size % 4, dtype=np.uint8)])


@pytest.mark.parametrize("element", sorted(BLOCKS))
@pytest.mark.parametrize("count,seed", [(5 * 96, 7), (3 * 33, 7), (7, 7), (256 * 64, 23), (256 * 3 + 100, 5)])
def test_pack_is_the_oracles_bytes_and_unpack_its_numbers(element, count, seed):
    values = oracle.random(count, seed)
    want = oracle_pack_ragged(element, values)
    got = host.pack(element, values)
    assert got.size == want.size and np.array_equal(got, want)
    per = BLOCKS[element][0]
    whole = -(-count // per) * per
    back = host.unpack(element, count, got)
    assert np.array_equal(back.view(np.uint32), oracle.unpack(element, want, whole)[:count].view(np.uint32))


@pytest.mark.parametrize("element", sorted(BLOCKS))
def test_pack_of_hard_blocks_is_the_oracles(element):
    rng = np.random.default_rng(40 + element)
    values = np.concatenate([
        rng.normal(0, 0.02, 256 * 32), np.zeros(256), np.full(256, 0.3), -np.abs(rng.normal(0, 1, 256)), np.abs(rng.normal(0, 1, 256)),
        rng.normal(0, 1, 256) * 10.0 ** rng.integers(-20, 4, 256), np.full(256, -1e-30), rng.integers(-3, 4, 256) * 0.5,
    ]).astype(np.float32)
    assert np.array_equal(host.pack(element, values), oracle_pack_ragged(element, values))


def test_half_bits_and_values_are_ieee_for_every_code_and_many_singles():
    lib = host.library()
    codes = np.arange(1 << 16, dtype=np.uint16)
    values = codes.view(np.float16).astype(np.float32)
    for code in range(0, 1 << 16, 7):
        got = np.float32(lib.nhost_half_value(code))
        assert got.view(np.uint32) == values[code].view(np.uint32) or (np.isnan(got) and np.isnan(values[code]))
    rng = np.random.default_rng(3)
    singles = np.concatenate([
        rng.integers(0, 1 << 32, 20000, dtype=np.uint64).astype(np.uint32).view(np.float32),
        np.array([0.0, -0.0, 65504.0, 65520.0, 65519.996, 5.9604645e-8, 2.9802322e-8, 2.9802326e-8, 6.1035156e-5, 6.0975552e-5, 8.940697e-8,
                  np.inf, -np.inf], dtype=np.float32),
        (values[:0x7C00:5].astype(np.float64) * (1 + 2.0 ** -11)).astype(np.float32),  # ties between neighbours
    ])
    singles = singles[~np.isnan(singles)]
    want = oracle.f32_to_f16(singles)
    for value, bits in zip(singles, want):
        assert lib.nhost_half_bits(float(value)) == int(bits), (value, bits)


def test_half_single_and_bfloat16_storage():
    values = oracle.random(101, 7)
    raw = host.pack(1, values)
    assert raw.size == 51 * 4 and np.array_equal(raw[:202].view(np.uint16), oracle.f32_to_f16(values)) and not raw[202:].any()
    assert np.array_equal(host.unpack(1, 101, raw), oracle.f16_to_f32(oracle.f32_to_f16(values)))
    assert np.array_equal(host.pack(0, values).view(np.float32), values)
    assert np.array_equal(host.unpack(0, 101, host.pack(0, values)), values)
    raw = host.pack(30, values)
    bits = values.view(np.uint32).astype(np.uint64)
    want = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16).astype(np.uint16)  # round to nearest even (lib.rs:325-329)
    assert np.array_equal(raw[:202].view(np.uint16), want)
    back = host.unpack(30, 101, raw)
    assert np.array_equal(back.view(np.uint32), want.astype(np.uint32) << 16)
    assert np.abs(back - values).max() <= 2.0 ** -8


def test_unpack_refuses_short_storage_in_the_reference_s_words():
    raw = host.pack(12, oracle.random(512, 7))
    with pytest.raises(host.Panic, match="unpacking 512 q4_k numbers out of 144 bytes where they pack 288"):
        host.unpack(12, 512, raw[:144])
    with pytest.raises(host.Panic, match="int8|storage packs numbers|unknown"):
        host.pack(2, np.zeros(4, dtype=np.float32))
