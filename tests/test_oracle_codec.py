"""Pins the CPU oracle's codecs (f16, PRNG, Q8_0, Q4_K) against what fixes them without the
reference binary: IEEE binary16 (numpy), the published ggml layouts restated in numpy,
hand-built blocks, and encode/decode invariants."""
import numpy as np
import pytest

import oracle
from neura_amd import synth


def test_f16_to_f32_matches_ieee_for_every_code():
    bits = np.arange(65536, dtype=np.uint16)
    ours = oracle.f16_to_f32(bits)
    theirs = bits.view(np.float16).astype(np.float32)
    assert np.array_equal(ours.view(np.uint32)[~np.isnan(theirs)], theirs.view(np.uint32)[~np.isnan(theirs)])
    assert np.all(np.isnan(ours[np.isnan(theirs)]))


def test_f32_to_f16_is_round_to_nearest_even():
    rng = np.random.default_rng(1)
    values = np.concatenate([
        rng.standard_normal(1 << 18).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 1 << 18).astype(np.float32),
        rng.integers(0, 1 << 32, 1 << 18, dtype=np.uint64).astype(np.uint32).view(np.float32),  # any bit pattern
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e9, -1e9, np.inf, -np.inf, 5.96e-8, 2.98e-8, 2.9802322e-8, 6.1e-5], dtype=np.float32),
    ])
    # every exact midpoint between neighbouring halves (ties) and both neighbours of it
    halves = np.arange(0, 0x7c00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mids = ((halves[:-1] + halves[1:]) / 2).astype(np.float32)
    values = np.concatenate([values, mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e9)), -mids])
    ours = oracle.f32_to_f16(values)
    with np.errstate(over="ignore"):
        theirs = values.astype(np.float16).view(np.uint16)
    nan = np.isnan(values)
    assert np.array_equal(ours[~nan], theirs[~nan])
    assert np.all((ours[nan] & 0x7fff) == 0x7e00)  # convert.rs:61-63: NaN -> sign | 0x7e00


def test_xorshift_unit_is_the_closed_form():
    entropy = 23 | 1
    expected = []
    for _ in range(1000):
        entropy ^= (entropy << 13) & 0xFFFFFFFF
        entropy ^= entropy >> 17
        entropy ^= (entropy << 5) & 0xFFFFFFFF
        expected.append(np.float32(-1.0) + np.float32(2.0) * (np.float32(entropy >> 8) / np.float32(1 << 24)))
    assert np.array_equal(oracle.random(1000, 23), np.array(expected, dtype=np.float32))
    assert np.array_equal(oracle.random(10, 22), oracle.random(10, 23))  # seed | 1
    held = oracle.random(100000, 29)
    assert held.min() >= -1.0 and held.max() < 1.0 and abs(float(held.mean())) < 0.01


def test_scale_min_k4_put_then_get_is_identity_everywhere():
    for at in range(8):
        for scale in range(64):
            for minimum in range(64):
                scales = np.zeros(12, dtype=np.uint8)
                oracle.put_scale_min_k4(scales, at, scale, minimum)
                assert oracle.scale_min_k4(scales, at) == (scale, minimum)


def test_scale_min_k4_matches_the_published_layout_on_random_bytes():
    rng = np.random.default_rng(2)
    scales = rng.integers(0, 256, (200, 12), dtype=np.uint8)
    sc, mn = synth.scale_min_k4(scales)
    for row in range(200):
        for at in range(8):
            assert oracle.scale_min_k4(scales[row], at) == (int(sc[row, at]), int(mn[row, at]))


def test_q8_0_unpack_every_code_is_the_closed_form():
    # all 256 codes under a spread of scales, block laid out by hand
    for scale in (np.float16(1.0), np.float16(0.0123), np.float16(6e-8), np.float16(65504.0), np.float16(0.0)):
        for first in range(0, 256, 32):
            codes = np.arange(first, first + 32, dtype=np.uint8)
            raw = np.concatenate([np.array([scale]).view(np.uint8), codes])
            got = oracle.unpack(oracle.EL_Q8_0, raw, 32)
            want = codes.view(np.int8).astype(np.float32) * np.float32(scale)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_q4_k_unpack_hand_built_block():
    # byte pattern in the manner of the reference's Q3_K known-answer test
    # (crates/neura-precision/tests/format.rs:221-234): quants (at*37+11), scales (at*53+7)
    raw = np.zeros(144, dtype=np.uint8)
    raw[0:2] = np.array([np.float16(0.5)]).view(np.uint8)
    raw[2:4] = np.array([np.float16(0.25)]).view(np.uint8)
    raw[4:16] = [(at * 53 + 7) & 0xFF for at in range(12)]
    raw[16:] = [(at * 37 + 11) & 0xFF for at in range(128)]
    got = oracle.unpack(oracle.EL_Q4_K, raw, 256)
    s = raw[4:16].astype(int)
    expected = []
    for j in range(8):
        if j < 4:
            sc, mn = s[j] & 63, s[j + 4] & 63
        else:
            sc, mn = (s[j + 4] & 15) | ((s[j - 4] >> 6) << 4), (s[j + 4] >> 4) | ((s[j] >> 6) << 4)
        for lane in range(32):
            byte = int(raw[16 + (j // 2) * 32 + lane])
            q = (byte >> 4) if j % 2 else (byte & 15)
            expected.append(np.float32(np.float32(0.5) * np.float32(sc)) * np.float32(q) - np.float32(np.float32(0.25) * np.float32(mn)))
    assert np.array_equal(got, np.array(expected, dtype=np.float32))
    # element order: 32 low nibbles then 32 high nibbles per 64-group (ggml.rs:339-348)
    assert got[0] == np.float32(0.5 * (s[0] & 63)) * np.float32(raw[16] & 15) - np.float32(0.25 * (s[4] & 63))
    assert got[32] == np.float32(0.5 * (s[1] & 63)) * np.float32(raw[16] >> 4) - np.float32(0.25 * (s[5] & 63))


def test_q6_k_unpack_hand_built_block():
    # one super-block whose element e carries code (7 e + 3) % 64 and whose sub-block s carries scale 5 s - 40, packed
    # here by ggml's published layout (crates/neura-precision/src/ggml.rs:394-407 reads it back)
    raw = np.zeros(210, dtype=np.uint8)
    codes = [(7 * e + 3) % 64 for e in range(256)]
    scales = [5 * s - 40 for s in range(16)]
    for e, code in enumerate(codes):
        half, group, seat = e // 128, (e % 128) // 32, e % 32
        at = half * 64 + (group % 2) * 32 + seat
        raw[at] |= (code & 15) << (4 if group >= 2 else 0)
        raw[128 + half * 32 + seat] |= (code >> 4) << (2 * group)
    raw[192:208] = np.array(scales, dtype=np.int8).view(np.uint8)
    raw[208:210] = np.array([0.25], dtype=np.float16).view(np.uint8)
    got = oracle.unpack(oracle.EL_Q6_K, raw, 256)
    want = np.array([np.float32(np.float32(0.25) * np.float32(scales[e // 16])) * np.float32(codes[e] - 32) for e in range(256)], dtype=np.float32)
    assert np.array_equal(got, want)


def test_q6_k_symmetric_quantizer_of_the_test_data_round_trips():
    # synth.q6_k_quantize makes the Q6_K matrices of the synthetic decoders; the oracle reads them back within half a step
    rng = np.random.default_rng(12)
    values = rng.normal(0, 0.02, 256 * 50).astype(np.float32)
    back = oracle.unpack(oracle.EL_Q6_K, synth.q6_k_quantize(values), values.size)
    step = np.abs(values).reshape(-1, 16).max(axis=1) / 31.0
    error = np.abs(back - values).reshape(-1, 16).max(axis=1)
    assert np.all(error <= step * 0.55 + np.abs(values).reshape(-1, 256).max(axis=1).repeat(16) * 2.0 ** -9)
    assert np.sign(back[np.abs(values) > 0.01]).tolist() == np.sign(values[np.abs(values) > 0.01]).tolist()


def test_q6_k_pack_invariants():
    # non-negative values survive within a step and a half of their sub-block (step = largest / 32, the largest itself
    # clamps to code 31, the int8 sub-scale rounds the step by up to a percent); the reference's unsigned conversion
    # (ggml.rs:120-125) drops every negative value to zero, and the restatement keeps that
    rng = np.random.default_rng(11)
    values = np.abs(rng.normal(0, 1, 256 * 40)).astype(np.float32)
    raw = oracle.pack(oracle.EL_Q6_K, values)
    assert raw.size == 40 * 210 == oracle.lib().oracle_payload_bytes(14, 256 * 40)
    back = oracle.unpack(oracle.EL_Q6_K, raw, values.size)
    step = np.abs(values).reshape(-1, 16).max(axis=1) / 32.0
    error = np.abs(back - values).reshape(-1, 16).max(axis=1)
    assert np.all(error <= step * 1.5)
    assert np.median(error / step) < 1.05  # the largest of sixteen draws usually sits on the clamped code
    negative = oracle.unpack(oracle.EL_Q6_K, oracle.pack(oracle.EL_Q6_K, -values), values.size)
    assert np.all(negative == 0.0)


def q3_k_walk(field):
    """ggml's published dequantize_row_q3_K as a scalar walk (the form the reference's own test checks its codec
    against, crates/neura-precision/tests/format.rs:173-219): scales through the three-word shuffle, then per half four
    shifts of two runs of 16, the mask bit moving up once per 32."""
    aux = [int.from_bytes(bytes(field[96 + 4 * at:100 + 4 * at]), "little") for at in range(3)] + [0]
    tmp = aux[2]
    k1, k2 = 0x03030303, 0x0F0F0F0F
    packed = [(aux[0] & k2) | ((tmp & k1) << 4), (aux[1] & k2) | (((tmp >> 2) & k1) << 4),
              ((aux[0] >> 4) & k2) | (((tmp >> 4) & k1) << 4), ((aux[1] >> 4) & k2) | (((tmp >> 6) & k1) << 4)]
    scales = [((packed[at // 4] >> ((at % 4) * 8)) & 0xFF) - 32 for at in range(16)]
    d = np.float32(np.array(field[108:110], dtype=np.uint8).view(np.float16)[0])
    out, walk, m = [], 0, 1
    for half in range(2):
        q = field[32 + half * 32:64 + half * 32]
        for shift in (0, 2, 4, 6):
            for run in range(2):
                dl = np.float32(d * np.float32(scales[walk]))
                walk += 1
                for l in range(16):
                    at = l + 16 * run
                    quant = ((int(q[at]) >> shift) & 3) - (0 if int(field[at]) & m else 4)
                    out.append(np.float32(dl * np.float32(quant)))
            m <<= 1
    return np.array(out, dtype=np.float32)


def test_q3_k_known_answer_block_of_the_reference():
    # the block of crates/neura-precision/tests/format.rs:221-234: third bits at*37+11, bit pairs at*53+7, scales at*19+3,
    # d = 0.25; the reference asserts its codec equals ggml's walk on it, bit for bit
    field = np.zeros(110, dtype=np.uint8)
    field[0:32] = [(at * 37 + 11) & 0xFF for at in range(32)]
    field[32:96] = [(at * 53 + 7) & 0xFF for at in range(64)]
    field[96:108] = [(at * 19 + 3) & 0xFF for at in range(12)]
    field[108:110] = np.array([0.25], dtype=np.float16).view(np.uint8)
    got = oracle.unpack(oracle.EL_Q3_K, field, 256)
    want = q3_k_walk(field)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(synth.q3_k_dequant(field, 256).view(np.uint32), want.view(np.uint32))
    # spot values worked by hand: element 0 has pair (7 >> 0) & 3 = 3, third bit 11 & 1 = 1 -> code 3; its scale is
    # (3 & 15) | ((155 & 3) << 4) = 51 - 32 = 19
    assert got[0] == np.float32(0.25 * 19 * 3)
    # element 16: pair (byte 32+16 = 16*53+7 = 855 & 255 = 87) & 3 = 3, third bit (16*37+11 = 603 & 255 = 91) & 1 = 1 -> 3;
    # scale 1 = (22 & 15) | ((174 & 3) << 4) = 6 | 32 = 38 - 32 = 6
    assert got[16] == np.float32(0.25 * 6 * 3)


def test_q3_k_round_trip_of_the_reference():
    # crates/neura-precision/tests/format.rs:236-245: a slow sine of amplitude 0.75 comes back within 0.25
    values = (np.sin(np.arange(256, dtype=np.float32) * np.float32(0.031)) * np.float32(0.75)).astype(np.float32)
    raw = oracle.pack(oracle.EL_Q3_K, values)
    assert raw.size == 110 == oracle.lib().oracle_payload_bytes(11, 256)
    back = oracle.unpack(oracle.EL_Q3_K, raw, 256)
    assert np.abs(back - values).max() <= 0.25
    # the scales are stored as codes 32..63 and every code is a pair plus a third bit
    scales = synth.q3_k_scales(raw[96:108].reshape(1, 12))
    assert scales.min() >= 0 and scales.max() <= 31


def test_q5_k_unpack_hand_built_block():
    # element e of sub-block s carries code (11 e + 5) % 32; scales and minimums through put_scale_min_k4's layout
    raw = np.zeros(176, dtype=np.uint8)
    raw[0:2] = np.array([np.float16(0.5)]).view(np.uint8)
    raw[2:4] = np.array([np.float16(0.125)]).view(np.uint8)
    raw[4:16] = [(at * 53 + 7) & 0xFF for at in range(12)]
    codes = [(11 * e + 5) % 32 for e in range(256)]
    for e, code in enumerate(codes):
        sub, l = e // 32, e % 32
        raw[48 + (sub // 2) * 32 + l] |= (code & 15) << (4 if sub % 2 else 0)
        raw[16 + l] |= (code >> 4) << sub
    got = oracle.unpack(oracle.EL_Q5_K, raw, 256)
    s = raw[4:16].astype(int)
    want = []
    for e, code in enumerate(codes):
        j = e // 32
        if j < 4:
            sc, mn = s[j] & 63, s[j + 4] & 63
        else:
            sc, mn = (s[j + 4] & 15) | ((s[j - 4] >> 6) << 4), (s[j + 4] >> 4) | ((s[j] >> 6) << 4)
        want.append(np.float32(np.float32(0.5) * np.float32(sc)) * np.float32(code) - np.float32(np.float32(0.125) * np.float32(mn)))
    assert np.array_equal(got, np.array(want, dtype=np.float32))


def test_q5_k_pack_invariants():
    values = oracle.random(256 * 200, 23)
    raw = oracle.pack(oracle.EL_Q5_K, values)
    assert oracle.lib().oracle_payload_bytes(13, 256 * 200) == raw.size == 200 * 176
    back = oracle.unpack(oracle.EL_Q5_K, raw, values.size)
    # 5-bit affine codes over a range of <= 2: step <= 2/31, and twice as fine as Q4_K on the same values
    assert np.abs(back - values).max() <= 2.0 / 31.0
    coarse = oracle.unpack(oracle.EL_Q4_K, oracle.pack(oracle.EL_Q4_K, values), values.size)
    assert np.abs(back - values).mean() < 0.6 * np.abs(coarse - values).mean()


@pytest.mark.parametrize("element", [8, 11, 12, 13, 14])
def test_unpack_matches_the_numpy_restatement_on_random_blocks(element):
    rng = np.random.default_rng(3 + element)
    elements = 256 * 300
    raw = synth.RANDOM[element](rng, elements)
    got = oracle.unpack(element, raw, elements)
    want = synth.DEQUANT[element](raw, elements)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("element", [8, 11, 12, 13])
def test_pack_matches_the_numpy_restatement(element):
    rng = np.random.default_rng(5 + element)
    values = np.concatenate([
        rng.normal(0, 0.02, 256 * 64), rng.uniform(-1, 1, 256 * 64), np.zeros(256), np.full(256, 0.3), -np.abs(rng.normal(0, 1, 256)),
        np.abs(rng.normal(0, 1, 256)),
    ]).astype(np.float32)
    assert np.array_equal(oracle.pack(element, values), synth.QUANTIZE[element](values))


def test_q8_0_pack_invariants():
    values = oracle.random(32 * 500, 7)  # the reference's own packing test draws seed 7 (runtime.rs:727)
    raw = oracle.pack(oracle.EL_Q8_0, values)
    back = oracle.unpack(oracle.EL_Q8_0, raw, values.size)
    blocks = raw.reshape(-1, 34)
    d = blocks[:, 0:2].copy().view(np.float16).astype(np.float32).reshape(-1)
    codes = blocks[:, 2:].view(np.int8)
    assert codes.min() >= -127 and codes.max() <= 127
    # every block holds a +-127 code: the scale is max|x| / 127
    assert np.all(np.abs(codes).max(axis=1) == 127)
    error = np.abs(back - values).reshape(-1, 32).max(axis=1)
    assert np.all(error <= d * 0.5 + np.abs(values).reshape(-1, 32).max(axis=1) * 2.0 ** -10)  # half a step + fp16 rounding of d


def test_q4_k_pack_invariants():
    values = oracle.random(256 * 200, 23)  # runtime.rs:24 draws seed 23
    raw = oracle.pack(oracle.EL_Q4_K, values)
    back = oracle.unpack(oracle.EL_Q4_K, raw, values.size)
    # 4-bit affine codes over a range of <= 2: step <= 2/15; error within a step
    assert np.abs(back - values).max() <= 2.0 / 15.0
    assert np.abs(back - values).mean() < 0.03
    assert oracle.lib().oracle_payload_bytes(12, 256 * 200) == raw.size == 200 * 144


def test_block_geometry():
    # crates/neura-abi/tests/layout.rs:147-158
    assert oracle.lib().oracle_payload_bytes(8, 32) == 34
    assert oracle.lib().oracle_payload_bytes(12, 256) == 144
    assert oracle.lib().oracle_payload_bytes(11, 256) == 110
    assert oracle.lib().oracle_payload_bytes(13, 256) == 176
    assert oracle.lib().oracle_payload_bytes(14, 256) == 210
    assert oracle.lib().oracle_payload_bytes(14, 256) == 210
    assert oracle.lib().oracle_payload_bytes(8, 4864 * 896) == 4630528
    assert oracle.lib().oracle_payload_bytes(12, 46792704) == 26320896
    assert oracle.lib().oracle_payload_bytes(12, 512 * 0 + 3584 * 18944) == 38191104
