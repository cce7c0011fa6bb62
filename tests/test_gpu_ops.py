"""GPU parity of every operator against the CPU oracle, through the C ABI.

Bars: dequantised weights and fp16 conversion bit-exact; products, norm, rope and attention
within 1e-3 relative or 1e-2 absolute of the oracle's fp32 accumulation (the tests assert much
tighter bounds where the arithmetic allows); argmax and gather exact."""
import json
import os

import numpy as np
import pytest

import cases
import oracle
from neura_amd import NH_Q3_K, NH_Q4_K, NH_Q5_K, NH_Q6_K, NH_Q8_0, NeuraError, synth

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def close(got, want, rel=1e-3, abs_=1e-2):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    bad = np.abs(got - want) > np.maximum(abs_, rel * np.abs(want))
    assert not bad.any(), "%d of %d outside tolerance, worst %g" % (bad.sum(), bad.size, np.abs(got - want).max())


def tight(got, want, scale=1e-5):
    """within `scale` of the largest expected magnitude: what fp32 reordering allows"""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    bound = scale * max(1.0, np.abs(want).max())
    assert np.abs(got - want).max() <= bound, (np.abs(got - want).max(), bound)


def as_exact_as_the_oracle(got, plain, exact, floor):
    """the device's distance from the exact (fp64) product is at most four times the oracle's own (or `floor` of the largest
    output where the oracle happens to sit on it); the measured ratio is printed so that a drift shows before it fails"""
    ours, theirs = float(np.abs(got - exact).max()), float(np.abs(plain - exact).max())
    print("distance from the exact product: device %.3g, oracle %.3g, ratio %.2f" % (ours, theirs, ours / theirs if theirs else float("inf")))
    assert ours <= max(4 * theirs, floor * max(1.0, float(np.abs(exact).max())))


# ------------------------------------------------------------------ codecs

@pytest.mark.parametrize("element", [NH_Q8_0, NH_Q3_K, NH_Q4_K, NH_Q5_K, NH_Q6_K])
def test_dequant_is_bit_exact(device, element):
    rng = np.random.default_rng(100 + element)
    elements = 256 * 4000
    raw = synth.RANDOM[element](rng, elements)
    got = device.dequant(element, raw, elements)
    want = oracle.unpack(element, raw, elements)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # packed real weights too (the reference's seeds)
    values = oracle.random(256 * 64, 23)
    raw = oracle.pack(element, values)
    assert np.array_equal(device.dequant(element, raw, values.size).view(np.uint32), oracle.unpack(element, raw, values.size).view(np.uint32))


@pytest.mark.parametrize("element", [NH_Q8_0, NH_Q3_K, NH_Q4_K, NH_Q5_K, NH_Q6_K])
def test_dequant_of_the_committed_blocks(device, element):
    """hand-built blocks stored under tests/golden/ with the float32 bit patterns they unpack to: the device against the
    file, not against an oracle run beside it"""
    held = np.load(os.path.join(GOLDEN, "hand_built_blocks.npz"))
    raw, bits = held["raw_%d" % element], held["bits_%d" % element]
    assert np.array_equal(device.dequant(element, raw, bits.size).view(np.uint32), bits)


def test_dequant_refuses_ragged_and_unknown(device):
    raw = np.zeros(144, dtype=np.uint8)
    with pytest.raises(NeuraError):
        device.dequant(NH_Q4_K, raw, 100)
    with pytest.raises(NeuraError):
        device.dequant(10, raw, 256)  # Q2_K: the reference reads it neither (crates/neura-gguf/src/header.rs:150-162)


def test_convert_half_is_bit_exact(device):
    rng = np.random.default_rng(101)
    values = np.concatenate([
        rng.standard_normal(100000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 100000).astype(np.float32),
        rng.integers(0, 1 << 32, 100000, dtype=np.uint64).astype(np.uint32).view(np.float32),
        np.array([0.0, -0.0, 65504.0, 65520.0, 65519.9, np.inf, -np.inf, np.nan, 5.96e-8, 2.98e-8, 6.1e-5], dtype=np.float32),
    ])
    assert np.array_equal(device.convert_half(values), oracle.f32_to_f16(values))


@pytest.mark.parametrize("count", [5 * 96, 3 * 33, 7, 32 * 100000 + 13])
def test_pack_q8_0_is_the_host_s_blocks(device, count):
    """the device encoder against the host's on the reference's own data (crates/neura-runtime/tests/runtime.rs:717-736: seed 7,
    shapes 5x96, 3x33 and 7) and on three million numbers: byte-equal, the padding behind the last block included"""
    values = oracle.random(count, 7)
    padded = np.zeros(-(-count // 32) * 32, dtype=np.float32)
    padded[:count] = values
    want = oracle.pack(NH_Q8_0, padded)
    want = np.concatenate([want, np.zeros(-want.size % 4, dtype=np.uint8)])
    got = device.pack_q8_0(values)
    assert got.size == want.size and np.array_equal(got, want)
    # and the blocks read back as the numbers the oracle reads
    back = device.dequant(NH_Q8_0, got[: padded.size // 32 * 34], padded.size)
    assert np.array_equal(back.view(np.uint32), oracle.unpack(NH_Q8_0, want, padded.size).view(np.uint32))


def test_pack_q8_0_of_hard_blocks(device):
    rng = np.random.default_rng(41)
    values = np.concatenate([
        np.zeros(64), np.full(32, 0.3), rng.normal(0, 1, 3200) * 10.0 ** rng.integers(-30, 30, 3200), np.full(32, -1e-38), np.full(32, 3e38),
        (rng.integers(-254, 255, 3200) * 0.5 / 127.0),  # quotients that land on halves
    ]).astype(np.float32)
    got, want = device.pack_q8_0(values), oracle.pack(NH_Q8_0, values)
    assert got.size == want.size + 2 and not got[want.size :].any()  # an odd number of blocks ends two bytes short of a word
    assert np.array_equal(got[: want.size], want)


@pytest.mark.parametrize("element,width", [(NH_Q8_0, 896), (NH_Q4_K, 1536), (NH_Q6_K, 768), (NH_Q5_K, 512), (NH_Q3_K, 768)])
def test_gather_is_the_dequantised_row_times_mask(device, element, width):
    rng = np.random.default_rng(102)
    vocab = 50
    raw = synth.RANDOM[element](rng, vocab * width)
    table = oracle.unpack(element, raw, vocab * width).reshape(vocab, width)
    tokens = np.array([0, 49, 7, 7, 13, 21], dtype=np.uint32)
    got = device.gather(element, raw, vocab, width, tokens, batch=2, mask=[1, 0])
    want = table[tokens] * np.array([1, 0, 1, 0, 1, 0], dtype=np.float32)[:, None]
    assert np.array_equal(got, want)
    with pytest.raises(NeuraError) as refused:  # refusal::INDEX (select.rs:38)
        device.gather(element, raw, vocab, width, np.array([50], dtype=np.uint32))
    assert refused.value.code == -4
    assert np.array_equal(device.gather(element, raw, vocab, width, tokens[:1]), table[:1])  # the refusal word was cleared


# ------------------------------------------------------------------ narrow products

def test_config1_q8_0_gemv_4864x896_seed0(device):
    rng = np.random.default_rng(0)
    N, K = 4864, 896
    raw = synth.q8_0_random(rng, N * K)
    x = rng.standard_normal(K).astype(np.float32)
    got = device.gemv(NH_Q8_0, raw, N, K, x)[0]
    want = oracle.gemv(NH_Q8_0, raw, N, K, x, threads=8)[0]
    close(got, want)
    tight(got, want, 2e-6)


def test_config1_against_the_committed_outputs(device):
    """configuration 1 from its seed, checked to be the stored inputs by SHA-256, against the outputs the oracle gave when the
    fixture was written; and the stored 64-row slice of W alone against the stored first 64 outputs"""
    held = np.load(os.path.join(GOLDEN, "config1_q8_0_gemv.npz"))
    with open(os.path.join(GOLDEN, "config1_q8_0_gemv.json")) as text:
        sums = json.load(text)
    N, K, raw, x = cases.config1()
    assert cases.sha256(raw) == sums["w_sha256"] and cases.sha256(x) == sums["x_sha256"]
    want = held["y_bits"].view(np.float32)
    tight(device.gemv(NH_Q8_0, raw, N, K, x)[0], want, 2e-6)
    tight(device.gemv(NH_Q8_0, held["w_first_64_rows"], 64, K, held["x"])[0], want[:64], 2e-6)


@pytest.mark.parametrize("element", [NH_Q3_K, NH_Q4_K, NH_Q5_K, NH_Q6_K])
def test_k_quant_products_against_the_committed_outputs(device, element):
    """a one-row product of each K-quant (the 16-row tiles take all four) against the outputs the oracle gave when the fixture
    was written, plain and with SwiGLU over the stored outputs' halves"""
    held = np.load(os.path.join(GOLDEN, "kquant_gemv.npz"))
    N, K, _, _ = cases.kquant_products(element)
    raw, x, want = held["raw_%d" % element], held["x_%d" % element], held["y_bits_%d" % element].view(np.float32)
    tight(device.gemv(element, raw, N, K, x)[0], want, 3e-6)
    gate, up = want[: N // 2].astype(np.float64), want[N // 2:].astype(np.float64)
    gated = gate / (1.0 + np.exp(-gate)) * up
    close(device.gemv(element, raw, N, K, x, swiglu=True)[0], gated, rel=1e-3, abs_=1e-4 * max(1.0, np.abs(gated).max()))


@pytest.mark.parametrize("name,N,K,seed", [("q", 1536, 1536, 201), ("k", 256, 1536, 202), ("o", 1536, 1536, 203), ("gate", 8960, 1536, 204),
                                           ("down", 1536, 8960, 205)])
def test_config2_q4_k_gemvs_of_a_1_5b_layer(device, name, N, K, seed):
    rng = np.random.default_rng(seed)
    raw = synth.q4_k_random(rng, N * K)
    x = rng.standard_normal(K).astype(np.float32)
    got = device.gemv(NH_Q4_K, raw, N, K, x)[0]
    want = oracle.gemv(NH_Q4_K, raw, N, K, x, threads=8)[0]
    close(got, want)
    tight(got, want, 2e-6)


@pytest.mark.parametrize("element", [NH_Q8_0, NH_Q3_K, NH_Q4_K, NH_Q5_K, NH_Q6_K])
@pytest.mark.parametrize("rows", [1, 2, 3, 4, 7, 8])
def test_reference_narrow_product_test(device, element, rows):
    # crates/neura-runtime/tests/runtime.rs:12-86 at its own shape, seeds and elements
    depth, columns = 2048, 1024
    payload = oracle.pack(element, oracle.random(columns * depth, 23))
    inputs = oracle.random(rows * depth, 29).reshape(rows, depth)
    got = device.gemv(element, payload, columns, depth, inputs)
    want = oracle.gemv(element, payload, columns, depth, inputs, threads=8)
    assert np.abs(got - want).max() <= 1e-3  # the reference's own bar
    tight(got, want, 2e-6)


@pytest.mark.parametrize("element,N,K", [(NH_Q8_0, 5, 32), (NH_Q8_0, 33, 96), (NH_Q8_0, 1, 2048 + 32), (NH_Q8_0, 130, 4864), (NH_Q8_0, 20, 8192), (NH_Q8_0, 6, 8160),
                                         (NH_Q8_0, 4, 1056), (NH_Q4_K, 3, 256),
                                         (NH_Q4_K, 17, 512), (NH_Q4_K, 1, 4096 + 256), (NH_Q4_K, 66, 18944), (NH_Q4_K, 9, 3584)])
def test_gemv_ragged_shapes(device, element, N, K):
    rng = np.random.default_rng(N * 7 + K)
    raw = synth.RANDOM[element](rng, N * K)
    for rows in (1, 2, 5):
        x = rng.standard_normal((rows, K)).astype(np.float32)
        got = device.gemv(element, raw, N, K, x)
        want = oracle.gemv(element, raw, N, K, x, threads=8)
        close(got, want)
        tight(got, want, 3e-6)


@pytest.mark.parametrize("element,N,K", [(NH_Q8_0, 64, 896), (NH_Q4_K, 64, 1536), (NH_Q4_K, 32, 8960)])
def test_gemv_epilogues(device, element, N, K):
    rng = np.random.default_rng(5)
    raw = synth.RANDOM[element](rng, N * K)
    for rows in (1, 4):
        x = rng.standard_normal((rows, K)).astype(np.float32)
        r = rng.standard_normal((rows, N)).astype(np.float32)
        plain = oracle.gemv(element, raw, N, K, x, threads=8)
        tight(device.gemv(element, raw, N, K, x, residual=r), r + plain, 3e-6)
        gate, up = plain[:, : N // 2], plain[:, N // 2:]
        want = gate * (np.float32(1) / (np.float32(1) + np.exp(-gate))) * up
        close(device.gemv(element, raw, N, K, x, swiglu=True), want, rel=1e-4, abs_=1e-4 * np.abs(want).max())


@pytest.mark.parametrize("mode", ["0", "2"])
@pytest.mark.parametrize("N,K,rows", [(16, 256, 1), (48, 512, 3), (272, 3584, 1), (64, 1536, 8), (32, 18944, 1), (32, 18944, 5), (1040, 768, 2)])
def test_q4_k_products_agree_in_every_form(device, monkeypatch, mode, N, K, rows):
    """NEURA_HIP_MFMA=0 forces the vector kernels, =2 the matrix-core kernel (integer MFMA over four-digit activations);
    both sit within fp32 reordering of the order-faithful oracle, plain, with a residual and with SwiGLU, for 1..8
    activation rows, rows deeper than one LDS stage, and activations that span many orders of magnitude."""
    monkeypatch.setenv("NEURA_HIP_MFMA", mode)
    rng = np.random.default_rng(N + K + rows)
    raw = synth.q4_k_random(rng, N * K)
    x = (rng.standard_normal((rows, K)) * np.exp(rng.uniform(-6, 6, (rows, K)))).astype(np.float32)  # wide dynamic range
    r = rng.standard_normal((rows, N)).astype(np.float32)
    plain = oracle.gemv(NH_Q4_K, raw, N, K, x, threads=8)
    exact = oracle.unpack(NH_Q4_K, raw, N * K).reshape(N, K).astype(np.float64) @ x.astype(np.float64).T
    scale = max(1.0, np.abs(exact).max())
    got = device.gemv(NH_Q4_K, raw, N, K, x)
    close(got, plain)
    # as close to the exact product as the oracle's own fp32 sums are, up to a small factor
    assert np.abs(got - exact.T).max() <= max(4 * np.abs(plain - exact.T).max(), 2e-6 * scale)
    tight(device.gemv(NH_Q4_K, raw, N, K, x, residual=r), r + plain, 1e-5)
    gate, up = plain[:, : N // 2].astype(np.float64), plain[:, N // 2:].astype(np.float64)
    want = gate / (1.0 + np.exp(-gate)) * up
    close(device.gemv(NH_Q4_K, raw, N, K, x, swiglu=True), want, rel=1e-3, abs_=1e-4 * max(1.0, np.abs(want).max()))


@pytest.mark.parametrize("N,K,rows", [(64, 3584, 1), (96, 2048, 4), (128, 256, 2), (2048, 3584, 7), (64, 4096, 3), (64, 1536, 8), (160, 768, 5),
                                      (64, 18944, 8), (96, 8960, 2), (32, 18944, 5)])
@pytest.mark.parametrize("forced", ["NEURA_HIP_MFMA32", "NEURA_HIP_F16_TILES"])
def test_q4_k_product_on_32_row_tiles(device, monkeypatch, forced, N, K, rows):
    """NEURA_HIP_MFMA32=2 forces the 32 x 32 x 32 integer MFMA kernel (weights as the B operand, the digit planes of up to
    eight activation rows as A, digits scaled per sub-block): plain, with a residual and with SwiGLU, for every count of
    activation rows, against the oracle and an fp64 product (the decoder tests run it with the fused norm).
    NEURA_HIP_F16_TILES=2 forces, for two rows and more, the 16-row tiles on half-precision MFMA (weights as exact halves
    code * sc, activations as value and residue half rows) through the same cases."""
    monkeypatch.setenv(forced, "2")
    rng = np.random.default_rng(N + K + rows)
    raw = synth.q4_k_random(rng, N * K)
    x = (rng.standard_normal((rows, K)) * np.exp(rng.uniform(-6, 6, (rows, K)))).astype(np.float32)  # wide dynamic range
    r = rng.standard_normal((rows, N)).astype(np.float32)
    plain = oracle.gemv(NH_Q4_K, raw, N, K, x, threads=8)
    exact = oracle.unpack(NH_Q4_K, raw, N * K).reshape(N, K).astype(np.float64) @ x.astype(np.float64).T
    got = device.gemv(NH_Q4_K, raw, N, K, x)
    close(got, plain)
    assert np.abs(got - exact.T).max() <= max(4 * np.abs(plain - exact.T).max(), 2e-6 * max(1.0, np.abs(exact).max()))
    tight(device.gemv(NH_Q4_K, raw, N, K, x, residual=r), r + plain, 1e-5)
    gate, up = plain[:, : N // 2].astype(np.float64), plain[:, N // 2:].astype(np.float64)
    want = gate / (1.0 + np.exp(-gate)) * up
    close(device.gemv(NH_Q4_K, raw, N, K, x, swiglu=True), want, rel=1e-3, abs_=1e-4 * max(1.0, np.abs(want).max()))
    x[0, 5] = np.inf
    assert not np.isfinite(device.gemv(NH_Q4_K, raw, N, K, x)[0]).any()


@pytest.mark.parametrize("tile16", ["1", "0"])
@pytest.mark.parametrize("N,K", [(16, 256), (64, 3584), (4608, 3584), (3584, 18944), (37888, 3584), (1040, 768), (48, 2048), (272, 8960), (2048, 1536),
                                 (17920, 1536), (1536, 1280)])
def test_q4_k_one_row_product_on_16_row_tiles(device, monkeypatch, tile16, N, K):
    """One activation row against Q4_K rows: the 16-row tiles on the 16 x 16 x 64 integer MFMA (weights as nibbles, the
    activation as three signed digit planes scaled per 64 numbers), and with NEURA_HIP_TILE16=0 the kernels that served
    before it.  Activations over many orders of magnitude, with outliers that set a group's scale from any seat of it;
    plain, with a residual (added in place), with SwiGLU; non-finite inputs stay visible and zeros give zeros."""
    monkeypatch.setenv("NEURA_HIP_TILE16", tile16)
    rng = np.random.default_rng(N + K)
    raw = synth.q4_k_random(rng, N * K)
    weights = oracle.unpack(NH_Q4_K, raw, N * K).reshape(N, K).astype(np.float64)
    r = rng.standard_normal((1, N)).astype(np.float32)
    for spread, outliers in ((2.0, False), (6.0, False), (6.0, True)):
        x = (rng.standard_normal((1, K)) * np.exp(rng.uniform(-spread, spread, (1, K)))).astype(np.float32)
        if outliers:
            x[0, rng.integers(0, K, 24)] *= 1e4  # at any seat of a group
        plain = oracle.gemv(NH_Q4_K, raw, N, K, x, threads=8)
        exact = weights @ x.astype(np.float64).T
        got = device.gemv(NH_Q4_K, raw, N, K, x)
        if spread == 2.0:
            close(got, plain)  # past this spread the oracle's own fp32 sums are the looser side: the exact product judges
        as_exact_as_the_oracle(got, plain, exact.T, 2e-6)
        tight(device.gemv(NH_Q4_K, raw, N, K, x, residual=r), r + plain, 1e-5)
    if N % 32 == 0:
        x = rng.standard_normal((1, K)).astype(np.float32)
        x[0, rng.integers(0, K, 8)] *= 50.0
        plain = oracle.gemv(NH_Q4_K, raw, N, K, x, threads=8)
        gate, up = plain[:, : N // 2].astype(np.float64), plain[:, N // 2 :].astype(np.float64)
        want = gate / (1.0 + np.exp(-gate)) * up
        close(device.gemv(NH_Q4_K, raw, N, K, x, swiglu=True), want, rel=1e-3, abs_=1e-4 * max(1.0, np.abs(want).max()))
    x[0, 5] = np.inf
    assert not np.isfinite(device.gemv(NH_Q4_K, raw, N, K, x)).any()
    assert not np.isfinite(device.gemv(NH_Q4_K, raw, N, K, np.full((1, K), np.nan, np.float32))).any()
    assert np.array_equal(device.gemv(NH_Q4_K, raw, N, K, np.zeros((1, K), np.float32)), np.zeros((1, N), np.float32))


@pytest.mark.parametrize("N,K,rows", [(16, 256, 2), (64, 3584, 4), (4608, 3584, 4), (3584, 3584, 3), (4608, 3584, 2), (1040, 768, 4), (48, 2048, 3),
                                      (272, 8960, 4), (96, 18944, 2), (37888, 3584, 4), (64, 10240, 3), (152064, 3584, 2)])
def test_q4_k_products_of_a_few_rows_on_16_row_tiles(device, monkeypatch, N, K, rows):
    """(NEURA_HIP_ROWS4=0: the form that serves where the kernel with four rows to an MFMA does not fit.)
    Two to four activation rows against Q4_K rows in one pass of the 16-row tiles (every row its own digit planes, the
    weights unpacked once a step): each row is, bit for bit, what the one-row product gives for it alone, plain, with a
    residual and with SwiGLU (the decoders' batches run it with the norm folded in); and the whole sits as close to the exact
    product as the oracle does.  A non-finite number stays in its own row."""
    monkeypatch.setenv("NEURA_HIP_ROWS4", "0")
    rng = np.random.default_rng(N + K + rows)
    raw = synth.q4_k_random(rng, N * K)
    x = (rng.standard_normal((rows, K)) * np.exp(rng.uniform(-2, 2, (rows, K)))).astype(np.float32)
    r = rng.standard_normal((rows, N)).astype(np.float32)
    if N * K <= 4608 * 3584:
        close(device.gemv(NH_Q4_K, raw, N, K, x), oracle.gemv(NH_Q4_K, raw, N, K, x, threads=8))
    x[rows - 1, rng.integers(0, K, 8)] *= 1e3  # with outliers the oracle's own fp32 sums are the looser side: the exact product judges
    got = device.gemv(NH_Q4_K, raw, N, K, x)
    if N * K <= 4608 * 3584:
        plain = oracle.gemv(NH_Q4_K, raw, N, K, x, threads=8)
        exact = oracle.unpack(NH_Q4_K, raw, N * K).reshape(N, K).astype(np.float64) @ x.astype(np.float64).T
        as_exact_as_the_oracle(got, plain, exact.T, 2e-6)
    with_residual = device.gemv(NH_Q4_K, raw, N, K, x, residual=r)
    gated = device.gemv(NH_Q4_K, raw, N, K, x, swiglu=True) if N % 32 == 0 else None
    for row in range(rows):
        one = x[row : row + 1]
        assert np.array_equal(got[row : row + 1], device.gemv(NH_Q4_K, raw, N, K, one)), row
        assert np.array_equal(with_residual[row : row + 1], device.gemv(NH_Q4_K, raw, N, K, one, residual=r[row : row + 1])), row
        if gated is not None:
            assert np.array_equal(gated[row : row + 1], device.gemv(NH_Q4_K, raw, N, K, one, swiglu=True)), row
    x[0, 5] = np.inf
    spoilt = device.gemv(NH_Q4_K, raw, N, K, x)
    assert not np.isfinite(spoilt[0]).any() and np.array_equal(spoilt[1:], got[1:])


@pytest.mark.parametrize("N,K,rows", [(16, 256, 3), (64, 3584, 4), (4608, 3584, 4), (3584, 3584, 3), (4608, 3584, 3), (1040, 768, 4), (48, 2048, 3),
                                      (272, 8960, 4), (37888, 3584, 4), (37888, 3584, 3), (64, 10240, 3), (152064, 3584, 3)])
def test_q4_k_products_of_several_rows_four_rows_to_an_mfma(device, N, K, rows):
    """Three and four activation rows against Q4_K rows, four activation rows in an MFMA's sixteen operand rows and the
    sub-block scales inside the weight operand: within the product's bar of the oracle and as close to the exact product as the oracle is, plain, with a residual
    and with SwiGLU; a row's numbers do not depend on the rows beside it (bit for bit what it gives next to rows of zeros),
    and a non-finite number stays in its own row."""
    rng = np.random.default_rng(N + K + rows)
    raw = synth.q4_k_random(rng, N * K)
    x = (rng.standard_normal((rows, K)) * np.exp(rng.uniform(-2, 2, (rows, K)))).astype(np.float32)
    r = rng.standard_normal((rows, N)).astype(np.float32)
    small = N * K <= 4608 * 3584
    if small:
        plain = oracle.gemv(NH_Q4_K, raw, N, K, x, threads=8)
        close(device.gemv(NH_Q4_K, raw, N, K, x), plain)
        tight(device.gemv(NH_Q4_K, raw, N, K, x, residual=r), r + plain, 1e-5)
    x[rows - 1, rng.integers(0, K, 8)] *= 1e3  # with outliers the oracle's own fp32 sums are the looser side: the exact product judges
    got = device.gemv(NH_Q4_K, raw, N, K, x)
    if small:
        plain = oracle.gemv(NH_Q4_K, raw, N, K, x, threads=8)
        exact = oracle.unpack(NH_Q4_K, raw, N * K).reshape(N, K).astype(np.float64) @ x.astype(np.float64).T
        # the digits' scale is a super-block's here: an outlier costs its 255 neighbours the bits it stands above them
        as_exact_as_the_oracle(got, plain, exact.T, 8e-6)
        if N % 32 == 0:
            gate, up = plain[:, : N // 2].astype(np.float64), plain[:, N // 2 :].astype(np.float64)
            want = gate / (1.0 + np.exp(-gate)) * up
            close(device.gemv(NH_Q4_K, raw, N, K, x, swiglu=True), want, rel=1e-3, abs_=1e-4 * max(1.0, np.abs(want).max()))
    with_residual = device.gemv(NH_Q4_K, raw, N, K, x, residual=r)
    gated = device.gemv(NH_Q4_K, raw, N, K, x, swiglu=True) if N % 32 == 0 else None
    for row in range(rows):
        beside_zeros = np.concatenate([x[row : row + 1], np.zeros((2, K), np.float32)])
        assert np.array_equal(got[row], device.gemv(NH_Q4_K, raw, N, K, beside_zeros)[0]), row
        assert np.array_equal(with_residual[row], device.gemv(NH_Q4_K, raw, N, K, beside_zeros, residual=np.stack([r[row], r[row], r[row]]))[0]), row
        if gated is not None:
            assert np.array_equal(gated[row], device.gemv(NH_Q4_K, raw, N, K, beside_zeros, swiglu=True)[0]), row
    # one row through the one-row kernel: the same numbers to the last few bits
    tight(got[0:1], device.gemv(NH_Q4_K, raw, N, K, x[0:1]), 8e-6)
    x[0, 5] = np.inf
    spoilt = device.gemv(NH_Q4_K, raw, N, K, x)
    assert not np.isfinite(spoilt[0]).any() and np.array_equal(spoilt[1:], got[1:])
    assert np.array_equal(device.gemv(NH_Q4_K, raw, N, K, np.zeros((rows, K), np.float32)), np.zeros((rows, N), np.float32))


def test_q4_k_product_on_the_matrix_cores_keeps_non_finite_inputs_visible(device, monkeypatch):
    monkeypatch.setenv("NEURA_HIP_MFMA", "2")
    rng = np.random.default_rng(2)
    N, K = 32, 512
    raw = synth.q4_k_random(rng, N * K)
    x = rng.standard_normal((2, K)).astype(np.float32)
    x[1, 77] = np.inf
    got = device.gemv(NH_Q4_K, raw, N, K, x)
    assert np.isfinite(got[0]).all() and not np.isfinite(got[1]).any()
    assert not np.isfinite(device.gemv(NH_Q4_K, raw, N, K, np.full((1, K), np.nan, np.float32))).any()
    assert np.array_equal(device.gemv(NH_Q4_K, raw, N, K, np.zeros((1, K), np.float32)), np.zeros((1, N), np.float32))


@pytest.mark.parametrize("element", [NH_Q6_K, NH_Q5_K, NH_Q3_K])
@pytest.mark.parametrize("N,K,rows", [(2, 256, 1), (7, 512, 3), (272, 3584, 1), (64, 1536, 8), (32, 18944, 1), (33, 18944, 5), (1040, 768, 2)])
def test_staged_super_block_products(device, element, N, K, rows):
    """Q6_K and Q3_K rows start on 2-byte boundaries (210- and 110-byte blocks), Q5_K rows on 16-byte ones: every alignment
    of a row, odd row counts, rows deeper than one LDS stage (K slices folded by a second kernel), 1..8 activation rows,
    plain, residual and SwiGLU."""
    rng = np.random.default_rng(N + K + rows + element)
    raw = synth.RANDOM[element](rng, N * K)
    x = rng.standard_normal((rows, K)).astype(np.float32)
    r = rng.standard_normal((rows, N)).astype(np.float32)
    plain = oracle.gemv(element, raw, N, K, x, threads=8)
    exact = oracle.unpack(element, raw, N * K).reshape(N, K).astype(np.float64) @ x.astype(np.float64).T
    got = device.gemv(element, raw, N, K, x)
    close(got, plain)
    tight(got, plain, 3e-6)
    assert np.abs(got - exact.T).max() <= max(4 * np.abs(plain - exact.T).max(), 2e-6 * max(1.0, np.abs(exact).max()))
    tight(device.gemv(element, raw, N, K, x, residual=r), r + plain, 1e-5)
    if N % 2 == 0:
        gate, up = plain[:, : N // 2].astype(np.float64), plain[:, N // 2:].astype(np.float64)
        want = gate / (1.0 + np.exp(-gate)) * up
        close(device.gemv(element, raw, N, K, x, swiglu=True), want, rel=1e-3, abs_=1e-4 * max(1.0, np.abs(want).max()))


@pytest.mark.parametrize("tile16", ["1", "0"])
@pytest.mark.parametrize("element,switch", [(NH_Q6_K, "NEURA_HIP_Q6K_TILE16"), (NH_Q5_K, "NEURA_HIP_Q5K_TILE16"), (NH_Q3_K, "NEURA_HIP_Q6K_TILE16")],
                         ids=["q6_k", "q5_k", "q3_k"])
@pytest.mark.parametrize("N,K", [(16, 256), (64, 3584), (3584, 18944), (4608, 3584), (1040, 768), (48, 2048), (272, 8960), (37888, 3584), (2048, 1536)])
def test_q6_k_and_q5_k_one_row_products_on_16_row_tiles(device, monkeypatch, tile16, element, switch, N, K):
    """One activation row against Q6_K rows on the 16 x 16 x 64 integer MFMA (the stored 6-bit codes as bytes, a scale per
    lane slice, the activation as three signed digit planes with a sum and a scale per 16 numbers), against Q3_K rows the
    same way (3-bit codes, 6-bit scales) and against Q5_K rows on the Q4_K tiles with the fifth bit beside the nibble; with
    NEURA_HIP_Q6K_TILE16=0 / NEURA_HIP_Q5K_TILE16=0 the staged kernel that served before them.  Rows of 210- and 110-byte
    blocks start on every alignment of a half word; activations over many
    orders of magnitude, with outliers at any seat; plain, with a residual (added in place) and with SwiGLU; non-finite
    inputs stay visible and zeros give zeros."""
    monkeypatch.setenv(switch, tile16)
    NH_Q6_K = element  # (the body below was written for Q6_K: the same checks serve both)
    rng = np.random.default_rng(N + K + 6)
    raw = synth.RANDOM[NH_Q6_K](rng, N * K)
    weights = oracle.unpack(NH_Q6_K, raw, N * K).reshape(N, K).astype(np.float64)
    r = rng.standard_normal((1, N)).astype(np.float32)
    for spread, outliers in ((0.0, False), (2.0, False), (6.0, False), (6.0, True)):
        x = (rng.standard_normal((1, K)) * np.exp(rng.uniform(-spread, spread, (1, K)))).astype(np.float32)
        if outliers:
            x[0, rng.integers(0, K, 24)] *= 1e4  # at any seat of a group
        plain = oracle.gemv(NH_Q6_K, raw, N, K, x, threads=8)
        exact = weights @ x.astype(np.float64).T
        got = device.gemv(NH_Q6_K, raw, N, K, x)
        if spread <= 2.0:
            close(got, plain)  # past this spread the oracle's own fp32 sums are the looser side: the exact product judges
        # (the digits keep 22 bits below the largest of 64 activations: what an outlier's neighbours lose is weighed by codes of
        # five bits where Q4_K's have four, so the floor under the bar is twice Q4_K's)
        as_exact_as_the_oracle(got, plain, exact.T, 2e-6 if element == 14 else 4e-6)
        tight(device.gemv(NH_Q6_K, raw, N, K, x, residual=r), r + plain, 1e-5)
    if N % 32 == 0:
        x = rng.standard_normal((1, K)).astype(np.float32)
        x[0, rng.integers(0, K, 8)] *= 50.0
        plain = oracle.gemv(NH_Q6_K, raw, N, K, x, threads=8)
        gate, up = plain[:, : N // 2].astype(np.float64), plain[:, N // 2:].astype(np.float64)
        with np.errstate(over="ignore"):
            want = gate / (1.0 + np.exp(-gate)) * up
        close(device.gemv(NH_Q6_K, raw, N, K, x, swiglu=True), want, rel=1e-3, abs_=1e-4 * max(1.0, np.abs(want).max()))
    x[0, 5] = np.inf
    assert not np.isfinite(device.gemv(NH_Q6_K, raw, N, K, x)).any()
    assert not np.isfinite(device.gemv(NH_Q6_K, raw, N, K, np.full((1, K), np.nan, np.float32))).any()
    assert np.array_equal(device.gemv(NH_Q6_K, raw, N, K, np.zeros((1, K), np.float32)), np.zeros((1, N), np.float32))


@pytest.mark.parametrize("element", [NH_Q6_K, NH_Q5_K, NH_Q3_K])
def test_staged_super_block_product_reads_packed_weights(device, element):
    N, K = 96, 2048
    values = oracle.random(N * K, 23)
    if element == NH_Q6_K:
        values = np.abs(values)  # the reference's Q6_K packing keeps non-negative values alone
    raw = oracle.pack(element, values)
    x = oracle.random(K, 29).reshape(1, K)
    tight(device.gemv(element, raw, N, K, x), oracle.gemv(element, raw, N, K, x, threads=8), 2e-6)


@pytest.mark.parametrize("element", [NH_Q4_K, NH_Q6_K, NH_Q5_K, NH_Q3_K])
def test_gemv_is_linear_and_matches_at_full_size(device, element):
    # size-independent properties at the 7B FFN shape: W(a x + b z) = a W x + b W z
    rng = np.random.default_rng(6)
    N, K = 18944, 3584
    host = synth.RANDOM[element](rng, N * K)
    raw = device.upload(host)
    x, z = rng.standard_normal(K).astype(np.float32), rng.standard_normal(K).astype(np.float32)
    yx, yz = device.gemv(element, raw, N, K, x)[0], device.gemv(element, raw, N, K, z)[0]
    both = device.gemv(element, raw, N, K, np.float32(0.5) * x - np.float32(2.0) * z)[0]
    tight(both, 0.5 * yx - 2.0 * yz, 1e-5)
    batched = device.gemv(element, raw, N, K, np.stack([x, z]))
    tight(batched[0], yx, 3e-6)  # (two rows of a K-quant other than Q4_K run the staged kernel: another order of the sums)
    tight(batched[1], yz, 3e-6)
    assert np.array_equal(yx, device.gemv(element, raw, N, K, x)[0])  # deterministic
    # and a handful of rows against the exact product of the unpacked weights
    row_bytes = host.nbytes // N
    for n in rng.integers(0, N, 8):
        weights = oracle.unpack(element, host[n * row_bytes:(n + 1) * row_bytes], K).astype(np.float64)
        assert abs(float(yx[n]) - float(weights @ x.astype(np.float64))) <= 2e-5 * max(1.0, float(np.abs(yx).max()))


def test_gemv_refuses_bad_shapes(device):
    raw = np.zeros(34 * 4, dtype=np.uint8)
    for args in ((NH_Q8_0, raw, 4, 33), (11, raw, 4, 32)):
        with pytest.raises(NeuraError):
            device.gemv(args[0], args[1], args[2], args[3], np.zeros(args[3], dtype=np.float32))
    with pytest.raises(NeuraError):
        device.gemv(NH_Q8_0, raw, 4, 32, np.zeros((9, 32), dtype=np.float32))


# ------------------------------------------------------------------ wide products

@pytest.mark.parametrize("element", [NH_Q8_0, NH_Q4_K, NH_Q5_K, NH_Q3_K])
def test_reference_wide_product_test(device, element):
    # crates/neura-runtime/tests/runtime.rs:88-144: 8 x 512 x 4096, seeds 23 / 29, tolerance 1e-3
    rows, depth, columns = 8, 512, 4096
    payload = oracle.pack(element, oracle.random(columns * depth, 23))
    inputs = oracle.random(rows * depth, 29).reshape(rows, depth)
    want = oracle.gemm(element, payload, columns, depth, inputs, threads=8)
    got = device.gemm(element, payload, columns, depth, inputs)
    assert np.abs(got - want).max() <= 1e-3


@pytest.mark.parametrize("element,M,N,K,half", [(NH_Q4_K, 70, 130, 512, True), (NH_Q4_K, 512, 256, 3584, True), (NH_Q4_K, 33, 64, 256, False),
                                                (NH_Q8_0, 100, 96, 896, False), (NH_Q8_0, 64, 64, 64, True), (NH_Q8_0, 200, 300, 4864, False),
                                                (NH_Q8_0, 130, 128, 192, True), (NH_Q8_0, 512, 1152, 896, False), (NH_Q8_0, 16, 32, 96, False),
                                                (NH_Q8_0, 9, 129, 320, False), (NH_Q6_K, 70, 130, 512, False),
                                                (NH_Q6_K, 40, 64, 3584, True), (NH_Q5_K, 70, 130, 512, True), (NH_Q5_K, 33, 64, 3584, False),
                                                (NH_Q3_K, 70, 130, 512, False), (NH_Q3_K, 40, 64, 3584, True)])
def test_gemm_matches_fp32_accumulation(device, element, M, N, K, half):
    rng = np.random.default_rng(M + N + K)
    raw = synth.RANDOM[element](rng, N * K)
    X = rng.standard_normal((M, K)).astype(np.float16 if half else np.float32)
    want = oracle.gemm(element, raw, N, K, X.astype(np.float32), threads=8)
    got = device.gemm(element, raw, N, K, X)
    close(got, want)
    r = rng.standard_normal((M, N)).astype(np.float32)
    close(device.gemm(element, raw, N, K, X, residual=r), want + r)


@pytest.mark.parametrize("element,M,N,K,half", [(NH_Q8_0, 100, 96, 896, False), (NH_Q8_0, 64, 64, 64, True), (NH_Q4_K, 70, 130, 512, True),
                                                (NH_Q4_K, 33, 64, 256, False), (NH_Q6_K, 70, 130, 512, True), (NH_Q6_K, 33, 64, 256, False),
                                                (NH_Q5_K, 70, 130, 512, False), (NH_Q3_K, 70, 130, 512, True)])
def test_gemm_on_the_vector_unit_matches_too(device, monkeypatch, element, M, N, K, half):
    """NEURA_HIP_GEMM_MFMA=0 keeps Q8_0 and K-quant wide products on the tiled vector kernel that serves the shapes the matrix
    cores do not take (rows that are not whole steps, unaligned operands)."""
    monkeypatch.setenv("NEURA_HIP_GEMM_MFMA", "0")
    rng = np.random.default_rng(M + N + K)
    raw = synth.RANDOM[element](rng, N * K)
    X = rng.standard_normal((M, K)).astype(np.float16 if half else np.float32)
    close(device.gemm(element, raw, N, K, X), oracle.gemm(element, raw, N, K, X.astype(np.float32), threads=8))


@pytest.mark.parametrize("M,N,K,half", [(70, 130, 512, True), (512, 256, 3584, True), (33, 64, 256, False), (130, 300, 1024, False)])
def test_q4_k_wide_product_with_weights_unpacked_into_lds(device, monkeypatch, M, N, K, half):
    """NEURA_HIP_GEMM_REGB=0: the Q4_K wide product whose stager waves unpack the weights into LDS (the default form keeps a
    lane's weight row in its registers); both are held to the same bar."""
    monkeypatch.setenv("NEURA_HIP_GEMM_REGB", "0")
    rng = np.random.default_rng(M * N + K)
    raw = synth.RANDOM[NH_Q4_K](rng, N * K)
    X = rng.standard_normal((M, K)).astype(np.float16 if half else np.float32)
    close(device.gemm(NH_Q4_K, raw, N, K, X), oracle.gemm(NH_Q4_K, raw, N, K, X.astype(np.float32), threads=8))


@pytest.mark.parametrize("element", [NH_Q6_K, NH_Q5_K, NH_Q3_K])
@pytest.mark.parametrize("M,N,K,half", [(70, 130, 512, False), (40, 64, 3584, True), (512, 256, 1280, True), (33, 200, 256, False),
                                        (130, 128, 768, True), (64, 256, 18944, False), (512, 512, 3584, False)])
def test_q6_k_q5_k_and_q3_k_wide_products_on_the_matrix_cores(device, element, M, N, K, half):
    """Q6_K rows as two exact half planes on the matrix cores ((q - 32) * (sc & 15) and 16 * (q - 32) * (sc >> 4)), Q5_K rows
    as Q4_K's with the fifth bit beside the nibble, Q3_K rows as the one exact plane (sc - 32) * code: against the oracle at the wide product's bar and against the exact
    product far inside it -- for Q6_K scales at both ends of a signed byte and at the seams of the split, blocks that start
    on either half of a word (210-byte blocks: every other one does; Q3_K's 110-byte blocks too); for Q5_K scales, minimums
    and codes at their largest; for Q3_K scales and codes at both ends;
    ragged tiles, half and fp32 activations, and a residual."""
    rng = np.random.default_rng(M + N + K + element)
    if element == NH_Q6_K:
        raw = np.array(synth.RANDOM[NH_Q6_K](rng, N * K), dtype=np.uint8).reshape(-1, 210)
        hard = rng.random(raw.shape[0]) < 0.25
        raw[hard, 192:208] = rng.choice(np.array([-128, 127, -1, 15, 16, -16, -17, 0], np.int8).view(np.uint8), (int(hard.sum()), 16))
    elif element == NH_Q3_K:
        raw = np.array(synth.RANDOM[NH_Q3_K](rng, N * K), dtype=np.uint8).reshape(-1, 110)
        hard = rng.random(raw.shape[0]) < 0.25
        raw[hard, 0:108] = rng.choice(np.array([0x00, 0xFF], np.uint8), (int(hard.sum()), 1))  # scales -32 and codes -4, or +31 and +3
    else:
        raw = np.array(synth.RANDOM[NH_Q5_K](rng, N * K), dtype=np.uint8).reshape(-1, 176)
        hard = rng.random(raw.shape[0]) < 0.25
        raw[hard, 4:16] = 0xFF   # every scale and minimum 63
        raw[hard, 16:176] = 0xFF  # every code 31
    raw = raw.reshape(-1)
    X = rng.standard_normal((M, K)).astype(np.float16 if half else np.float32)
    want = oracle.gemm(element, raw, N, K, X.astype(np.float32), threads=8)
    got = device.gemm(element, raw, N, K, X)
    close(got, want)
    exact = X.astype(np.float64) @ oracle.unpack(element, raw, N * K).reshape(N, K).astype(np.float64).T
    assert np.abs(got - exact).max() <= max(4 * np.abs(want - exact).max(), 2e-6 * max(1.0, np.abs(exact).max()))
    r = rng.standard_normal((M, N)).astype(np.float32)
    close(device.gemm(element, raw, N, K, X, residual=r), want + r)


def test_q8_0_wide_product_of_the_small_decoder_s_shapes(device):
    """The Q8_0 products of a 512-token fill of the 0.5B-shape decoder (hidden 896, FFN 4864, 14 heads of 64, 2 key heads), weights
    N(0, 0.02) quantised as a checkpoint's are, fp32 activations over a few orders of magnitude: every output against fp32
    accumulation."""
    rng = np.random.default_rng(8)
    for N, K in [(1152, 896), (896, 896), (4864, 896), (896, 4864)]:
        raw = oracle.pack(NH_Q8_0, (rng.standard_normal(N * K) * 0.02).astype(np.float32))
        X = (rng.standard_normal((512, K)) * np.exp(rng.uniform(-3, 3, (512, K)))).astype(np.float32)
        want = oracle.gemm(NH_Q8_0, raw, N, K, X, threads=16)
        got = device.gemm(NH_Q8_0, raw, N, K, X)
        close(got, want, rel=1e-3, abs_=1e-2)
        tight(got, want, 1e-5)


def test_config3_wide_product_at_full_size(device):
    """The wide product of the benchmark as it is timed: M = 512, K = 3584, N = 18944 (148 column tiles by 4 row tiles),
    random Q4_K blocks, half activations N(0,1), every one of the 9.7 million outputs against fp32 accumulation."""
    M, K, N = 512, 3584, 18944
    rng = np.random.default_rng(33)
    raw = synth.q4_k_random(rng, N * K)
    X = rng.standard_normal((M, K)).astype(np.float16)
    want = oracle.gemm(NH_Q4_K, raw, N, K, X.astype(np.float32), threads=16)
    got = device.gemm(NH_Q4_K, raw, N, K, X)
    close(got, want)
    # and with the decoder's fp32 activations
    X32 = rng.standard_normal((M, K)).astype(np.float32)
    close(device.gemm(NH_Q4_K, raw, N, K, X32), oracle.gemm(NH_Q4_K, raw, N, K, X32, threads=16))


# ------------------------------------------------------------------ row operators

@pytest.mark.parametrize("C", [896, 1536, 3584, 100])
def test_rmsnorm_matches_bit_for_bit(device, C):
    rng = np.random.default_rng(C)
    x = rng.standard_normal((5, C)).astype(np.float32)
    w = rng.standard_normal(C).astype(np.float32)
    r = rng.standard_normal((5, C)).astype(np.float32)
    want, _ = oracle.rmsnorm(x, w, 1e-6)
    assert np.array_equal(device.rmsnorm(x, w, 1e-6), want)  # same summation order, same roundings
    want, total = oracle.rmsnorm(x, w, 1e-6, residual=r)
    got, got_total = device.rmsnorm(x, w, 1e-6, residual=r, want_sum=True)
    assert np.array_equal(got, want) and np.array_equal(got_total, total)


def test_gemv_with_fused_norm_equals_norm_then_gemv(device):
    # the decoder fuses the norm into the product's prologue; the C ABI exposes both halves
    rng = np.random.default_rng(8)
    N, K = 64, 3584
    raw = synth.q4_k_random(rng, N * K)
    x = rng.standard_normal((1, K)).astype(np.float32)
    w = rng.standard_normal(K).astype(np.float32)
    normed = device.rmsnorm(x, w, 1e-6)
    want = oracle.gemv(NH_Q4_K, raw, N, K, oracle.rmsnorm(x, w, 1e-6)[0])
    tight(device.gemv(NH_Q4_K, raw, N, K, normed), want, 2e-6)


@pytest.mark.parametrize("width,base,origin", [(64, 1e6, 0), (128, 1e6, 1023), (128, 1e6, 4095), (8, 10000.0, 3)])
def test_rope_matches_oracle(device, width, base, origin):
    rng = np.random.default_rng(71)  # runtime.rs:539 draws seed 71
    x = rng.standard_normal((3, 2, 4, width)).astype(np.float32)
    cursor = np.array([origin, origin // 2], dtype=np.uint32)
    got = device.rope(x, cursor, base)
    for plane in range(3):
        for b in range(2):
            want = oracle.rope(x[plane, b], int(cursor[b]), base)
            assert np.abs(got[plane, b] - want).max() <= 1e-4  # the reference's bar (runtime.rs:468-549)
            assert np.abs(got[plane, b] - want).max() <= 4e-6 * max(1.0, np.abs(want).max())


def test_cache_write_casts_and_scatters(device):
    rng = np.random.default_rng(9)
    kv_heads, batch, rows, width, capacity, window = 2, 3, 2, 64, 12, 10
    k = rng.standard_normal((kv_heads, batch, rows, width)).astype(np.float32)
    v = rng.standard_normal((kv_heads, batch, rows, width)).astype(np.float32)
    ck = device.alloc(kv_heads * batch * capacity * width * 2)
    cv = device.alloc(kv_heads * batch * capacity * width * 2)
    cursor = [0, 5, 8]
    device.cache_write(k, v, ck, cv, capacity, window, cursor, mask=[1, 1, 0])
    gk = ck.numpy(np.uint16, (kv_heads, batch, capacity, width))
    gv = cv.numpy(np.uint16, (kv_heads, batch, capacity, width))
    wk, wv = np.zeros_like(gk), np.zeros_like(gv)
    for b, (at, active) in enumerate(zip(cursor, [1, 1, 0])):
        first = at if active else window  # an inactive plane writes the scratch rows (cache.rs:336, :360-364)
        wk[:, b, first:first + rows] = oracle.f32_to_f16(k[:, b])
        wv[:, b, first:first + rows] = oracle.f32_to_f16(v[:, b])
    assert np.array_equal(gk, wk) and np.array_equal(gv, wv)
    with pytest.raises(NeuraError) as refused:  # a cursor past the capacity: refusal::ORIGIN
        device.cache_write(k, v, ck, cv, capacity, window, [0, 11, 0])
    assert refused.value.code == -4
    with pytest.raises(NeuraError):  # rows <= window <= capacity (cache.rs:117-125)
        device.cache_write(k, v, ck, cv, capacity, capacity + 1, cursor)


# ------------------------------------------------------------------ attention, choice

@pytest.mark.parametrize("heads,kv_heads,batch,rows,keys,width,origins", [
    (4, 2, 2, 3, 12, 32, [9, 4]),
    (14, 2, 1, 1, 1100, 64, [1024]),       # the 0.5B decode shape at context 1024
    (28, 4, 1, 1, 4200, 128, [4095]),      # the 7B decode shape at context 4096
    (28, 4, 8, 1, 600, 128, [0, 1, 63, 64, 65, 300, 511, 599]),
    (12, 2, 1, 17, 300, 128, [200]),       # a fill chunk
    (8, 8, 2, 5, 40, 256, [35, 0]),
    (6, 1, 1, 2, 70, 64, [3]),
    (8, 1, 1, 1, 333, 128, [331]),         # one plane, eight query heads a group: sections of 64 keys, tiles of sixteen
    (7, 7, 1, 1, 90, 64, [17]),            # seven planes of one query head; the cursor inside the second tile
])
def test_attention_matches_oracle_and_f64(device, heads, kv_heads, batch, rows, keys, width, origins):
    rng = np.random.default_rng(17)  # runtime.rs:594-605 draws seeds 17 / 29 / 43
    capacity = keys + 3
    q = rng.standard_normal((heads, batch, rows, width)).astype(np.float32)
    K = rng.standard_normal((kv_heads, batch, capacity, width)).astype(np.float16)
    V = rng.standard_normal((kv_heads, batch, capacity, width)).astype(np.float16)
    scale = 1.0 / np.sqrt(width)
    got = device.attention(q, K.view(np.uint16), V.view(np.uint16), kv_heads, capacity, keys, origins, scale)
    want = oracle.attention(q, K.view(np.uint16), V.view(np.uint16), kv_heads, capacity, keys, origins, scale)
    close(got, want)
    assert np.abs(got - want).max() <= 1e-5
    if batch == 1:
        exact = oracle.attention_f64(q, K[:, :, :keys].astype(np.float32), V[:, :, :keys].astype(np.float32), kv_heads, origins[0], True, scale)
        assert np.abs(got - exact).max() <= 1e-5  # the reference's bar against fp64 (runtime.rs:551-619)


@pytest.mark.parametrize("element", [0, 30])  # Element::Single, Element::Bfloat16 (crates/neura-decoder/src/cache.rs:130-134)
@pytest.mark.parametrize("heads,kv_heads,batch,rows,keys,width,origins", [
    (4, 2, 2, 3, 12, 32, [9, 4]),
    (14, 2, 1, 1, 1100, 64, [1024]),
    (28, 4, 2, 1, 600, 128, [63, 599]),
    (12, 2, 1, 17, 300, 128, [200]),
    (8, 8, 2, 5, 40, 256, [35, 0]),
])
def test_attention_over_single_and_bfloat16_states(device, element, heads, kv_heads, batch, rows, keys, width, origins):
    """Keys and values cast into states of another element by the device (nh_cache_write_element), bit for bit what the
    oracle's cast holds, then weighed (nh_attention_element) as the oracle weighs them and within 1e-5 of the f64 reference
    over the numbers the states hold."""
    rng = np.random.default_rng(17 + element)
    capacity = keys + rows
    wide = 4 if element == 0 else 2
    stored = np.float32 if element == 0 else np.uint16
    ck, cv = device.alloc(kv_heads * batch * capacity * width * wide), device.alloc(kv_heads * batch * capacity * width * wide)
    K = rng.standard_normal((kv_heads, batch, capacity, width)).astype(np.float32)
    V = rng.standard_normal((kv_heads, batch, capacity, width)).astype(np.float32)
    want_k, want_v = oracle.cache_cast(K, element), oracle.cache_cast(V, element)
    for first in range(0, capacity - rows + 1, rows):  # the states are filled a chunk at a time through the writer
        device.cache_write(K[:, :, first : first + rows], V[:, :, first : first + rows], ck, cv, capacity, keys, [first] * batch, element=element)
    filled = (capacity - rows) // rows * rows + rows
    got_k, got_v = ck.numpy(stored, K.shape), cv.numpy(stored, K.shape)
    assert np.array_equal(got_k[:, :, :filled].view(np.uint8), want_k[:, :, :filled].view(np.uint8))
    assert np.array_equal(got_v[:, :, :filled].view(np.uint8), want_v[:, :, :filled].view(np.uint8))
    ck, cv = device.upload(want_k), device.upload(want_v)  # every slot now, the ones no chunk reached too
    q = rng.standard_normal((heads, batch, rows, width)).astype(np.float32)
    scale = 1.0 / np.sqrt(width)
    got = device.attention(q, ck, cv, kv_heads, capacity, keys, origins, scale, element=element)
    want = oracle.attention(q, want_k, want_v, kv_heads, capacity, keys, origins, scale, element=element)
    close(got, want)
    assert np.abs(got - want).max() <= 1e-5
    if batch == 1:
        held_k = want_k if element == 0 else (want_k.astype(np.uint32) << 16).view(np.float32)
        held_v = want_v if element == 0 else (want_v.astype(np.uint32) << 16).view(np.float32)
        exact = oracle.attention_f64(q, held_k[:, :, :keys], held_v[:, :, :keys], kv_heads, origins[0], True, scale)
        assert np.abs(got - exact).max() <= 1e-5


def test_attention_of_equal_scores_is_the_running_mean(device):
    # crates/neura-runtime/tests/runtime.rs:813-875
    rng = np.random.default_rng(43)
    V = rng.standard_normal((2, 1, 100, 64)).astype(np.float16)
    q = np.zeros((4, 1, 1, 64), dtype=np.float32)
    for origin in (0, 7, 99):
        got = device.attention(q, np.zeros_like(V).view(np.uint16), V.view(np.uint16), 2, 100, 100, [origin], 0.125)
        for head in range(4):
            assert np.allclose(got[head, 0, 0], V[head // 2, 0, : origin + 1].astype(np.float32).mean(axis=0), atol=1e-5)


@pytest.mark.parametrize("element", [1, 0, 30])
def test_a_ring_cache_weighs_the_last_window_of_keys(device, element):
    # crates/neura-decoder/tests/cache.rs:11-51 (the reference runs it in single and half storage): equal scores,
    # value = step -> the mean of the last WINDOW steps
    WINDOW, CAPACITY, WIDTH = 5, 7, 32
    ck = device.alloc(CAPACITY * WIDTH * 4)
    cv = device.alloc(CAPACITY * WIDTH * 4)
    q = np.zeros((1, 1, 1, WIDTH), dtype=np.float32)
    q[..., 0] = 1.0
    key = np.zeros((1, 1, 1, WIDTH), dtype=np.float32)
    key[..., 0] = 1.0
    for step in range(2 * WINDOW + 2):
        value = np.zeros((1, 1, 1, WIDTH), dtype=np.float32)
        value[..., 0] = float(step)
        device.cache_write(key, value, ck, cv, CAPACITY, WINDOW, [step], ring=True, element=element)
        got = device.attention(q, ck, cv, 1, CAPACITY, WINDOW, [step], 1.0, reach=WINDOW, element=element)
        first = max(0, step - (WINDOW - 1))
        expected = sum(range(first, step + 1)) / (step - first + 1)
        assert abs(got[0, 0, 0, 0] - expected) < 1e-5 and got[0, 0, 0, 1] == 0.0, (step, got[0, 0, 0, :2])


def test_a_masked_chunk_leaves_the_ring_it_wraps_into_alone(device):
    # crates/neura-decoder/tests/cache.rs:53-95: an inactive plane whose cursor wraps onto slot 0 writes the scratch row
    WINDOW, WIDTH = 4, 32
    ck = device.alloc((WINDOW + 1) * WIDTH * 2)
    cv = device.alloc((WINDOW + 1) * WIDTH * 2)
    key = np.ones((1, 1, 1, WIDTH), dtype=np.float32)
    values = np.zeros((1, 1, 1, WIDTH), dtype=np.float32)
    values[..., 0] = 7.0
    masked = np.zeros((1, 1, 1, WIDTH), dtype=np.float32)
    masked[..., 0] = 9.0
    device.cache_write(key, values, ck, cv, WINDOW + 1, WINDOW, [0], ring=True)
    device.cache_write(key, masked, ck, cv, WINDOW + 1, WINDOW, [WINDOW], mask=[0], ring=True)
    got = device.attention(np.zeros((1, 1, 1, WIDTH), dtype=np.float32), ck, cv, 1, WINDOW + 1, WINDOW, [0], 1.0, reach=WINDOW)
    assert abs(got[0, 0, 0, 0] - 7.0) < 1e-5


@pytest.mark.parametrize("heads,kv_heads,batch,width,window,chunks", [
    (4, 2, 1, 32, 6, (1, 3, 2, 6, 1, 1, 4, 5, 2)),         # the row-at-a-time kernel
    (12, 2, 2, 128, 40, (1, 17, 30, 1, 40, 8, 1, 1, 25)),  # chunks of four rows and more: the matrix cores
    (14, 2, 1, 64, 100, (64, 1, 50, 1, 1, 100, 7)),
    (28, 4, 1, 128, 300, (250, 1, 1, 120, 1, 1)),          # several sections of the ring, folded
])
def test_ring_attention_matches_the_oracle(device, heads, kv_heads, batch, width, window, chunks):
    """Chunks of rows written into a ring and attended as they go, planes at different cursors: device against oracle on
    the same cache bytes, before the ring wraps, as it wraps inside a chunk, and several turns in."""
    rng = np.random.default_rng(29)
    widest = max(chunks)
    capacity = window + widest
    scale = 1.0 / np.sqrt(width)
    K = np.zeros((kv_heads, batch, capacity, width), dtype=np.uint16)
    V = np.zeros_like(K)
    origins = np.array([0] + [3 * b + 2 for b in range(1, batch)], dtype=np.uint32)
    for rows in chunks:
        k = rng.standard_normal((kv_heads, batch, rows, width)).astype(np.float32)
        v = rng.standard_normal((kv_heads, batch, rows, width)).astype(np.float32)
        q = rng.standard_normal((heads, batch, rows, width)).astype(np.float32)
        for b in range(batch):
            for row in range(rows):
                K[:, b, (origins[b] + row) % window] = oracle.f32_to_f16(k[:, b, row])
                V[:, b, (origins[b] + row) % window] = oracle.f32_to_f16(v[:, b, row])
        ck, cv = device.upload(K), device.upload(V)
        got = device.attention(q, ck, cv, kv_heads, capacity, window, origins, scale, reach=window)
        want = oracle.attention(q, K, V, kv_heads, capacity, window, origins, scale, reach=window)
        assert np.abs(got - want).max() <= 1e-5, (rows, origins)
        # the device's own ring write lands on the same slots
        dk, dv = device.upload(np.zeros_like(K)), device.upload(np.zeros_like(V))
        device.cache_write(k, v, dk, dv, capacity, window, origins, ring=True)
        mine = dk.numpy(np.uint16, K.shape)
        for b in range(batch):
            for row in range(rows):
                if origins[b] + row + window >= origins[b] + rows:  # not overwritten by a later row of the same chunk
                    assert np.array_equal(mine[:, b, (origins[b] + row) % window], oracle.f32_to_f16(k[:, b, row]))
        ck.release(), cv.release(), dk.release(), dv.release()
        origins = origins + rows


def test_attention_refuses_a_cursor_past_its_keys(device):
    q = np.zeros((2, 1, 1, 64), dtype=np.float32)
    K = np.zeros((2, 1, 8, 64), dtype=np.uint16)
    with pytest.raises(NeuraError) as refused:  # attention.rs:250-252
        device.attention(q, K, K, 2, 8, 8, [8], 1.0)
    assert refused.value.code == -4
    with pytest.raises(NeuraError):
        device.attention(q, K, K, 2, 8, 8, [0], 0.0)  # refusal::KNOB (attention.rs:128-132)


@pytest.mark.parametrize("n", [1, 32, 1000, 4096, 4097, 20000, 152064])
def test_sample_matches_the_oracle(device, n):
    """nh_sample against the oracle's restatement of sample_row on the same logits: every keep from 1 to 64, tight and open
    nuclei, temperatures either side of one, many seeds.  Columns can only differ where two candidates' value + noise tie
    within the last bits of the device's and the host's logarithms, which these seeds do not meet."""
    rng = np.random.default_rng(n)
    rows = 96
    logits = (rng.standard_normal((rows, n)) * 3.0).astype(np.float32)
    drawn = oracle.draws([(int(rng.integers(0, 2 ** 32)), float(rng.choice([0.25, 0.7, 1.0, 1.5, 4.0])), int(rng.integers(1, 65)),
                           float(rng.choice([0.05, 0.5, 0.85, 0.95, 1.0]))) for _ in range(rows)])
    got = device.sample(logits, drawn)
    want = oracle.sample(logits, drawn)
    assert list(got) == list(want)
    # the reference's own properties (crates/neura-runtime/tests/choice.rs:41-126)
    first = oracle.draws([(s, 1.0, 1, 1.0) for s in range(rows)])
    assert list(device.sample(logits, first)) == [int(np.argmax(row)) for row in logits]
    if n >= 32:
        pair = oracle.draws([(0x2F0F1A3B, 1.0, 6, 0.85), (0x91E10D57, 1.0, 6, 0.85)])
        alone = [int(device.sample(logits[r:r + 1], pair[r:r + 1])[0]) for r in range(2)]
        assert list(device.sample(logits[:2], pair)) == alone


def test_sample_ranks_ties_by_column_and_refuses_what_the_reference_refuses(device):
    # equal logits rank by column: keep 4 of 5000 equal columns leaves the first four, in any section
    flat = np.zeros((256, 5000), dtype=np.float32)
    got = device.sample(flat, oracle.draws([(seed, 1.0, 4, 1.0) for seed in range(256)]))
    assert set(got) == {0, 1, 2, 3}
    assert list(got) == list(oracle.sample(flat, oracle.draws([(seed, 1.0, 4, 1.0) for seed in range(256)])))
    # integers in a narrow range: many exact ties across sections
    rng = np.random.default_rng(3)
    tied = rng.integers(0, 40, (64, 152064)).astype(np.float32)
    drawn = oracle.draws([(seed * 977, 1.0, 64, 1.0) for seed in range(64)])
    assert list(device.sample(tied, drawn)) == list(oracle.sample(tied, drawn))
    one = np.zeros((1, 8), dtype=np.float32)
    for bad in ((1, 0.0, 4, 1.0), (1, np.inf, 4, 1.0), (1, np.nan, 4, 1.0), (1, 1.0, 0, 1.0), (1, 1.0, 65, 1.0), (1, 1.0, 4, 0.0), (1, 1.0, 4, 1.5)):
        with pytest.raises(NeuraError):  # crates/neura-generate/src/sampling.rs:16-29
            device.sample(one, oracle.draws([bad]))
    with pytest.raises(NeuraError):
        device.sample(np.zeros((1, 262145), dtype=np.float32), oracle.draws([(1, 1.0, 4, 1.0)]))


def test_sample_frequencies_follow_the_softmax_of_the_kept_candidates(device):
    # Gumbel-max on the device: 4096 rows of the same logits under 4096 seeds
    rng = np.random.default_rng(5)
    row = rng.normal(0, 1.5, 12).astype(np.float32)
    logits = np.tile(row, (4096, 1))
    for temperature, keep in ((1.0, 12), (0.5, 12), (2.0, 5)):
        scaled = row.astype(np.float64) / temperature
        kept = np.argsort(-scaled, kind="stable")[:keep]
        p = np.zeros(12)
        p[kept] = np.exp(scaled[kept] - scaled.max())
        p /= p.sum()
        counts = np.zeros(12)
        for batch in range(5):
            drawn = oracle.draws([((batch * 4096 + seed) * 2654435761 % 2 ** 32, temperature, keep, 1.0) for seed in range(4096)])
            counts += np.bincount(device.sample(logits, drawn), minlength=12)
        assert counts[p == 0].sum() == 0
        expected = p * counts.sum()
        chi2 = ((counts - expected) ** 2 / np.maximum(expected, 1e-9))[p > 0].sum()
        assert chi2 < 45, (temperature, keep, chi2)


def test_argmax_lowest_index_on_ties(device):
    rng = np.random.default_rng(10)
    values = rng.integers(0, 1000, (3, 151936)).astype(np.float32)  # many exact ties
    got = device.argmax(values)
    assert list(got) == [oracle.argmax(row) for row in values] == [int(np.argmax(row)) for row in values]
    values = rng.standard_normal((8, 152064)).astype(np.float32)
    assert list(device.argmax(values)) == [int(np.argmax(row)) for row in values]
    assert list(device.argmax(np.full((1, 5000), -np.inf, dtype=np.float32))) == [0]
    assert list(device.argmax(np.array([[1.0]], dtype=np.float32))) == [0]
    edge = np.zeros((1, 4097), dtype=np.float32)
    edge[0, 4096] = 1.0
    assert list(device.argmax(edge)) == [4096]
