"""The CPU oracle against the fixtures committed under tests/golden/ (written by tests/golden/make_fixtures.py), and the
check that the decoders the parity tests run are not degenerate."""
import json
import os

import numpy as np
import pytest

import cases
import oracle
from neura_amd import synth

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.mark.parametrize("element", [cases.Q8_0, cases.Q3_K, cases.Q4_K, cases.Q5_K, cases.Q6_K])
def test_the_oracle_unpacks_the_committed_blocks_to_the_committed_bits(element):
    held = np.load(os.path.join(GOLDEN, "hand_built_blocks.npz"))
    raw, elements = cases.hand_built_blocks(element)
    assert np.array_equal(raw, held["raw_%d" % element])  # the pattern is the one the fixture was written from
    assert np.array_equal(oracle.unpack(element, raw, elements).view(np.uint32), held["bits_%d" % element])
    # and the numpy restatement of ggml's published walk gives the same bits
    assert np.array_equal(synth.DEQUANT[element](raw, elements).view(np.uint32), held["bits_%d" % element])


def test_the_oracle_answers_configuration_1_as_committed():
    held = np.load(os.path.join(GOLDEN, "config1_q8_0_gemv.npz"))
    with open(os.path.join(GOLDEN, "config1_q8_0_gemv.json")) as text:
        sums = json.load(text)
    N, K, raw, x = cases.config1()
    assert cases.sha256(raw) == sums["w_sha256"] and cases.sha256(x) == sums["x_sha256"]  # the seeded inputs are the ones stored
    row_bytes = raw.size // N
    assert np.array_equal(raw[: 64 * row_bytes], held["w_first_64_rows"]) and np.array_equal(x, held["x"])
    y = oracle.gemv(cases.Q8_0, raw, N, K, x, threads=4)[0]
    assert np.array_equal(y.view(np.uint32), held["y_bits"]) and cases.sha256(y) == sums["y_sha256"]
    # the stored slice alone gives the stored first 64 outputs, and they are the fp64 product to fp32 rounding of the sums
    first = oracle.gemv(cases.Q8_0, held["w_first_64_rows"], 64, K, held["x"])[0]
    assert np.array_equal(first.view(np.uint32), held["y_bits"][:64])
    exact = synth.q8_0_dequant(held["w_first_64_rows"], 64 * K).reshape(64, K).astype(np.float64) @ held["x"].astype(np.float64)
    assert np.abs(first - exact).max() <= 2e-5 * np.abs(exact).max()


@pytest.mark.parametrize("element", [cases.Q3_K, cases.Q4_K, cases.Q5_K, cases.Q6_K])
def test_the_oracle_answers_the_k_quant_products_as_committed(element):
    held = np.load(os.path.join(GOLDEN, "kquant_gemv.npz"))
    N, K, raw, x = cases.kquant_products(element)
    assert np.array_equal(raw, held["raw_%d" % element]) and np.array_equal(x, held["x_%d" % element])  # the seeded inputs are the ones stored
    y = oracle.gemv(element, held["raw_%d" % element], N, K, held["x_%d" % element], threads=4)[0]
    assert np.array_equal(y.view(np.uint32), held["y_bits_%d" % element])
    # and the stored outputs are the fp64 product of ggml's published walk (in numpy) to the rounding of fp32 sums
    exact = synth.DEQUANT[element](held["raw_%d" % element], N * K).reshape(N, K).astype(np.float64) @ held["x_%d" % element].astype(np.float64)
    assert np.abs(held["y_bits_%d" % element].view(np.float32) - exact).max() <= 2e-5 * np.abs(exact).max()


SMALL_Q4 = dict(layers=3, hidden=512, heads=8, kv_heads=2, head_dim=128, ffn=1024, vocab=1000, tied=False)
TINY = dict(layers=2, hidden=256, heads=4, kv_heads=2, head_dim=64, ffn=512, vocab=320, tied=True)
CUT_7B = dict(synth.SHAPES["qwen2.5-7b"], vocab=4096)  # the 7B shape's layers behind a short vocabulary


def moved_by_the_input(shape, element, mode, layers, threads=None):
    rng = np.random.default_rng(50)
    host = {name: raw for name, _, _, raw in synth.model_tensors(shape, element, rng, mode=mode, layers=layers, threads=threads)}
    ref = oracle.Model(shape, element, host, 1, 8, 1, layers=layers)
    first, chosen_first = ref.forward([1234 % shape["vocab"]], 1, [0], threads=8)
    first = first.copy()
    second, chosen_second = ref.forward([7], 1, [0], threads=8)
    return float(np.abs(first - second).max() / np.abs(first).max()), int(chosen_first[0]), int(chosen_second[0])


@pytest.mark.parametrize("shape,element,layers,threads", [(TINY, cases.Q8_0, None, None), (SMALL_Q4, cases.Q4_K, None, None), (CUT_7B, cases.Q4_K, 2, 8)],
                         ids=["tiny-q8_0", "small-q4_k", "7b-cut-q4_k"])
def test_the_decoders_the_parity_tests_run_depend_on_their_input(shape, element, layers, threads):
    """Greedy ids identical to the oracle's prove something only on a network whose logits depend on the token fed: with
    N(0, 0.02) weights another token moves the logits by far more than the 1e-2 of the largest asked for here (and by far
    more than the 1e-3 the parity tests allow the device)."""
    moved, _, _ = moved_by_the_input(shape, element, "normal", layers, threads)
    assert moved > 1e-2, moved


def test_random_q4_k_blocks_make_a_degenerate_decoder():
    """Why the 7B-shape parity tests run N(0, 0.02) weights beside BASELINE's random blocks: random nibbles and scales under
    positive d and dmin give every weight a large positive mean, the network collapses onto one direction, and another input
    token moves the logits by less than the parity bar -- the same token comes out whatever goes in."""
    moved, first, second = moved_by_the_input(CUT_7B, cases.Q4_K, "blocks", 2)
    assert moved < 1e-3 and first == second, (moved, first, second)
