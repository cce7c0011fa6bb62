"""Seeded inputs that more than one test, and the script that writes the committed fixtures, build the same way.

Everything here is data: weights, cache contents, first tokens, hand-built blocks.  The GPU tests feed it to the device
and to the oracle; tests/golden/make_fixtures.py feeds it to the oracle alone and stores what comes out."""
import hashlib

import numpy as np

from neura_amd import synth

Q8_0, Q3_K, Q4_K, Q5_K, Q6_K = 8, 11, 12, 13, 14
BLOCK_ELEMENTS = {Q8_0: 32, Q3_K: 256, Q4_K: 256, Q5_K: 256, Q6_K: 256}


def hand_built_blocks(element, blocks=4):
    """Raw blocks whose every byte follows a fixed pattern (the idea of crates/neura-precision/tests/format.rs:221-234:
    bytes (at * 37 + 11), (at * 53 + 7), (at * 19 + 3) over the fields of a block), with half-precision scales that are
    ordinary finite numbers: the same bytes in every process, no generator involved."""
    per, size = synth.BLOCK_BYTES[element]
    raw = np.zeros((blocks, size), dtype=np.uint8)
    at = np.arange(size, dtype=np.uint32)
    for block in range(blocks):
        mult = (37, 53, 19, 71)[block % 4]
        raw[block] = ((at + 1 + block * 5) * mult + (11, 7, 3, 29)[block % 4]) & 0xFF
    scales = {Q8_0: [(0, 0.0078125)], Q4_K: [(0, 0.015625), (2, 0.00390625)], Q5_K: [(0, 0.0078125), (2, 0.001953125)],
              Q6_K: [(208, 0.00048828125)], Q3_K: [(108, 0.0009765625)]}[element]
    for block in range(blocks):
        for offset, value in scales:
            half = np.array([value * (1 + block) * (1.0 if block % 2 == 0 else 1.5)], dtype=np.float16)
            raw[block, offset:offset + 2] = half.view(np.uint8)
    return raw.reshape(-1), blocks * per


def config1():
    """BASELINE configuration 1: W 4864 x 896 in Q8_0 (codes uniform in [-127, 127], fp16 scales |N(0, 0.02)|), x N(0, 1), seed 0."""
    rng = np.random.default_rng(0)
    N, K = 4864, 896
    raw = synth.q8_0_random(rng, N * K)
    x = rng.standard_normal(K).astype(np.float32)
    return N, K, raw, x


def kquant_products(element):
    """A narrow product of each K-quant at a shape every one-row form takes (48 rows of three super-blocks: whole 16-row tiles,
    rows of 210- and 110-byte blocks on both alignments): seeded random blocks, activations over a few orders of magnitude."""
    N, K = 48, 768
    rng = np.random.default_rng(900 + element)
    raw = synth.RANDOM[element](rng, N * K)
    x = (rng.standard_normal(K) * np.exp(rng.uniform(-2.0, 2.0, K))).astype(np.float32)
    return N, K, raw, x


def sha256(array):
    return hashlib.sha256(np.ascontiguousarray(array).view(np.uint8).tobytes()).hexdigest()


def decoder_case(shape, element, mode, seed, layers, batch, filled, cache_seed=None, threads=16):
    """(tensors, host tensors by name, the N(0,1) halves every state holds below `filled`, the first token)

    The halves are a list over layers of (key halves, value halves), each [kv_heads][batch][filled][head_dim] float16.
    `cache_seed`: the states and the token come from a generator of their own (configuration 4 was written that way);
    otherwise from the one that drew the weights, in this order."""
    rng = np.random.default_rng(seed)
    tensors = list(synth.model_tensors(shape, element, rng, mode=mode, layers=layers, threads=threads if mode == "normal" and threads else None))
    host = {name: raw for name, _, _, raw in tensors}
    if cache_seed is not None:
        rng = np.random.default_rng(cache_seed)
    count = shape["layers"] if layers is None else layers
    halves = []
    for _ in range(count):
        pair = []
        for _ in range(2):
            pair.append(rng.standard_normal((shape["kv_heads"], batch, filled, shape["head_dim"])).astype(np.float16))
        halves.append(tuple(pair))
    token = int(rng.integers(0, shape["vocab"]))
    return tensors, host, halves, token


def hold(halves, cache_shape, ref, model=None):
    """puts the halves of decoder_case into the oracle's states and, where one is given, the device model's"""
    filled = halves[0][0].shape[2]
    for layer, pair in enumerate(halves):
        for which, (values, held) in enumerate(zip(pair, (ref.cache_k, ref.cache_v))):
            whole = np.zeros(cache_shape, dtype=np.float16)
            whole[:, :, :filled] = values
            held[layer][:] = whole.view(np.uint16).reshape(-1)
            if model is not None:
                model.cache_write(layer, which, whole.view(np.uint16))


def config4_case(threads=None):
    """BASELINE configuration 4: the 0.5B shape in Q8_0 (N(0, 0.02) weights through the reference's encoder, one generator
    in order), states holding 1024 positions, one random first token."""
    shape = synth.SHAPES["qwen2.5-0.5b"]
    tensors, host, halves, token = decoder_case(shape, Q8_0, "normal", 0, None, 1, 1024, cache_seed=40, threads=threads)
    return shape, tensors, host, halves, token


def config5_case(mode):
    """BASELINE configuration 5, the whole 7B shape with states holding 4032 positions.  "normal": weights a test can see
    through, N(0, 0.02) packed to Q4_K by the reference's encoder; "blocks": the benchmark's random Q4_K blocks."""
    shape = synth.SHAPES["qwen2.5-7b"]
    tensors, host, halves, token = decoder_case(shape, Q4_K, mode, 52, None, 1, 4096 - 64)
    return shape, tensors, host, halves, token


def config5_normal_case():
    return config5_case("normal")
