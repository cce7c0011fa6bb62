"""GPU parity of the decoder (decode step, fill, greedy loop) against the CPU oracle."""
import json
import os

import numpy as np
import pytest

import cases
import oracle
from neura_amd import NH_Q3_K, NH_Q4_K, NH_Q5_K, NH_Q6_K, NH_Q8_0, NeuraError, synth
from neura_amd.loader import Model, Weights

pytestmark = pytest.mark.gpu

TINY = dict(layers=2, hidden=256, heads=4, kv_heads=2, head_dim=64, ffn=512, vocab=320, tied=True)
SMALL_Q4 = dict(layers=3, hidden=512, heads=8, kv_heads=2, head_dim=128, ffn=1024, vocab=1000, tied=False)


def build(device, shape, element, batch, context, max_rows=1, seed=0, mode="normal", layers=None, window=None, cache_element=1, elements=None):
    rng = np.random.default_rng(seed)
    tensors = list(synth.model_tensors(shape, element, rng, mode=mode, layers=layers, elements=elements))
    host = {name: raw for name, _, _, raw in tensors}
    weights = Weights(device, tensors)
    model = Model(device, weights, shape, element, batch, context, max_rows, layers=layers, window=window, cache_element=cache_element)
    ref = oracle.Model(shape, element, host, batch, context, max_rows, layers=layers, window=window, cache_element=cache_element, elements=elements)
    return model, ref, weights


def margins(logits):
    top = np.sort(logits, axis=1)[:, -2:]
    return top[:, 1] - top[:, 0]


@pytest.mark.parametrize("shape,element", [(TINY, NH_Q8_0), (SMALL_Q4, NH_Q4_K)])
def test_decode_steps_match_oracle_logits_and_tokens(device, shape, element):
    model, ref, weights = build(device, shape, element, batch=2, context=32)
    rng = np.random.default_rng(1)
    tokens = rng.integers(0, shape["vocab"], 2)
    for step in range(6):
        cursors = [step, step]
        want_logits, want = ref.forward(tokens, 1, cursors)
        got = model.decode_step(tokens, cursors)
        logits = model.logits()
        scale = np.abs(want_logits).max()
        # a 1e-6 reordering difference now and then flips the fp16 rounding of a cached key or
        # value (one half ulp = 5e-4 relative); the oracle sits as far from an fp64 forward pass
        assert np.abs(logits - want_logits).max() <= 1e-3 * scale, step
        assert list(got) == list(want), (step, margins(want_logits))
        tokens = got
    for layer in range(shape["layers"]):  # the caches hold the same halves
        for which, held in ((0, ref.cache_k), (1, ref.cache_v)):
            got_cache = oracle.f16_to_f32(model.cache_read(layer, which).reshape(-1))
            want_cache = oracle.f16_to_f32(held[layer])
            assert np.abs(got_cache - want_cache).max() <= 2e-3 * max(1.0, np.abs(want_cache).max())
    model.release(), weights.release()


@pytest.mark.parametrize("cache_element", [0, 30], ids=["single", "bfloat16"])
@pytest.mark.parametrize("shape,element", [(TINY, NH_Q8_0), (SMALL_Q4, NH_Q4_K)])
def test_decoders_keep_their_states_in_single_or_bfloat16(device, shape, element, cache_element):
    """Cache::new(.., Element::Single | Bfloat16) (crates/neura-decoder/src/cache.rs:130-134; the reference's own example
    keeps single precision states, examples/qwen/main.rs:107): a fill chunk with one plane masked, then decode steps of
    both planes -- logits and greedy tokens as the oracle's with the same states, and the states themselves equal."""
    model, ref, weights = build(device, shape, element, batch=2, context=40, max_rows=8, seed=5, cache_element=cache_element)
    rng = np.random.default_rng(6)
    prompt = rng.integers(0, shape["vocab"], (8, 2))
    model.prefill(prompt.reshape(-1), 8, [0, 0], mask=[1, 0])
    ref.forward(prompt.reshape(-1), 8, [0, 0], mask=[1, 0], want_logits=False)
    model.prefill(prompt.reshape(-1), 8, [8, 0], mask=[1, 1])
    ref.forward(prompt.reshape(-1), 8, [8, 0], mask=[1, 1], want_logits=False)
    tokens = rng.integers(0, shape["vocab"], 2)
    for step in range(5):
        cursors = [16 + step, 8 + step]
        want_logits, want = ref.forward(tokens, 1, cursors)
        got = model.decode_step(tokens, cursors)
        assert np.abs(model.logits() - want_logits).max() <= 1e-3 * np.abs(want_logits).max(), step
        assert list(got) == list(want), (step, margins(want_logits))
        tokens = got
    for layer in range(shape["layers"]):
        for which, held in ((0, ref.cache_k), (1, ref.cache_v)):
            got_cache, want_cache = model.cache_read(layer, which).reshape(-1), held[layer]
            if cache_element == 30:
                got_cache, want_cache = (got_cache.astype(np.uint32) << 16).view(np.float32), (want_cache.astype(np.uint32) << 16).view(np.float32)
            assert got_cache.dtype == np.float32 and np.abs(got_cache - want_cache).max() <= 1e-2 * max(1.0, np.abs(want_cache).max())
    # a state written through the C ABI reads back as it was written, in the states' element
    written = (rng.standard_normal(model.cache_shape).astype(np.float32) if cache_element == 0
               else rng.integers(0, 1 << 15, model.cache_shape).astype(np.uint16))
    model.cache_write(0, 1, written)
    assert np.array_equal(model.cache_read(0, 1), written)
    model.release(), weights.release()


@pytest.mark.parametrize("cache_element", [0, 30], ids=["single", "bfloat16"])
@pytest.mark.parametrize("shape,element", [(TINY, NH_Q8_0), (SMALL_Q4, NH_Q4_K)])
def test_one_plane_steps_over_single_or_bfloat16_states_ride_the_fused_kernels(device, monkeypatch, shape, element, cache_element):
    """One plane, one token a step: the rotation and the append ride in the q|k|v product's epilogue, which casts what it
    appends into the states' element, and the attention walks single and bfloat16 states on the matrix cores.  Logits and
    tokens as the oracle's over the same states, the appended rows equal to its rows, and the same steps with the rotation in
    a kernel of its own and the plain fp32 attention (the forms these replaced) within the same bar."""
    monkeypatch.setenv("NEURA_HIP_GRAPH", "0")  # the twins launch eagerly, so the switches below are read at every step
    fused, ref, weights_a = build(device, shape, element, batch=1, context=40, max_rows=8, seed=5, cache_element=cache_element)
    plain, _, weights_b = build(device, shape, element, batch=1, context=40, max_rows=8, seed=5, cache_element=cache_element)
    rng = np.random.default_rng(6)
    prompt = rng.integers(0, shape["vocab"], 8)
    for model in (fused, plain):
        model.prefill(prompt, 8, [0])
    ref.forward(prompt, 8, [0], want_logits=False)
    token = int(rng.integers(0, shape["vocab"]))
    for step in range(6):
        want_logits, want = ref.forward([token], 1, [8 + step])
        monkeypatch.setenv("NEURA_HIP_FUSE_ROPE", "1"), monkeypatch.setenv("NEURA_HIP_ATTENTION_ANY", "0")
        got = fused.decode_step([token], [8 + step])
        logits = fused.logits()
        monkeypatch.setenv("NEURA_HIP_FUSE_ROPE", "0"), monkeypatch.setenv("NEURA_HIP_ATTENTION_ANY", "1")
        got_plain = plain.decode_step([token], [8 + step])
        scale = np.abs(want_logits).max()
        assert np.abs(logits - want_logits).max() <= 1e-3 * scale and np.abs(plain.logits() - want_logits).max() <= 1e-3 * scale, step
        assert list(got) == list(got_plain) == list(want), (step, margins(want_logits))
        token = int(got[0])
    for layer in range(shape["layers"]):
        for which, held in ((0, ref.cache_k), (1, ref.cache_v)):
            rows = []
            for model in (fused, plain):
                got_cache = model.cache_read(layer, which).reshape(-1)
                rows.append((got_cache.astype(np.uint32) << 16).view(np.float32) if cache_element == 30 else got_cache)
            want_cache = (held[layer].astype(np.uint32) << 16).view(np.float32) if cache_element == 30 else held[layer]
            bar = 1e-2 * max(1.0, np.abs(want_cache).max())
            assert np.abs(rows[0] - want_cache).max() <= bar and np.abs(rows[1] - want_cache).max() <= bar
            assert np.any(rows[0].reshape(fused.cache_shape)[:, 0, 8:14])  # the decode steps' rows are there
    for held in (fused, plain, weights_a, weights_b):
        held.release()


def test_a_decoder_names_the_element_of_its_states(device):
    with pytest.raises(NeuraError, match="single, half or bfloat16"):
        build(device, TINY, NH_Q8_0, batch=1, context=8, cache_element=12)


def test_masked_planes_and_chunked_fill(device):
    shape = SMALL_Q4
    model, ref, weights = build(device, shape, NH_Q4_K, batch=2, context=40, max_rows=16, seed=3)
    rng = np.random.default_rng(4)
    prompt = rng.integers(0, shape["vocab"], (16, 2))  # tokens[row * batch + plane]
    # plane 0 fills 16 rows at cursor 0 while plane 1 is inactive
    model.prefill(prompt.reshape(-1), 16, [0, 0], mask=[1, 0])
    ref.forward(prompt.reshape(-1), 16, [0, 0], mask=[1, 0], want_logits=False)
    # then both planes decode: plane 0 at cursor 16, plane 1 starts at 0
    tokens = [7, 9]
    for step in range(3):
        cursors = [16 + step, step]
        want_logits, want = ref.forward(tokens, 1, cursors)
        got = model.decode_step(tokens, cursors)
        assert np.abs(model.logits() - want_logits).max() <= 1e-3 * np.abs(want_logits).max()
        assert list(got) == list(want)
        tokens = got
    k = model.cache_read(0, 0)
    assert np.any(k[:, 0, :16]) and not np.any(k[:, 1, 3:40])  # the inactive plane wrote scratch rows only
    # chunked fill == token by token (generation.rs:458-470): replay plane 0 alone, one token at a time
    model.reset([1, 1])
    assert not np.any(model.cache_read(0, 0)[:, :, :40])
    for at in range(16):
        model.decode_step([prompt[at, 0], 0], [at, 0], mask=[1, 0])
    k_single = oracle.f16_to_f32(model.cache_read(0, 0)[:, 0, :16].reshape(-1))
    k_chunk = oracle.f16_to_f32(k[:, 0, :16].reshape(-1))
    assert np.abs(k_single - k_chunk).max() <= 2e-3 * max(1.0, np.abs(k_chunk).max())
    model.release(), weights.release()


MIXED = {"output.weight": NH_Q6_K, "blk.0.attn_v.weight": NH_Q6_K, "blk.2.ffn_down.weight": NH_Q6_K, "blk.2.ffn_gate.weight": NH_Q6_K}
# the way Q3_K_M files are: Q3_K for most, Q5_K and Q4_K for some projections, a Q6_K head
MIXED_3 = {"output.weight": NH_Q6_K, "blk.0.attn_v.weight": NH_Q5_K, "blk.1.attn_v.weight": NH_Q4_K, "blk.1.ffn_down.weight": NH_Q5_K, "blk.1.attn_output.weight": NH_Q4_K,
           "blk.2.attn_q.weight": NH_Q4_K, "blk.2.attn_k.weight": NH_Q4_K, "blk.2.attn_v.weight": NH_Q4_K, "blk.2.ffn_up.weight": NH_Q5_K}


@pytest.mark.parametrize("base,mixed", [(NH_Q4_K, MIXED), (NH_Q3_K, MIXED_3), (NH_Q6_K, {}), (NH_Q5_K, {}), (NH_Q3_K, {})],
                         ids=["q4_k_m", "q3_k_m", "q6_k", "q5_k", "q3_k"])
@pytest.mark.parametrize("batch", [1, 2, 8])
def test_mixed_elements_and_projection_biases(device, batch, base, mixed):
    """A decoder stored the way Q4_K_M files are (Q6_K for some matrices, Q4_K for the rest) whose q, k and v projections
    carry Qwen2's biases: layer 0 (a Q6_K value projection, biases) takes one product per matrix, layer 1 (one element,
    biases) folds rotation and biases into the stacked product at batch 1, layer 2 (gate and up stored differently) runs
    the two halves apart.  Decode steps, a 16-row fill and the caches against the oracle.  The same for decoders stored in
    one K-quant throughout (the fill's q|k|v is then one stacked wide product of that element on the matrix cores).  In the
    Q3_K_M mix layers 0 and 1 rotate q|k in a Q3_K product and cast the rows of a Q5_K and a Q4_K value projection into the
    value state from those products' own epilogues."""
    shape = SMALL_Q4
    rng = np.random.default_rng(21)
    tensors = list(synth.model_tensors(shape, base, rng, mode="normal", elements=mixed, biases=(0, 1)))
    host = {name: (raw.view(np.float32) if name.endswith(".bias") else raw) for name, _, _, raw in tensors}
    weights = Weights(device, tensors)
    model = Model(device, weights, shape, base, batch, 40, 16)
    ref = oracle.Model(shape, base, host, batch, 40, 16, elements=mixed)
    prompt = rng.integers(0, shape["vocab"], (16, batch))
    model.prefill(prompt.reshape(-1), 16, [0] * batch)
    ref.forward(prompt.reshape(-1), 16, [0] * batch, want_logits=False)
    tokens = rng.integers(0, shape["vocab"], batch)
    for step in range(5):
        cursors = [16 + step] * batch
        want_logits, want = ref.forward(tokens, 1, cursors)
        got = model.decode_step(tokens, cursors)
        assert np.abs(model.logits() - want_logits).max() <= 1e-3 * np.abs(want_logits).max(), step
        assert list(got) == list(want), (step, margins(want_logits))
        tokens = got
    for layer in range(shape["layers"]):
        for which, held in ((0, ref.cache_k), (1, ref.cache_v)):
            got_cache = oracle.f16_to_f32(model.cache_read(layer, which).reshape(-1))
            want_cache = oracle.f16_to_f32(held[layer])
            assert np.abs(got_cache - want_cache).max() <= 2e-3 * max(1.0, np.abs(want_cache).max())
    model.release(), weights.release()


def test_sampled_decode_steps_draw_as_the_oracle_draws(device):
    """A sampled answer program: the same forward pass, the choice drawn per plane with its own seed, temperature,
    candidate count and nucleus, all written by the host before each step (the recorded graph is replayed with new
    draws).  The draw is checked on the device's own logits, the logits against the oracle's as in the greedy test."""
    shape = SMALL_Q4
    model, ref, weights = build(device, shape, NH_Q4_K, batch=3, context=40)
    rng = np.random.default_rng(9)
    tokens = rng.integers(0, shape["vocab"], 3)
    seeds = [oracle.lib().oracle_plane_seed(1234, slot) for slot in range(3)]
    for step in range(8):
        cursors = [step] * 3
        mask = [1, 1, 1] if step % 3 else [1, 0, 1]
        drawn = oracle.draws([(oracle.lib().oracle_seed_bits((seeds[slot] + step) & 0xFFFFFFFF), [0.8, 1.0, 1.3][slot], [40, 1, 64][slot],
                               [0.9, 1.0, 0.5][slot]) for slot in range(3)])
        want_logits, greedy = ref.forward(tokens, 1, cursors, mask=mask)
        got = model.decode_step_sampled(tokens, cursors, drawn, mask=mask)
        logits = model.logits()
        live = [slot for slot in range(3) if mask[slot]]
        assert np.abs(logits[live] - want_logits[live]).max() <= 1e-3 * np.abs(want_logits[live]).max(), step
        want = oracle.sample(logits, drawn)
        assert [got[slot] for slot in live] == [want[slot] for slot in live], step
        if mask[1]:
            assert got[1] == greedy[1]  # a plane that keeps one candidate answers greedily
        tokens = [int(got[slot]) if mask[slot] else int(tokens[slot]) for slot in range(3)]
    # a greedy step after sampled ones still answers with the argmax
    want_logits, greedy = ref.forward(tokens, 1, [8] * 3)
    assert list(model.decode_step(tokens, [8] * 3)) == list(greedy)
    with pytest.raises(NeuraError):
        model.decode_step_sampled(tokens, [9] * 3, oracle.draws([(1, 1.0, 70, 1.0)] * 3))
    model.release(), weights.release()


@pytest.mark.parametrize("shape,element,batch", [(TINY, NH_Q8_0, 2), (SMALL_Q4, NH_Q4_K, 1)])
def test_a_windowed_model_keeps_a_ring_of_its_last_tokens(device, shape, element, batch):
    """BatchSpec::window (crates/neura-generate/src/batch.rs:148-152, :313-325): caches of window + chunk rows written as
    rings, attention over the last `window` positions.  A chunked fill that wraps inside a chunk, then decode steps two
    turns round the ring (batch 1 folds the rotation and the ring seat into the q|k|v product), against the oracle."""
    window, rows, context = 12, 8, 64
    model, ref, weights = build(device, shape, element, batch=batch, context=context, max_rows=rows, seed=5, window=window)
    assert model.capacity == window + rows
    rng = np.random.default_rng(6)
    cursor = 0
    for chunk in range(2):  # the second chunk wraps: positions 8..15 over a ring of 12
        prompt = rng.integers(0, shape["vocab"], (rows, batch))
        model.prefill(prompt.reshape(-1), rows, [cursor] * batch)
        ref.forward(prompt.reshape(-1), rows, [cursor] * batch, want_logits=False)
        cursor += rows
    tokens = rng.integers(0, shape["vocab"], batch)
    for step in range(2 * window + 3):
        want_logits, want = ref.forward(tokens, 1, [cursor] * batch)
        got = model.decode_step(tokens, [cursor] * batch)
        assert np.abs(model.logits() - want_logits).max() <= 1e-3 * np.abs(want_logits).max(), step
        assert list(got) == list(want), (step, margins(want_logits))
        tokens = got
        cursor += 1
    for layer in range(shape["layers"]):
        for which, held in ((0, ref.cache_k), (1, ref.cache_v)):
            got_cache = oracle.f16_to_f32(model.cache_read(layer, which)[:, :, :window].reshape(-1))
            want_cache = oracle.f16_to_f32(held[layer].reshape(shape["kv_heads"], batch, window + rows, shape["head_dim"])[:, :, :window].reshape(-1))
            assert np.abs(got_cache - want_cache).max() <= 2e-3 * max(1.0, np.abs(want_cache).max())
    with pytest.raises(NeuraError) as refused:  # batch.rs:315-318
        Model(device, weights, shape, element, batch, 8, 1, window=9)
    assert "a batch keeps a window of 9 tokens over a context of 8" in str(refused.value)
    with pytest.raises(NeuraError) as refused:  # batch.rs:319-322
        Model(device, weights, shape, element, batch, 32, 8, window=6)
    assert "a batch fills chunks of 8 rows into a window of 6 tokens" in str(refused.value)
    model.release(), weights.release()


def test_a_ring_of_several_sections_merged_by_the_output_projection(device):
    """A Q8_0 decoder of one plane whose window is a ring of 140 keys: three attention sections, left unmerged for the output
    projection to merge as it stages its row.  Filled to four keys short of a full ring, then decode steps that wrap it:
    logits and tokens as the oracle's."""
    window, rows = 140, 8
    model, ref, weights = build(device, TINY, NH_Q8_0, batch=1, context=400, max_rows=rows, seed=9, window=window)
    rng = np.random.default_rng(10)
    cursor = 0
    for chunk in range(17):
        prompt = rng.integers(0, TINY["vocab"], (rows, 1))
        model.prefill(prompt.reshape(-1), rows, [cursor])
        ref.forward(prompt.reshape(-1), rows, [cursor], want_logits=False)
        cursor += rows
    tokens = [7]
    for step in range(12):
        want_logits, want = ref.forward(tokens, 1, [cursor])
        got = model.decode_step(tokens, [cursor])
        assert np.abs(model.logits() - want_logits).max() <= 1e-3 * np.abs(want_logits).max(), step
        assert list(got) == list(want), (step, margins(want_logits))
        tokens, cursor = got, cursor + 1
    model.release(), weights.release()


def test_a_window_as_wide_as_what_was_fed_changes_nothing(device):
    """Until the ring wraps a windowed model holds every key an unbounded one holds: the same tokens."""
    shape = TINY
    bounded, _, held = build(device, shape, NH_Q8_0, batch=1, context=32, seed=7, window=16)
    open_, _, held2 = build(device, shape, NH_Q8_0, batch=1, context=32, seed=7)
    token_a = token_b = [3]
    for step in range(16):
        token_a = bounded.decode_step(token_a, [step])
        token_b = open_.decode_step(token_b, [step])
        assert list(token_a) == list(token_b), step
        assert np.array_equal(bounded.logits(), open_.logits())
    bounded.release(), open_.release(), held.release(), held2.release()


@pytest.mark.parametrize("batch", [2, 6, 8])
def test_decode_on_half_precision_tiles_matches_the_oracle(device, monkeypatch, batch):
    """NEURA_HIP_F16_TILES=2 sends every product of a 2..8 plane step to the 16-row half-precision tiles: stacked q|k|v and
    gate|up with the fused norm, the residual epilogues, SwiGLU, against the oracle's logits and tokens."""
    monkeypatch.setenv("NEURA_HIP_F16_TILES", "2")
    shape = SMALL_Q4
    model, ref, weights = build(device, shape, NH_Q4_K, batch=batch, context=24, seed=8)
    rng = np.random.default_rng(9)
    tokens = rng.integers(0, shape["vocab"], batch)
    for step in range(5):
        cursors = [step] * batch
        want_logits, want = ref.forward(tokens, 1, cursors)
        got = model.decode_step(tokens, cursors)
        assert np.abs(model.logits() - want_logits).max() <= 1e-3 * np.abs(want_logits).max(), step
        assert list(got) == list(want), (step, margins(want_logits))
        tokens = got
    model.release(), weights.release()


def test_decode_refuses_what_the_reference_refuses(device):
    model, ref, weights = build(device, TINY, NH_Q8_0, batch=1, context=8)
    with pytest.raises(NeuraError):   # cursor at the context (batch.rs:1627-1632)
        model.decode_step([1], [8])
    with pytest.raises(NeuraError) as refused:  # token id past the vocabulary: refusal::INDEX
        model.decode_step([TINY["vocab"]], [0])
    assert refused.value.code == -4
    assert model.decode_step([1], [0])[0] == ref.forward([1], 1, [0])[1][0]  # and the model still answers
    with pytest.raises(NeuraError):
        model.prefill([1, 2], 2, [0])  # built for chunks of one row
    model.release(), weights.release()


def golden_ids(name):
    """the ids the oracle chose when tests/golden/make_fixtures.py wrote the fixture"""
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", name)) as held:
        return json.load(held)["ids"]


def test_config4_greedy_64_steps_qwen2_5_0_5b_shape_q8_0(device):
    """Random-init 0.5B-shape Q8_0 decoder, fp16 caches prefilled to 1024 random tokens' worth
    of N(0,1) halves, 64 greedy steps from a random prompt id: token ids identical to the
    oracle's, and the oracle's identical to the committed ids.  The oracle follows the reference's summation order;
    identity against the reference binary itself is unpinned (it cannot be run here)."""
    shape, tensors, host, halves, token = cases.config4_case(threads=16)
    context, filled, steps = 1024 + 64, 1024, 64
    weights = Weights(device, tensors)
    model = Model(device, weights, shape, NH_Q8_0, 1, context, 1)
    ref = oracle.Model(shape, NH_Q8_0, host, 1, context, 1)
    cases.hold(halves, model.cache_shape, ref, model)
    got_tokens, want_tokens, gaps = [], [], []
    got = want = token
    for step in range(steps):
        want_logits, chosen = ref.forward([want], 1, [filled + step], threads=16)
        want = int(chosen[0])
        got = int(model.decode_step([got], [filled + step])[0])
        want_tokens.append(want), got_tokens.append(got)
        gaps.append(float(margins(want_logits)[0]))
        if got != want:
            break
    print("greedy margins (top1 - top2): min %.3g median %.3g" % (min(gaps), float(np.median(gaps))))
    assert got_tokens == want_tokens, "first divergence at step %d, margin %g" % (len(got_tokens) - 1, gaps[-1])
    assert want_tokens == golden_ids("config4_greedy_ids.json")
    same_cache_rows(model, ref, shape["layers"], [list(range(filled, filled + steps))], "rows the 64 steps appended")
    model.release(), weights.release()


def fill_caches(model, ref, rng, shape, layers, batch, filled):
    """positions below `filled` of every state of both decoders hold the same N(0,1) halves"""
    for layer in range(layers):
        for which, held in ((0, ref.cache_k), (1, ref.cache_v)):
            halves = np.zeros(model.cache_shape, dtype=np.float16)
            halves[:, :, :filled] = rng.standard_normal((shape["kv_heads"], batch, filled, shape["head_dim"])).astype(np.float16)
            held[layer][:] = halves.view(np.uint16).reshape(-1)
            model.cache_write(layer, which, halves.view(np.uint16))


def same_cache_rows(model, ref, layers, rows_of_plane, what):
    """the key and value rows at the given positions (a list per plane) hold the oracle's halves: what a decode step or a
    fill appended, rotation included"""
    for layer in range(layers):
        for which, held in ((0, ref.cache_k), (1, ref.cache_v)):
            got_all = model.cache_read(layer, which)
            want_all = held[layer].reshape(model.cache_shape)
            for plane, positions in enumerate(rows_of_plane):
                got_rows = oracle.f16_to_f32(np.ascontiguousarray(got_all[:, plane, positions]).reshape(-1))
                want_rows = oracle.f16_to_f32(np.ascontiguousarray(want_all[:, plane, positions]).reshape(-1))
                assert np.any(want_rows), (what, layer, which, plane)
                assert np.abs(got_rows - want_rows).max() <= 2e-3 * max(1.0, np.abs(want_rows).max()), (what, layer, which, plane)


def input_moves_the_logits(ref, batch, cursors, vocab, least=1e-2):
    """A test network must not be degenerate: another input token moves the oracle's logits by more than `least` of the
    largest (random Q4_K blocks have a large positive mean: every matrix is all ones plus noise, the network collapses onto
    one direction and its logits hardly depend on the token -- parity of ids proves nothing there).  Both passes write the
    same cache rows, which the step under test then writes again."""
    first, _ = ref.forward([1234 % vocab] * batch, 1, cursors, threads=16)
    first = first.copy()
    second, _ = ref.forward([7] * batch, 1, cursors, threads=16)
    moved = float(np.abs(first - second).max() / np.abs(first).max())
    print("another input token moves the oracle's logits by %.3g of the largest" % moved, flush=True)
    return moved > least


@pytest.mark.parametrize("mode", ["blocks", "normal"])
def test_config5_shape_two_layers_qwen2_5_7b_q4_k(device, mode):
    """The 7B shape itself (hidden 3584, 28 query heads over 4 key heads of 128, ffn 18944, vocabulary 152064, separate head)
    cut to two layers, at context 4096: decode steps at batch 1 on caches filled with N(0,1) halves
    (the products at their real depths and row counts, the rotation folded in, attention over 4000 keys in sections), a
    512-row fill, the prompt chunk of the benchmark (wide products with stacked q|k|v and fused packing passes, attention
    over a chunk), and steps of eight planes (the half-precision tiles on gate|up and the head, the integer tiles on the
    rest), each against the oracle: logits within 1e-3 of the largest, the greedy token identical at every step, and the key
    and value rows the steps and the fill appended equal to the oracle's.

    "blocks": random Q4_K blocks, the distribution BASELINE's product configurations name -- a degenerate network (its
    logits do not depend on the token), which holds the products' bulk accuracy and nothing else.  "normal": N(0, 0.02)
    weights packed by the reference's Q4_K encoder -- a network whose logits, tokens and appended rows depend on every
    input-dependent piece (embedding row, rotation at the cursor, cache append, attention over the appended rows)."""
    shape = synth.SHAPES["qwen2.5-7b"]
    # (the degenerate twin fills 128 rows -- the same kernels over one tile of rows -- which spares the oracle half a minute)
    layers, context, filled, rows = 2, 4096, 3500, 512 if mode == "normal" else 128
    rng = np.random.default_rng(50)
    tensors = list(synth.model_tensors(shape, NH_Q4_K, rng, mode=mode, layers=layers, threads=16))
    host = {name: raw for name, _, _, raw in tensors}
    weights = Weights(device, tensors)

    def pair(batch, max_rows):
        model = Model(device, weights, shape, NH_Q4_K, batch, context, max_rows, layers=layers)
        ref = oracle.Model(shape, NH_Q4_K, host, batch, context, max_rows, layers=layers)
        fill_caches(model, ref, rng, shape, layers, batch, filled)
        return model, ref

    seen = []

    def same(model, ref, tokens, cursors, what):
        want_logits, want = ref.forward(tokens, 1, cursors, threads=16)
        got = model.decode_step(tokens, cursors)
        logits = model.logits()
        scale = np.abs(want_logits).max()
        assert np.abs(logits - want_logits).max() <= 1e-3 * scale, what
        gaps = margins(want_logits)
        print("%s (%s): tokens %s, top-2 margins min %.3g of a largest logit of %.3g, logits within %.3g" %
              (what, mode, [int(t) for t in want], gaps.min(), scale, np.abs(logits - want_logits).max()), flush=True)
        assert [int(t) for t in got] == [int(t) for t in want], (what, gaps)
        seen.extend(int(t) for t in want)
        return [int(t) for t in want]

    model, ref = pair(1, rows)
    assert input_moves_the_logits(ref, 1, [filled], shape["vocab"]) or mode == "blocks"
    token = [int(rng.integers(0, shape["vocab"]))]
    for step in range(3):
        token = same(model, ref, token, [filled + step], "batch 1, step %d" % step)
    # what the three steps appended: the rotated key rows and the value rows at the stepped cursors (the epilogue of the
    # q|k|v product at 4608 x 3584)
    same_cache_rows(model, ref, layers, [[filled, filled + 1, filled + 2]], "rows the batch-1 steps appended")
    # a fill of 512 (128) rows behind the keys already held (positions 3503 .. 4014), then a step that weighs what it wrote
    prompt = rng.integers(0, shape["vocab"], rows)
    first = filled + 3
    model.prefill(prompt, rows, [first])
    ref.forward(prompt, rows, [first], want_logits=False, threads=16)
    same_cache_rows(model, ref, layers, [list(range(first, first + rows))], "rows the fill appended")
    same(model, ref, token, [first + rows], "batch 1 after the %d-row fill" % rows)
    same_cache_rows(model, ref, layers, [[first + rows]], "the row behind the fill")
    model.release()
    model, ref = pair(8, 1)
    tokens = [int(t) for t in rng.integers(0, shape["vocab"], 8)]
    for step in range(2):
        tokens = same(model, ref, tokens, [filled - 7 * plane + step for plane in range(8)], "batch 8, step %d" % step)
    same_cache_rows(model, ref, layers, [[filled - 7 * plane, filled - 7 * plane + 1] for plane in range(8)], "rows the batch-8 steps appended")
    if mode == "normal":
        assert len(set(seen)) > len(seen) // 2, seen  # the chosen tokens differ from step to step and plane to plane
    model.release(), weights.release()


@pytest.mark.parametrize("mode", ["blocks", "normal"])
def test_config5_full_depth_greedy_64_steps_qwen2_5_7b_shape_q4_k(device, mode):
    """The model the benchmark times, whole: 28 layers of the 7B shape, a separate head, fp16 caches
    holding 4032 positions of N(0,1) halves, then 64 greedy steps up to the end of the context of 4096 -- every token
    identical to the oracle's, with no allowance for close calls.  "blocks": the benchmark's random Q4_K blocks (a
    degenerate network: one token, margins in the hundreds -- the products' bulk accuracy); "normal": N(0, 0.02) weights
    packed by the reference's encoder (tokens vary, margins are small and printed; nothing is gated on them).

    The oracle's 64 ids are the committed ones (tests/golden/make_fixtures.py wrote them from these same seeded inputs: two
    minutes of host time a file).  Beside the device the oracle itself runs the first NEURA_TEST_ORACLE_STEPS steps (default 8;
    64 runs it all the way): its ids must be the file's, the device's logits must lie within 1e-3 of its largest, and the key
    and value rows those steps append must be its rows.  The oracle follows the reference's summation order; identity against
    the reference binary itself is unpinned (it cannot be run here)."""
    shape = synth.SHAPES["qwen2.5-7b"]
    context, steps = 4096, 64
    live = max(1, min(steps, int(os.environ.get("NEURA_TEST_ORACLE_STEPS", "8"))))
    filled = context - steps
    shape_, tensors, host, halves, token = cases.config5_case(mode)
    assert shape_ is shape
    stored = golden_ids("config5_%s_greedy_ids.json" % mode)
    assert len(stored) == steps
    weights = Weights(device, tensors)
    model = Model(device, weights, shape, NH_Q4_K, 1, context, 1)
    ref = oracle.Model(shape, NH_Q4_K, host, 1, context, 1)
    cases.hold(halves, model.cache_shape, ref, model)
    del halves
    got = want = token
    got_tokens, want_tokens, gaps, apart = [], [], [], []
    for step in range(steps):
        got = int(model.decode_step([got], [filled + step])[0])
        got_tokens.append(got)
        if step < live:
            want_logits, chosen = ref.forward([want], 1, [filled + step], threads=16)
            want = int(chosen[0])
            want_tokens.append(want)
            gaps.append(float(margins(want_logits)[0]))
            apart.append(float(np.abs(model.logits() - want_logits).max() / np.abs(want_logits).max()))
        if got != stored[step]:
            break
    print("greedy tokens (%s): %s" % (mode, got_tokens))
    print("the oracle beside the device over %d steps: top-2 margins min %.3g median %.3g; logits within %.3g of the largest" %
          (len(gaps), min(gaps), float(np.median(gaps)), max(apart)))
    assert want_tokens == stored[:len(want_tokens)], "the oracle no longer chooses what it chose when the fixture was written"
    assert max(apart) <= 1e-3
    assert got_tokens == stored, "first divergence from the oracle's ids at step %d" % (len(got_tokens) - 1)
    if mode == "normal":
        assert len(set(got_tokens)) > steps // 2, got_tokens
        same_cache_rows(model, ref, shape["layers"], [list(range(filled, filled + live))], "rows the first steps appended")
    model.release(), weights.release()


@pytest.mark.parametrize("mode", ["blocks", "normal"])
def test_config5_shape_stored_as_a_q4_k_m_file_stores_it(device, mode):
    """The 7B shape cut to two layers, stored the way llama.cpp's Q4_K_M recipe stores Qwen2.5-7B: the head and the first
    layer's value and down projections in Q6_K, q, k and v biases on every layer.  Batch-1 steps at context 4096: the
    Q6_K products at their real shapes (a 152064-row head, a down projection), q|k rotated from one
    product with the value row appended behind it, the layer of one element with biases in the folded rotation.  Random
    blocks and N(0, 0.02) weights (Q6_K through the symmetric numpy quantizer), as above."""
    shape = synth.SHAPES["qwen2.5-7b"]
    layers, context, filled = 2, 4096, 4000
    mixed = {"output.weight": NH_Q6_K, "blk.0.attn_v.weight": NH_Q6_K, "blk.0.ffn_down.weight": NH_Q6_K}
    rng = np.random.default_rng(51)
    tensors = list(synth.model_tensors(shape, NH_Q4_K, rng, mode=mode, layers=layers, elements=mixed, biases=(0, 1), threads=16))
    host = {name: (raw.view(np.float32) if name.endswith(".bias") else raw) for name, _, _, raw in tensors}
    weights = Weights(device, tensors)
    model = Model(device, weights, shape, NH_Q4_K, 1, context, 1, layers=layers)
    ref = oracle.Model(shape, NH_Q4_K, host, 1, context, 1, layers=layers, elements=mixed)
    fill_caches(model, ref, rng, shape, layers, 1, filled)
    assert input_moves_the_logits(ref, 1, [filled], shape["vocab"]) or mode == "blocks"
    token = [int(rng.integers(0, shape["vocab"]))]
    chosen = []
    for step in range(3):
        want_logits, want = ref.forward(token, 1, [filled + step], threads=16)
        got = model.decode_step(token, [filled + step])
        scale = np.abs(want_logits).max()
        print("step %d (%s): token %d, margin %.3g, logits within %.3g of %.3g" % (step, mode, int(want[0]), margins(want_logits)[0],
                                                                                 np.abs(model.logits() - want_logits).max(), scale), flush=True)
        assert np.abs(model.logits() - want_logits).max() <= 1e-3 * scale, step
        assert int(got[0]) == int(want[0]), (step, margins(want_logits))
        token = [int(want[0])]
        chosen.append(token[0])
    same_cache_rows(model, ref, layers, [[filled, filled + 1, filled + 2]], "rows the steps appended")
    if mode == "normal":
        assert len(set(chosen)) > 1, chosen
    model.release(), weights.release()


def test_recorded_steps_are_refused_in_a_traced_process(device, monkeypatch):
    """rocprofv3 names its tool library in the environment of what it runs; hipGraphLaunch has crashed under it, so a traced
    process steps eagerly and NEURA_HIP_GRAPH=1 there is an error at nh_model_create, not a crash later.  (No graph is
    launched here: the environment alone is what the library looks at.)"""
    monkeypatch.setenv("ROCP_TOOL_LIBRARIES", "librocprofiler-sdk-tool.so")
    monkeypatch.setenv("NEURA_HIP_GRAPH", "1")
    with pytest.raises(NeuraError, match="traced"):
        build(device, TINY, NH_Q8_0, batch=1, context=8)
    monkeypatch.delenv("NEURA_HIP_GRAPH")
    model, ref, weights = build(device, TINY, NH_Q8_0, batch=1, context=8)  # without the switch: eager steps, same answers
    for step in range(3):
        assert model.decode_step([5], [step])[0] == ref.forward([5], 1, [step])[1][0]
    model.release(), weights.release()


def test_graph_replays_match_eager_steps(device, monkeypatch):
    """The decode step replayed from its captured HIP graph gives, on every replay, exactly the
    logits and tokens of the same step launched eagerly -- with eager work (fills, operator
    calls, synchronisations) between the replays, masked and unmasked variants interleaved."""
    shape = SMALL_Q4
    monkeypatch.setenv("NEURA_HIP_GRAPH", "1")
    replayed, _, weights_a = build(device, shape, NH_Q4_K, batch=2, context=48, max_rows=8, seed=5)
    monkeypatch.setenv("NEURA_HIP_GRAPH", "0")
    eager, _, weights_b = build(device, shape, NH_Q4_K, batch=2, context=48, max_rows=8, seed=5)
    rng = np.random.default_rng(6)
    prompt = rng.integers(0, shape["vocab"], (8, 2)).reshape(-1)
    tokens_a = tokens_b = [3, 4]
    cursor = [0, 0]
    for step in range(12):
        if step == 4:  # a chunked fill between replays moves both cursors on by 8
            for model in (replayed, eager):
                model.prefill(prompt, 8, cursor)
            cursor = [cursor[0] + 8, cursor[1] + 8]
        mask = [1, 0] if step % 3 == 2 else None
        got_a = replayed.decode_step(tokens_a, cursor, mask=mask)
        got_b = eager.decode_step(tokens_b, cursor, mask=mask)
        logits_a, logits_b = replayed.logits(), eager.logits()
        rows = [0] if mask else [0, 1]
        assert np.array_equal(logits_a[rows], logits_b[rows]), step
        assert list(got_a[rows]) == list(got_b[rows]), step
        # eager operator work on the same stream before the next replay
        x = rng.standard_normal((1, shape["hidden"])).astype(np.float32)
        device.rmsnorm(x, np.ones(shape["hidden"], np.float32), 1e-6)
        device.sync()
        tokens_a, tokens_b = [int(got_a[0]), 4], [int(got_b[0]), 4]
        cursor = [cursor[0] + 1, cursor[1] + (0 if mask else 1)]
    for layer in range(shape["layers"]):
        for which in (0, 1):
            assert np.array_equal(replayed.cache_read(layer, which)[:, :, :40], eager.cache_read(layer, which)[:, :, :40])
    for held in (replayed, eager, weights_a, weights_b):
        held.release()


WIDE_CUT = dict(layers=2, hidden=3584, heads=28, kv_heads=4, head_dim=128, ffn=2048, vocab=512, tied=False)


@pytest.mark.parametrize("shape,element,same_sums", [(SMALL_Q4, NH_Q4_K, True), (TINY, NH_Q8_0, True), (SMALL_Q4, NH_Q6_K, False), (SMALL_Q4, NH_Q3_K, False),
                                                     (WIDE_CUT, NH_Q6_K, False), (WIDE_CUT, NH_Q3_K, False), (SMALL_Q4, NH_Q5_K, False)],
                         ids=["q4_k", "q8_0", "q6_k", "q3_k", "q6_k-3584", "q3_k-3584", "q5_k"])
def test_rotation_folded_into_the_product_matches_the_separate_kernel(device, monkeypatch, shape, element, same_sums):
    """At batch 1 the q|k|v product of a decoder rotates q and k and appends k and v to the caches in its epilogue; the same
    steps with the rotation as its own kernel give the same bits in the caches and the logits where both run the same
    product kernel (Q4_K, Q8_0).  Q6_K, Q3_K and Q5_K fold the rotation into their 16-row tile product, and the twin with the
    rotation apart multiplies on the staged kernel: another order of the sums, so logits and caches are held to the
    decoder's bar and to the oracle, and the tokens to each other."""
    monkeypatch.setenv("NEURA_HIP_GRAPH", "0")  # both twins launch eagerly, so the switch below is read at every step
    mode = "normal" if shape is not WIDE_CUT else "blocks"
    folded, ref, weights_a = build(device, shape, element, batch=1, context=24, seed=9, mode=mode)
    apart, _, weights_b = build(device, shape, element, batch=1, context=24, seed=9, mode=mode)
    token_a = token_b = 5
    for step in range(8):
        monkeypatch.setenv("NEURA_HIP_FUSE_ROPE", "1")
        got_a = folded.decode_step([token_a], [step])
        logits_a = folded.logits()
        monkeypatch.setenv("NEURA_HIP_FUSE_ROPE", "0")
        got_b = apart.decode_step([token_b], [step])
        logits_b = apart.logits()
        want_logits, want = ref.forward([token_a], 1, [step])
        scale = np.abs(want_logits).max()
        if same_sums:
            assert np.array_equal(logits_a, logits_b), step
        else:
            assert np.abs(logits_a - logits_b).max() <= 1e-3 * scale, step
        assert np.abs(logits_a - want_logits).max() <= 1e-3 * scale
        assert list(got_a) == list(got_b) == list(want), (step, margins(want_logits))
        token_a = token_b = int(got_a[0])
    for layer in range(shape["layers"]):
        for which, held in ((0, ref.cache_k), (1, ref.cache_v)):
            mine, twin = folded.cache_read(layer, which), apart.cache_read(layer, which)
            if same_sums:
                assert np.array_equal(mine, twin), (layer, which)
            else:
                bar = 1e-2 * max(1.0, np.abs(held[layer]).max())
                mine, twin, want_rows = mine.astype(np.float32).reshape(-1), twin.astype(np.float32).reshape(-1), held[layer].astype(np.float32).reshape(-1)
                assert np.abs(mine - want_rows).max() <= bar and np.abs(mine - twin).max() <= bar, (layer, which)
                assert np.any(mine.reshape(folded.cache_shape)[:, 0, :8])  # the steps' rows are there
    # a cursor past the window is refused by the folded form as by the separate kernel
    monkeypatch.setenv("NEURA_HIP_FUSE_ROPE", "1")
    with pytest.raises(NeuraError):
        folded.decode_step([1], [folded.capacity + 3])
    for held in (folded, apart, weights_a, weights_b):
        held.release()


@pytest.mark.parametrize("shape,biased", [(SMALL_Q4, False), (SMALL_Q4, True), (WIDE_CUT, False)], ids=["small", "small-biased", "3584"])
@pytest.mark.parametrize("batch", [5, 8])
def test_rotation_folded_into_the_product_of_several_planes(device, monkeypatch, shape, biased, batch):
    """Five to eight planes of one token each: the q|k|v product of a Q4_K decoder (the 32-row integer tiles) rotates q and k
    and appends k and v in its epilogue, every plane at its own cursor.  The twin with the rotation as a kernel of its own runs
    the same product kernel and the same table of cosines and sines, so logits and caches agree bit for bit; both are held to
    the oracle (logits, tokens, and the rows the steps appended).  With q, k and v biases the twin multiplies the three
    matrices one by one: each row's sums are the same, and so are the bits."""
    monkeypatch.setenv("NEURA_HIP_GRAPH", "0")  # both twins launch eagerly, so the switch below is read at every step
    layers = list(range(shape["layers"])) if biased else []

    def pair():
        rng = np.random.default_rng(31)
        tensors = list(synth.model_tensors(shape, NH_Q4_K, rng, mode="normal" if shape is not WIDE_CUT else "blocks", biases=layers))
        weights = Weights(device, tensors)
        return Model(device, weights, shape, NH_Q4_K, batch, 40, 1), weights, {name: (raw.view(np.float32) if name.endswith(".bias") else raw) for name, _, _, raw in tensors}

    folded, weights_a, host = pair()
    apart, weights_b, _ = pair()
    ref = oracle.Model(shape, NH_Q4_K, host, batch, 40, 1)
    tokens = [3 + 7 * plane for plane in range(batch)]
    first = [3 * plane for plane in range(batch)]  # every plane at a cursor of its own
    steps = 5
    for step in range(steps):
        cursors = [at + step for at in first]
        monkeypatch.setenv("NEURA_HIP_FUSE_ROPE", "1")
        got_a = folded.decode_step(tokens, cursors)
        logits_a = folded.logits()
        monkeypatch.setenv("NEURA_HIP_FUSE_ROPE", "0")
        got_b = apart.decode_step(tokens, cursors)
        logits_b = apart.logits()
        want_logits, want = ref.forward(tokens, 1, cursors)
        assert np.array_equal(logits_a, logits_b), step
        assert np.abs(logits_a - want_logits).max() <= 1e-3 * np.abs(want_logits).max()
        assert list(got_a) == list(got_b) == list(want), (step, margins(want_logits))
        tokens = [int(t) for t in got_a]
    for layer in range(shape["layers"]):
        for which in (0, 1):
            assert np.array_equal(folded.cache_read(layer, which), apart.cache_read(layer, which)), (layer, which)
    same_cache_rows(folded, ref, shape["layers"], [list(range(at, at + steps)) for at in first], "rows the planes' steps appended")
    # a cursor past the window is refused by the folded form as by the separate kernel
    monkeypatch.setenv("NEURA_HIP_FUSE_ROPE", "1")
    with pytest.raises(NeuraError):
        folded.decode_step(tokens, [folded.capacity + 3] * batch)
    for held in (folded, apart, weights_a, weights_b):
        held.release()


# (a chained launch hands ffn_down's first weights across the seam: it takes rows of sixteen super-blocks and more)
CHAIN_SMALL = dict(layers=2, hidden=512, heads=8, kv_heads=2, head_dim=128, ffn=4096, vocab=1000, tied=False)
CHAIN_SHAPES = [CHAIN_SMALL, dict(layers=2, hidden=3584, heads=28, kv_heads=4, head_dim=128, ffn=18944, vocab=2048, tied=False)]


@pytest.mark.parametrize("shape", CHAIN_SHAPES, ids=["small", "7b-layers"])
@pytest.mark.parametrize("chain", ["1", "2"])
def test_products_chained_into_one_launch_match_one_launch_a_product(device, monkeypatch, shape, chain):
    """At batch 1 the products between two attentions can run as one launch with seams between them (NEURA_HIP_CHAIN=1: gate|up
    and ffn_down; 2: attn_output in front; the default is one launch a product).  What crosses a seam crosses it at device
    scope and carries tag words: a reader that finds a piece without this step's tag reads it again.  The same steps one launch
    a product (NEURA_HIP_CHAIN=0) give the same logits to the last few bits (the chained stages split a row's super-blocks over
    eight waves where the launches of their own take four or seven, so sums associate differently), the same tokens and the
    same cache rows; both sit within the decoder's bar of the oracle.  No step fell back."""
    monkeypatch.setenv("NEURA_HIP_GRAPH", "0")  # both twins launch eagerly, so the switch below is read at every step
    tensors = list(synth.model_tensors(shape, NH_Q4_K, np.random.default_rng(21), mode="normal", threads=16))
    weights = Weights(device, tensors)
    chained, apart = Model(device, weights, shape, NH_Q4_K, 1, 40), Model(device, weights, shape, NH_Q4_K, 1, 40)
    ref = oracle.Model(shape, NH_Q4_K, {name: raw for name, _, _, raw in tensors}, 1, 40)
    token_a = token_b = 11
    for step in range(6):
        monkeypatch.setenv("NEURA_HIP_CHAIN", chain)
        got_a = chained.decode_step([token_a], [step])
        logits_a = chained.logits()
        monkeypatch.setenv("NEURA_HIP_CHAIN", "0")
        got_b = apart.decode_step([token_b], [step])
        logits_b = apart.logits()
        want_logits, want = ref.forward([token_a], 1, [step], threads=16)
        scale = np.abs(want_logits).max()
        assert np.abs(logits_a - logits_b).max() <= 2e-5 * scale, step
        assert np.abs(logits_a - want_logits).max() <= 1e-3 * scale, step
        assert list(got_a) == list(got_b) == list(want), (step, margins(want_logits))
        token_a = token_b = int(got_a[0])
    same_cache_rows(chained, ref, shape["layers"], [list(range(6))], "rows the chained steps appended")
    assert chained.seam_fallbacks() == 0 and apart.seam_fallbacks() == 0
    for held in (chained, apart, weights):
        held.release()


@pytest.mark.parametrize("graph", ["0", "1"])
def test_a_seam_that_gives_up_sends_the_step_down_the_path_of_one_launch_a_product(device, monkeypatch, graph):
    """NEURA_HIP_CHAIN_SPIN=0: every reader at a seam gives up before it looks twice (the kernels all end; no wait is ever
    unbounded, and no wave leaves early).  The step that met it is run again one launch a product and answers as the oracle
    does, the model counts one fallback and stays on that path, eager or recorded."""
    monkeypatch.setenv("NEURA_HIP_GRAPH", graph)
    monkeypatch.setenv("NEURA_HIP_CHAIN", "2")
    monkeypatch.setenv("NEURA_HIP_CHAIN_SPIN", "0")
    model, ref, weights = build(device, CHAIN_SMALL, NH_Q4_K, batch=1, context=40, seed=22)
    monkeypatch.delenv("NEURA_HIP_CHAIN_SPIN")
    token = 5
    for step in range(5):
        want_logits, want = ref.forward([token], 1, [step])
        got = model.decode_step([token], [step])
        assert np.abs(model.logits() - want_logits).max() <= 1e-3 * np.abs(want_logits).max(), step
        assert list(got) == list(want), step
        assert model.seam_fallbacks() == 1, step
        token = int(got[0])
    # a model built without the hook chains, and never falls back
    healthy, ref, weights_b = build(device, CHAIN_SMALL, NH_Q4_K, batch=1, context=40, seed=22)
    token = 5
    for step in range(5):
        want_logits, want = ref.forward([token], 1, [step])
        got = healthy.decode_step([token], [step])
        assert np.abs(healthy.logits() - want_logits).max() <= 1e-3 * np.abs(want_logits).max(), step
        assert list(got) == list(want), step
        token = int(got[0])
    assert healthy.seam_fallbacks() == 0
    for held in (model, healthy, weights, weights_b):
        held.release()


@pytest.mark.parametrize("base,down", [(NH_Q4_K, NH_Q4_K), (NH_Q4_K, NH_Q6_K), (NH_Q6_K, NH_Q6_K), (NH_Q3_K, NH_Q3_K), (NH_Q3_K, NH_Q4_K), (NH_Q5_K, NH_Q6_K)],
                         ids=["q4_k ffn_down", "q6_k ffn_down", "q6_k throughout", "q3_k throughout", "q3_k into q4_k", "q5_k into q6_k"])
def test_swiglu_outputs_handed_on_as_digit_planes_match_the_floats(device, monkeypatch, base, down):
    """At batch 1 the gate|up product of a decoder leaves silu(gate) * up as the digit planes ffn_down multiplies (a
    power-of-two scale per 16 outputs where ffn_down's own staging takes one per 64); NEURA_HIP_TILE16_HANDED=0 hands the
    floats on instead.  Both stay within the decoder's bar of the oracle and of each other (a difference in the last bits of
    a key now and then flips its rounding to half, 5e-4 of it) and choose the same tokens.  With Q6_K down projections (a
    Q4_K_M file's) the planes feed the Q6_K tiles, which read the same pieces; gate|up products of Q6_K, Q3_K and Q5_K leave
    the same pieces, for down projections of any K-quant."""
    monkeypatch.setenv("NEURA_HIP_GRAPH", "0")  # both twins launch eagerly, so the switch below is read at every step
    elements = {"blk.%d.ffn_down.weight" % layer: down for layer in range(SMALL_Q4["layers"])} if down != base else None
    handed, ref, weights_a = build(device, SMALL_Q4, base, batch=1, context=24, seed=11, elements=elements)
    floats, _, weights_b = build(device, SMALL_Q4, base, batch=1, context=24, seed=11, elements=elements)
    token = 7
    for step in range(8):
        monkeypatch.setenv("NEURA_HIP_TILE16_HANDED", "1")
        got_a = handed.decode_step([token], [step])
        logits_a = handed.logits()
        monkeypatch.setenv("NEURA_HIP_TILE16_HANDED", "0")
        got_b = floats.decode_step([token], [step])
        logits_b = floats.logits()
        want_logits, want = ref.forward([token], 1, [step])
        scale = np.abs(want_logits).max()
        assert np.abs(logits_a - want_logits).max() <= 1e-3 * scale and np.abs(logits_b - want_logits).max() <= 1e-3 * scale, step
        assert np.abs(logits_a - logits_b).max() <= 1e-3 * scale, step
        assert list(got_a) == list(got_b) == list(want), (step, margins(want_logits))
        token = int(got_a[0])
    for held in (handed, floats, weights_a, weights_b):
        held.release()


def test_attention_sections_merged_by_the_output_projection_match_the_fold(device, monkeypatch):
    """At batch 1 the attention of a Q8_0 decoder leaves the sums of its sections unmerged and the output projection merges
    them as it stages its row (one launch fewer a layer); NEURA_HIP_MERGE_IN_PRODUCT=0 keeps the fold's own launch.  The
    window is three sections of 54 keys: the steps walk from one section seen (the others empty: no mass) into the second.
    Both twins stay within the decoder's bar of the oracle and choose its tokens."""
    monkeypatch.setenv("NEURA_HIP_GRAPH", "0")  # both twins launch eagerly, so the switch below is read at every step
    merged, ref, weights_a = build(device, TINY, NH_Q8_0, batch=1, context=160, seed=31)
    folded, _, weights_b = build(device, TINY, NH_Q8_0, batch=1, context=160, seed=31)
    token = 5
    for step in range(70):
        monkeypatch.setenv("NEURA_HIP_MERGE_IN_PRODUCT", "1")
        got_a = merged.decode_step([token], [step])
        logits_a = merged.logits()
        monkeypatch.setenv("NEURA_HIP_MERGE_IN_PRODUCT", "0")
        got_b = folded.decode_step([token], [step])
        logits_b = folded.logits()
        want_logits, want = ref.forward([token], 1, [step])
        scale = np.abs(want_logits).max()
        assert np.abs(logits_a - want_logits).max() <= 1e-3 * scale and np.abs(logits_b - want_logits).max() <= 1e-3 * scale, step
        assert np.abs(logits_a - logits_b).max() <= 1e-4 * scale, step
        assert list(got_a) == list(got_b) == list(want), (step, margins(want_logits))
        token = int(got_a[0])
    for held in (merged, folded, weights_a, weights_b):
        held.release()


@pytest.mark.parametrize("base,mixed", [(NH_Q4_K, MIXED), (NH_Q5_K, MIXED), (NH_Q3_K, MIXED_3)], ids=["q4_k_m", "q5_k_m", "q3_k_m"])
@pytest.mark.parametrize("pair", ["1", "0"], ids=["one launch", "two launches"])
def test_value_rows_appended_by_their_product_equal_the_append_kernels(device, monkeypatch, pair, base, mixed):
    """Where q|k go out rotated from one product and the value projection is stored otherwise (layer 0 of the Q4_K_M-like
    mix: Q6_K; the same mix over Q5_K; layers 0 and 1 of the Q3_K_M-like mix: Q5_K and Q4_K), the value product casts its
    rows (+ bias) into the value state itself -- beside a Q4_K or Q5_K q|k product in one launch, or (NEURA_HIP_PAIR=0, and
    wherever no pair is built) in a launch of its own; NEURA_HIP_APPEND_VALUE=0 leaves the cast to the append kernel.
    The same sums either way: states and logits equal bit for bit, and the oracle's tokens."""
    monkeypatch.setenv("NEURA_HIP_GRAPH", "0")  # both twins launch eagerly, so the switch below is read at every step
    monkeypatch.setenv("NEURA_HIP_PAIR", pair)
    shape = SMALL_Q4
    tensors = list(synth.model_tensors(shape, base, np.random.default_rng(21), mode="normal", elements=mixed, biases=(0, 1)))
    host = {name: (raw.view(np.float32) if name.endswith(".bias") else raw) for name, _, _, raw in tensors}
    weights = Weights(device, tensors)
    fused, apart = Model(device, weights, shape, base, 1, 24, 1), Model(device, weights, shape, base, 1, 24, 1)
    ref = oracle.Model(shape, base, host, 1, 24, 1, elements=mixed)
    token = 11
    for step in range(6):
        monkeypatch.setenv("NEURA_HIP_APPEND_VALUE", "1")
        got_a = fused.decode_step([token], [step])
        logits_a = fused.logits()
        monkeypatch.setenv("NEURA_HIP_APPEND_VALUE", "0")
        got_b = apart.decode_step([token], [step])
        assert np.array_equal(logits_a, apart.logits()), step
        want_logits, want = ref.forward([token], 1, [step])
        assert np.abs(logits_a - want_logits).max() <= 1e-3 * np.abs(want_logits).max(), step
        assert list(got_a) == list(got_b) == list(want), (step, margins(want_logits))
        token = int(got_a[0])
    for layer in range(shape["layers"]):
        assert np.array_equal(fused.cache_read(layer, 1), apart.cache_read(layer, 1)), layer
    assert np.any(fused.cache_read(0, 1)[:, 0, :6])
    fused.release(), apart.release(), weights.release()


def test_rows_packed_through_lds_equal_the_rows_packed_from_memory(device, monkeypatch):
    """A fill's wide products take their fp32 rows (as they lie, normalised, or gated by silu) packed into half rows; the
    packing stages a row in LDS and crosses memory once, NEURA_HIP_PACK_STAGED=0 walks the row in memory three times.  The
    same arithmetic on the same numbers: states and the next step's logits equal bit for bit, and within the oracle's bar."""
    staged, ref, weights_a = build(device, SMALL_Q4, NH_Q4_K, batch=2, context=48, max_rows=20, seed=41)
    walked, _, weights_b = build(device, SMALL_Q4, NH_Q4_K, batch=2, context=48, max_rows=20, seed=41)
    prompt = np.random.default_rng(42).integers(0, SMALL_Q4["vocab"], (20, 2))
    monkeypatch.setenv("NEURA_HIP_PACK_STAGED", "1")
    staged.prefill(prompt.reshape(-1), 20, [0, 0])
    monkeypatch.setenv("NEURA_HIP_PACK_STAGED", "0")
    walked.prefill(prompt.reshape(-1), 20, [0, 0])
    monkeypatch.delenv("NEURA_HIP_PACK_STAGED")
    ref.forward(prompt.reshape(-1), 20, [0, 0], want_logits=False)
    for layer in range(SMALL_Q4["layers"]):
        for which in (0, 1):
            assert np.array_equal(staged.cache_read(layer, which), walked.cache_read(layer, which)), (layer, which)
    want_logits, want = ref.forward([3, 4], 1, [20, 20])
    got_a, got_b = staged.decode_step([3, 4], [20, 20]), walked.decode_step([3, 4], [20, 20])
    assert np.array_equal(staged.logits(), walked.logits())
    assert np.abs(staged.logits() - want_logits).max() <= 1e-3 * np.abs(want_logits).max()
    assert list(got_a) == list(got_b) == list(want), margins(want_logits)
    for held in (staged, walked, weights_a, weights_b):
        held.release()


def test_decoders_of_different_rope_bases_step_in_turn(device):
    """Two decoders of different rope bases and head widths stepping alternately at batch 2 (the rotation as its own
    kernel, read from the device's table of inverse frequencies): each keeps answering from its own recorded step as the
    oracle does, whatever table the other one asked for in between."""
    first, ref_a, weights_a = build(device, SMALL_Q4, NH_Q4_K, batch=2, context=24, seed=21)
    tensors_b = list(synth.model_tensors(TINY, NH_Q8_0, np.random.default_rng(22), mode="normal"))
    weights_b = Weights(device, tensors_b)
    second = Model(device, weights_b, TINY, NH_Q8_0, 2, 24, 1, rope_base=1e4)
    ref_b = oracle.Model(TINY, NH_Q8_0, {name: raw for name, _, _, raw in tensors_b}, 2, 24, 1, rope_base=1e4)
    tokens_a, tokens_b = [3, 4], [5, 6]
    for step in range(6):
        want_logits, want = ref_a.forward(tokens_a, 1, [step, step])
        tokens_a = list(first.decode_step(tokens_a, [step, step]))
        assert np.abs(first.logits() - want_logits).max() <= 1e-3 * np.abs(want_logits).max(), step
        assert tokens_a == list(want), step
        want_logits, want = ref_b.forward(tokens_b, 1, [step, step])
        tokens_b = list(second.decode_step(tokens_b, [step, step]))
        assert np.abs(second.logits() - want_logits).max() <= 1e-3 * np.abs(want_logits).max(), step
        assert tokens_b == list(want), step
    first.release(), second.release(), weights_a.release(), weights_b.release()


def test_a_recorded_step_survives_a_scratch_that_moves(device):
    """The recorded decode step holds addresses inside the device scratch; an operator call that makes the
    scratch grow (and move) in between must not leave the replay reading freed memory."""
    shape = SMALL_Q4
    model, ref, weights = build(device, shape, NH_Q4_K, batch=2, context=16, seed=13)
    tokens = [3, 4]
    for step in range(2):
        want_logits, want = ref.forward(tokens, 1, [step, step])
        tokens = list(model.decode_step(tokens, [step, step]))
        assert tokens == list(want)
    # a wide product with fp32 activations large enough to outgrow whatever scratch the device holds now
    rng = np.random.default_rng(1)
    M, N, K = 2048, 128, 16384
    device.gemm(NH_Q4_K, synth.q4_k_random(rng, N * K), N, K, rng.standard_normal((M, K)).astype(np.float32))
    for step in range(2, 5):
        want_logits, want = ref.forward(tokens, 1, [step, step])
        tokens = list(model.decode_step(tokens, [step, step]))
        assert np.abs(model.logits() - want_logits).max() <= 1e-3 * np.abs(want_logits).max()
        assert tokens == list(want)
    model.release(), weights.release()
