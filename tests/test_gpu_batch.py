"""The host layer end to end on the GPU: a Qwen2 GGUF file is opened by the C++ reader, poured
into the weight arena, and generated from by the greedy batch; the tokens are checked against
the CPU oracle run one sequence at a time.  The equivalences are the reference's own
(crates/neura-generate/tests/generation.rs:430-470): a sequence answers in a batch as it does
alone, and a prompt filled in chunks answers as one fed token by token."""
import numpy as np
import pytest

import oracle
from gguf_fixture import build as build_gguf
from neura_amd import NH_Q3_K, NH_Q4_K, NH_Q5_K, NH_Q6_K, NH_Q8_0, host, synth

pytestmark = pytest.mark.gpu

SHAPE = dict(layers=2, hidden=256, heads=4, kv_heads=2, head_dim=64, ffn=512, vocab=320, tied=True)
SHAPE_Q4 = dict(layers=2, hidden=512, heads=4, kv_heads=2, head_dim=128, ffn=1024, vocab=600, tied=False)
CONTEXT = 96


def qwen2_gguf(path, shape, element, seed, elements=None, biases=()):
    rng = np.random.default_rng(seed)
    tensors = list(synth.model_tensors(shape, element, rng, mode="normal", elements=elements, biases=biases))
    metadata = [("general.alignment", "u32", 32), ("general.architecture", "string", "qwen2"),
                ("qwen2.block_count", "u32", shape["layers"]), ("qwen2.embedding_length", "u32", shape["hidden"]),
                ("qwen2.feed_forward_length", "u32", shape["ffn"]), ("qwen2.attention.head_count", "u32", shape["heads"]),
                ("qwen2.attention.head_count_kv", "u32", shape["kv_heads"]), ("qwen2.context_length", "u32", 32768),
                ("qwen2.rope.freq_base", "f32", 1e6), ("qwen2.attention.layer_norm_rms_epsilon", "f32", 1e-6)]
    if shape["hidden"] // shape["heads"] != shape["head_dim"]:
        metadata.append(("qwen2.attention.key_length", "u32", shape["head_dim"]))
    data, _, _ = build_gguf(32, metadata, [(name, kind, list(dims), raw.tobytes()) for name, kind, dims, raw in tensors])
    path.write_bytes(data)
    return {name: (raw.view(np.float32) if name.endswith(".bias") else raw) for name, _, _, raw in tensors}


def alone(shape, element, tensors, prompt, count, elements=None):
    """The oracle's greedy answer to one prompt: fed token by token, then `count` choices."""
    ref = oracle.Model(shape, element, tensors, batch=1, context=CONTEXT, elements=elements)
    margins = []
    for at, token in enumerate(prompt):
        logits, chosen = ref.forward([token], 1, [at])
    out = []
    for step in range(count):
        top = np.sort(logits[0])[-2:]
        margins.append(top[1] - top[0])
        out.append(int(chosen[0]))
        if step + 1 < count:
            logits, chosen = ref.forward([out[-1]], 1, [len(prompt) + step])
    return out, min(margins)


def run(batch, wanted):
    """Steps until every plane of `wanted` {slot: count} has emitted its count."""
    got = {slot: [] for slot in wanted}
    for _ in range(400):
        for slot, token in batch.step():
            if slot in wanted and len(got[slot]) < wanted[slot]:
                got[slot].append(token)
        if all(len(got[slot]) >= wanted[slot] for slot in wanted):
            return got
    raise AssertionError("the batch never answered")


@pytest.fixture(scope="module")
def runtime():
    held = host.Runtime(0)
    yield held
    held.close()


@pytest.mark.parametrize("shape,element,chunks", [(SHAPE, NH_Q8_0, [16, 4]), (SHAPE_Q4, NH_Q4_K, [16, 4]), (SHAPE, NH_Q8_0, [])])
def test_a_batched_sequence_answers_as_it_does_alone(runtime, tmp_path, shape, element, chunks):
    tensors = qwen2_gguf(tmp_path / "model.gguf", shape, element, seed=11)
    archive = host.GgufFile.open(tmp_path / "model.gguf")
    batch = host.Batch(runtime, archive, shape["vocab"], CONTEXT, 3, chunks)
    assert archive.reads() > 0
    rng = np.random.default_rng(12)
    prompts = [list(rng.integers(0, shape["vocab"], n)) for n in (1, 23, 40)]  # no chunk, 16+4+3 single, 16+16+4+4 single
    slots = [batch.admit(prompt) for prompt in prompts]
    assert slots == [0, 1, 2] and batch.active() == [0, 1, 2]
    got = run(batch, {slot: 8 for slot in slots})
    for slot, prompt in zip(slots, prompts):
        want, margin = alone(shape, element, tensors, prompt, 8)
        assert got[slot] == want, (slot, margin)
    batch.close()
    archive.close()


MIXED_FILES = {
    # the way Q4_K_M files of Qwen2 checkpoints come: q6_k for the head, some value and down projections; biases on q, k, v
    "q4_k_m": (NH_Q4_K, {"output.weight": NH_Q6_K, "blk.0.attn_v.weight": NH_Q6_K, "blk.1.ffn_down.weight": NH_Q6_K}),
    # and Q3_K_M files: q3_k for most, q5_k and q4_k for some projections, a q6_k head
    "q3_k_m": (NH_Q3_K, {"output.weight": NH_Q6_K, "blk.0.attn_v.weight": NH_Q5_K, "blk.1.ffn_down.weight": NH_Q5_K, "blk.1.attn_output.weight": NH_Q4_K}),
}


@pytest.mark.parametrize("kind", sorted(MIXED_FILES))
def test_a_file_of_mixed_storage_with_projection_biases_generates(runtime, tmp_path, kind):
    shape = SHAPE_Q4
    base, mixed = MIXED_FILES[kind]
    tensors = qwen2_gguf(tmp_path / "model.gguf", shape, base, seed=31, elements=mixed, biases=(0, 1))
    archive = host.GgufFile.open(tmp_path / "model.gguf")
    batch = host.Batch(runtime, archive, shape["vocab"], CONTEXT, 2, [16])
    rng = np.random.default_rng(32)
    prompts = [list(rng.integers(0, shape["vocab"], n)) for n in (5, 21)]
    slots = [batch.admit(prompt) for prompt in prompts]
    got = run(batch, {slot: 6 for slot in slots})
    for slot, prompt in zip(slots, prompts):
        want, margin = alone(shape, base, tensors, prompt, 6, elements=mixed)
        assert got[slot] == want, (slot, margin)
    batch.close()
    archive.close()


def test_a_batch_keeps_the_planes_it_is_told_to(runtime, tmp_path):
    shape, element = SHAPE, NH_Q8_0
    tensors = qwen2_gguf(tmp_path / "model.gguf", shape, element, seed=21)
    archive = host.Gguf.decode((tmp_path / "model.gguf").read_bytes())
    batch = host.Batch(runtime, archive, shape["vocab"], CONTEXT, 2, [8])
    assert batch.step() == [] and batch.active() == [] and batch.cursor(0) is None
    first, second = [5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15], [3, 1, 4]
    assert batch.admit(first) == 0 and batch.admit(second) == 1
    with pytest.raises(host.Panic, match="all 2 planes of this batch hold a sequence"):
        batch.admit([1])
    with pytest.raises(host.Panic, match="still holds 11 prompt tokens"):
        batch.suspend(0)
    with pytest.raises(host.Panic, match="resumes only after it is suspended"):
        batch.resume(0, [1])
    with pytest.raises(host.Panic, match="at least one token"):
        batch.restart(0, [])
    with pytest.raises(host.Panic, match="the prompt holds 96 tokens where this batch holds 96 of context"):
        batch.restart(0, [1] * 96)
    batch.restart(0, first)
    # step 1: plane 0 fills 8 rows then feeds one more; plane 1 feeds its first token
    assert batch.step() == []
    assert batch.cursor(0) == 9 and batch.cursor(1) == 1 and batch.remaining(0) == CONTEXT - 9
    got = run(batch, {0: 3, 1: 3})
    want0, _ = alone(shape, element, tensors, first, 3)
    want1, _ = alone(shape, element, tensors, second, 3)
    assert got[0] == want0 and got[1] == want1
    # a suspended plane stands still while the other goes on, and answers on as if it never had
    # (crates/neura-generate/src/batch.rs:1015-1054, :1107-1123)
    at = batch.cursor(1)
    batch.suspend(1)
    assert batch.active() == [0] and batch.occupied() == [0, 1]
    batch.step(), batch.step()
    assert batch.cursor(1) == at
    with pytest.raises(host.Panic, match="already suspended"):
        batch.suspend(1)
    # the sequence so far: prompt + every token fed; resuming with one more token continues it
    emitted1 = got[1]
    fed = at - len(second)           # answer tokens already fed back into plane 1
    assert fed <= len(emitted1)
    more = [17, 18]
    batch.resume(1, more)
    assert batch.active() == [0, 1]
    tail = run(batch, {1: 2})[1]
    history = second + emitted1[:fed] + more
    want_tail, _ = alone(shape, element, tensors, history, 2)
    assert tail == want_tail
    batch.finish(0)
    assert batch.occupied() == [1] and batch.cursor(0) is None
    assert batch.admit([2, 2]) == 0
    batch.close()
    archive.close()


def test_a_model_refuses_a_gguf_of_another_architecture(runtime, tmp_path):
    data, _, _ = build_gguf(32, [("general.architecture", "string", "llama")], [])
    archive = host.Gguf.decode(data)
    with pytest.raises(host.Panic, match="names llama as its general.architecture"):
        host.Batch(runtime, archive, 10, 16, 1, [])
    data, _, _ = build_gguf(32, [("general.architecture", "string", "qwen2")], [])
    with pytest.raises(host.Panic, match="this gguf holds no qwen2.block_count"):
        host.Batch(runtime, host.Gguf.decode(data), 10, 16, 1, [])
