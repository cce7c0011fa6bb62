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


def alone(shape, element, tensors, prompt, count, elements=None, window=None, cache_element=1):
    """The oracle's greedy answer to one prompt: fed token by token, then `count` choices."""
    ref = oracle.Model(shape, element, tensors, batch=1, context=CONTEXT, elements=elements, window=window, cache_element=cache_element)
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


@pytest.mark.parametrize("cache,dtype", [(0, np.float32), (30, None)], ids=["single", "bfloat16"])
def test_a_batch_keeps_its_states_in_the_element_it_is_given(runtime, tmp_path, cache, dtype):
    """The model function hands its caches an element (examples/qwen/main.rs:107 keeps single precision states): a batch over such
    a model answers as the oracle with the same states does, and its state file holds them in that element."""
    from safetensors.numpy import load_file

    shape, element = SHAPE, NH_Q8_0
    tensors = qwen2_gguf(tmp_path / "model.gguf", shape, element, seed=71)
    archive = host.GgufFile.open(tmp_path / "model.gguf")
    batch = host.Batch(runtime, archive, shape["vocab"], CONTEXT, 2, [8], cache=cache)
    rng = np.random.default_rng(72)
    prompts = [list(rng.integers(0, shape["vocab"], n)) for n in (5, 21)]
    slots = [batch.admit(prompt) for prompt in prompts]
    got = run(batch, {slot: 6 for slot in slots})
    for slot, prompt in zip(slots, prompts):
        want, margin = alone(shape, element, tensors, prompt, 6, cache_element=cache)
        assert got[slot] == want, (slot, margin)
    batch.save_state(tmp_path / "state.safetensors")
    raw = open(tmp_path / "state.safetensors", "rb").read()
    assert (b'"dtype":"F32"' if cache == 0 else b'"dtype":"BF16"') in raw
    if dtype is not None:  # numpy holds no bfloat16: the single precision file is opened by the package, the other by its header
        held = load_file(str(tmp_path / "state.safetensors"))
        assert all(tensor.dtype == dtype and tensor.shape == (shape["kv_heads"], 2, CONTEXT + 8, shape["head_dim"]) for tensor in held.values())
        assert held["blk.1.cache.key"][:, 1, :20].any()
    second = host.Batch(runtime, archive, shape["vocab"], CONTEXT, 2, [8], cache=cache)
    second.restore_state(tmp_path / "state.safetensors", batch.snapshot())
    assert run(second, {0: 4, 1: 4}) == run(batch, {0: 4, 1: 4})
    other = host.Batch(runtime, archive, shape["vocab"], CONTEXT, 2, [8])
    with pytest.raises(host.Panic, match="is not in half storage"):
        other.restore_state(tmp_path / "state.safetensors", batch.snapshot())
    with pytest.raises(host.Panic, match="single, half or bfloat16"):
        host.Batch(runtime, archive, shape["vocab"], CONTEXT, 2, [8], cache=8)
    for held_batch in (batch, second, other):
        held_batch.close()
    archive.close()


@pytest.mark.parametrize("chunks", [[], [8, 4]])
def test_a_batch_keeps_only_the_window_of_tokens_it_declares(runtime, tmp_path, chunks):
    """crates/neura-generate/tests/generation.rs:521-560 on the real decoder: a batch of a 10 token window answers as the
    oracle's ring of 10 does, alone or beside another plane, with prompts longer than the window (the fill wraps)."""
    WINDOW = 10
    tensors = qwen2_gguf(tmp_path / "model.gguf", SHAPE, NH_Q8_0, seed=21)
    archive = host.GgufFile.open(tmp_path / "model.gguf")
    batch = host.Batch(runtime, archive, SHAPE["vocab"], CONTEXT, 2, chunks, window=WINDOW)
    assert batch.window() == WINDOW
    rng = np.random.default_rng(22)
    prompts = [list(rng.integers(0, SHAPE["vocab"], n)) for n in (27, 5)]
    slots = [batch.admit(prompt) for prompt in prompts]
    got = run(batch, {slot: 14 for slot in slots})
    for slot, prompt in zip(slots, prompts):
        want, margin = alone(SHAPE, NH_Q8_0, tensors, prompt, 14, window=WINDOW)
        assert got[slot] == want, (slot, margin)
    unbounded, _ = alone(SHAPE, NH_Q8_0, tensors, prompts[0], 14)
    assert unbounded != got[slots[0]]  # the window is felt: 27 prompt tokens in, only 10 are weighed
    batch.close()
    archive.close()
    with pytest.raises(host.Panic) as refused:  # batch.rs:149, :315-322
        host.batch_spec_check(16, 1, [], window=0)
    assert "a batch keeps a window of no token" in str(refused.value)
    with pytest.raises(host.Panic) as refused:
        host.batch_spec_check(16, 1, [], window=17)
    assert "a batch keeps a window of 17 tokens over a context of 16" in str(refused.value)
    with pytest.raises(host.Panic) as refused:
        host.batch_spec_check(16, 1, [8, 4], window=6)
    assert "a batch fills chunks of 8 rows into a window of 6 tokens" in str(refused.value)


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


def test_a_sampled_batch_draws_by_plane_seeds_the_host_can_write(runtime, tmp_path):
    """BatchSpec::sampled: every plane draws with its own seed (plane_seed of the batch seed, one further per draw),
    temperature, candidate count and nucleus (crates/neura-generate/src/batch.rs:643-732, :829-864, :1688-1709).  Each
    emitted token is checked against the oracle's draw from the logits the device answered with one step earlier."""
    shape, element = SHAPE, NH_Q8_0
    qwen2_gguf(tmp_path / "model.gguf", shape, element, seed=41)
    archive = host.GgufFile.open(tmp_path / "model.gguf")
    batch = host.Batch(runtime, archive, shape["vocab"], CONTEXT, 2, [8], sampling=(0.9, 40, 0.95))
    assert [batch.seed_of(slot) for slot in range(2)] == [host.plane_seed(0, slot) for slot in range(2)]
    batch.set_seed(1234)
    batch.set_temperature(1.4, slot=1)
    batch.set_cumulative(0.8, slot=1)
    batch.set_keep(17, slot=1)
    settings = [(0.9, 40, 0.95), (1.4, 17, 0.8)]
    rng = np.random.default_rng(42)
    prompts = [list(rng.integers(0, shape["vocab"], n)) for n in (3, 12)]
    slots = [batch.admit(prompt) for prompt in prompts]
    draws = [0, 0]
    pending = {}  # slot -> the token the oracle expects the plane to emit next
    emitted = {0: [], 1: []}
    for step in range(30):
        before = [batch.seed_of(slot) for slot in slots]
        out = batch.step()
        for slot, token in out:
            assert token == pending[slot], (step, slot)
            emitted[slot].append(token)
        logits = batch.logits()
        for slot in slots:
            if batch.seed_of(slot) != before[slot]:  # the plane drew on this step
                assert batch.seed_of(slot) == (before[slot] + 1) & 0xFFFFFFFF
                assert before[slot] == (host.plane_seed(1234, slot) + draws[slot]) & 0xFFFFFFFF
                draws[slot] += 1
                temperature, keep, cumulative = settings[slot]
                pending[slot] = int(oracle.sample(logits[slot:slot + 1], oracle.draws([(host.seed_bits(before[slot]), temperature, keep, cumulative)]))[0])
    assert len(emitted[0]) >= 20 and len(emitted[1]) >= 15
    assert len(set(emitted[0])) > 3  # a temperature near one spreads the answers of a random-init decoder
    batch.close()

    # the same seed answers the same; another seed answers otherwise
    streams = []
    for seed in (1234, 1234, 99):
        again = host.Batch(runtime, archive, shape["vocab"], CONTEXT, 2, [8], sampling=(0.9, 40, 0.95))
        again.set_seed(seed)
        again.set_temperature(1.4, slot=1), again.set_cumulative(0.8, slot=1), again.set_keep(17, slot=1)
        for prompt in prompts:
            again.admit(prompt)
        streams.append(run(again, {0: 20, 1: 15}))
        again.close()
    assert streams[0] == {0: emitted[0][:20], 1: emitted[1][:15]} == streams[1]
    assert streams[2] != streams[0]
    archive.close()


def test_a_temperature_and_a_candidate_count_the_host_writes_steer_the_draws(runtime, tmp_path):
    # crates/neura-generate/tests/generation.rs:564-627 and the test after it, on a decoder instead of constant logits
    shape, element = SHAPE, NH_Q8_0
    tensors = qwen2_gguf(tmp_path / "model.gguf", shape, element, seed=43)
    archive = host.GgufFile.open(tmp_path / "model.gguf")
    prompt = [5, 9, 2, 77]
    greedy, margin = alone(shape, element, tensors, prompt, 12)
    batch = host.Batch(runtime, archive, shape["vocab"], CONTEXT, 2, [], sampling=(1.0, 64, 1.0))
    batch.set_temperature(1e-4)  # logits 10^4 apart leave the noise nothing to move
    batch.admit(prompt), batch.admit(prompt)
    assert run(batch, {0: 12, 1: 12}) == {0: greedy, 1: greedy}, margin
    # plane 0 hot, plane 1 keeping one candidate: the one stays greedy while the other spreads
    batch.restart(0, prompt), batch.restart(1, prompt)
    batch.set_temperature(1000.0)
    batch.set_keep(1, slot=1)
    got = run(batch, {0: 40, 1: 12})
    assert got[1] == greedy, margin
    assert len(set(got[0])) > 10 and got[0][:12] != greedy
    with pytest.raises(host.Panic, match="a batch of 2 planes names no plane 2"):
        batch.set_keep(3, slot=2)
    with pytest.raises(host.Panic, match="a batch keeps 65 candidates where a row holds between one and 64"):
        batch.set_keep(65)
    with pytest.raises(host.Panic, match="a sampling temperature of 0 spreads no logits"):
        batch.set_temperature(0.0)
    with pytest.raises(host.Panic, match="a cumulative mass of 2 keeps no candidate"):
        batch.set_cumulative(2.0)
    batch.close()
    plain = host.Batch(runtime, archive, shape["vocab"], CONTEXT, 1, [])
    for refused, sentence in ((lambda: plain.set_temperature(1.0), "a greedy batch draws no temperature"), (lambda: plain.set_keep(4), "a greedy batch draws no candidate count"),
                              (lambda: plain.set_cumulative(0.5), "a greedy batch draws no cumulative mass"), (lambda: plain.set_seed(1), "a greedy batch draws no seed"),
                              (lambda: plain.seed_of(0), "a greedy batch draws no seed")):
        with pytest.raises(host.Panic, match=sentence):
            refused()
    plain.close()
    archive.close()


@pytest.mark.parametrize("sampling", [None, (0.9, 40, 0.95)], ids=["greedy", "sampled"])
def test_a_batch_restored_from_its_snapshot_and_state_file_answers_on(runtime, tmp_path, sampling):
    """Batch::snapshot + save_state, then restore_state into another batch (crates/neura-generate/src/batch.rs:484-628):
    the second batch goes on with the tokens the first would have answered with.  The state file is a container any
    safetensors reader opens; its tensors are the caches as the C ABI reads them."""
    from safetensors.numpy import load_file

    shape, element = SHAPE, NH_Q8_0
    qwen2_gguf(tmp_path / "model.gguf", shape, element, seed=51)
    archive = host.GgufFile.open(tmp_path / "model.gguf")
    first = host.Batch(runtime, archive, shape["vocab"], CONTEXT, 3, [8], sampling=sampling)
    if sampling:
        first.set_seed(77)
        first.set_temperature(1.3, slot=2)
    rng = np.random.default_rng(52)
    prompts = [list(rng.integers(0, shape["vocab"], n)) for n in (4, 30)]
    for prompt in prompts:
        first.admit(prompt)
    for _ in range(9):   # plane 0 answers already, plane 1 still feeds its prompt, plane 2 is empty
        first.step()
    first.suspend(0)
    snapshot = first.snapshot()
    assert snapshot[:4] == b"NBS1" and host.snapshot_round_trip(snapshot) == snapshot
    first.save_state(tmp_path / "state.safetensors")
    held = load_file(str(tmp_path / "state.safetensors"))
    capacity = CONTEXT + 8
    assert sorted(held) == sorted("blk.%d.cache.%s" % (layer, which) for layer in range(shape["layers"]) for which in ("key", "value"))
    assert all(tensor.dtype == np.float16 and tensor.shape == (shape["kv_heads"], 3, capacity, shape["head_dim"]) for tensor in held.values())
    assert np.abs(held["blk.1.cache.key"][:, 1, :20].astype(np.float32)).max() > 0  # plane 1 has written twenty-odd keys
    assert not held["blk.1.cache.key"][:, 2].any()                                    # plane 2 none

    second = host.Batch(runtime, archive, shape["vocab"], CONTEXT, 3, [8], sampling=sampling)
    second.restore_state(tmp_path / "state.safetensors", snapshot)
    assert second.active() == [1] and second.occupied() == [0, 1]
    assert [second.cursor(slot) for slot in range(3)] == [first.cursor(slot) for slot in range(3)]
    if sampling:
        assert [second.seed_of(slot) for slot in range(3)] == [first.seed_of(slot) for slot in range(3)]
    for batch in (first, second):
        batch.resume(0, [3, 1, 4])
    want = run(first, {0: 10, 1: 10})
    assert run(second, {0: 10, 1: 10}) == want
    # a batch of another shape refuses the snapshot, and a file that misses a state is refused
    other = host.Batch(runtime, archive, shape["vocab"], CONTEXT, 2, [8], sampling=sampling)
    with pytest.raises(host.Panic, match="a batch of 2 planes restores a snapshot of 3 planes"):
        other.restore(snapshot)
    if sampling is None:
        drawing = host.Batch(runtime, archive, shape["vocab"], CONTEXT, 3, [8], sampling=(1.0, 4, 1.0))
        with pytest.raises(host.Panic, match="a batch draws true restores a snapshot of a batch that draws false"):
            drawing.restore(snapshot)
        drawing.close()
    for batch in (first, second, other):
        batch.close()
    archive.close()


@pytest.mark.parametrize("chunks", [[], [4, 2]])
@pytest.mark.parametrize("sampling", [None, (1.0, 4, 1.0)], ids=["greedy", "sampled"])
def test_a_batch_reuses_the_prefix_its_planes_share(runtime, tmp_path, chunks, sampling):
    """crates/neura-generate/tests/generation.rs:379-405: two prompts that start alike answer the same whether each feeds its
    whole prompt or the batch keeps their common start as a shared prefix (fed once, copied into a plane as it starts);
    the greedy answers are also the oracle's answers to the whole prompts."""
    shape, element = SHAPE, NH_Q8_0
    tensors = qwen2_gguf(tmp_path / "model.gguf", shape, element, seed=61)
    archive = host.GgufFile.open(tmp_path / "model.gguf")
    rng = np.random.default_rng(62)
    common = list(rng.integers(0, shape["vocab"], 7))
    prompts = [common + list(rng.integers(0, shape["vocab"], n)) for n in (3, 5)]

    def batched(prefix):
        batch = host.Batch(runtime, archive, shape["vocab"], CONTEXT, 2, chunks, sampling=sampling, shared=prefix is not None)
        if prefix is not None:
            batch.prefix(prefix)
            batch.prefix(prefix)  # the prefix it already keeps: nothing to do (batch.rs:913-915)
        slots = [batch.admit(prompt) for prompt in prompts]
        if prefix is not None:
            assert [batch.cursor(slot) for slot in slots] == [len(prefix)] * 2
        got = run(batch, {slot: 6 for slot in slots})
        batch.close()
        return [got[slot] for slot in slots]

    plain = batched(None)
    assert batched(common) == plain
    if sampling is None:
        assert plain == [alone(shape, element, tensors, prompt, 6)[0] for prompt in prompts]
    archive.close()


def test_a_shared_prefix_is_refused_where_the_reference_refuses_it_and_travels_in_a_state_file(runtime, tmp_path):
    from safetensors.numpy import load_file

    shape, element = SHAPE, NH_Q8_0
    qwen2_gguf(tmp_path / "model.gguf", shape, element, seed=63)
    archive = host.GgufFile.open(tmp_path / "model.gguf")
    rng = np.random.default_rng(64)
    common = list(rng.integers(0, shape["vocab"], 9))
    plain = host.Batch(runtime, archive, shape["vocab"], CONTEXT, 2, [4])
    with pytest.raises(host.Panic, match="a batch fills a shared prefix only when it declares one"):  # batch.rs:895-898
        plain.prefix(common)
    plain.close()
    first = host.Batch(runtime, archive, shape["vocab"], CONTEXT, 3, [4], shared=True)
    with pytest.raises(host.Panic, match="a shared prefix holds at least one token"):
        first.prefix([])
    with pytest.raises(host.Panic, match="a shared prefix holds 96 tokens where this batch holds 96 of context"):
        first.prefix([1] * CONTEXT)
    first.prefix(common)
    with pytest.raises(host.Panic, match="a batch shares a prefix of 9 tokens, and this prompt does not start with it"):  # batch.rs:1078-1082
        first.admit([common[0] + 1] + common[1:] + [5])
    with pytest.raises(host.Panic, match="a prompt of 9 tokens holds no token after the shared prefix of 9 tokens"):
        first.admit(common)
    first.admit(common + [5, 6, 7])
    with pytest.raises(host.Panic, match="a batch fills a shared prefix while no plane holds a sequence"):  # batch.rs:899-902
        first.prefix(common + [1])
    first.admit(common + [8])
    for _ in range(5):
        first.step()
    # the prefix and the shared plane travel with the snapshot and the state file
    snapshot = first.snapshot()
    assert host.snapshot_round_trip(snapshot) == snapshot
    first.save_state(tmp_path / "state.safetensors")
    held = load_file(str(tmp_path / "state.safetensors"))
    assert sorted(held) == sorted("blk.%d.cache.%s%s" % (layer, shared, which) for layer in range(shape["layers"]) for shared in ("", "shared.")
                                  for which in ("key", "value"))
    capacity = CONTEXT + 4
    assert held["blk.0.cache.shared.key"].shape == (shape["kv_heads"], 1, capacity, shape["head_dim"])
    assert held["blk.1.cache.shared.value"][:, 0, :9].any() and not held["blk.1.cache.shared.value"][:, 0, 9:].any()
    assert np.array_equal(held["blk.1.cache.key"][:, 1, :9], held["blk.1.cache.shared.key"][:, 0, :9])  # a plane started from it
    second = host.Batch(runtime, archive, shape["vocab"], CONTEXT, 3, [4], shared=True)
    second.restore_state(tmp_path / "state.safetensors", snapshot)
    for batch in (first, second):
        assert batch.admit(common + [11, 12]) == 2  # starts from the prefix the state file brought
    want = run(first, {0: 6, 1: 6, 2: 6})
    assert run(second, {0: 6, 1: 6, 2: 6}) == want
    undeclared = host.Batch(runtime, archive, shape["vocab"], CONTEXT, 3, [4])
    with pytest.raises(host.Panic, match="a snapshot holds a shared prefix where this batch declares none"):  # batch.rs:564-567
        undeclared.restore(snapshot)
    # a forgotten prefix: prompts are whole again
    second.finish(0)
    second.forget_prefix()
    assert second.admit([4, 5]) == 0 and second.cursor(0) == 0
    for batch in (first, second, undeclared):
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
