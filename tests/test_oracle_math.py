"""Pins the CPU oracle's arithmetic (products, norm, rope, attention, choice, decoder) against
the closed forms the reference's own tests use and independent numpy / fp64 restatements."""
import numpy as np
import pytest

import oracle
from neura_amd import synth


@pytest.mark.parametrize("element", [8, 12])
@pytest.mark.parametrize("rows", [1, 2, 4])
def test_narrow_product_is_the_references_test_definition(element, rows):
    # crates/neura-runtime/tests/runtime.rs:12-86: seeds 23 / 29, 1024 x 2048, tolerance 1e-3
    depth, columns = 2048, 256  # a 256-column slice of the reference's 1024 keeps the CPU suite short
    values = oracle.random(columns * depth, 23)
    payload = oracle.pack(element, values)
    weight = oracle.unpack(element, payload, values.size).reshape(columns, depth)
    inputs = oracle.random(rows * depth, 29).reshape(rows, depth)
    expected = np.zeros((rows, columns), dtype=np.float32)
    for step in range(depth):  # fp32 running sum over the depth, as the test's triple loop
        expected += weight[:, step][None, :] * inputs[:, step][:, None]
    got = oracle.gemv(element, payload, columns, depth, inputs)
    assert np.abs(got - expected).max() <= 1e-3
    exact = inputs.astype(np.float64) @ weight.astype(np.float64).T
    assert np.abs(got - exact).max() <= 1e-3
    wide = oracle.gemm(element, payload, columns, depth, inputs)
    assert np.array_equal(wide, expected)  # the wide oracle IS that running sum


def test_narrow_product_handles_a_depth_that_is_no_multiple_of_1024():
    rng = np.random.default_rng(11)
    for element, depth in ((8, 896), (8, 4864), (12, 1536), (12, 3584), (12, 8960)):
        raw = synth.RANDOM[element](rng, 8 * depth)
        x = rng.standard_normal(depth).astype(np.float32)
        w = synth.DEQUANT[element](raw, 8 * depth).reshape(8, depth).astype(np.float64)
        exact = w @ x.astype(np.float64)
        got = oracle.gemv(element, raw, 8, depth, x)[0]
        assert np.allclose(got, exact, rtol=1e-5, atol=1e-3 * np.abs(exact).max() * 1e-2)
        assert np.array_equal(got, oracle.gemv(element, raw, 8, depth, x, threads=4)[0])  # threads keep the order


def test_rmsnorm_is_the_composed_form():
    # crates/neura-runtime/tests/norm.rs:21-26: mean(x^2), 1/sqrt(mean + eps), * w; tolerance 1e-5
    rng = np.random.default_rng(12)
    for C in (896, 1536, 3584, 100):
        x = rng.standard_normal((3, C)).astype(np.float32)
        w = rng.standard_normal(C).astype(np.float32)
        r = rng.standard_normal((3, C)).astype(np.float32)
        got, _ = oracle.rmsnorm(x, w, 1e-6)
        want = x.astype(np.float64) / np.sqrt((x.astype(np.float64) ** 2).mean(axis=1, keepdims=True) + 1e-6) * w
        assert np.abs(got - want).max() <= 1e-5 * max(1.0, np.abs(want).max())
        got, total = oracle.rmsnorm(x, w, 1e-6, residual=r)
        assert np.array_equal(total, x + r)
        v = (x + r).astype(np.float64)
        want = v / np.sqrt((v ** 2).mean(axis=1, keepdims=True) + 1e-6) * w
        assert np.abs(got - want).max() <= 1e-5 * max(1.0, np.abs(want).max())


def test_rope_is_rotate_half():
    # crates/neura-runtime/tests/runtime.rs:468-494
    rng = np.random.default_rng(13)
    for width, base, origin in ((64, 1e6, 0), (128, 1e6, 1024), (128, 10000.0, 4095), (8, 10000.0, 3)):
        x = rng.standard_normal((5, width)).astype(np.float32)
        got = oracle.rope(x, origin, base)
        half = width // 2
        pos = (origin + np.arange(5))[:, None].astype(np.float64)
        freq = np.float64(base) ** (-2.0 * np.arange(half) / width)
        angle = pos * freq
        lo, hi = x[:, :half].astype(np.float64), x[:, half:].astype(np.float64)
        want = np.concatenate([lo * np.cos(angle) - hi * np.sin(angle), hi * np.cos(angle) + lo * np.sin(angle)], axis=1)
        # fp32 angles at position p carry an error of about p * 2^-24 radians
        assert np.abs(got - want).max() <= 1e-4 + (origin + 5) * 2.0 ** -22
        assert np.allclose(np.linalg.norm(got, axis=1), np.linalg.norm(x, axis=1), rtol=1e-5)  # a rotation keeps the norm
    assert np.array_equal(oracle.rope(x, 0, 1e6)[0], x[0])  # position 0 turns nothing


@pytest.mark.parametrize("heads,kv_heads,batch,rows,keys,width,origin", [
    (4, 2, 2, 3, 12, 8, 9),      # the shape family of runtime.rs:551-619
    (14, 2, 1, 1, 70, 64, 69),
    (8, 8, 1, 5, 40, 16, 35),
    (6, 2, 2, 1, 33, 128, 20),
])
def test_attention_matches_the_f64_reference(heads, kv_heads, batch, rows, keys, width, origin):
    rng = np.random.default_rng(17)
    q = rng.standard_normal((heads, batch, rows, width)).astype(np.float32)
    K = rng.standard_normal((kv_heads, batch, keys, width)).astype(np.float32)
    V = rng.standard_normal((kv_heads, batch, keys, width)).astype(np.float32)
    scale = 1.0 / np.sqrt(width)
    want = oracle.attention_f64(q, K, V, kv_heads, origin, True, scale)
    got = oracle.attention(q, K, V, kv_heads, keys, keys, [origin] * batch, scale)
    assert np.abs(got - want).max() <= 1e-5
    # independent numpy check of the fp64 reference itself on one plane
    groups = heads // kv_heads
    h, b, r = heads - 1, batch - 1, rows - 1
    s = (K[h // groups, b].astype(np.float64) @ q[h, b, r].astype(np.float64)) * scale
    s[np.arange(keys) > origin + r] = -np.inf
    p = np.exp(s - s.max())
    p /= p.sum()
    assert np.abs(want[h, b, r] - p @ V[h // groups, b].astype(np.float64)).max() <= 1e-6
    # fp16 cache: same numbers once K and V are rounded to half
    K16, V16 = K.astype(np.float16), V.astype(np.float16)
    want16 = oracle.attention_f64(q, K16.astype(np.float32), V16.astype(np.float32), kv_heads, origin, True, scale)
    got16 = oracle.attention(q, K16.view(np.uint16), V16.view(np.uint16), kv_heads, keys, keys, [origin] * batch, scale)
    assert np.abs(got16 - want16).max() <= 1e-5


def test_attention_over_equal_scores_is_the_running_mean_of_the_values():
    # crates/neura-runtime/tests/runtime.rs:813-875: all-zero q -> mean of the visible V rows
    rng = np.random.default_rng(19)
    V = rng.standard_normal((2, 1, 10, 8)).astype(np.float32)
    q = np.zeros((4, 1, 1, 8), dtype=np.float32)
    for origin in (0, 3, 9):
        got = oracle.attention(q, np.zeros_like(V), V, 2, 10, 10, [origin], 0.35)
        for head in range(4):
            assert np.allclose(got[head, 0, 0], V[head // 2, 0, : origin + 1].mean(axis=0), atol=1e-6)


@pytest.mark.parametrize("half", [False, True])
def test_a_ring_weighs_the_last_window_of_keys(half):
    # crates/neura-decoder/tests/cache.rs:11-51: equal scores, value = step -> the mean of the last WINDOW steps
    WINDOW, CAPACITY, WIDTH = 5, 7, 2
    K = np.zeros((1, 1, CAPACITY, WIDTH), dtype=np.float32)
    V = np.zeros((1, 1, CAPACITY, WIDTH), dtype=np.float32)
    q = np.array([1.0, 0.0], dtype=np.float32).reshape(1, 1, 1, WIDTH)
    for step in range(2 * WINDOW + 3):
        K[0, 0, step % WINDOW] = [1.0, 0.0]
        V[0, 0, step % WINDOW] = [float(step), 0.0]
        if half:
            got = oracle.attention(q, K.astype(np.float16).view(np.uint16), V.astype(np.float16).view(np.uint16), 1, CAPACITY, WINDOW, [step], 1.0, reach=WINDOW)
        else:
            got = oracle.attention(q, K, V, 1, CAPACITY, WINDOW, [step], 1.0, reach=WINDOW)
        first = max(0, step - (WINDOW - 1))
        expected = sum(range(first, step + 1)) / (step - first + 1)
        assert abs(got[0, 0, 0, 0] - expected) < 1e-5 and got[0, 0, 0, 1] == 0.0, (step, got)


def test_a_ring_equals_attention_over_the_positions_it_still_holds():
    # An independent reading of the ring: keep every position ever written; the query at position p weighs positions
    # p - reach + 1 .. p that no later row of the same chunk has overwritten (position j leaves when j + window is written).
    rng = np.random.default_rng(31)
    heads, kv_heads, width, window, capacity = 4, 2, 8, 6, 9
    scale = 1.0 / np.sqrt(width)
    K = np.zeros((kv_heads, 1, capacity, width), dtype=np.float32)
    V = np.zeros_like(K)
    history_k, history_v = [], []
    origin = 0
    for rows in (1, 3, 2, 6, 1, 1, 4, 5, 2):
        k = rng.standard_normal((kv_heads, rows, width)).astype(np.float32)
        v = rng.standard_normal((kv_heads, rows, width)).astype(np.float32)
        q = rng.standard_normal((heads, 1, rows, width)).astype(np.float32)
        for row in range(rows):
            K[:, 0, (origin + row) % window] = k[:, row]
            V[:, 0, (origin + row) % window] = v[:, row]
            history_k.append(k[:, row])
            history_v.append(v[:, row])
        got = oracle.attention(q, K, V, kv_heads, capacity, window, [origin], scale, reach=window)
        written = origin + rows
        for head in range(heads):
            for row in range(rows):
                position = origin + row
                seen = [j for j in range(max(0, position - window + 1), position + 1) if j + window >= written]
                keys = np.array([history_k[j][head // 2] for j in seen], dtype=np.float64)
                values = np.array([history_v[j][head // 2] for j in seen], dtype=np.float64)
                scores = keys @ q[head, 0, row].astype(np.float64) * scale
                weights = np.exp(scores - scores.max())
                want = (weights / weights.sum()) @ values
                assert np.abs(got[head, 0, row] - want).max() <= 1e-5, (origin, rows, head, row)
        origin += rows


def test_argmax_breaks_ties_toward_the_lowest_index():
    assert oracle.argmax([1.0, 3.0, 3.0, 2.0]) == 1
    assert oracle.argmax([5.0]) == 0
    assert oracle.argmax([-np.inf, -np.inf]) == 0
    rng = np.random.default_rng(23)
    values = rng.integers(0, 50, 10000).astype(np.float32)
    assert oracle.argmax(values) == int(np.argmax(values))


def numpy_decoder(shape, element, tensors, tokens, cursor, layers, context, rope_base=1e6, eps=1e-6):
    """An independent fp64 forward pass of one token per plane against an EMPTY cache history
    of `cursor` zero keys (what a fresh cache holds), for pinning the oracle's composition."""
    H, hd = shape["hidden"], shape["head_dim"]
    heads, kvh, F = shape["heads"], shape["kv_heads"], shape["ffn"]

    def mat(name, rows, cols):
        return synth.DEQUANT[element](tensors[name], rows * cols).reshape(rows, cols).astype(np.float64)

    def vec(name):
        return np.asarray(tensors[name]).view(np.float32).astype(np.float64)

    def rms(x, w):
        return x / np.sqrt((x * x).mean() + eps) * w

    def rope(x, position):
        half = hd // 2
        freq = np.float64(rope_base) ** (-2.0 * np.arange(half) / hd)
        a = position * freq
        lo, hi = x[:half], x[half:]
        return np.concatenate([lo * np.cos(a) - hi * np.sin(a), hi * np.cos(a) + lo * np.sin(a)])

    E = mat("token_embd.weight", shape["vocab"], H)
    out = []
    for token, position in zip(tokens, cursor):
        h = E[token].copy()
        for L in range(layers):
            p = "blk.%d." % L
            xn = rms(h, vec(p + "attn_norm.weight"))
            q = mat(p + "attn_q.weight", heads * hd, H) @ xn
            k = mat(p + "attn_k.weight", kvh * hd, H) @ xn
            v = mat(p + "attn_v.weight", kvh * hd, H) @ xn
            att = np.zeros(heads * hd)
            for head in range(heads):
                g = head // (heads // kvh)
                qh = rope(q[head * hd:(head + 1) * hd], position)
                kh = rope(k[g * hd:(g + 1) * hd], position).astype(np.float16).astype(np.float64)
                vh = v[g * hd:(g + 1) * hd].astype(np.float16).astype(np.float64)
                # `position` zero keys (score 0, value 0) then this key
                s = np.concatenate([np.zeros(position), [qh @ kh / np.sqrt(hd)]])
                w = np.exp(s - s.max())
                w /= w.sum()
                att[head * hd:(head + 1) * hd] = w[-1] * vh
            h = h + mat(p + "attn_output.weight", H, heads * hd) @ att
            xn = rms(h, vec(p + "ffn_norm.weight"))
            g_ = mat(p + "ffn_gate.weight", F, H) @ xn
            u = mat(p + "ffn_up.weight", F, H) @ xn
            h = h + mat(p + "ffn_down.weight", H, F) @ (g_ / (1 + np.exp(-g_)) * u)
        head_w = mat("output.weight", shape["vocab"], H) if "output.weight" in tensors else E
        out.append(head_w @ rms(h, vec("output_norm.weight")))
    return np.array(out)


TINY = dict(layers=2, hidden=256, heads=4, kv_heads=2, head_dim=64, ffn=512, vocab=320, tied=True)


@pytest.mark.parametrize("element,tied", [(8, True), (12, False)])
def test_decoder_step_matches_an_independent_numpy_forward(element, tied):
    shape = dict(TINY, tied=tied)
    rng = np.random.default_rng(29)
    tensors = {name: raw for name, _, _, raw in synth.model_tensors(shape, element, rng, mode="normal")}
    model = oracle.Model(shape, element, tensors, batch=2, context=16)
    tokens, cursor = [5, 319], [0, 7]
    logits, chosen = model.forward(tokens, 1, cursor)
    want = numpy_decoder(shape, element, tensors, tokens, cursor, shape["layers"], 16)
    assert np.abs(logits - want).max() <= 2e-4 * max(1.0, np.abs(want).max())
    assert list(chosen) == [int(np.argmax(row)) for row in logits]
    # the new key landed in the cache at its cursor, as fp16
    hd = shape["head_dim"]
    k = model.cache_k[0].reshape(shape["kv_heads"], 2, model.capacity, hd)
    assert np.any(k[0, 0, 0] != 0) and np.any(k[0, 1, 7] != 0) and not np.any(k[0, 0, 1]) and not np.any(k[0, 1, 6])


def test_decoder_chunked_fill_equals_token_by_token():
    # crates/neura-generate/tests/generation.rs:458-470: chunked prefill == unchunked
    shape = TINY
    rng = np.random.default_rng(31)
    tensors = {name: raw for name, _, _, raw in synth.model_tensors(shape, 8, rng, mode="normal")}
    prompt = rng.integers(0, shape["vocab"], 6)
    one = oracle.Model(shape, 8, tensors, batch=1, context=16, max_rows=4)
    for at, token in enumerate(prompt):
        logits_one, _ = one.forward([token], 1, [at])
    two = oracle.Model(shape, 8, tensors, batch=1, context=16, max_rows=4)
    two.forward(prompt[:4], 4, [0], want_logits=False)
    two.forward(prompt[4:5], 1, [4])
    logits_two, _ = two.forward(prompt[5:6], 1, [5])
    assert np.abs(logits_one - logits_two).max() <= 1e-4
    for a, b in zip(one.cache_k, two.cache_k):
        ka = oracle.f16_to_f32(a).reshape(-1)
        kb = oracle.f16_to_f32(b).reshape(-1)
        assert np.abs(ka - kb).max() <= 2e-3


def test_decoder_inactive_plane_writes_scratch_rows_only():
    shape = TINY
    rng = np.random.default_rng(37)
    tensors = {name: raw for name, _, _, raw in synth.model_tensors(shape, 8, rng, mode="normal")}
    both = oracle.Model(shape, 8, tensors, batch=2, context=8, max_rows=1)
    logits, _ = both.forward([3, 4], 1, [2, 0], mask=[1, 0])
    alone = oracle.Model(shape, 8, tensors, batch=1, context=8, max_rows=1)
    logits_alone, _ = alone.forward([3], 1, [2])
    assert np.array_equal(logits[0], logits_alone[0])  # batched == alone (generation.rs:365-377)
    k = both.cache_k[0].reshape(shape["kv_heads"], 2, both.capacity, shape["head_dim"])
    assert not np.any(k[:, 1, :8])       # the window of the inactive plane is untouched
    assert np.any(k[:, 0, 2])
