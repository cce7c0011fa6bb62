"""Pins the oracle's sampled choice (crates/neura-kernel/src/task/choice.rs:81-89, :933-989) without the reference:
the hash against a numpy restatement, the reference's own two properties (crates/neura-runtime/tests/choice.rs:41-126),
a nucleus worked by hand, and the draw frequencies against the softmax over what the nucleus keeps."""
import numpy as np

import oracle

CLASSES = 32


def noise(seed, columns):
    """-log(-log(u)) of the reference's integer mixer, in numpy"""
    m = np.uint64(0xFFFFFFFF)
    column = np.asarray(columns, dtype=np.uint64)
    key = (column * np.uint64(0x27D4EB2F)) & m
    h = (np.uint64(seed) ^ ((key * np.uint64(0x9E3779B9)) & m)) & m
    h ^= h >> np.uint64(16)
    h = (h * np.uint64(0x7FEB352D)) & m
    h ^= h >> np.uint64(15)
    h = (h * np.uint64(0x846CA68B)) & m
    h ^= h >> np.uint64(16)
    u = (h >> np.uint64(8)).astype(np.float32) * np.float32(1.0 / 16777216.0)
    with np.errstate(divide="ignore"):
        return -np.log(-np.log(u.astype(np.float64)))


def test_gumbel_noise_is_the_closed_form():
    for seed in (0, 1, 0x2F0F1A3B, 0x91E10D57, 0xFFFFFFFF):
        columns = np.array([0, 1, 2, 31, 151935, 152063, 2 ** 24 + 5], dtype=np.uint32)
        want = noise(seed, columns)
        got = np.array([oracle.lib().oracle_gumbel_noise(seed, int(c)) for c in columns])
        finite = np.isfinite(want)
        assert np.allclose(got[finite], want[finite], rtol=2e-6, atol=2e-6)
    # uniform numbers: the mean of -log(-log(u)) over many columns is Euler's constant, its variance pi^2 / 6
    drawn = np.array([oracle.lib().oracle_gumbel_noise(12345, c) for c in range(200000)])
    drawn = drawn[np.isfinite(drawn)]
    assert abs(drawn.mean() - 0.5772) < 0.01 and abs(drawn.var() - np.pi ** 2 / 6) < 0.03


def test_a_nucleus_that_keeps_one_candidate_draws_the_argmax():
    # crates/neura-runtime/tests/choice.rs:92-126: seed 73, 4 rows of 32, keep 1, cumulative 1, whatever the seeds
    logits = oracle.random(4 * CLASSES, 73).reshape(4, CLASSES)
    for bump in (0, 0x9E3779B9):
        seeds = [((0x3C6EF372 ^ row) + bump) & 0xFFFFFFFF for row in range(4)]
        got = oracle.sample(logits, oracle.draws([(s, 1.0, 1, 1.0) for s in seeds]))
        assert list(got) == [int(np.argmax(row)) for row in logits]
    # and keeping one candidate under any nucleus is the argmax too
    assert list(oracle.sample(logits, oracle.draws([(7, 0.7, 1, 0.3)] * 4))) == [int(np.argmax(row)) for row in logits]


def test_a_row_seed_draws_the_numbers_its_own_row_holds():
    # crates/neura-runtime/tests/choice.rs:41-90: a row draws the same column alone and beside another row
    logits = oracle.random(2 * CLASSES, 71).reshape(2, CLASSES)
    seeds = [0x2F0F1A3B, 0x91E10D57]
    alone = [int(oracle.sample(logits[row:row + 1], oracle.draws([(seeds[row], 1.0, 6, 0.85)]))[0]) for row in range(2)]
    together = oracle.sample(logits, oracle.draws([(seed, 1.0, 6, 0.85) for seed in seeds]))
    assert list(together) == alone
    swapped = oracle.sample(logits[::-1], oracle.draws([(seed, 1.0, 6, 0.85) for seed in seeds[::-1]]))
    assert list(swapped) == alone[::-1]


def test_a_nucleus_worked_by_hand():
    # probabilities 0.5, 0.25, 0.125, 0.0625, 0.0625 (logits = log p): keep 4 leaves a tail of 0.0625 outside the candidates;
    # cumulative 0.8: running + tail reaches 0.8 * total at the second candidate (0.75 + 0.0625), so two columns remain
    p = np.array([0.0625, 0.5, 0.125, 0.25, 0.0625], dtype=np.float64)
    logits = np.log(p).astype(np.float32).reshape(1, -1)
    seen = set()
    for seed in range(400):
        seen.add(int(oracle.sample(logits, oracle.draws([(seed, 1.0, 4, 0.8)]))[0]))
    assert seen == {1, 3}
    # cumulative 0.55: 0.5 + 0.0625 reaches 0.55 at the first candidate
    assert {int(oracle.sample(logits, oracle.draws([(seed, 1.0, 4, 0.55)]))[0]) for seed in range(100)} == {1}
    # cumulative 1: the boundary never closes before the last kept candidate (0.9375 + 0.0625 reaches it there): all four
    assert {int(oracle.sample(logits, oracle.draws([(seed, 1.0, 4, 1.0)]))[0]) for seed in range(2000)} == {1, 3, 2, 0}
    # equal logits rank by column: keep 4 of the five leaves out the last
    flat = np.zeros((1, 5), dtype=np.float32)
    assert {int(oracle.sample(flat, oracle.draws([(seed, 1.0, 4, 1.0)]))[0]) for seed in range(400)} == {0, 1, 2, 3}


def test_draw_frequencies_follow_the_softmax_of_the_kept_candidates():
    # Gumbel-max: the largest of logit + noise is a draw from softmax(logits); temperature divides the logits first
    rng = np.random.default_rng(5)
    logits = rng.normal(0, 1.5, (1, 12)).astype(np.float32)
    for temperature, keep in ((1.0, 12), (0.5, 12), (2.0, 5)):
        scaled = logits[0].astype(np.float64) / temperature
        kept = np.argsort(-scaled, kind="stable")[:keep]
        p = np.zeros(12)
        p[kept] = np.exp(scaled[kept] - scaled.max())
        p /= p.sum()
        draws = 20000
        chosen = np.array([int(oracle.sample(logits, oracle.draws([(seed * 2654435761 % 2 ** 32, temperature, keep, 1.0)]))[0]) for seed in range(draws)])
        counts = np.bincount(chosen, minlength=12)
        assert counts[p == 0].sum() == 0
        expected = p * draws
        chi2 = ((counts - expected) ** 2 / np.maximum(expected, 1e-9))[p > 0].sum()
        assert chi2 < 45, (temperature, keep, chi2)  # 11 degrees of freedom: 45 is far in the tail


def test_seed_plumbing_of_a_batch():
    # crates/neura-generate/src/batch.rs:1841-1847
    assert oracle.lib().oracle_plane_seed(0, 0) == 0x9E3779B9
    assert oracle.lib().oracle_plane_seed(5, 1) == 5 ^ ((2 * 0x9E3779B9) & 0xFFFFFFFF)
    for seed in (0, 1, 0x9E3779B9, 0xFFFFFFFF, 0x12345678):
        bits = oracle.lib().oracle_seed_bits(seed)
        assert bits >> 23 == 0x7F and bits & 0x7FFFFF == (seed ^ (seed >> 23)) & 0x7FFFFF
        assert 1.0 <= np.array([bits], dtype=np.uint32).view(np.float32)[0] < 2.0
