"""Writes the committed fixtures of tests/golden/ from the CPU oracle (run from the repository root):

    python tests/golden/make_fixtures.py [blocks] [config1] [kquants] [config4] [config5] [config5_blocks]

A fixture is data -- inputs and the outputs the oracle gave for them on the day it was written -- so that an oracle and a
kernel that drift together no longer agree with what is stored here.  The tests that read them:
tests/test_oracle_golden.py (CPU: the oracle against the files) and the GPU tests named below (the device against the files).

  hand_built_blocks.npz        raw blocks of every block format built from fixed byte patterns, and the float32 bit patterns
                               they unpack to                                  (test_gpu_ops.py::test_dequant_of_the_committed_blocks)
  config1_q8_0_gemv.npz/.json  BASELINE configuration 1: the first 64 rows of W, x, every output, and SHA-256 of the whole W
                               and of the outputs                              (test_gpu_ops.py::test_config1_against_the_committed_outputs)
  kquant_gemv.npz              a one-row product of Q3_K, Q4_K, Q5_K and Q6_K each (48 x 768): blocks, activations and the
                               oracle's outputs, plain and as silu(gate) * up  (test_gpu_ops.py::test_k_quant_products_against_the_committed_outputs)
  config4_greedy_ids.json      the 64 greedy ids of configuration 4            (test_gpu_decoder.py::test_config4_...)
  config5_normal_greedy_ids.json  the 64 greedy ids of the whole 7B shape with N(0, 0.02) weights packed to Q4_K
                                                                               (test_gpu_decoder.py::test_config5_full_depth_...[normal])
  config5_blocks_greedy_ids.json  the same with the benchmark's random Q4_K blocks (test_gpu_decoder.py::test_config5_full_depth_...[blocks])
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for path in (ROOT, os.path.join(ROOT, "tests")):
    if path not in sys.path:
        sys.path.insert(0, path)

import cases  # noqa: E402
import oracle  # noqa: E402

THREADS = int(os.environ.get("ORACLE_THREADS", "8"))


def blocks():
    held = {}
    for element in (cases.Q8_0, cases.Q3_K, cases.Q4_K, cases.Q5_K, cases.Q6_K):
        raw, elements = cases.hand_built_blocks(element)
        values = oracle.unpack(element, raw, elements)
        assert np.isfinite(values).all() and np.abs(values).max() > 0
        held["raw_%d" % element] = raw
        held["bits_%d" % element] = values.view(np.uint32)
    np.savez_compressed(os.path.join(HERE, "hand_built_blocks.npz"), **held)


def config1():
    N, K, raw, x = cases.config1()
    y = oracle.gemv(cases.Q8_0, raw, N, K, x, threads=THREADS)[0]
    row_bytes = raw.size // N
    np.savez_compressed(os.path.join(HERE, "config1_q8_0_gemv.npz"), w_first_64_rows=raw[: 64 * row_bytes], x=x, y_bits=y.view(np.uint32))
    with open(os.path.join(HERE, "config1_q8_0_gemv.json"), "w") as out:
        json.dump({"N": N, "K": K, "seed": 0, "w_sha256": cases.sha256(raw), "x_sha256": cases.sha256(x), "y_sha256": cases.sha256(y)}, out, indent=1)
        out.write("\n")


def kquants():
    held = {}
    for element in (cases.Q3_K, cases.Q4_K, cases.Q5_K, cases.Q6_K):
        N, K, raw, x = cases.kquant_products(element)
        y = oracle.gemv(element, raw, N, K, x, threads=THREADS)[0]
        exact = oracle.unpack(element, raw, N * K).reshape(N, K).astype(np.float64) @ x.astype(np.float64)
        assert np.abs(y - exact).max() <= 2e-5 * np.abs(exact).max()
        held["raw_%d" % element], held["x_%d" % element], held["y_bits_%d" % element] = raw, x, y.view(np.uint32)
    np.savez_compressed(os.path.join(HERE, "kquant_gemv.npz"), **held)


def greedy(shape, element, host, halves, token, context, filled, steps, name, note):
    ref = oracle.Model(shape, element, host, 1, context, 1)
    cache_shape = (shape["kv_heads"], 1, context + 1, shape["head_dim"])
    cases.hold(halves, cache_shape, ref)
    ids, gaps = [], []
    want = token
    for step in range(steps):
        logits, chosen = ref.forward([want], 1, [filled + step], threads=THREADS)
        want = int(chosen[0])
        top = np.sort(logits[0])[-2:]
        ids.append(want), gaps.append(float(top[1] - top[0]))
        print(name, step, want, gaps[-1], flush=True)
    with open(os.path.join(HERE, name), "w") as out:
        json.dump({"note": note, "first_token": token, "cursor_of_first_step": filled, "ids": ids,
                   "smallest_top2_margin": min(gaps), "median_top2_margin": float(np.median(gaps))}, out, indent=1)
        out.write("\n")


def config4():
    shape, _, host, halves, token = cases.config4_case(threads=THREADS)
    greedy(shape, cases.Q8_0, host, halves, token, 1024 + 64, 1024, 64, "config4_greedy_ids.json",
           "cases.config4_case: 0.5B shape, Q8_0, states holding 1024 positions of N(0,1) halves, 64 greedy steps of the oracle")


def config5():
    shape, _, host, halves, token = cases.config5_normal_case()
    greedy(shape, cases.Q4_K, host, halves, token, 4096, 4096 - 64, 64, "config5_normal_greedy_ids.json",
           "cases.config5_normal_case: 7B shape, N(0, 0.02) weights packed to Q4_K, states holding 4032 positions, 64 greedy steps of the oracle")


def config5_blocks():
    shape, _, host, halves, token = cases.config5_case("blocks")
    greedy(shape, cases.Q4_K, host, halves, token, 4096, 4096 - 64, 64, "config5_blocks_greedy_ids.json",
           "cases.config5_case('blocks'): 7B shape, random Q4_K blocks (a degenerate network), states holding 4032 positions, 64 greedy steps of the oracle")


if __name__ == "__main__":
    wanted = sys.argv[1:] or ["blocks", "config1", "kquants", "config4", "config5", "config5_blocks"]
    for name in wanted:
        {"blocks": blocks, "config1": config1, "kquants": kquants, "config4": config4, "config5": config5, "config5_blocks": config5_blocks}[name]()
