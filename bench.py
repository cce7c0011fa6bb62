#!/usr/bin/env python3
"""Headline benchmark: batch-1 greedy decode of a random-init Qwen2.5-7B-shaped decoder with
Q4_K weights and an fp16 KV cache at context 4096, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step (one token): input upload, every kernel of the 28 layers, the
output head, the greedy choice and the read-back of the chosen token.  Weights and caches are
resident in HBM before the timed region.  Prints ONE JSON line:
  value        tokens/s over the K timed steps (host clock around device-synchronised steps)
  roofline     the Q4_K narrow product: weight bytes each launch walks / its device time,
               measured with HIP events around back-to-back passes over the 113 product
               launches of a decode step on the same stream, against MI355X's 8 TB/s HBM peak
  cpu_baseline the CPU oracle (a port of the reference path, OpenMP over output columns) on
               the host cores, timed on a bounded sample of the same workload
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes one Q4_K product launch of the 7B-shape decode step moves on average come from the rocprofv3 FETCH_SIZE /
# WRITE_SIZE runs summarised in this file (each counter scaled by its reading for a plain 1 GiB copy); they cannot be
# measured inside this script, so the summary carries one machine-readable line and the commit it was measured at
TRAFFIC_SUMMARY = os.path.join("profiles", "gemv_q4k_tile16_hbm_counters.md")


def measured_traffic(name):
    """(bytes per launch, "file @ commit") from the line `traffic <workload> <bytes> at <commit>` of the summary, or (None, None)"""
    try:
        with open(os.path.join(ROOT, TRAFFIC_SUMMARY)) as held:
            for line in held:
                words = line.strip().strip("`").split()
                if len(words) == 5 and words[0] == "traffic" and words[1] == name and words[3] == "at":
                    return float(words[2]), "%s @ %s" % (TRAFFIC_SUMMARY, words[4])
    except OSError:
        pass
    return None, None


def note(text):
    """progress on stderr (stdout carries the one JSON line): names the leg a failure belongs to"""
    print("[bench] " + text, file=sys.stderr, flush=True)


def workload(name):
    """(shape, element of the matrices, context, matrices stored otherwise, layers whose q/k/v carry biases)"""
    from neura_amd import synth

    if name == "qwen2.5-7b-q4k":
        return synth.SHAPES["qwen2.5-7b"], 12, 4096, {}, ()
    if name == "qwen2.5-0.5b-q8_0":
        return synth.SHAPES["qwen2.5-0.5b"], 8, 1088, {}, ()
    if name == "qwen2.5-1.5b-q4k":  # the shape whose layer products are BASELINE's second configuration
        return synth.SHAPES["qwen2.5-1.5b"], 12, 1088, {}, ()
    if name in ("qwen2.5-7b-q4_k_m", "qwen2.5-7b-q5_k_m", "qwen2.5-7b-q3_k_m"):
        # the mix llama.cpp's Q4_K_M recipe gives a Qwen2.5-7B file: the head and, in the first and last eighth of the layers
        # and every third between, the value and down projections in Q6_K, the rest Q4_K; q, k and v biases everywhere.
        # Q5_K_M: the same over Q5_K.  Q3_K_M: Q3_K for q, k, gate and up, Q4_K for o, Q5_K for v and down in those
        # layers and Q4_K in the others.
        shape = synth.SHAPES["qwen2.5-7b"]
        count = shape["layers"]
        more_bits = [i for i in range(count) if i < count // 8 or i >= 7 * count // 8 or (i - count // 8) % 3 == 2]
        mixed = {"output.weight": 14}
        base = {"qwen2.5-7b-q4_k_m": 12, "qwen2.5-7b-q5_k_m": 13, "qwen2.5-7b-q3_k_m": 11}[name]
        for i in range(count):
            if base == 11:
                mixed["blk.%d.attn_output.weight" % i] = 12
                mixed["blk.%d.attn_v.weight" % i] = mixed["blk.%d.ffn_down.weight" % i] = 13 if i in more_bits else 12
            elif i in more_bits:
                mixed["blk.%d.attn_v.weight" % i] = mixed["blk.%d.ffn_down.weight" % i] = 14
        return shape, base, 4096, mixed, tuple(range(count))
    raise SystemExit("unknown workload %s" % name)


def weight_bytes_per_token(shape, element, layers, mixed=None):
    from neura_amd import synth

    mixed = mixed or {}
    total = synth.matrix_bytes(mixed.get("output.weight", element), shape["vocab"], shape["hidden"])
    for layer in range(layers):
        for name, rows, columns in synth.layer_matrices(shape):
            total += synth.matrix_bytes(mixed.get("blk.%d.%s.weight" % (layer, name), element), rows, columns)
    return total


def host_threads():
    """(threads the CPU legs use, cores the machine shows): the scheduler's affinity mask, at most the 16 cores a one-GPU
    job is given on a shared host whatever the machine shows"""
    shown = os.cpu_count() or 1
    try:
        allowed = len(os.sched_getaffinity(0))
    except AttributeError:
        allowed = shown
    return max(1, min(allowed, int(os.environ.get("NEURA_BENCH_CPU_THREADS", "16")))), shown


def native_oracle():
    """Compiles the oracle for this machine (-O3 -march=native -ffp-contract=off) and returns the build's flags; the
    portable build the parity tests use is timed instead where no compiler is at hand."""
    import subprocess

    directory = os.path.join(ROOT, "oracle")
    try:
        subprocess.run(["make", "-B", "-C", directory, "native"], check=True, capture_output=True, timeout=120)
        os.environ["NEURA_ORACLE_LIBRARY"] = os.path.join(directory, "libneura_oracle_native.so")
        return "-O3 -march=native -ffp-contract=off"
    except (OSError, subprocess.SubprocessError):
        return "-O2 -march=x86-64-v2 -ffp-contract=off (no native build here)"


def cpu_baseline(shape, element, host_tensors, context, layers, seconds_budget=12.0):
    """Times the oracle's decode step (the checker, used here only as the reported CPU baseline)
    on a bounded sample: a decoder cut to `sample_layers` layers plus the output head, at the
    same context length; the full-depth rate is extrapolated from the per-layer and head times.
    Two legs: every core this job may use, and one thread."""
    flags = native_oracle()
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle

    cores, shown = host_threads()
    rng = np.random.default_rng(7)
    cursor = context - 1

    def step_seconds(threads, sample_layers, budget, most):
        model = oracle.Model(shape, element, host_tensors, batch=1, context=context, layers=sample_layers)
        for held in model.cache_k + model.cache_v:  # a filled cache, as on the device
            held[:] = rng.standard_normal(held.size).astype(np.float16).view(np.uint16)
        model.forward([1], 1, [cursor], threads=threads)  # warm-up
        began = time.perf_counter()
        runs = 0
        while runs < 2 or (time.perf_counter() - began < budget and runs < most):
            model.forward([1], 1, [cursor], threads=threads)
            runs += 1
        with_head = (time.perf_counter() - began) / runs
        # head alone: a zero-layer model
        head_model = oracle.Model(shape, element, host_tensors, batch=1, context=context, layers=0)
        head_model.forward([1], 1, [cursor], threads=threads)
        began = time.perf_counter()
        for _ in range(2):
            head_model.forward([1], 1, [cursor], threads=threads)
        head = (time.perf_counter() - began) / 2
        per_layer = max(with_head - head, 0.0) / sample_layers
        return head + per_layer * layers, runs

    sample_layers = min(layers, 4)
    step, runs = step_seconds(cores, sample_layers, seconds_budget, 50)
    single, single_runs = step_seconds(1, 1, seconds_budget / 2, 3)
    return {
        "value": 1.0 / step,
        "unit": "tokens/s",
        "cores": cores,
        "kind": "port",
        "single_thread": {"value": 1.0 / single, "unit": "tokens/s", "cores": 1},
        "host_cores_shown": shown,
        "build": flags,
        "sample": "%d decode steps of a %d-layer cut of the %d-layer decoder plus the output head at context %d on %d threads (this job's "
                  "share of a host that shows %d cores); full depth extrapolated as head + %d x per-layer time (%.3f s/step); the "
                  "single-thread figure from %d steps of a 1-layer cut the same way (%.2f s/step)" %
                  (runs, sample_layers, layers, context, cores, shown, layers, step, single_runs, single),
    }


def gemm_config3(device, rng, repeats=10):
    """The wide-product configuration of the benchmark: the Q4_K product M=512, K=3584, N=18944 (the 7B-shape FFN up projection), with half
    activations as the configuration states them and with fp32 activations as the decoder's fill passes them; and the same shape in
    Q8_0 blocks (the element of the small decoder's fill) and in Q6_K, Q5_K and Q3_K blocks (what a K-quant mix stores beside Q4_K),
    half activations."""
    from neura_amd import synth

    M, K, N = 512, 3584, 18944
    y = device.alloc(M * N * 4)
    out = {"workload": "Q4_K wide product M=%d K=%d N=%d, random blocks, N(0,1) activations" % (M, K, N), "flop": 2.0 * M * N * K,
           "mfma_peak_tflops": 2500.0}
    for name, element, dtype, code in (("half_activations", 12, np.float16, 1), ("fp32_activations", 12, np.float32, 0),
                                       ("q8_0_half_activations", 8, np.float16, 1), ("q6_k_half_activations", 14, np.float16, 1),
                                       ("q5_k_half_activations", 13, np.float16, 1), ("q3_k_half_activations", 11, np.float16, 1)):
        raw = device.upload(synth.RANDOM[element](rng, N * K))
        x = device.upload(rng.standard_normal((M, K)).astype(dtype))
        for timed in (False, True):
            if timed:
                device.sync()
                device.timer_start()
            for _ in range(repeats if timed else 3):
                status = device.lib.nh_gemm(device.handle, element, raw.pointer, N, K, x.pointer, code, M, y.pointer, None)
                assert status == 0, device.lib.nh_last_error()
        seconds = device.timer_stop() / repeats
        out[name] = {"us": seconds * 1e6, "tflops": 2.0 * M * N * K / seconds / 1e12, "frac_of_mfma_peak": 2.0 * M * N * K / seconds / 2.5e15}
        x.release()
        raw.release()
    y.release()
    return out


def decode_batch8(device, weights, shape, element, context, layers):
    """Eight sequences at the end of their context stepping together: 4 warm-up steps, then 16 timed."""
    from neura_amd.loader import Model

    batch = 8
    model = Model(device, weights, shape, element, batch=batch, context=context, layers=layers)
    steps, warm = 16, 4
    tokens = list(range(1, batch + 1))
    first = context - (steps + warm)
    for step in range(warm):
        tokens = [int(t) for t in model.decode_step(tokens, [first + step] * batch)]
    device.sync()
    began = time.perf_counter()
    for step in range(steps):
        tokens = [int(t) for t in model.decode_step(tokens, [first + warm + step] * batch)]
    device.sync()
    elapsed = time.perf_counter() - began
    model.release()
    return {"value": batch * steps / elapsed, "unit": "tokens/s", "ms_per_step": elapsed / steps * 1e3,
            "note": "8 planes, caches not pre-filled (zeros), cursors at the end of context %d" % context}


def extras(device, weights, shape, element, context, layers, rng):
    """The other two measurements the workload names, on the same resident weights: decode at
    batch 8 (eight sequences at the end of their context) and a 512-token prompt fill."""
    from neura_amd.loader import Model

    import neura_amd

    out = {}
    note("extras: sampled decode, batch 1")
    # batch 1 again with a sampled choice (temperature 0.8, 40 candidates, nucleus 0.95; the seed one further a step)
    model = Model(device, weights, shape, element, batch=1, context=context, layers=layers)
    steps, warm = 32, 4
    first, token = context - (steps + warm), 1
    for step in range(warm + steps):
        if step == warm:
            device.sync()
            began = time.perf_counter()
        draws = np.array([(0x3F800000 | (step & 0x7FFFFF), 0.8, 40, 0.95)], dtype=neura_amd.DRAW)
        token = int(model.decode_step_sampled([token], [first + step], draws)[0])
    device.sync()
    elapsed = time.perf_counter() - began
    out["decode_sampled_batch1"] = {"value": steps / elapsed, "unit": "tokens/s", "ms_per_step": elapsed / steps * 1e3,
                                    "note": "as the headline step with the greedy choice replaced by the sampled one; caches not pre-filled (zeros)"}
    model.release()
    note("extras: decode, batch 1, single precision states")
    model = Model(device, weights, shape, element, batch=1, context=context, layers=layers, cache_element=0)
    steps, warm = 32, 4
    first, token = context - (steps + warm), 1
    for step in range(warm + steps):
        if step == warm:
            device.sync()
            began = time.perf_counter()
        token = int(model.decode_step([token], [first + step])[0])
    device.sync()
    elapsed = time.perf_counter() - began
    out["decode_single_states_batch1"] = {"value": steps / elapsed, "unit": "tokens/s", "ms_per_step": elapsed / steps * 1e3,
                                          "note": "as the headline step with the key and value states in single precision (the element the "
                                                  "reference's example keeps); caches not pre-filled (zeros)"}
    model.release()
    note("extras: decode, batch 8")
    out["decode_batch8"] = decode_batch8(device, weights, shape, element, context, layers)
    note("extras: 512-token fill")
    out["prefill_512"] = fill_512(device, weights, shape, element, context, layers, rng)
    note("extras: wide product of configuration 3")
    out["gemm_config3"] = gemm_config3(device, rng)
    if element == 12 and not os.environ.get("NEURA_BENCH_SKIP_Q8"):
        note("extras: 0.5B-shape Q8_0 decode")
        out["decode_0_5b_q8_0"] = small_q8_0_decode(device)
        note("extras: Q4_K products of one 1.5B-shape layer")
        out["layer_products_1_5b_q4k"] = layer_products_1_5b(device)
    return out


def small_q8_0_decode(device):
    """The 0.5B-shape Q8_0 decoder (the model of the reference's own CPU-runnable decode case): batch 1, cache filled to 1024,
    64 greedy steps after 8."""
    from neura_amd import synth
    from neura_amd.loader import Model, Weights

    shape, element, context, _, _ = workload("qwen2.5-0.5b-q8_0")
    rng = np.random.default_rng(0)
    tensors = list(synth.model_tensors(shape, element, rng, mode="normal"))
    weights = Weights(device, tensors)
    model = Model(device, weights, shape, element, batch=1, context=context)
    for layer in range(shape["layers"]):
        for which in (0, 1):
            model.cache_write(layer, which, rng.standard_normal(model.cache_shape).astype(np.float16).view(np.uint16))
    steps, warm = 64, 8
    first, token = context - (steps + warm), 1
    for step in range(warm + steps):
        if step == warm:
            device.sync()
            began = time.perf_counter()
        token = int(model.decode_step([token], [first + step])[0])
    device.sync()
    elapsed = time.perf_counter() - began
    model.release()
    weights.release()
    walked = weight_bytes_per_token(shape, element, shape["layers"])
    return {"value": steps / elapsed, "unit": "tokens/s", "ms_per_step": elapsed / steps * 1e3,
            "weight_bytes_per_token": walked, "hbm_frac_whole_step": walked / (elapsed / steps) / 1e9 / HBM_PEAK_GBS,
            "note": "qwen2.5-0.5b shape, Q8_0, 24 layers, batch 1, fp16 KV cache at context %d; hbm_frac_whole_step = weight bytes of a "
                    "step over the whole step's time (every kernel and the read-back), against 8 TB/s" % context}


def layer_products_1_5b(device):
    """The Q4_K narrow products of one Qwen2.5-1.5B-shaped layer at batch 1 (hidden 1536, 12 query and 2 key heads of 128,
    FFN 8960: q|k|v, attn_output, gate|up, ffn_down), launched back to back between one pair of events.  The timed pass of a
    decoder also walks its output head: a decoder of two such layers and one of one are timed and their difference is the layer."""
    from neura_amd import synth
    from neura_amd.loader import Model, Weights

    rng = np.random.default_rng(2)
    passes = 64
    measured = []
    for layers in (2, 1):
        shape = dict(synth.SHAPES["qwen2.5-1.5b"], layers=layers)
        weights = Weights(device, list(synth.model_tensors(shape, 12, rng, mode="blocks", layers=layers)))
        model = Model(device, weights, shape, 12, batch=1, context=64, layers=layers)
        model.decode_step([1], [0])
        measured.append(model.time_products(passes))
        model.release()
        weights.release()
    seconds = measured[0][0] - measured[1][0]
    launches = (measured[0][1] - measured[1][1]) / passes
    walked = (measured[0][2] - measured[1][2]) / passes
    return {"us_per_layer": seconds / passes * 1e6, "launches": launches, "weight_bytes": walked, "hbm_gbs": walked * passes / seconds / 1e9,
            "hbm_frac": walked * passes / seconds / 1e9 / HBM_PEAK_GBS,
            "note": "q|k|v, attn_output, gate|up and ffn_down of one layer: a pass over a two-layer decoder's products minus a pass over "
                    "a one-layer decoder's (the output head, which both walk, drops out)"}


def fill_512(device, weights, shape, element, context, layers, rng):
    """One 512-token prompt filled into an empty cache at cursor 0: a warm-up, then the mean of three."""
    from neura_amd.loader import Model

    rows = 512
    model = Model(device, weights, shape, element, batch=1, context=context, max_rows=rows, layers=layers)
    prompt = rng.integers(0, shape["vocab"], rows)
    model.prefill(prompt, rows, [0])
    device.sync()
    began = time.perf_counter()
    repeats = 3
    for _ in range(repeats):
        model.prefill(prompt, rows, [0])
    device.sync()
    elapsed = (time.perf_counter() - began) / repeats
    per_layer = sum(2.0 * rows * n * k for _, n, k in __import__("neura_amd").synth.layer_matrices(shape))
    model.release()
    return {"value": rows / elapsed, "unit": "tokens/s", "ms": elapsed * 1e3, "product_tflops": layers * per_layer / elapsed / 1e12,
            "note": "one 512-row fill at cursor 0, all products on f16 MFMA; the decoder's fp32 activations enter as two half rows each "
                    "(the value rounded to half and its residue), 22 bits of every activation, so the matrix cores do twice the work of "
                    "a half-activation product; "
                    "product_tflops counts 2*M*N*K of the products over the whole fill time"}


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--workload", default="qwen2.5-7b-q4k")
    parser.add_argument("--layers", type=int, default=None, help="cut the decoder (for quick checks; the result is then not the headline)")
    parser.add_argument("--sampled", action="store_true",
                        help="draw every token (temperature 0.8, 40 candidates, nucleus 0.95) instead of taking the largest logit; not the headline")
    parser.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    parser.add_argument("--no-extras", action="store_true", help="skip the batch-8 decode, 512-token fill and wide-product measurements")
    parser.add_argument("--gemm-only", action="store_true", help="run only the wide product (M=512, K=3584, N=18944) and print its line")
    parser.add_argument("--fill-only", action="store_true", help="run only the 512-token fill of the workload and print its line")
    parser.add_argument("--batch8-only", action="store_true", help="run only the 8-plane decode of the workload and print its line")
    parser.add_argument("--calibrate-copy", type=int, default=0, metavar="MIB",
                        help="also run one plain device-to-device copy of MIB MiB (a known-size reference for HBM byte counters)")
    args = parser.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        raise SystemExit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import neura_amd
    from neura_amd import synth
    from neura_amd.loader import Model, Weights

    if args.gemm_only:
        device = neura_amd.Device(0)
        print(json.dumps({"gemm_config3": gemm_config3(device, np.random.default_rng(0))}))
        device.close()
        return
    shape, element, context, mixed, biases = workload(args.workload)
    layers = shape["layers"] if args.layers is None else args.layers
    rng = np.random.default_rng(0)
    mode = "blocks" if element == 12 else "normal"
    tensors = list(synth.model_tensors(shape, element, rng, mode=mode, layers=layers, elements=mixed, biases=biases))
    note("weights synthesised; opening the device")
    device = neura_amd.Device(0)
    weights = Weights(device, tensors)
    note("weights resident")
    if args.fill_only:
        print(json.dumps({"prefill_512": fill_512(device, weights, shape, element, context, layers, rng)}))
        weights.release()
        device.close()
        return
    if args.batch8_only:
        print(json.dumps({"decode_batch8": decode_batch8(device, weights, shape, element, context, layers)}))
        weights.release()
        device.close()
        return
    model = Model(device, weights, shape, element, batch=1, context=context, layers=layers)
    # fp16 caches filled up to the context with N(0,1) halves
    for layer in range(layers):
        for which in (0, 1):
            model.cache_write(layer, which, rng.standard_normal(model.cache_shape).astype(np.float16).view(np.uint16))

    if args.calibrate_copy:
        nbytes = args.calibrate_copy << 20
        source, target = device.alloc(nbytes), device.alloc(nbytes)
        for _ in range(4):
            assert device.lib.nh_copy(device.handle, target.pointer, source.pointer, nbytes) == 0
        device.sync()

    total = args.warmup + args.steps
    first_cursor = context - total  # the last timed step sits at cursor context - 1
    assert first_cursor >= 0, "more steps than the context holds"
    token = 1

    def one_step(token, step):
        if args.sampled:
            draws = np.array([(0x3F800000 | (step & 0x7FFFFF), 0.8, 40, 0.95)], dtype=neura_amd.DRAW)
            return int(model.decode_step_sampled([token], [first_cursor + step], draws)[0])
        return int(model.decode_step([token], [first_cursor + step])[0])

    note("caches filled; warm-up steps")
    for step in range(args.warmup):
        token = one_step(token, step)
        note("warm-up step %d done" % step)
    device.sync()
    note("timed steps")
    began = time.perf_counter()
    for step in range(args.steps):
        token = one_step(token, args.warmup + step)
    device.sync()
    elapsed = time.perf_counter() - began

    note("timed steps done; product-only passes")
    # the dominant kernel alone: every narrow product of a decode step (same matrices, shapes
    # and buffers), launched back to back between one pair of HIP events on the same stream
    profiled = min(args.steps, 32)
    gemv_seconds, launches, walked = model.time_products(profiled)
    per_launch_bytes = walked / launches
    per_launch_seconds = gemv_seconds / launches
    achieved = per_launch_bytes / per_launch_seconds / 1e9

    traffic, traffic_source = measured_traffic(args.workload)
    result = {
        "metric": "decode tok/s (bs=1) Qwen2.5-7B-shape Q4_K; quant-GEMV HBM GB/s (% peak)",
        "value": args.steps / elapsed,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "%s decode, batch 1, %d layers, fp16 KV cache at context %d, random-init %s weights%s" %
                        (args.workload, layers, context, ("Q4_K" if element == 12 else "Q8_0") + (" and Q6_K" if mixed else ""),
                         ", sampled choice" if args.sampled else ""),
            "weight_bytes_per_token": weight_bytes_per_token(shape, element, layers, mixed),
            "arithmetic": "dtype f32 = what activations, sums, logits and every scale are held and joined in; inside a Q4_K product "
                          "the 4-bit codes meet each activation as three signed base-256 digit planes (22 bits below a power-of-two "
                          "scale of its 64-element group, of its 16-element chunk where ffn_down takes them from the SwiGLU epilogue) "
                          "on v_mfma_i32_16x16x64_i8 -- exact integer sums, weighed by d * sc and dmin * m in fp32; keys and values "
                          "are stored as fp16 and attention multiplies them on v_mfma_f32_16x16x{32,16}_f16 with fp32 sums",
        },
        "roofline": {
            "bound": "hbm",
            "kernel": ("all narrow products: gemv_q4k_tile16_kernel, gemv_q6k_tile16_kernel" if mixed else
                       "gemv_q4k_tile16_kernel (q|k|v with the rotation, attn_output, gate|up with SwiGLU, ffn_down, output head)" if element == 12
                       else "gemv_q8_0_decode_kernel"),
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": traffic if args.layers is None else None,
            "traffic_source": traffic_source if args.layers is None else None,
            "bytes_per_launch": per_launch_bytes,
            "us_per_launch": per_launch_seconds * 1e6,
            "launches_per_step": launches / profiled,
            "gemv_ms_per_step": gemv_seconds / profiled * 1e3,
        },
    }
    if not args.no_extras:
        result["extras"] = extras(device, weights, shape, element, context, layers, rng)
    if not args.no_cpu and not mixed:
        note("CPU baseline")
        host = {name: raw for name, _, _, raw in tensors}
        result["cpu_baseline"] = cpu_baseline(shape, element, host, context, layers)
    else:
        result["cpu_baseline"] = None
    model.release()
    weights.release()
    device.close()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
