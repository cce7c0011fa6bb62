"""Seeded synthetic GGUF payloads of the benchmark configurations, and vectorised numpy
codecs of the block formats.

The numpy codecs restate ggml's published Q8_0 / Q3_K / Q4_K / Q5_K / Q6_K layouts independently of the C oracle
(they are how the tests pin it) and quantize random-init model weights fast enough for the
0.5B-shape configuration.  They run on the host only.
"""
import numpy as np

Q8_0_BLOCK, Q8_0_BYTES = 32, 34
Q4_K_BLOCK, Q4_K_BYTES = 256, 144
Q6_K_BLOCK, Q6_K_BYTES = 256, 210
Q5_K_BLOCK, Q5_K_BYTES = 256, 176
Q3_K_BLOCK, Q3_K_BYTES = 256, 110


def q8_0_random(rng, elements):
    """Blocks of 32 int8 drawn uniformly from [-127, 127] with fp16 scale |N(0, 0.02)|."""
    blocks = elements // Q8_0_BLOCK
    raw = np.empty((blocks, Q8_0_BYTES), dtype=np.uint8)
    scale = np.abs(rng.normal(0.0, 0.02, blocks)).astype(np.float16)
    raw[:, 0:2] = scale.view(np.uint8).reshape(blocks, 2)
    raw[:, 2:] = rng.integers(-127, 128, (blocks, 32), dtype=np.int8).view(np.uint8)
    return raw.reshape(-1)


def q4_k_random(rng, elements):
    """Super-blocks of random nibbles, uniform 6-bit sub-scales / mins (any scale byte is a
    valid packing) and fp16 d, dmin drawn |N(0, 0.01)|."""
    blocks = elements // Q4_K_BLOCK
    raw = np.empty((blocks, Q4_K_BYTES), dtype=np.uint8)
    d = np.abs(rng.normal(0.0, 0.01, (blocks, 2))).astype(np.float16)
    raw[:, 0:4] = d.view(np.uint8).reshape(blocks, 4)
    raw[:, 4:] = rng.integers(0, 256, (blocks, 140), dtype=np.uint8)
    return raw.reshape(-1)


def q6_k_random(rng, elements):
    """Super-blocks of random 6-bit codes (128 nibble bytes, 64 bytes of bit pairs), int8 sub-scales drawn uniformly
    from [-64, 63] and fp16 d drawn |N(0, 0.001)| (weights of the order of 0.01..1, as d * scale * (code - 32))."""
    blocks = elements // Q6_K_BLOCK
    raw = np.empty((blocks, Q6_K_BYTES), dtype=np.uint8)
    raw[:, 0:192] = rng.integers(0, 256, (blocks, 192), dtype=np.uint8)
    raw[:, 192:208] = rng.integers(-64, 64, (blocks, 16), dtype=np.int8).view(np.uint8)
    raw[:, 208:210] = np.abs(rng.normal(0.0, 0.001, (blocks, 1))).astype(np.float16).view(np.uint8).reshape(blocks, 2)
    return raw.reshape(-1)


def q6_k_dequant(raw, elements):
    """ggml's dequantize_row_q6_K, vectorised: per half of 128, element l of groups 0..3 takes nibble ql[l] & 15,
    ql[l + 32] & 15, ql[l] >> 4, ql[l + 32] >> 4 and bit pairs 0, 2, 4, 6 of qh[l]; scale sc[l // 16 + 2 * group]."""
    f32 = np.float32
    blocks = np.asarray(raw, dtype=np.uint8).reshape(-1, Q6_K_BYTES)[: elements // Q6_K_BLOCK]
    d = blocks[:, 208:210].copy().view(np.float16).astype(f32)              # [blocks, 1]
    sc = blocks[:, 192:208].view(np.int8).astype(f32).reshape(-1, 2, 8)      # [blocks, half, 8]
    ql = blocks[:, 0:128].reshape(-1, 2, 2, 32)                              # [blocks, half, low/high 32, l]
    qh = blocks[:, 128:192].reshape(-1, 2, 32)
    out = np.empty((blocks.shape[0], 2, 4, 32), dtype=f32)
    for group in range(4):
        nibble = (ql[:, :, group % 2, :] >> 4) if group >= 2 else (ql[:, :, group % 2, :] & 0x0F)
        code = (nibble | (((qh >> (2 * group)) & 3) << 4)).astype(f32) - f32(32)
        scale = np.repeat(sc[:, :, 2 * group:2 * group + 2], 16, axis=2)      # [blocks, half, 32]
        out[:, :, group, :] = (d[:, :, None] * scale).astype(f32) * code
    return out.reshape(-1)


def q5_k_random(rng, elements):
    """Super-blocks of random 5-bit codes (32 bytes of fifth bits, 128 nibble bytes), uniform 6-bit sub-scales / mins and
    fp16 d, dmin drawn |N(0, 0.005)|."""
    blocks = elements // Q5_K_BLOCK
    raw = np.empty((blocks, Q5_K_BYTES), dtype=np.uint8)
    d = np.abs(rng.normal(0.0, 0.005, (blocks, 2))).astype(np.float16)
    raw[:, 0:4] = d.view(np.uint8).reshape(blocks, 4)
    raw[:, 4:] = rng.integers(0, 256, (blocks, Q5_K_BYTES - 4), dtype=np.uint8)
    return raw.reshape(-1)


def q3_k_random(rng, elements):
    """Super-blocks of random 3-bit codes (32 bytes of third bits, 64 bytes of bit pairs), random 6-bit sub-scales and
    fp16 d drawn |N(0, 0.002)| (weights d * (scale - 32) * code with |scale - 32| <= 32, code in -4..3)."""
    blocks = elements // Q3_K_BLOCK
    raw = np.empty((blocks, Q3_K_BYTES), dtype=np.uint8)
    raw[:, 0:108] = rng.integers(0, 256, (blocks, 108), dtype=np.uint8)
    raw[:, 108:110] = np.abs(rng.normal(0.0, 0.002, (blocks, 1))).astype(np.float16).view(np.uint8).reshape(blocks, 2)
    return raw.reshape(-1)


def q5_k_dequant(raw, elements):
    """ggml's dequantize_row_q5_K, vectorised: per 64 elements two sub-blocks share 32 nibble bytes (low nibbles first);
    the fifth bit of element l of sub-block s is bit s of qh[l]; value = d * sc * code - dmin * m."""
    f32 = np.float32
    blocks = np.asarray(raw, dtype=np.uint8).reshape(-1, Q5_K_BYTES)[: elements // Q5_K_BLOCK]
    d = blocks[:, 0:2].copy().view(np.float16).astype(f32)
    dmin = blocks[:, 2:4].copy().view(np.float16).astype(f32)
    sc, mn = scale_min_k4(blocks[:, 4:16])
    quantum = (d * sc.astype(f32)).astype(f32)
    low = (dmin * mn.astype(f32)).astype(f32)
    qh = blocks[:, 16:48]
    ql = blocks[:, 48:176].reshape(-1, 4, 32)
    out = np.empty((blocks.shape[0], 8, 32), dtype=f32)
    for sub in range(8):
        nibble = (ql[:, sub // 2, :] >> 4) if sub % 2 else (ql[:, sub // 2, :] & 0x0F)
        code = (nibble + np.where(qh & (1 << sub), 16, 0)).astype(f32)
        out[:, sub, :] = (quantum[:, sub:sub + 1] * code).astype(f32) - low[:, sub:sub + 1]
    return out.reshape(-1)


def q3_k_scales(scales):
    """[blocks, 12] uint8 -> [blocks, 16] scale codes minus 32, by the word shuffle of ggml's dequantize_row_q3_K
    (kmask1 = 0x03030303, kmask2 = 0x0f0f0f0f over three little-endian words)."""
    aux = np.ascontiguousarray(scales).view("<u4").reshape(-1, 3).astype(np.uint32)
    tmp = aux[:, 2]
    k1, k2 = np.uint32(0x03030303), np.uint32(0x0F0F0F0F)
    packed = np.stack([
        (aux[:, 0] & k2) | ((tmp & k1) << 4),
        (aux[:, 1] & k2) | (((tmp >> 2) & k1) << 4),
        ((aux[:, 0] >> 4) & k2) | (((tmp >> 4) & k1) << 4),
        ((aux[:, 1] >> 4) & k2) | (((tmp >> 6) & k1) << 4),
    ], axis=1).astype("<u4")
    return packed.view(np.uint8).reshape(-1, 16).astype(np.int32) - 32


def q3_k_dequant(raw, elements):
    """ggml's dequantize_row_q3_K, vectorised: per half of 128 and shift 0, 2, 4, 6 two runs of 16 (bytes l and l + 16 of
    the half's 32 quant bytes), each with its own scale; the code is the bit pair minus 4 unless mask bit `m` of
    hmask[l] is set, m walking 1, 2, 4, ... over the eight runs of 32."""
    f32 = np.float32
    blocks = np.asarray(raw, dtype=np.uint8).reshape(-1, Q3_K_BYTES)[: elements // Q3_K_BLOCK]
    d = blocks[:, 108:110].copy().view(np.float16).astype(f32)               # [blocks, 1]
    scales = q3_k_scales(blocks[:, 96:108]).astype(f32)                       # [blocks, 16]
    hmask = blocks[:, 0:32]
    qs = blocks[:, 32:96].reshape(-1, 2, 32)
    out = np.empty((blocks.shape[0], 2, 4, 32), dtype=f32)
    walk = 0
    for half in range(2):
        for j in range(4):
            pair = ((qs[:, half, :] >> (2 * j)) & 3).astype(np.int32)
            code = (pair - np.where(hmask & (1 << (half * 4 + j)), 0, 4)).astype(f32)
            scale = np.repeat(scales[:, walk:walk + 2], 16, axis=1)          # [blocks, 32]
            out[:, half, j, :] = (d * scale).astype(f32) * code
            walk += 2
    return out.reshape(-1)


def q8_0_dequant(raw, elements):
    blocks = np.asarray(raw, dtype=np.uint8).reshape(-1, Q8_0_BYTES)[: elements // Q8_0_BLOCK]
    d = blocks[:, 0:2].copy().view(np.float16).astype(np.float32)  # [blocks, 1]
    q = blocks[:, 2:].view(np.int8).astype(np.float32)
    return (q * d).reshape(-1)


def scale_min_k4(scales):
    """[blocks, 12] uint8 -> (sc [blocks, 8], m [blocks, 8]) as ggml's get_scale_min_k4."""
    s = scales.astype(np.uint32)
    sc = np.empty((s.shape[0], 8), dtype=np.uint32)
    mn = np.empty((s.shape[0], 8), dtype=np.uint32)
    sc[:, :4] = s[:, 0:4] & 63
    mn[:, :4] = s[:, 4:8] & 63
    sc[:, 4:] = (s[:, 8:12] & 0x0F) | ((s[:, 0:4] >> 6) << 4)
    mn[:, 4:] = (s[:, 8:12] >> 4) | ((s[:, 4:8] >> 6) << 4)
    return sc, mn


def q4_k_dequant(raw, elements):
    blocks = np.asarray(raw, dtype=np.uint8).reshape(-1, Q4_K_BYTES)[: elements // Q4_K_BLOCK]
    d = blocks[:, 0:2].copy().view(np.float16).astype(np.float32)    # [blocks, 1]
    dmin = blocks[:, 2:4].copy().view(np.float16).astype(np.float32)
    sc, mn = scale_min_k4(blocks[:, 4:16])
    quantum = d * sc.astype(np.float32)                              # rounded fp32 product
    low = dmin * mn.astype(np.float32)
    qs = blocks[:, 16:].reshape(-1, 4, 32)
    codes = np.stack([qs & 0x0F, qs >> 4], axis=2).astype(np.float32)  # [blocks, group, seat, 32]
    quantum = quantum.reshape(-1, 4, 2, 1)
    low = low.reshape(-1, 4, 2, 1)
    return (quantum * codes - low).astype(np.float32).reshape(-1)


def _round_away(values):
    return np.sign(values) * np.floor(np.abs(values) + np.float32(0.5))


def q8_0_quantize(values):
    """ggml.rs:201-209: d = max|x| / 127 in fp32, codes from the fp32 d, fp16 d stored."""
    x = np.asarray(values, dtype=np.float32).reshape(-1, Q8_0_BLOCK)
    size = np.abs(x).max(axis=1, keepdims=True)
    quantum = (size / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        inverse = np.where(quantum == 0, np.float32(0), np.float32(1.0) / quantum).astype(np.float32)
    codes = np.clip(_round_away((x * inverse).astype(np.float32)), -127, 127).astype(np.int8)
    raw = np.empty((x.shape[0], Q8_0_BYTES), dtype=np.uint8)
    raw[:, 0:2] = quantum.astype(np.float16).view(np.uint8).reshape(-1, 2)
    raw[:, 2:] = codes.view(np.uint8)
    return raw.reshape(-1)


def q4_k_quantize(values):
    """ggml.rs:149-199 (affine_block with 15 steps over 32-element sub-blocks)."""
    f32 = np.float32
    x = np.asarray(values, dtype=f32).reshape(-1, 8, 32)
    lows = np.minimum(f32(0), x.min(axis=2))
    highs = np.maximum(f32(0), x.max(axis=2))
    quantums = ((highs - lows) / f32(15)).astype(f32)
    scale = (quantums.max(axis=1, keepdims=True) / f32(63)).astype(f32)
    minimum = ((-lows).max(axis=1, keepdims=True) / f32(63)).astype(f32)
    with np.errstate(divide="ignore", invalid="ignore"):
        codes = np.where(scale == 0, f32(0), quantums / scale).astype(f32)
        mins = np.where(minimum == 0, f32(0), -lows / minimum).astype(f32)
    codes = np.clip(_round_away(codes), 0, 63).astype(np.uint32)
    mins = np.clip(_round_away(mins), 0, 63).astype(np.uint32)
    raw = np.zeros((x.shape[0], Q4_K_BYTES), dtype=np.uint8)
    raw[:, 0:2] = scale.astype(np.float16).view(np.uint8).reshape(-1, 2)
    raw[:, 2:4] = minimum.astype(np.float16).view(np.uint8).reshape(-1, 2)
    s = raw[:, 4:16]
    s[:, 0:4] = (codes[:, 0:4] | ((codes[:, 4:8] >> 4) << 6)).astype(np.uint8)
    s[:, 4:8] = (mins[:, 0:4] | ((mins[:, 4:8] >> 4) << 6)).astype(np.uint8)
    s[:, 8:12] = ((codes[:, 4:8] & 0x0F) | ((mins[:, 4:8] & 0x0F) << 4)).astype(np.uint8)
    quantum = (scale * codes.astype(f32)).astype(f32)[:, :, None]
    low = (minimum * mins.astype(f32)).astype(f32)[:, :, None]
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(quantum == 0, f32(0), ((x + low).astype(f32) / quantum).astype(f32))
    q = np.clip(_round_away(q.astype(f32)), 0, 15).astype(np.uint8).reshape(-1, 4, 2, 32)
    raw[:, 16:] = (q[:, :, 0, :] | (q[:, :, 1, :] << 4)).reshape(-1, 128)
    return raw.reshape(-1)


def q5_k_quantize(values):
    """ggml.rs:149-199 (affine_block with 31 steps over 32-element sub-blocks; the fifth bit of sub-block s, element l is
    bit s of byte 16 + l)."""
    f32 = np.float32
    x = np.asarray(values, dtype=f32).reshape(-1, 8, 32)
    lows = np.minimum(f32(0), x.min(axis=2))
    highs = np.maximum(f32(0), x.max(axis=2))
    quantums = ((highs - lows) / f32(31)).astype(f32)
    scale = (quantums.max(axis=1, keepdims=True) / f32(63)).astype(f32)
    minimum = ((-lows).max(axis=1, keepdims=True) / f32(63)).astype(f32)
    with np.errstate(divide="ignore", invalid="ignore"):
        codes = np.where(scale == 0, f32(0), quantums / scale).astype(f32)
        mins = np.where(minimum == 0, f32(0), -lows / minimum).astype(f32)
    codes = np.clip(_round_away(codes), 0, 63).astype(np.uint32)
    mins = np.clip(_round_away(mins), 0, 63).astype(np.uint32)
    raw = np.zeros((x.shape[0], Q5_K_BYTES), dtype=np.uint8)
    raw[:, 0:2] = scale.astype(np.float16).view(np.uint8).reshape(-1, 2)
    raw[:, 2:4] = minimum.astype(np.float16).view(np.uint8).reshape(-1, 2)
    s = raw[:, 4:16]
    s[:, 0:4] = (codes[:, 0:4] | ((codes[:, 4:8] >> 4) << 6)).astype(np.uint8)
    s[:, 4:8] = (mins[:, 0:4] | ((mins[:, 4:8] >> 4) << 6)).astype(np.uint8)
    s[:, 8:12] = ((codes[:, 4:8] & 0x0F) | ((mins[:, 4:8] & 0x0F) << 4)).astype(np.uint8)
    quantum = (scale * codes.astype(f32)).astype(f32)[:, :, None]
    low = (minimum * mins.astype(f32)).astype(f32)[:, :, None]
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(quantum == 0, f32(0), ((x + low).astype(f32) / quantum).astype(f32))
    q = np.clip(_round_away(q.astype(f32)), 0, 31).astype(np.uint8)             # [blocks, 8, 32]
    nib = (q & 0x0F).reshape(-1, 4, 2, 32)
    raw[:, 48:176] = (nib[:, :, 0, :] | (nib[:, :, 1, :] << 4)).reshape(-1, 128)
    fifth = np.zeros((x.shape[0], 32), dtype=np.uint8)
    for sub in range(8):
        fifth |= ((q[:, sub, :] >> 4) & 1) << sub
    raw[:, 16:48] = fifth
    return raw.reshape(-1)


def q3_k_quantize(values):
    """ggml.rs:242-289: d = widest magnitude / 4 / 31, sub-scales round(peak / 4 / d) + 32 per 16 elements, codes
    round(x / (d * (scale - 32))) in -4..3; the fp32 d quantizes and the fp16 d is stored."""
    f32 = np.float32
    x = np.asarray(values, dtype=f32).reshape(-1, 16, 16)
    peaks = np.abs(x).max(axis=2)                                               # [blocks, 16]
    widest = np.maximum(peaks.max(axis=1, keepdims=True), np.finfo(f32).tiny).astype(f32)
    d = ((widest / f32(4)).astype(f32) / f32(31)).astype(f32)
    codes = np.clip(_round_away(((peaks / f32(4)).astype(f32) / d).astype(f32)), 0, 31).astype(np.uint32) + 32
    quantum = (d * (codes.astype(f32) - f32(32))).astype(f32)[:, :, None]
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(quantum == 0, f32(0), (x / quantum).astype(f32))
    q = np.clip(_round_away(q.astype(f32)), -4, 3).astype(np.int32)             # [blocks, sub 16, lane 16]
    q = q.reshape(-1, 2, 4, 2, 16)                                              # [blocks, half, j, second, lane]
    raw = np.zeros((x.shape[0], Q3_K_BYTES), dtype=np.uint8)
    quants = np.zeros((x.shape[0], 2, 2, 16), dtype=np.uint8)                   # [blocks, half, second, lane]
    high = np.zeros((x.shape[0], 2, 16), dtype=np.uint8)                        # [blocks, second, lane]
    for half in range(2):
        for j in range(4):
            quants[:, half] |= ((q[:, half, j] & 3) << (2 * j)).astype(np.uint8)
            high |= ((q[:, half, j] >= 0).astype(np.uint8) << (half * 4 + j)).astype(np.uint8)
    raw[:, 0:32] = high.reshape(-1, 32)
    raw[:, 32:96] = quants.reshape(-1, 64)
    low4, high2 = (codes & 0x0F).astype(np.uint8), ((codes >> 4) & 3).astype(np.uint8)
    raw[:, 96:104] = low4[:, 0:8] | (low4[:, 8:16] << 4)
    for at in range(16):
        raw[:, 104 + at % 4] |= high2[:, at] << (2 * (at // 4))
    raw[:, 108:110] = d.astype(np.float16).view(np.uint8).reshape(-1, 2)
    return raw.reshape(-1)


def q6_k_quantize(values):
    """Symmetric 6-bit codes in ggml's Q6_K layout: per 16 elements a step of largest / 31, int8 sub-scales against a
    super scale of largest step / 127, codes round(x / step) + 32.  (Test data only: the reference's own Q6_K packer,
    ggml.rs:352-392, keeps non-negative values alone, which no model's weights are.)"""
    f32 = np.float32
    x = np.asarray(values, dtype=f32).reshape(-1, 16, 16)
    steps = (np.abs(x).max(axis=2) / f32(31)).astype(f32)                      # [blocks, 16]
    d = (steps.max(axis=1, keepdims=True) / f32(127)).astype(f32)
    with np.errstate(divide="ignore", invalid="ignore"):
        sc = np.where(d == 0, f32(0), steps / d)
    sc = np.clip(_round_away(sc.astype(f32)), 0, 127).astype(np.int8)
    d16 = d.astype(np.float16)
    step = (d16.astype(f32) * sc.astype(f32)).astype(f32)[:, :, None]
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(step == 0, f32(0), x / step)
    codes = (np.clip(_round_away(q.astype(f32)), -32, 31) + 32).astype(np.uint8).reshape(-1, 2, 4, 32)  # [blocks, half, group, l]
    raw = np.zeros((codes.shape[0], Q6_K_BYTES), dtype=np.uint8)
    low = codes & 0x0F
    ql = np.empty((codes.shape[0], 2, 2, 32), dtype=np.uint8)
    ql[:, :, 0, :] = low[:, :, 0, :] | (low[:, :, 2, :] << 4)
    ql[:, :, 1, :] = low[:, :, 1, :] | (low[:, :, 3, :] << 4)
    raw[:, 0:128] = ql.reshape(-1, 128)
    high = codes >> 4
    raw[:, 128:192] = (high[:, :, 0, :] | (high[:, :, 1, :] << 2) | (high[:, :, 2, :] << 4) | (high[:, :, 3, :] << 6)).reshape(-1, 64)
    raw[:, 192:208] = sc.view(np.uint8)
    raw[:, 208:210] = d16.view(np.uint8).reshape(-1, 2)
    return raw.reshape(-1)


QUANTIZE = {8: q8_0_quantize, 11: q3_k_quantize, 12: q4_k_quantize, 13: q5_k_quantize, 14: q6_k_quantize}
RANDOM = {8: q8_0_random, 11: q3_k_random, 12: q4_k_random, 13: q5_k_random, 14: q6_k_random}
DEQUANT = {8: q8_0_dequant, 11: q3_k_dequant, 12: q4_k_dequant, 13: q5_k_dequant, 14: q6_k_dequant}
BLOCK_BYTES = {8: (Q8_0_BLOCK, Q8_0_BYTES), 11: (Q3_K_BLOCK, Q3_K_BYTES), 12: (Q4_K_BLOCK, Q4_K_BYTES), 13: (Q5_K_BLOCK, Q5_K_BYTES),
               14: (Q6_K_BLOCK, Q6_K_BYTES)}


def matrix_bytes(element, rows, columns):
    per, size = BLOCK_BYTES[element]
    return rows * (columns // per) * size


# ---- decoder shapes of the benchmark configurations --------------------------------------

SHAPES = {
    # name: layers, hidden, heads, kv_heads, head_dim, ffn, vocab, tied head
    "qwen2.5-0.5b": dict(layers=24, hidden=896, heads=14, kv_heads=2, head_dim=64, ffn=4864, vocab=151936, tied=True),
    "qwen2.5-1.5b": dict(layers=28, hidden=1536, heads=12, kv_heads=2, head_dim=128, ffn=8960, vocab=151936, tied=True),
    "qwen2.5-7b": dict(layers=28, hidden=3584, heads=28, kv_heads=4, head_dim=128, ffn=18944, vocab=152064, tied=False),
}


def layer_matrices(shape):
    """(name, rows N, columns K) of the seven matrices of one layer."""
    H, QW, KW, F = shape["hidden"], shape["heads"] * shape["head_dim"], shape["kv_heads"] * shape["head_dim"], shape["ffn"]
    return [("attn_q", QW, H), ("attn_k", KW, H), ("attn_v", KW, H), ("attn_output", H, QW), ("ffn_gate", F, H), ("ffn_up", F, H),
            ("ffn_down", H, F)]


def _normal_matrix(held, rows, columns, seed, threads):
    """N(0, 0.02) weights of one matrix quantized chunk by chunk on `threads` threads: every chunk of rows draws from its own
    generator (seeded by the matrix's seed and the chunk's index, so the bytes do not depend on the thread count) and is packed
    by the host layer's encoder where that is the reference's (Q8_0, Q4_K, Q5_K, Q3_K) and by the numpy one for Q6_K."""
    from concurrent.futures import ThreadPoolExecutor

    pack = None
    if held != 14:
        from . import host  # the C++ packer, byte for byte the numpy one and some ten times faster

        pack = lambda values: np.asarray(host.pack(held, values.reshape(-1))).view(np.uint8).reshape(-1)
    else:
        pack = QUANTIZE[held]
    out = np.empty(matrix_bytes(held, rows, columns), dtype=np.uint8)
    row_bytes = matrix_bytes(held, 1, columns)
    step = max(1, (1 << 22) // columns)

    def chunk(index):
        first = index * step
        n = min(step, rows - first)
        values = np.random.default_rng([seed, index]).standard_normal((n, columns), dtype=np.float32) * np.float32(0.02)
        out[first * row_bytes:(first + n) * row_bytes] = pack(values)

    with ThreadPoolExecutor(max_workers=threads) as pool:
        list(pool.map(chunk, range((rows + step - 1) // step)))
    return out


def model_tensors(shape, element, rng, mode="blocks", layers=None, elements=None, biases=(), threads=None):
    """Yields (name, element, dims (GGUF order: K first), raw bytes) of a random-init decoder.

    `elements`: name -> element of the matrices stored otherwise than `element` (a Q4_K_M file keeps some in Q6_K);
    `biases`: layers whose q, k and v projections carry an fp32 bias (Qwen2 checkpoints do).

    mode "blocks": matrices are random raw blocks (the Q4_K distribution of the GEMV
    configurations); mode "normal": N(0, 0.02) weights quantized with the reference's encoder
    (`threads`: on that many threads, a generator per chunk of rows -- the way to build the 7B shape in seconds;
    without it one generator draws everything in order).
    Norm weights are fp32.
    """
    H = shape["hidden"]
    count = shape["layers"] if layers is None else layers

    elements = elements or {}

    def matrix(name, rows, columns):
        held = elements.get(name, element)
        if mode == "blocks":
            return held, RANDOM[held](rng, rows * columns)
        if threads:
            return held, _normal_matrix(held, rows, columns, int(rng.integers(0, 1 << 62)), threads)
        out = np.empty(matrix_bytes(held, rows, columns), dtype=np.uint8)
        step = max(1, (1 << 24) // columns)
        row_bytes = matrix_bytes(held, 1, columns)
        for first in range(0, rows, step):
            n = min(step, rows - first)
            values = rng.normal(0.0, 0.02, (n, columns)).astype(np.float32)
            out[first * row_bytes:(first + n) * row_bytes] = QUANTIZE[held](values)
        return held, out

    def norm():
        return (1.0 + 0.1 * rng.standard_normal(H)).astype(np.float32).view(np.uint8)

    held, raw = matrix("token_embd.weight", shape["vocab"], H)
    yield "token_embd.weight", held, (H, shape["vocab"]), raw
    for layer in range(count):
        yield "blk.%d.attn_norm.weight" % layer, 0, (H,), norm()
        yield "blk.%d.ffn_norm.weight" % layer, 0, (H,), norm()
        for name, rows, columns in layer_matrices(shape):
            held, raw = matrix("blk.%d.%s.weight" % (layer, name), rows, columns)
            yield "blk.%d.%s.weight" % (layer, name), held, (columns, rows), raw
            if layer in biases and name in ("attn_q", "attn_k", "attn_v"):
                yield "blk.%d.%s.bias" % (layer, name), 0, (rows,), rng.normal(0.0, 0.5, rows).astype(np.float32).view(np.uint8)
    yield "output_norm.weight", 0, (H,), norm()
    if not shape["tied"]:
        held, raw = matrix("output.weight", shape["vocab"], H)
        yield "output.weight", held, (H, shape["vocab"]), raw
