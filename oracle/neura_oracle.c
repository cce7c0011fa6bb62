/*
 * neura_oracle.c -- CPU restatement of the reference's quantized-GGUF decoder path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test suite, the
 * smoke check and the cpu_baseline leg of the benchmark may load it.  The HIP
 * library never links, loads or calls anything in this file.
 *
 * Every function follows one piece of /root/reference (cited as path:line under
 * that root).  Arithmetic is scalar fp32 in the reference's summation order and
 * the file must be compiled with -ffp-contract=off so that no multiply-add is
 * fused (the reference's host codec rounds the product before the subtract).
 *
 * Pinning status of each function (what fixes its answer without running the
 * reference, which cannot be built here: Rust, no toolchain):
 *   f16 <-> f32 ............ pinned: IEEE binary16 RNE == numpy.float16, all 65536
 *                            codes + 2^20 sampled floats incl. ties/subnormals
 *   xorshift unit .......... pinned: closed form init.rs:86-91, brute force in python
 *   scale_min_k4 / put ..... pinned: put-then-get identity over all 8*64*64 cases
 *   q8_0 / q4_k unpack ..... pinned: independent numpy restatement of ggml's published
 *                            dequantize_row_q8_0 / dequantize_row_q4_K + hand-built blocks
 *   q8_0 / q4_k pack ....... pinned: invariants (|unpack(pack(x)) - x| <= d/2, codes in
 *                            range) + independent numpy restatement
 *   q3_k unpack ............ pinned: the reference's own known-answer block (bytes at*37+11, at*53+7, at*19+3,
 *                            d = 0.25: crates/neura-precision/tests/format.rs:221-234) walked by a numpy
 *                            restatement of ggml's published dequantize_row_q3_K, + its round-trip bound (:236-245)
 *   q5_k / q6_k unpack ..... pinned: numpy restatements of ggml's published dequantize_row_q5_K / _q6_K + hand-built blocks
 *   q3_k / q5_k / q6_k pack  pinned: round-trip bounds and field invariants
 *   gemv / gemm ............ pinned: the reference's own test definition (fp32 triple
 *                            loop over unpack, runtime.rs:72-83) + fp64 numpy
 *   rmsnorm ................ pinned: composed form tests/norm.rs:21-26
 *   rope ................... pinned: closed form runtime.rs:468-494 (rotate-half)
 *   attention .............. pinned: f64 reference tests/support/attention.rs:38-109
 *   argmax ................. pinned: ties -> lowest index, brute force
 *   sample ................. pinned: the hash against a numpy restatement; keep == 1 is the argmax and a row draws by
 *                            its own seed (the reference's own tests, crates/neura-runtime/tests/choice.rs:41-126); the
 *                            draw frequencies against the softmax over the kept nucleus (Gumbel-max); a nucleus worked
 *                            by hand.  The rounding of the shader's log and exp is PARITY UNPINNED (no fixture holds it).
 *   decode step / greedy ... PARITY UNPINNED against the reference binary (no reference
 *                            test runs a transformer); pinned only by composition of the
 *                            pinned parts above plus an independent numpy forward pass.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define Q8_0_BLOCK 32   /* neura-abi/src/element.rs:33-40 */
#define Q8_0_BYTES 34
#define Q4_K_BLOCK 256
#define Q4_K_BYTES 144
#define Q6_K_BLOCK 256
#define Q6_K_BYTES 210 /* 128 low nibbles, 64 bytes of high bit pairs, 16 int8 scales, f16 d: neura-abi/src/element.rs:167-170 */
#define Q5_K_BLOCK 256
#define Q5_K_BYTES 176 /* f16 d, f16 dmin, 12 scale bytes, 32 bytes of fifth bits, 128 nibble bytes: neura-abi/src/element.rs:163-166 */
#define Q3_K_BLOCK 256
#define Q3_K_BYTES 110 /* 32 bytes of third bits, 64 bytes of bit pairs, 12 scale bytes, f16 d: neura-abi/src/element.rs:171-174 */
#define SUB_BLOCK 32
#define FOLDED_LANES 32   /* neura-profile/src/profile.rs:1327 */
#define FOLDED_STAGE 1024 /* neura-profile/src/profile.rs:1358 */
#define WORKGROUP 256     /* neura-profile/src/profile.rs:2086-2089 */
#define ATTN_KEYS 16      /* neura-profile/src/profile.rs:70 */

enum { EL_F32 = 0, EL_F16 = 1, EL_BF16 = 30, EL_Q8_0 = 8, EL_Q3_K = 11, EL_Q4_K = 12, EL_Q5_K = 13, EL_Q6_K = 14 }; /* ggml ids, neura-gguf/src/header.rs:150-162 */

/* ---------------------------------------------------------------- f16 ---- */

/* crates/neura-kernel/src/task/convert.rs:57-84 (half_bits); equals half::f16::from_f32 */
uint16_t oracle_f32_to_f16(float value) {
    uint32_t bits;
    memcpy(&bits, &value, 4);
    uint32_t sign = (bits >> 16) & 0x8000u;
    uint32_t magnitude = bits & 0x7fffffffu;
    if (magnitude > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (magnitude >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);
    if (magnitude < 0x33000000u) return (uint16_t)sign;
    if (magnitude < 0x38800000u) {
        uint32_t exponent = (bits >> 23) & 0xffu;
        uint32_t significand = (bits & 0x007fffffu) | 0x00800000u;
        uint32_t shift = 126u - exponent;
        uint32_t rounded = significand + ((1u << (shift - 1u)) - 1u) + ((significand >> shift) & 1u);
        return (uint16_t)(sign | (rounded >> shift));
    }
    uint32_t rounded = bits + 0x0fffu + ((bits >> 13) & 1u);
    uint32_t exponent = (rounded >> 23) & 0xffu;
    if (exponent >= 143u) return (uint16_t)(sign | 0x7c00u);
    return (uint16_t)(sign | ((exponent - 112u) << 10) | ((rounded >> 13) & 0x3ffu));
}

/* crates/neura-precision/src/ggml.rs:74-76 (half_at -> half::f16::to_f32), exact */
float oracle_f16_to_f32(uint16_t half) {
    uint32_t sign = ((uint32_t)half & 0x8000u) << 16;
    uint32_t exponent = (half >> 10) & 0x1fu;
    uint32_t fraction = half & 0x3ffu;
    uint32_t bits;
    if (exponent == 0) {
        if (fraction == 0) {
            bits = sign;
        } else {
            int shift = 0;
            while (!(fraction & 0x400u)) { fraction <<= 1; shift++; }
            fraction &= 0x3ffu;
            bits = sign | ((uint32_t)(113 - shift) << 23) | (fraction << 13);
        }
    } else if (exponent == 31) {
        bits = sign | 0x7f800000u | (fraction << 13);
    } else {
        bits = sign | ((exponent + 112u) << 23) | (fraction << 13);
    }
    float out;
    memcpy(&out, &bits, 4);
    return out;
}

void oracle_f32_to_f16_many(const float *in, uint64_t n, uint16_t *out) {
    for (uint64_t i = 0; i < n; i++) out[i] = oracle_f32_to_f16(in[i]);
}
void oracle_f16_to_f32_many(const uint16_t *in, uint64_t n, float *out) {
    for (uint64_t i = 0; i < n; i++) out[i] = oracle_f16_to_f32(in[i]);
}

/* --------------------------------------------------------------- PRNG ---- */

/* crates/neura-graph/src/init.rs:86-91 */
float oracle_unit(uint32_t *entropy) {
    *entropy ^= *entropy << 13;
    *entropy ^= *entropy >> 17;
    *entropy ^= *entropy << 5;
    return (float)(*entropy >> 8) / (float)(1u << 24);
}

/* crates/neura-runtime/tests/support/mod.rs:41-48 with init.rs:61-69: uniform in [-1,1) */
void oracle_random(uint32_t count, uint32_t seed, float *out) {
    uint32_t entropy = seed | 1u;
    for (uint32_t i = 0; i < count; i++) out[i] = -1.0f + (1.0f - -1.0f) * oracle_unit(&entropy);
}

/* -------------------------------------------------------- block codecs ---- */

/* crates/neura-precision/src/ggml.rs:127-136 */
void oracle_scale_min_k4(const uint8_t *scales, uint32_t at, uint32_t *scale, uint32_t *min) {
    if (at < 4) {
        *scale = scales[at] & 63u;
        *min = scales[at + 4] & 63u;
    } else {
        *scale = (uint32_t)(scales[at + 4] & 0x0fu) | ((uint32_t)(scales[at - 4] >> 6) << 4);
        *min = (uint32_t)(scales[at + 4] >> 4) | ((uint32_t)(scales[at] >> 6) << 4);
    }
}

/* crates/neura-precision/src/ggml.rs:138-147 (scales must start zeroed) */
void oracle_put_scale_min_k4(uint8_t *scales, uint32_t at, uint32_t scale, uint32_t min) {
    if (at < 4) {
        scales[at] = (uint8_t)scale;
        scales[at + 4] = (uint8_t)min;
    } else {
        scales[at + 4] = (uint8_t)((scale & 0x0fu) | ((min & 0x0fu) << 4));
        scales[at - 4] |= (uint8_t)((scale >> 4) << 6);
        scales[at] |= (uint8_t)((min >> 4) << 6);
    }
}

/* crates/neura-precision/src/ggml.rs:211-216 */
static void q8_0_values(const uint8_t *field, float *out) {
    uint16_t h;
    memcpy(&h, field, 2);
    float quantum = oracle_f16_to_f32(h);
    for (int at = 0; at < Q8_0_BLOCK; at++) out[at] = (float)(int8_t)field[2 + at] * quantum;
}

/* crates/neura-precision/src/ggml.rs:336-350 */
static void q4_k_values(const uint8_t *field, float *out) {
    uint16_t h0, h1;
    memcpy(&h0, field, 2);
    memcpy(&h1, field + 2, 2);
    float scale = oracle_f16_to_f32(h0);
    float min = oracle_f16_to_f32(h1);
    int o = 0;
    for (uint32_t group = 0; group < 4; group++) {
        for (uint32_t seat = 0; seat < 2; seat++) {
            uint32_t code, offset;
            oracle_scale_min_k4(field + 4, group * 2 + seat, &code, &offset);
            float quantum = scale * (float)code;
            float low = min * (float)offset;
            for (uint32_t within = 0; within < SUB_BLOCK; within++) {
                uint8_t byte = field[16 + group * 32 + within];
                uint32_t quant = seat ? (uint32_t)(byte >> 4) : (uint32_t)(byte & 0x0f);
                out[o++] = quantum * (float)quant - low;
            }
        }
    }
}

/* crates/neura-precision/src/ggml.rs:394-407: two halves of 128, four groups of 32 in each; the 6-bit code is a
 * nibble (groups 0, 1 low and 2, 3 high of bytes half*64 + (group%2)*32 + within) plus two bits
 * (byte 128 + half*32 + within, shifted by 2*group); one int8 scale per 16 elements; value = d * scale * (code - 32),
 * left to right, every product rounded. */
static void q6_k_values(const uint8_t *field, float *out) {
    uint16_t h;
    memcpy(&h, field + 208, 2);
    float scale = oracle_f16_to_f32(h);
    for (uint32_t seat = 0; seat < 2; seat++)
        for (uint32_t group = 0; group < 4; group++)
            for (uint32_t within = 0; within < 32; within++) {
                uint32_t index = group * 2 + within / 16;
                int8_t sub = (int8_t)field[192 + seat * 8 + index];
                uint8_t byte = field[seat * 64 + (group % 2) * 32 + within];
                uint32_t nibble = group >= 2 ? (uint32_t)(byte >> 4) : (uint32_t)(byte & 0x0f);
                uint32_t quant = nibble | (((uint32_t)(field[128 + seat * 32 + within] >> (2 * group)) & 3u) << 4);
                float product = scale * (float)sub;
                *out++ = product * ((float)quant - 32.0f);
            }
}

/* crates/neura-precision/src/ggml.rs:321-335: Q4_K's walk with a fifth bit per code, bit 2*group + seat of byte 16 + within */
static void q5_k_values(const uint8_t *field, float *out) {
    uint16_t h0, h1;
    memcpy(&h0, field, 2);
    memcpy(&h1, field + 2, 2);
    float scale = oracle_f16_to_f32(h0);
    float min = oracle_f16_to_f32(h1);
    for (uint32_t group = 0; group < 4; group++) {
        for (uint32_t seat = 0; seat < 2; seat++) {
            uint32_t code, offset;
            oracle_scale_min_k4(field + 4, group * 2 + seat, &code, &offset);
            float quantum = scale * (float)code;
            float low = min * (float)offset;
            for (uint32_t within = 0; within < SUB_BLOCK; within++) {
                uint32_t high = ((uint32_t)field[16 + within] >> (2 * group + seat)) & 1u;
                uint8_t byte = field[48 + group * 32 + within];
                uint32_t quant = (seat ? (uint32_t)(byte >> 4) : (uint32_t)(byte & 0x0f)) | (high << 4);
                *out++ = quantum * (float)quant - low;
            }
        }
    }
}

/* 6-bit scale `at` (0..15) of a Q3_K super-block: crates/neura-precision/src/ggml.rs:224-229 */
static uint32_t q3_k_scale(const uint8_t *field, uint32_t at) {
    uint8_t low = field[96 + at % 8];
    uint32_t nibble = at < 8 ? (uint32_t)(low & 0x0f) : (uint32_t)(low >> 4);
    uint8_t high = field[96 + 8 + at % 4];
    return nibble | ((((uint32_t)high >> (2 * (at / 4))) & 3u) << 4);
}

/* crates/neura-precision/src/ggml.rs:291-306: sixteen sub-blocks of 16; code = two bits minus 4 unless the third bit is set;
 * value = d * (scale - 32) * code, left to right */
static void q3_k_values(const uint8_t *field, float *out) {
    uint16_t h;
    memcpy(&h, field + 108, 2);
    float d = oracle_f16_to_f32(h);
    for (uint32_t at = 0; at < Q3_K_BLOCK; at++) {
        uint32_t sub = at / 16, lane = at % 16;
        uint32_t half = sub / 8, within = sub % 8, j = within / 2, second = within % 2;
        uint32_t low = ((uint32_t)field[32 + half * 32 + second * 16 + lane] >> (2 * j)) & 3u;
        int high = (field[second * 16 + lane] & (1u << (half * 4 + j))) != 0;
        int quant = (int)low - (high ? 0 : 4);
        float product = d * ((float)(uint8_t)q3_k_scale(field, sub) - 32.0f);
        out[at] = product * (float)quant;
    }
}

/* crates/neura-precision/src/ggml.rs:22-38 (unpack); elements must be whole blocks */
int oracle_unpack(int element, const uint8_t *bytes, uint64_t elements, float *out) {
    if (element == EL_Q8_0) {
        if (elements % Q8_0_BLOCK) return -1;
        for (uint64_t b = 0; b < elements / Q8_0_BLOCK; b++) q8_0_values(bytes + b * Q8_0_BYTES, out + b * Q8_0_BLOCK);
        return 0;
    }
    if (element == EL_Q4_K) {
        if (elements % Q4_K_BLOCK) return -1;
        for (uint64_t b = 0; b < elements / Q4_K_BLOCK; b++) q4_k_values(bytes + b * Q4_K_BYTES, out + b * Q4_K_BLOCK);
        return 0;
    }
    if (element == EL_Q6_K) {
        if (elements % Q6_K_BLOCK) return -1;
        for (uint64_t b = 0; b < elements / Q6_K_BLOCK; b++) q6_k_values(bytes + b * Q6_K_BYTES, out + b * Q6_K_BLOCK);
        return 0;
    }
    if (element == EL_Q5_K) {
        if (elements % Q5_K_BLOCK) return -1;
        for (uint64_t b = 0; b < elements / Q5_K_BLOCK; b++) q5_k_values(bytes + b * Q5_K_BYTES, out + b * Q5_K_BLOCK);
        return 0;
    }
    if (element == EL_Q3_K) {
        if (elements % Q3_K_BLOCK) return -1;
        for (uint64_t b = 0; b < elements / Q3_K_BLOCK; b++) q3_k_values(bytes + b * Q3_K_BYTES, out + b * Q3_K_BLOCK);
        return 0;
    }
    if (element == EL_F16) {
        oracle_f16_to_f32_many((const uint16_t *)bytes, elements, out);
        return 0;
    }
    if (element == EL_F32) {
        memcpy(out, bytes, elements * 4);
        return 0;
    }
    return -2;
}

/* Rust f32::round: half away from zero */
static float round_away(float v) { return roundf(v); }
static float clampf(float v, float lo, float hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* crates/neura-precision/src/ggml.rs:201-209 with peak :98-108 */
static void q8_0_encode(const float *values, uint8_t *out) {
    float size = 0.0f;
    for (int i = 0; i < Q8_0_BLOCK; i++)
        if (size < fabsf(values[i])) size = fabsf(values[i]);
    float quantum = size / 127.0f;
    float inverse = quantum == 0.0f ? 0.0f : 1.0f / quantum;
    uint16_t h = oracle_f32_to_f16(quantum);
    memcpy(out, &h, 2);
    for (int i = 0; i < Q8_0_BLOCK; i++) out[2 + i] = (uint8_t)(int8_t)clampf(round_away(values[i] * inverse), -127.0f, 127.0f);
}

static float least(float a, float b) { return a < b ? a : b; }
static float greatest(float a, float b) { return a > b ? a : b; }

/* crates/neura-precision/src/ggml.rs:149-199 (affine_block; Q4K: steps 15, nibbles at 16; Q5K: steps 31, fifth bits at 16, nibbles at 48) */
static void affine_encode(const float *values, uint8_t *field, int fifth) {
    const int count = Q4_K_BLOCK / SUB_BLOCK;
    const float steps = fifth ? 31.0f : 15.0f;
    const int quants = fifth ? 48 : 16;
    float lows[8], quantums[8];
    for (int at = 0; at < count; at++) {
        float low = 0.0f, high = 0.0f; /* span folds from (0,0): ggml.rs:110-114 */
        for (int i = 0; i < SUB_BLOCK; i++) {
            low = least(low, values[at * SUB_BLOCK + i]);
            high = greatest(high, values[at * SUB_BLOCK + i]);
        }
        lows[at] = least(0.0f, low);
        quantums[at] = (high - lows[at]) / steps;
    }
    float scale = 0.0f, min = 0.0f;
    for (int at = 0; at < count; at++) scale = greatest(scale, quantums[at]);
    scale = scale / 63.0f;
    for (int at = 0; at < count; at++) min = greatest(min, -lows[at]);
    min = min / 63.0f;
    uint8_t codes[8], mins[8];
    for (int at = 0; at < count; at++) {
        float c = scale == 0.0f ? 0.0f : quantums[at] / scale; /* scale_of(quantum, low) = low/quantum */
        float m = min == 0.0f ? 0.0f : -lows[at] / min;
        codes[at] = (uint8_t)clampf(round_away(c), 0.0f, 63.0f);
        mins[at] = (uint8_t)clampf(round_away(m), 0.0f, 63.0f);
    }
    memset(field, 0, fifth ? Q5_K_BYTES : Q4_K_BYTES);
    for (int at = 0; at < count; at++) oracle_put_scale_min_k4(field + 4, (uint32_t)at, codes[at], mins[at]);
    uint16_t h = oracle_f32_to_f16(scale);
    memcpy(field, &h, 2);
    h = oracle_f32_to_f16(min);
    memcpy(field + 2, &h, 2);
    for (int at = 0; at < count; at++) {
        float quantum = scale * (float)codes[at];
        float low = min * (float)mins[at];
        for (int within = 0; within < SUB_BLOCK; within++) {
            uint32_t code = 0;
            if (quantum != 0.0f) code = (uint32_t)clampf(round_away((values[at * SUB_BLOCK + within] + low) / quantum), 0.0f, steps);
            int group = at / 2;
            int seat = at % 2;
            field[quants + group * SUB_BLOCK + within] |= (uint8_t)((code & 0x0f) << (seat ? 4 : 0));
            if (fifth && (code & 0x10)) field[16 + within] |= (uint8_t)(1u << (2 * group + seat));
        }
    }
}

static void q4_k_encode(const float *values, uint8_t *field) { affine_encode(values, field, 0); }
static void q5_k_encode(const float *values, uint8_t *field) { affine_encode(values, field, 1); } /* ggml.rs:313-315 */

/* crates/neura-precision/src/ggml.rs:242-289: sixteen sub-blocks of 16, d = widest / 4 / 31, scale codes 32..63
 * (stored six bits: four in a nibble of bytes 96..103, two in bytes 104..107), codes round(x / (d * scale)) in -4..3 */
static void q3_k_encode(const float *values, uint8_t *field) {
    float peaks[16];
    for (int at = 0; at < 16; at++) {
        float peak = 0.0f;
        for (int i = 0; i < 16; i++) peak = greatest(peak, fabsf(values[at * 16 + i]));
        peaks[at] = peak;
    }
    float widest = 0.0f;
    for (int at = 0; at < 16; at++) widest = greatest(widest, peaks[at]);
    if (!(widest >= 1.17549435e-38f)) widest = 1.17549435e-38f; /* f32::max(MIN_POSITIVE) */
    float d = widest / 4.0f / 31.0f;
    uint32_t codes[16];
    for (int at = 0; at < 16; at++) codes[at] = (uint32_t)clampf(round_away(peaks[at] / 4.0f / d), 0.0f, 31.0f) + 32u;
    memset(field, 0, Q3_K_BYTES);
    for (uint32_t at = 0; at < 16; at++) { /* put_q3_k_scale, ggml.rs:231-240 */
        uint8_t low = (uint8_t)(codes[at] & 0x0f), high = (uint8_t)((codes[at] >> 4) & 3u);
        if (at < 8)
            field[96 + at] |= low;
        else
            field[96 + at - 8] |= (uint8_t)(low << 4);
        field[96 + 8 + at % 4] |= (uint8_t)(high << (2 * (at / 4)));
    }
    for (uint32_t at = 0; at < Q3_K_BLOCK; at++) {
        uint32_t sub = at / 16, lane = at % 16;
        float quantum = d * (float)(codes[sub] - 32u);
        int quant = 0;
        if (quantum != 0.0f) quant = (int)clampf(round_away(values[at] / quantum), -4.0f, 3.0f);
        uint32_t half = sub / 8, within = sub % 8, j = within / 2, second = within % 2;
        field[32 + half * 32 + second * 16 + lane] |= (uint8_t)(((uint32_t)quant & 3u) << (2 * j));
        if (quant >= 0) field[second * 16 + lane] |= (uint8_t)(1u << (half * 4 + j));
    }
    uint16_t h = oracle_f32_to_f16(d);
    memcpy(field + 108, &h, 2);
}

/* crates/neura-precision/src/ggml.rs:352-392.  Sixteen sub-blocks of 16: factor = largest magnitude / 32, super scale =
 * largest factor / 127 stored as f16 while the f32 value quantizes.  `quantized` (ggml.rs:120-125) converts the
 * rounded, clamped quotient to an unsigned integer, which in Rust saturates: every negative quotient becomes 0, so
 * negative values pack as code 32 (zero).  This follows the reference; a decoder never notices. */
static void q6_k_encode(const float *values, uint8_t *field) {
    float factors[16];
    for (int at = 0; at < 16; at++) {
        float size = 0.0f;
        for (int i = 0; i < 16; i++) {
            float a = fabsf(values[at * 16 + i]);
            if (size < a) size = a;
        }
        factors[at] = size / 32.0f;
    }
    float scale = 0.0f;
    for (int at = 0; at < 16; at++) scale = greatest(scale, fabsf(factors[at]));
    scale = scale / 127.0f;
    memset(field, 0, Q6_K_BYTES);
    uint16_t h = oracle_f32_to_f16(scale);
    memcpy(field + 208, &h, 2);
    for (int at = 0; at < 16; at++) {
        int8_t code = 0;
        if (scale != 0.0f) code = (int8_t)clampf(round_away(factors[at] / scale), -127.0f, 127.0f);
        field[192 + at] = (uint8_t)code;
        float factor = scale * (float)code;
        for (int within = 0; within < 16; within++) {
            int element = at * 16 + within;
            int half = element / 128, group = (element % 128) / 32, seat = element % 32;
            uint32_t quant = 0;
            if (factor != 0.0f) {
                float q = clampf(round_away(values[element] / factor), -32.0f, 31.0f);
                quant = q < 0.0f ? 0u : (uint32_t)q; /* a saturating float -> u32 cast */
            }
            quant += 32;
            uint8_t *byte = &field[half * 64 + (group % 2) * 32 + seat];
            if (group >= 2)
                *byte = (uint8_t)((*byte & 0x0f) | ((quant & 15u) << 4));
            else
                *byte = (uint8_t)((*byte & 0xf0) | (quant & 15u));
            field[128 + half * 32 + seat] |= (uint8_t)(((quant >> 4) & 3u) << (2 * group));
        }
    }
}

/* crates/neura-precision/src/ggml.rs:8-20 (pack); n must be whole blocks here */
int oracle_pack(int element, const float *values, uint64_t n, uint8_t *out) {
    if (element == EL_Q8_0) {
        if (n % Q8_0_BLOCK) return -1;
        for (uint64_t b = 0; b < n / Q8_0_BLOCK; b++) q8_0_encode(values + b * Q8_0_BLOCK, out + b * Q8_0_BYTES);
        return 0;
    }
    if (element == EL_Q4_K) {
        if (n % Q4_K_BLOCK) return -1;
        for (uint64_t b = 0; b < n / Q4_K_BLOCK; b++) q4_k_encode(values + b * Q4_K_BLOCK, out + b * Q4_K_BYTES);
        return 0;
    }
    if (element == EL_Q6_K) {
        if (n % Q6_K_BLOCK) return -1;
        for (uint64_t b = 0; b < n / Q6_K_BLOCK; b++) q6_k_encode(values + b * Q6_K_BLOCK, out + b * Q6_K_BYTES);
        return 0;
    }
    if (element == EL_Q5_K) {
        if (n % Q5_K_BLOCK) return -1;
        for (uint64_t b = 0; b < n / Q5_K_BLOCK; b++) q5_k_encode(values + b * Q5_K_BLOCK, out + b * Q5_K_BYTES);
        return 0;
    }
    if (element == EL_Q3_K) {
        if (n % Q3_K_BLOCK) return -1;
        for (uint64_t b = 0; b < n / Q3_K_BLOCK; b++) q3_k_encode(values + b * Q3_K_BLOCK, out + b * Q3_K_BYTES);
        return 0;
    }
    if (element == EL_F16) {
        oracle_f32_to_f16_many(values, n, (uint16_t *)out);
        return 0;
    }
    if (element == EL_F32) {
        memcpy(out, values, n * 4);
        return 0;
    }
    return -2;
}

uint64_t oracle_payload_bytes(int element, uint64_t elements) { /* neura-abi/src/element.rs:231-240 */
    switch (element) {
    case EL_Q8_0: return (elements + Q8_0_BLOCK - 1) / Q8_0_BLOCK * Q8_0_BYTES;
    case EL_Q4_K: return (elements + Q4_K_BLOCK - 1) / Q4_K_BLOCK * Q4_K_BYTES;
    case EL_Q6_K: return (elements + Q6_K_BLOCK - 1) / Q6_K_BLOCK * Q6_K_BYTES;
    case EL_Q5_K: return (elements + Q5_K_BLOCK - 1) / Q5_K_BLOCK * Q5_K_BYTES;
    case EL_Q3_K: return (elements + Q3_K_BLOCK - 1) / Q3_K_BLOCK * Q3_K_BYTES;
    case EL_F16: return elements * 2;
    case EL_F32: return elements * 4;
    default: return 0;
    }
}

/* ------------------------------------------------------------- matmul ---- */

/* one 32-element run of row `w_row` starting at element k0: Σ x[i]·w[i] in order.
 * Q8_0: crates/neura-kernel/src/dot.rs:471-542 (weight = f32(i8)·scale, then ·x)
 * Q4_K: crates/neura-kernel/src/dot.rs:583-619 (weight = scale·f32(q) − min) */
static float run_dot(int element, const uint8_t *w_row, uint32_t k0, const float *x, uint32_t last) {
    float total = 0.0f;
    if (element == EL_Q8_0) {
        const uint8_t *field = w_row + (size_t)(k0 / Q8_0_BLOCK) * Q8_0_BYTES;
        uint16_t h;
        memcpy(&h, field, 2);
        float scale = oracle_f16_to_f32(h);
        for (uint32_t at = 0; at < last; at++) total = total + x[k0 + at] * ((float)(int8_t)field[2 + at] * scale);
        return total;
    }
    if (element == EL_Q4_K) {
        const uint8_t *field = w_row + (size_t)(k0 / Q4_K_BLOCK) * Q4_K_BYTES;
        uint32_t within = k0 % Q4_K_BLOCK;
        uint32_t group = within / 64u, seat = (within % 64u) / SUB_BLOCK;
        uint32_t sc, m;
        oracle_scale_min_k4(field + 4, group * 2 + seat, &sc, &m);
        uint16_t h0, h1;
        memcpy(&h0, field, 2);
        memcpy(&h1, field + 2, 2);
        float scale = oracle_f16_to_f32(h0) * (float)sc;
        float min = oracle_f16_to_f32(h1) * (float)m;
        for (uint32_t at = 0; at < last; at++) {
            uint8_t byte = field[16 + group * 32 + at];
            uint32_t quant = seat ? (uint32_t)(byte >> 4) : (uint32_t)(byte & 0x0f);
            total = total + x[k0 + at] * (scale * (float)quant - min);
        }
        return total;
    }
    if (element == EL_Q6_K) { /* crates/neura-kernel/src/dot.rs:663-797: weight = (d * scale) * (code - 32), one scale per 16 */
        const uint8_t *field = w_row + (size_t)(k0 / Q6_K_BLOCK) * Q6_K_BYTES;
        uint32_t within = k0 % Q6_K_BLOCK;
        uint32_t side = within / 128u, group = (within % 128u) / SUB_BLOCK;
        uint16_t h;
        memcpy(&h, field + 208, 2);
        float width = oracle_f16_to_f32(h);
        float lower = width * (float)(int8_t)field[192 + side * 8 + group * 2];
        float upper = width * (float)(int8_t)field[192 + side * 8 + group * 2 + 1];
        for (uint32_t at = 0; at < last; at++) {
            uint8_t byte = field[side * 64 + (group % 2) * 32 + at];
            uint32_t nibble = group >= 2 ? (uint32_t)(byte >> 4) : (uint32_t)(byte & 0x0f);
            uint32_t quant = nibble | (((uint32_t)(field[128 + side * 32 + at] >> (2 * group)) & 3u) << 4);
            float weight = at >= 16 ? upper : lower;
            total = total + x[k0 + at] * (weight * ((float)quant - 32.0f));
        }
        return total;
    }
    if (element == EL_Q5_K) { /* crates/neura-kernel/src/dot.rs:621-661: weight = scale * f32(nibble | fifth << 4) - min */
        const uint8_t *field = w_row + (size_t)(k0 / Q5_K_BLOCK) * Q5_K_BYTES;
        uint32_t within = k0 % Q5_K_BLOCK;
        uint32_t group = within / 64u, seat = (within % 64u) / SUB_BLOCK;
        uint32_t sc, m;
        oracle_scale_min_k4(field + 4, group * 2 + seat, &sc, &m);
        uint16_t h0, h1;
        memcpy(&h0, field, 2);
        memcpy(&h1, field + 2, 2);
        float scale = oracle_f16_to_f32(h0) * (float)sc;
        float min = oracle_f16_to_f32(h1) * (float)m;
        for (uint32_t at = 0; at < last; at++) {
            uint8_t byte = field[48 + group * 32 + at];
            uint32_t nibble = seat ? (uint32_t)(byte >> 4) : (uint32_t)(byte & 0x0f);
            uint32_t quant = nibble | ((((uint32_t)field[16 + at] >> (2 * group + seat)) & 1u) << 4);
            total = total + x[k0 + at] * (scale * (float)quant - min);
        }
        return total;
    }
    if (element == EL_Q3_K) { /* crates/neura-kernel/src/dot.rs:544-581: weight = (d * (scale - 32)) * (pair - 4 unless the third bit is set) */
        const uint8_t *field = w_row + (size_t)(k0 / Q3_K_BLOCK) * Q3_K_BYTES;
        uint32_t within = k0 % Q3_K_BLOCK;
        uint32_t group = within / SUB_BLOCK, half = group / 4u, j = group % 4u;
        uint16_t h;
        memcpy(&h, field + 108, 2);
        float width = oracle_f16_to_f32(h);
        float scale0 = width * ((float)q3_k_scale(field, half * 8 + j * 2) - 32.0f);
        float scale1 = width * ((float)q3_k_scale(field, half * 8 + j * 2 + 1) - 32.0f);
        for (uint32_t at = 0; at < last; at++) {
            uint32_t low = ((uint32_t)field[32 + half * 32 + at] >> (2 * j)) & 3u;
            uint32_t high = ((uint32_t)field[at] >> (half * 4 + j)) & 1u;
            float scale = at >= 16 ? scale1 : scale0;
            float weight = scale * ((float)low - (high == 0u ? 4.0f : 0.0f));
            total = total + x[k0 + at] * weight;
        }
        return total;
    }
    if (element == EL_F16) {
        const uint16_t *w = (const uint16_t *)w_row;
        for (uint32_t at = 0; at < last; at++) total = total + x[k0 + at] * oracle_f16_to_f32(w[k0 + at]);
        return total;
    }
    const float *w = (const float *)w_row;
    for (uint32_t at = 0; at < last; at++) total = total + x[k0 + at] * w[k0 + at];
    return total;
}

static size_t row_bytes(int element, uint32_t K) { return (size_t)oracle_payload_bytes(element, K); }

/* One output of the folded narrow product, in the reference's order:
 * crates/neura-kernel/src/task/matmul.rs:376-517 (lane ℓ of 32 sums runs ℓ, ℓ+32, … of a
 * ≤1024-deep slot; the 32 lane partials are added serially :493-500) and
 * :1318-1333 (slot partials added serially); slots = ⌈K/1024⌉ (profile.rs:1503). */
static float folded_dot(int element, const uint8_t *w_row, uint32_t K, const float *x) {
    uint32_t depth_blocks = (K + SUB_BLOCK - 1) / SUB_BLOCK;
    uint32_t splits = (K + FOLDED_STAGE - 1) / FOLDED_STAGE;
    float out = 0.0f;
    for (uint32_t slot = 0; slot < splits; slot++) {
        uint32_t first_block = (uint32_t)(((uint64_t)slot * depth_blocks) / splits);
        uint32_t last_block = (uint32_t)(((uint64_t)(slot + 1) * depth_blocks) / splits);
        uint32_t blocks = last_block - first_block;
        float partial[FOLDED_LANES];
        for (uint32_t lane = 0; lane < FOLDED_LANES; lane++) {
            float acc = 0.0f;
            for (uint32_t chunk = 0; chunk < (blocks + FOLDED_LANES - 1) / FOLDED_LANES; chunk++) {
                uint32_t step = chunk * FOLDED_LANES + lane;
                uint32_t at = (first_block + step) * SUB_BLOCK;
                if (step < blocks && at < K) {
                    uint32_t last = (at + SUB_BLOCK < K ? at + SUB_BLOCK : K) - at;
                    acc = acc + run_dot(element, w_row, at, x, last);
                }
            }
            partial[lane] = acc;
        }
        float total = 0.0f;
        for (uint32_t other = 0; other < FOLDED_LANES; other++) total = total + partial[other];
        if (splits == 1) return total;
        out = out + total;
    }
    return out;
}

/* y[r][n] = Σ_k x[r][k]·W[n][k], W row-major [N][K] in `element` storage, order as above.
 * threads > 1 splits the N loop (every output keeps its own serial order). */
int oracle_gemv(int element, const uint8_t *W, uint32_t N, uint32_t K, const float *x, uint32_t rows, float *y, int threads) {
    if (element != EL_Q8_0 && element != EL_Q4_K && element != EL_Q6_K && element != EL_Q5_K && element != EL_Q3_K && element != EL_F16 && element != EL_F32) return -2;
    size_t stride = row_bytes(element, K);
    (void)threads;
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
    for (int64_t n = 0; n < (int64_t)N; n++)
        for (uint32_t r = 0; r < rows; r++) y[(size_t)r * N + n] = folded_dot(element, W + (size_t)n * stride, K, x + (size_t)r * K);
    return 0;
}

/* The reference's own test definition of a product: fp32 running sum over k of
 * unpack(W)[n][k]·x[m][k] (crates/neura-runtime/tests/runtime.rs:72-83, :130-142).
 * X is fp32 [M][K]; Y fp32 [M][N]. */
int oracle_gemm(int element, const uint8_t *W, uint32_t N, uint32_t K, const float *X, uint32_t M, float *Y, int threads) {
    size_t stride = row_bytes(element, K);
    if (!stride) return -2;
    int fail = 0;
    (void)threads;
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
    for (int64_t n = 0; n < (int64_t)N; n++) {
        float *w = (float *)malloc((size_t)K * 4);
        if (!w || oracle_unpack(element, W + (size_t)n * stride, K, w)) {
            fail = 1;
        } else {
            for (uint32_t m = 0; m < M; m++) {
                float total = 0.0f;
                const float *x = X + (size_t)m * K;
                for (uint32_t k = 0; k < K; k++) total += w[k] * x[k];
                Y[(size_t)m * N + n] = total;
            }
        }
        free(w);
    }
    return fail ? -1 : 0;
}

/* ------------------------------------------------------------ rmsnorm ---- */

/* crates/neura-kernel/src/task/norm.rs:55-130 (NORM_RMS branch) with the 256-thread tree
 * of crates/neura-kernel/src/task/reduce.rs:21-38.  residual (may be NULL) is the prelude
 * add read: value = x + residual; when sum_out != NULL it receives that sum (the staged row). */
void oracle_rmsnorm(const float *x, const float *residual, const float *w, float eps, uint32_t rows, uint32_t C, float *out, float *sum_out) {
    for (uint32_t row = 0; row < rows; row++) {
        const float *xr = x + (size_t)row * C;
        const float *rr = residual ? residual + (size_t)row * C : NULL;
        float scratch[WORKGROUP];
        for (uint32_t lid = 0; lid < WORKGROUP; lid++) {
            float square = 0.0f;
            for (uint32_t c = lid; c < C; c += WORKGROUP) {
                float value = rr ? xr[c] + rr[c] : xr[c];
                square = square + value * value;
            }
            scratch[lid] = square;
        }
        for (uint32_t stride = WORKGROUP / 2; stride > 0; stride /= 2)
            for (uint32_t lid = 0; lid < stride; lid++) scratch[lid] = scratch[lid] + scratch[lid + stride];
        float mean_square = scratch[0] / (float)C;
        float scale = 1.0f / sqrtf(mean_square + eps);
        for (uint32_t c = 0; c < C; c++) {
            float value = rr ? xr[c] + rr[c] : xr[c];
            if (sum_out) sum_out[(size_t)row * C + c] = value;
            float result = value * scale;
            if (w) result = result * w[c];
            out[(size_t)row * C + c] = result;
        }
    }
}

/* --------------------------------------------------------------- rope ---- */

/* crates/neura-kernel/src/task/rope.rs:48-50 */
float oracle_rope_angle(uint32_t position, uint32_t channel, uint32_t width, float base) {
    return (float)position * powf(base, -2.0f * (float)channel / (float)width);
}

/* crates/neura-kernel/src/task/rope.rs:95-122 on one [rows][width] head: rotate-half over all
 * `width` channels, position = origin + row.  In place is not allowed (reads partner). */
void oracle_rope(const float *in, uint32_t rows, uint32_t width, uint32_t origin, float base, float *out) {
    uint32_t half = width / 2;
    for (uint32_t row = 0; row < rows; row++) {
        for (uint32_t c = 0; c < width; c++) {
            int high = c >= half;
            uint32_t channel = high ? c - half : c;
            float angle = oracle_rope_angle(origin + row, channel, width, base);
            float value = in[(size_t)row * width + c];
            float partner = in[(size_t)row * width + (high ? c - half : c + half)];
            float cosine = cosf(angle), sine = sinf(angle);
            out[(size_t)row * width + c] = high ? value * cosine + partner * sine : value * cosine - partner * sine;
        }
    }
}

/* ---------------------------------------------------------- attention ---- */

static float softmax_exp(float a) { return expf(a > -104.0f ? a : -104.0f); } /* substrate.rs:110-116 */

/* crates/neura-kernel/src/task/attention.rs:103-108: the position the key in slot `at` of a ring of `keys` slots holds
 * once `written` positions have gone in -- the latest one below `written` that lands on the slot */
static uint32_t key_position(uint32_t at, uint32_t keys, uint32_t written) {
    if (written <= keys) return at;
    return at + keys * ((written - 1u - at) / keys);
}

/* crates/neura-kernel/src/task/attention.rs:136-163 (causal): the key in slot `at` is weighed by the query at `position` */
static int key_seen(uint32_t at, uint32_t keys, uint32_t written, uint32_t position, uint32_t reach) {
    if (at >= keys) return 0;
    uint32_t held = reach > 0 ? key_position(at, keys, written) : at;
    if (held > position) return 0;
    if (reach > 0 && position - held >= reach) return 0;
    return 1;
}

/* One number of a key / value state (crates/neura-kernel/src/fetch.rs:95-107: a half, the upper half of a single, or a single),
 * and the cast that puts it there (graph.cast, crates/neura-decoder/src/cache.rs:347-348; bfloat16 rounds to nearest even,
 * crates/neura-kernel/src/task/convert.rs:86-89 and crates/neura-precision/src/lib.rs:325-329). */
static float cache_value(const void *held, int element, size_t at) {
    if (element == EL_F32) return ((const float *)held)[at];
    if (element == EL_BF16) {
        uint32_t bits = (uint32_t)((const uint16_t *)held)[at] << 16;
        float value;
        memcpy(&value, &bits, 4);
        return value;
    }
    return oracle_f16_to_f32(((const uint16_t *)held)[at]);
}
static void cache_put(void *held, int element, size_t at, float value) {
    if (element == EL_F32) {
        ((float *)held)[at] = value;
    } else if (element == EL_BF16) {
        uint32_t bits;
        memcpy(&bits, &value, 4);
        ((uint16_t *)held)[at] = (uint16_t)((bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16);
    } else {
        ((uint16_t *)held)[at] = oracle_f32_to_f16(value);
    }
}
void oracle_cache_put_many(void *held, int element, uint64_t at, const float *values, uint64_t count) {
    for (uint64_t i = 0; i < count; i++) cache_put(held, element, at + i, values[i]);
}

/* Causal GQA attention over an fp16, bf16 or fp32 KV cache, fp32 online softmax in key blocks of 16
 * (crates/neura-kernel/src/task/attention.rs:309-617; visible :151-163; GQA head :327-334).
 *   q    [heads][batch][rows][width] f32
 *   K,V  [kv_heads][batch][capacity][width]  (kv_element: EL_F16, EL_BF16 or EL_F32)
 *   cursor[batch] = origin of each plane; key `at` visible iff at <= origin+row and at < keys
 *   reach: 0, or the span of a ring (Cache::windowed, crates/neura-decoder/src/cache.rs:366-406): slot `at` then holds
 *          position key_position(at), and a query weighs the last `reach` positions up to its own
 *   out  [heads][batch][rows][width]
 */
int oracle_attention(const float *q, const void *K, const void *V, int kv_element, uint32_t heads, uint32_t kv_heads, uint32_t batch,
                     uint32_t rows, uint32_t width, uint32_t capacity, uint32_t keys, uint32_t reach, const uint32_t *cursor, float scale,
                     float *out) {
    if (kv_element != EL_F16 && kv_element != EL_F32 && kv_element != EL_BF16) return -2;
    if (heads % kv_heads || width > 512) return -1;
    uint32_t groups = heads / kv_heads;
    for (uint32_t h = 0; h < heads; h++)
        for (uint32_t b = 0; b < batch; b++)
            for (uint32_t row = 0; row < rows; row++) {
                const float *qr = q + (((size_t)h * batch + b) * rows + row) * width;
                size_t plane = ((size_t)(h / groups) * batch + b) * capacity;
                uint32_t origin = cursor[b];
                uint32_t position = origin + row, written = origin + rows;
                uint32_t walked_keys = origin + rows < keys ? origin + rows : keys;
                float acc[512];
                for (uint32_t d = 0; d < width; d++) acc[d] = 0.0f;
                float largest = -INFINITY, total = 0.0f;
                for (uint32_t block = 0; block * ATTN_KEYS < walked_keys; block++) {
                    float weights[ATTN_KEYS];
                    float block_largest = -INFINITY;
                    uint32_t block_keys = 0;
                    for (uint32_t s = 0; s < ATTN_KEYS; s++) {
                        uint32_t at = block * ATTN_KEYS + s;
                        int seen = key_seen(at, keys, written, position, reach);
                        weights[s] = -INFINITY;
                        if (!seen) continue;
                        float score = 0.0f;
                        for (uint32_t d = 0; d < width; d++) {
                            float kv = cache_value(K, kv_element, (plane + at) * width + d);
                            score = score + qr[d] * kv;
                        }
                        weights[s] = score * scale;
                        block_keys++;
                        if (weights[s] > block_largest) block_largest = weights[s];
                    }
                    float next = largest > block_largest ? largest : block_largest;
                    float rescale = largest != -INFINITY ? softmax_exp(largest - next) : 1.0f;
                    largest = next;
                    total = total * rescale;
                    for (uint32_t d = 0; d < width; d++) acc[d] = acc[d] * rescale;
                    for (uint32_t s = 0; s < ATTN_KEYS; s++) {
                        uint32_t at = block * ATTN_KEYS + s;
                        if (!key_seen(at, keys, written, position, reach)) continue; /* an unseen key weighs exp(-104) ~ 0 there */
                        float weight = block_keys > 0 ? softmax_exp(weights[s] - largest) : 0.0f;
                        total = total + weight;
                        for (uint32_t d = 0; d < width; d++) {
                            float vv = cache_value(V, kv_element, (plane + at) * width + d);
                            acc[d] = acc[d] + weight * vv;
                        }
                    }
                }
                float normalized = total > 0.0f ? 1.0f / total : 0.0f;
                float *o = out + (((size_t)h * batch + b) * rows + row) * width;
                for (uint32_t d = 0; d < width; d++) o[d] = acc[d] * normalized;
            }
    return 0;
}

/* fp64 reference in the shape of crates/neura-runtime/tests/support/attention.rs:38-109
 * (no ring window: reach = 0).  K,V fp32 [kv_heads][batch][keys][width]. */
void oracle_attention_f64(const float *q, const float *K, const float *V, uint32_t heads, uint32_t kv_heads, uint32_t batch, uint32_t rows,
                          uint32_t width, uint32_t keys, uint32_t origin, int causal, float scale, float *out) {
    uint32_t groups = heads / kv_heads;
    double *logits = (double *)malloc(sizeof(double) * keys);
    for (uint32_t plane = 0; plane < heads * batch; plane++) {
        uint32_t head = plane / batch;
        size_t source = (size_t)(head / groups) * batch + plane % batch;
        for (uint32_t row = 0; row < rows; row++) {
            double largest = -INFINITY;
            for (uint32_t c = 0; c < keys; c++) {
                if (causal && c > origin + row) {
                    logits[c] = -INFINITY;
                    continue;
                }
                double s = 0.0;
                for (uint32_t d = 0; d < width; d++)
                    s += (double)q[((size_t)plane * rows + row) * width + d] * (double)K[(source * keys + c) * width + d];
                logits[c] = s * (double)scale;
                if (logits[c] > largest) largest = logits[c];
            }
            double total = 0.0;
            for (uint32_t c = 0; c < keys; c++) {
                logits[c] = exp(logits[c] - largest);
                total += logits[c];
            }
            for (uint32_t d = 0; d < width; d++) {
                double sum = 0.0;
                for (uint32_t c = 0; c < keys; c++) sum += logits[c] / total * (double)V[(source * keys + c) * width + d];
                out[((size_t)plane * rows + row) * width + d] = (float)sum;
            }
        }
    }
    free(logits);
}

/* ------------------------------------------------------------- argmax ---- */

/* crates/neura-kernel/src/task/choice.rs:46-51, :396-404: largest value, lowest index on ties */
uint32_t oracle_argmax(const float *values, uint32_t n) {
    uint32_t best = 0;
    for (uint32_t i = 1; i < n; i++)
        if (values[i] > values[best]) best = i;
    return best;
}

/* the two largest values (for reporting the greedy margin) */
void oracle_top2(const float *values, uint32_t n, float *first, float *second) {
    float a = -INFINITY, b = -INFINITY;
    for (uint32_t i = 0; i < n; i++) {
        if (values[i] > a) {
            b = a;
            a = values[i];
        } else if (values[i] > b) {
            b = values[i];
        }
    }
    *first = a;
    *second = b;
}

/* ------------------------------------------------------------- sample ---- */

typedef struct {
    uint32_t seed;     /* the 32 bits the kernel hashes (a batch writes seed_bits(seed), crates/neura-generate/src/batch.rs:1845-1847) */
    float temperature; /* logits * recip(temperature), crates/neura-generate/src/sampling.rs:82 */
    uint32_t keep;     /* 1..64 */
    float cumulative;  /* (0, 1] */
} oracle_draw;

/* crates/neura-kernel/src/task/choice.rs:81-89 over element_key((0, 0, 0, column)) (substrate.rs:146-152;
 * coordinates(column, dims) of a [1, 1, rows, columns] value puts the column in w and zero elsewhere, choice.rs:102-107) */
float oracle_gumbel_noise(uint32_t seed, uint32_t column) {
    uint32_t key = 0u * 0x9e3779b9u;
    key = (key ^ 0u) * 0x85ebca6bu;
    key = (key ^ 0u) * 0xc2b2ae35u;
    key = (key ^ column) * 0x27d4eb2fu;
    uint32_t hash = seed ^ (key * 0x9e3779b9u);
    hash = hash ^ (hash >> 16);
    hash = hash * 0x7feb352du;
    hash = hash ^ (hash >> 15);
    hash = hash * 0x846ca68bu;
    hash = hash ^ (hash >> 16);
    return -logf(-logf((float)(hash >> 8) * (1.0f / 16777216.0f)));
}

/* One row of crates/neura-kernel/src/task/choice.rs:933-989 (sample_row): the keep largest values (larger first, lower
 * column first among equals, :396-404), the nucleus boundary against cumulative * total, then the largest
 * value + noise (choice_precedes, :46-51).  The row's mass is summed in column order here; the reference sums it
 * over a workgroup tree (:891-931), which differs in the last bits only. */
static uint32_t sample_row(const float *logits, uint32_t n, oracle_draw draw) {
    float scale = 1.0f / draw.temperature;
    float *values = (float *)malloc((size_t)n * 4);
    for (uint32_t i = 0; i < n; i++) values[i] = logits[i] * scale;
    uint32_t chosen = 0xffffffffu;
    if (draw.keep == 1 && draw.cumulative == 1.0f) { /* :943-947 */
        chosen = oracle_argmax(values, n);
        free(values);
        return chosen;
    }
    float row_max = -INFINITY;
    for (uint32_t i = 0; i < n; i++)
        if (values[i] > row_max) row_max = values[i];
    float total = 0.0f;
    for (uint32_t i = 0; i < n; i++) total = total + softmax_exp(values[i] - row_max);
    /* rank_row: the next candidate is the best of those that rank after the previous one */
    float kept_value[64];
    uint32_t kept_index[64];
    uint32_t count = 0;
    float previous_value = INFINITY;
    uint32_t previous_index = 0xffffffffu;
    while (count < draw.keep && count < 64) {
        uint32_t best = 0xffffffffu;
        for (uint32_t i = 0; i < n; i++) {
            int after = previous_index == 0xffffffffu || values[i] < previous_value || (values[i] == previous_value && i > previous_index);
            if (!after) continue;
            if (best == 0xffffffffu || values[i] > values[best]) best = i; /* equal values: the lower index stays */
        }
        if (best == 0xffffffffu) break;
        kept_value[count] = values[best], kept_index[count] = best;
        previous_value = values[best], previous_index = best;
        count++;
    }
    float mass = 0.0f;
    for (uint32_t c = 0; c < count; c++) mass = mass + softmax_exp(kept_value[c] - row_max);
    float tail = total - mass;
    float threshold = draw.cumulative * total;
    uint32_t boundary = count;
    float running = 0.0f;
    for (uint32_t c = 0; c < count; c++) {
        running = running + softmax_exp(kept_value[c] - row_max);
        if (running + tail >= threshold && c + 1 < boundary) boundary = c + 1;
    }
    float best = -INFINITY;
    for (uint32_t c = 0; c < boundary; c++) {
        float weight = kept_value[c] + oracle_gumbel_noise(draw.seed, kept_index[c]);
        if (chosen == 0xffffffffu || weight > best || (weight == best && kept_index[c] < chosen)) best = weight, chosen = kept_index[c];
    }
    free(values);
    return chosen == 0xffffffffu ? 0u : chosen;
}

/* graph.sample over rows of n logits: out[r] drawn with draws[r] */
int oracle_sample(const float *logits, uint32_t rows, uint32_t n, const oracle_draw *draws, uint32_t *out) {
    for (uint32_t r = 0; r < rows; r++) {
        oracle_draw d = draws[r];
        if (!(d.temperature > 0.0f) || isinf(d.temperature) || d.keep < 1 || d.keep > 64 || !(d.cumulative > 0.0f) || !(d.cumulative <= 1.0f)) return -1;
        out[r] = sample_row(logits + (size_t)r * n, n, d);
    }
    return 0;
}

/* crates/neura-generate/src/batch.rs:1841-1847: the seed of plane `slot` under a batch seed, and the bits a batch writes */
uint32_t oracle_plane_seed(uint32_t seed, uint32_t slot) { return seed ^ ((slot + 1u) * 0x9e3779b9u); }
uint32_t oracle_seed_bits(uint32_t seed) { return 0x3f800000u | ((seed ^ (seed >> 23)) & 0x007fffffu); }

/* -------------------------------------------------------------- model ---- */

/* Qwen2-style decoder in the composition of examples/qwen/model.rs:92-103,
 * examples/qwen/attention.rs:98-154 (without the qwen35 q-gate and q/k norms) and
 * examples/qwen/mlp.rs:29-36.  All pointers are borrowed from the caller. */
typedef struct {
    uint32_t layers, hidden, heads, kv_heads, head_dim, ffn, vocab;
    uint32_t capacity; /* cache rows per (head, plane) */
    uint32_t window;   /* visible keys; scratch rows start at `window` */
    uint32_t batch;
    uint32_t ring;     /* 1: the window is a ring (Cache::windowed): position p sits in slot p % window */
    float rope_base, eps;
    int matrix_element;          /* element of every matrix (EL_Q8_0 / EL_Q4_K / EL_F16 / EL_F32) */
    const uint8_t *token_embd;   /* [vocab][hidden] in matrix_element */
    const uint8_t *output;       /* [vocab][hidden] or NULL = tied to token_embd */
    const float *output_norm;    /* [hidden] */
    const float **attn_norm;     /* [layers] -> [hidden] */
    const uint8_t **attn_q, **attn_k, **attn_v, **attn_o;
    const float **ffn_norm;
    const uint8_t **ffn_gate, **ffn_up, **ffn_down;
    uint16_t **cache_k, **cache_v; /* [layers] -> f16 [kv_heads][batch][capacity][head_dim] */
    /* optional (NULL = absent).  matrix_elements: the element of each matrix where they differ -- [token_embd, output, then per
     * layer attn_q, attn_k, attn_v, attn_output, ffn_gate, ffn_up, ffn_down].  attn_*_bias [layers] -> f32 [rows] or NULL entries:
     * Qwen2 checkpoints add a bias to q, k and v before the rotation; the reference's qwen example has none
     * (examples/qwen/attention.rs:98-154). */
    const int *matrix_elements;
    const float **attn_q_bias, **attn_k_bias, **attn_v_bias;
    int cache_element; /* what cache_k / cache_v hold: EL_F16, EL_BF16 or EL_F32 (Cache::new(.., element), cache.rs:130-134) */
} oracle_model;

static int element_of(const oracle_model *m, uint32_t slot) { return m->matrix_elements ? m->matrix_elements[slot] : m->matrix_element; }
static void add_bias(float *y, const float *bias, uint32_t rows, uint32_t n) {
    if (!bias) return;
    for (uint32_t r = 0; r < rows; r++)
        for (uint32_t c = 0; c < n; c++) y[(size_t)r * n + c] = y[(size_t)r * n + c] + bias[c];
}

/* crates/neura-kernel/src/pointwise.rs:66-68 and neura-pointwise/src/op.rs:163 */
static float silu(float a) { return a * (1.0f / (1.0f + expf(-a))); }

/* One forward pass of `rows` consecutive tokens per plane (rows = 1: the answer program of
 * crates/neura-generate/src/batch.rs:1716-1725; rows > 1: a fill chunk, :1434-1501).
 *   tokens [rows][batch] (row-major by row then plane, batch.rs:1450-1452)
 *   cursor [batch], mask [batch] (0 = inactive plane: hidden zeroed, K/V go to scratch rows)
 *   logits_out: NULL or [batch][vocab] for the LAST row; chosen_out: NULL or [batch]
 */
int oracle_model_forward(const oracle_model *m, const uint32_t *tokens, uint32_t rows, const uint32_t *cursor, const uint8_t *mask,
                         float *logits_out, uint32_t *chosen_out, int threads) {
    const uint32_t H = m->hidden, B = m->batch, hd = m->head_dim, QW = m->heads * hd, KW = m->kv_heads * hd, F = m->ffn;
    const uint32_t T = rows * B; /* flattened rows: index t = row*B + plane */
    const int el_embd = element_of(m, 0), el_head = m->output ? element_of(m, 1) : element_of(m, 0);
    const size_t embd_stride = row_bytes(el_embd, H);
    float *h = (float *)calloc((size_t)T * H, 4), *xn = (float *)malloc((size_t)T * H * 4);
    float *q = (float *)malloc((size_t)T * QW * 4), *k = (float *)malloc((size_t)T * KW * 4), *v = (float *)malloc((size_t)T * KW * 4);
    float *qh = (float *)malloc((size_t)T * QW * 4), *att = (float *)malloc((size_t)T * QW * 4), *attj = (float *)malloc((size_t)T * QW * 4);
    float *proj = (float *)malloc((size_t)T * H * 4), *g = (float *)malloc((size_t)T * F * 4), *u = (float *)malloc((size_t)T * F * 4);
    float *tmp = (float *)malloc((size_t)(hd > H ? hd : H) * 4);
    if (!h || !xn || !q || !k || !v || !qh || !att || !attj || !proj || !g || !u || !tmp) return -1;
    for (uint32_t t = 0; t < T; t++) {
        uint32_t b = t % B;
        if (tokens[t] >= m->vocab) return -3; /* refusal::INDEX, select.rs:38 */
        oracle_unpack(el_embd, m->token_embd + (size_t)tokens[t] * embd_stride, H, tmp);
        for (uint32_t c = 0; c < H; c++) h[(size_t)t * H + c] = tmp[c] * (mask[b] ? 1.0f : 0.0f);
    }
    for (uint32_t b = 0; b < B; b++)
        if (mask[b] && !m->ring && cursor[b] + rows > m->window) return -4; /* refusal::ORIGIN, attention.rs:250-252 (reach == 0) */
    float scale = 1.0f / sqrtf((float)hd);
    for (uint32_t L = 0; L < m->layers; L++) {
        oracle_rmsnorm(h, NULL, m->attn_norm[L], m->eps, T, H, xn, NULL);
        const uint32_t slot0 = 2 + 7 * L;
        oracle_gemv(element_of(m, slot0 + 0), m->attn_q[L], QW, H, xn, T, q, threads);
        oracle_gemv(element_of(m, slot0 + 1), m->attn_k[L], KW, H, xn, T, k, threads);
        oracle_gemv(element_of(m, slot0 + 2), m->attn_v[L], KW, H, xn, T, v, threads);
        add_bias(q, m->attn_q_bias ? m->attn_q_bias[L] : NULL, T, QW);
        add_bias(k, m->attn_k_bias ? m->attn_k_bias[L] : NULL, T, KW);
        add_bias(v, m->attn_v_bias ? m->attn_v_bias[L] : NULL, T, KW);
        /* heads + as_planes: q [T][heads*hd] -> qh [heads][B][rows][hd], roped at cursor+row */
        for (uint32_t t = 0; t < T; t++) {
            uint32_t row = t / B, b = t % B;
            for (uint32_t head = 0; head < m->heads; head++) {
                oracle_rope(q + (size_t)t * QW + head * hd, 1, hd, cursor[b] + row, m->rope_base, tmp);
                memcpy(qh + (((size_t)head * B + b) * rows + row) * hd, tmp, hd * 4);
            }
            for (uint32_t head = 0; head < m->kv_heads; head++) {
                /* slot math crates/neura-decoder/src/cache.rs:311-337, layout.rs:10-24 */
                /* a ring seats position p at p - window * floor(p / window) (layout.rs:32-36) */
                uint32_t seat = m->ring ? (cursor[b] + row) % m->window : cursor[b] + row;
                size_t slot = ((size_t)head * B + b) * m->capacity + (mask[b] ? seat : m->window + row);
                oracle_rope(k + (size_t)t * KW + head * hd, 1, hd, cursor[b] + row, m->rope_base, tmp);
                oracle_cache_put_many(m->cache_k[L], m->cache_element, slot * hd, tmp, hd);
                oracle_cache_put_many(m->cache_v[L], m->cache_element, slot * hd, v + (size_t)t * KW + head * hd, hd);
            }
        }
        oracle_attention(qh, m->cache_k[L], m->cache_v[L], m->cache_element, m->heads, m->kv_heads, B, rows, hd, m->capacity, m->window, m->ring ? m->window : 0u, cursor, scale, att);
        /* joined + as_rows: [heads][B][rows][hd] -> [T][heads*hd] */
        for (uint32_t t = 0; t < T; t++) {
            uint32_t row = t / B, b = t % B;
            for (uint32_t head = 0; head < m->heads; head++)
                memcpy(attj + (size_t)t * QW + head * hd, att + (((size_t)head * B + b) * rows + row) * hd, hd * 4);
        }
        oracle_gemv(element_of(m, slot0 + 3), m->attn_o[L], H, QW, attj, T, proj, threads);
        for (size_t i = 0; i < (size_t)T * H; i++) h[i] = h[i] + proj[i];
        oracle_rmsnorm(h, NULL, m->ffn_norm[L], m->eps, T, H, xn, NULL);
        oracle_gemv(element_of(m, slot0 + 4), m->ffn_gate[L], F, H, xn, T, g, threads);
        oracle_gemv(element_of(m, slot0 + 5), m->ffn_up[L], F, H, xn, T, u, threads);
        for (size_t i = 0; i < (size_t)T * F; i++) g[i] = silu(g[i]) * u[i];
        oracle_gemv(element_of(m, slot0 + 6), m->ffn_down[L], H, F, g, T, proj, threads);
        for (size_t i = 0; i < (size_t)T * H; i++) h[i] = (h[i] + proj[i]) * (mask[(i / H) % B] ? 1.0f : 0.0f);
    }
    if (logits_out || chosen_out) {
        float *logits = logits_out ? logits_out : (float *)malloc((size_t)B * m->vocab * 4);
        const float *last = h + (size_t)(rows - 1) * B * H;
        oracle_rmsnorm(last, NULL, m->output_norm, m->eps, B, H, xn, NULL);
        oracle_gemv(el_head, m->output ? m->output : m->token_embd, m->vocab, H, xn, B, logits, threads);
        if (chosen_out)
            for (uint32_t b = 0; b < B; b++) chosen_out[b] = oracle_argmax(logits + (size_t)b * m->vocab, m->vocab);
        if (!logits_out) free(logits);
    }
    free(h); free(xn); free(q); free(k); free(v); free(qh); free(att); free(attj); free(proj); free(g); free(u); free(tmp);
    return 0;
}
