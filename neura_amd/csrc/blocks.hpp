// Device-side readers of raw ggml blocks and fp16 helpers.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

#include "../../include/neura_hip.h"

namespace nh {

__device__ __forceinline__ float half_to_float(uint16_t bits) {
    return (float)__builtin_bit_cast(_Float16, bits);  // exact
}

// fp32 -> fp16, round to nearest even, subnormals kept, NaN -> sign|0x7e00
// (crates/neura-kernel/src/task/convert.rs:57-84)
__device__ __forceinline__ uint16_t float_to_half(float value) {
    uint32_t bits = __builtin_bit_cast(uint32_t, value);
    if ((bits & 0x7fffffffu) > 0x7f800000u) return (uint16_t)(((bits >> 16) & 0x8000u) | 0x7e00u);
    return __builtin_bit_cast(uint16_t, (_Float16)value);
}

// exp(max(argument, -104)) (crates/neura-kernel/src/substrate.rs:110-116)
// e^argument for the arguments a running softmax meets (never above zero; -inf gives 0, below -104 the result is zero in
// single precision anyway).  One hardware exp2 of argument * log2(e), the product carried in two parts so the result keeps
// the accuracy of the instruction; no branches, so a lane's eight weights of a tile stay one straight run of instructions.
__device__ __forceinline__ float softmax_exp(float argument) {
    const float x = fmaxf(argument, -104.0f);
    const float scaled = x * 1.44269502e+00f;
    const float rest = fmaf(x, 1.44269502e+00f, -scaled) + x * 1.92596299e-08f;  // what the rounded product left out
    const float power = __builtin_amdgcn_exp2f(scaled);
    return fmaf(power, rest * 6.93147182e-01f, power);
}

// round to nearest even, as the reference's device casts (crates/neura-kernel/src/task/convert.rs:86-89)
__device__ __forceinline__ uint16_t float_to_bfloat16(float value) {
    const uint32_t bits = __builtin_bit_cast(uint32_t, value);
    return (uint16_t)((bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16);
}

// one number of a key / value state held in CE = NH_F16, NH_BF16 or NH_F32 (crates/neura-kernel/src/fetch.rs:95-107)
template <int CE>
__device__ __forceinline__ void cache_store(void *base, uint64_t at, float value) {
    if (CE == NH_F32) static_cast<float *>(base)[at] = value;
    else if (CE == NH_BF16) static_cast<uint16_t *>(base)[at] = float_to_bfloat16(value);
    else static_cast<uint16_t *>(base)[at] = float_to_half(value);
}
template <int CE>
__device__ __forceinline__ float cache_load(const void *base, uint64_t at) {
    if (CE == NH_F32) return static_cast<const float *>(base)[at];
    if (CE == NH_BF16) return __builtin_bit_cast(float, (uint32_t)static_cast<const uint16_t *>(base)[at] << 16);
    return half_to_float(static_cast<const uint16_t *>(base)[at]);
}

__device__ __forceinline__ uint16_t load_u16(const uint8_t *p) { return *reinterpret_cast<const uint16_t *>(p); }

// 6-bit scale and min `j` (0..7) of a Q4_K super-block from its 12 scale bytes
// (crates/neura-precision/src/ggml.rs:127-136)
__device__ __forceinline__ void scale_min_k4(const uint8_t *s, uint32_t j, uint32_t &scale, uint32_t &min) {
    if (j < 4) {
        scale = s[j] & 63u;
        min = s[j + 4] & 63u;
    } else {
        scale = (uint32_t)(s[j + 4] & 0x0fu) | ((uint32_t)(s[j - 4] >> 6) << 4);
        min = (uint32_t)(s[j + 4] >> 4) | ((uint32_t)(s[j] >> 6) << 4);
    }
}

// element `i` of a row of Q8_0 blocks (crates/neura-precision/src/ggml.rs:211-216)
__device__ __forceinline__ float q8_0_element(const uint8_t *row, uint64_t i) {
    const uint8_t *block = row + (i / 32) * 34;
    float quantum = half_to_float(load_u16(block));
    return (float)(int8_t)block[2 + (i % 32)] * quantum;
}

// element `i` of a row of Q4_K blocks (crates/neura-precision/src/ggml.rs:336-350): the product
// scale*code and the product min*offset are each rounded before the subtract
__device__ __forceinline__ float q4_k_element(const uint8_t *row, uint64_t i) {
    const uint8_t *block = row + (i / 256) * 144;
    uint32_t within = (uint32_t)(i % 256);
    uint32_t group = within / 64, seat = (within % 64) / 32, lane = within % 32;
    uint32_t code, offset;
    scale_min_k4(block + 4, group * 2 + seat, code, offset);
    float quantum = __fmul_rn(half_to_float(load_u16(block)), (float)code);
    float low = __fmul_rn(half_to_float(load_u16(block + 2)), (float)offset);
    uint8_t byte = block[16 + group * 32 + lane];
    uint32_t quant = seat ? (uint32_t)(byte >> 4) : (uint32_t)(byte & 0x0f);
    return __fsub_rn(__fmul_rn(quantum, (float)quant), low);
}

// element `i` of a row of Q6_K blocks (crates/neura-precision/src/ggml.rs:394-407): d * scale, rounded, times (code - 32)
__device__ __forceinline__ float q6_k_element(const uint8_t *row, uint64_t i) {
    const uint8_t *block = row + (i / 256) * 210;
    uint32_t within = (uint32_t)(i % 256);
    uint32_t half = within / 128, group = (within % 128) / 32, lane = within % 32;
    uint8_t packed = block[half * 64 + (group % 2) * 32 + lane];
    uint32_t low = group >= 2 ? (uint32_t)(packed >> 4) : (uint32_t)(packed & 0x0f);
    uint32_t high = ((uint32_t)block[128 + half * 32 + lane] >> (2 * group)) & 3u;
    float scale = (float)(int8_t)block[192 + half * 8 + group * 2 + lane / 16];
    float quantum = __fmul_rn(half_to_float(load_u16(block + 208)), scale);
    return __fmul_rn(quantum, (float)(low | (high << 4)) - 32.0f);
}

// element `i` of a row of Q5_K blocks (crates/neura-precision/src/ggml.rs:321-335): Q4_K's walk with a fifth bit per code
__device__ __forceinline__ float q5_k_element(const uint8_t *row, uint64_t i) {
    const uint8_t *block = row + (i / 256) * 176;
    uint32_t within = (uint32_t)(i % 256);
    uint32_t group = within / 64, seat = (within % 64) / 32, lane = within % 32;
    uint32_t code, offset;
    scale_min_k4(block + 4, group * 2 + seat, code, offset);
    float quantum = __fmul_rn(half_to_float(load_u16(block)), (float)code);
    float low = __fmul_rn(half_to_float(load_u16(block + 2)), (float)offset);
    uint8_t byte = block[48 + group * 32 + lane];
    uint32_t quant = (seat ? (uint32_t)(byte >> 4) : (uint32_t)(byte & 0x0f)) | ((((uint32_t)block[16 + lane] >> (2 * group + seat)) & 1u) << 4);
    return __fsub_rn(__fmul_rn(quantum, (float)quant), low);
}

// 6-bit scale `at` (0..15) of a Q3_K super-block, as stored (32 too large): crates/neura-precision/src/ggml.rs:224-229
__device__ __forceinline__ uint32_t q3_k_scale(const uint8_t *block, uint32_t at) {
    uint32_t low = block[96 + at % 8];
    uint32_t nibble = at < 8 ? (low & 0x0fu) : (low >> 4);
    uint32_t high = block[104 + at % 4];
    return nibble | (((high >> (2 * (at / 4))) & 3u) << 4);
}

// element `i` of a row of Q3_K blocks (crates/neura-precision/src/ggml.rs:291-306): d * (scale - 32), rounded, times the
// code: the bit pair, less 4 unless the third bit is set
__device__ __forceinline__ float q3_k_element(const uint8_t *row, uint64_t i) {
    const uint8_t *block = row + (i / 256) * 110;
    uint32_t within = (uint32_t)(i % 256);
    uint32_t sub = within / 16, lane = within % 16;
    uint32_t half = sub / 8, j = (sub % 8) / 2, second = sub % 2;
    uint32_t low = ((uint32_t)block[32 + half * 32 + second * 16 + lane] >> (2 * j)) & 3u;
    uint32_t high = ((uint32_t)block[second * 16 + lane] >> (half * 4 + j)) & 1u;
    float quantum = __fmul_rn(half_to_float(load_u16(block + 108)), (float)q3_k_scale(block, sub) - 32.0f);
    return __fmul_rn(quantum, (float)low - (high ? 0.0f : 4.0f));
}

// element `i` of a row stored as ELEMENT
template <int ELEMENT>
__device__ __forceinline__ float stored_element(const uint8_t *row, uint64_t i) {
    if (ELEMENT == NH_Q8_0) return q8_0_element(row, i);
    if (ELEMENT == NH_Q3_K) return q3_k_element(row, i);
    if (ELEMENT == NH_Q4_K) return q4_k_element(row, i);
    if (ELEMENT == NH_Q5_K) return q5_k_element(row, i);
    if (ELEMENT == NH_Q6_K) return q6_k_element(row, i);
    if (ELEMENT == NH_F16) return half_to_float(reinterpret_cast<const uint16_t *>(row)[i]);
    return reinterpret_cast<const float *>(row)[i];
}

// 1 / sqrt(total / columns + eps) with every step rounded to fp32 exactly as IEEE does
// (crates/neura-kernel/src/task/norm.rs:102-104).  Each step runs in fp64 and is rounded
// once more to fp32, which for /, + and sqrt equals the correctly rounded fp32 operation.
__device__ __forceinline__ float rms_scale_of(float total, uint32_t columns, float eps) {
    float mean = (float)((double)total / (double)(float)columns);
    float shifted = (float)((double)mean + (double)eps);
    float root = (float)sqrt((double)shifted);
    return (float)(1.0 / (double)root);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, 64);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset, 64));
    return v;
}

}  // namespace nh
