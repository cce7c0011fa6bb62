// Causal grouped-query attention over an fp16 K/V cache (flash-decoding form).
//
// One workgroup serves one (kv head, plane, query row, key section): the `groups` query
// heads that share the kv head ride along, so every K/V row is fetched once for all of them.
// A key row of `WIDTH` halves is read by WIDTH/8 lanes with one 128-bit load each; a wave
// therefore walks 64/(WIDTH/8) keys per step and the four waves of a workgroup interleave.
// Every lane keeps a running (max, sum, accumulator) for its own key stream; streams are
// merged with shuffles inside a wave, through LDS across waves, and across sections by a
// second kernel (crates/neura-kernel/src/task/attention.rs:619-671 does the same fold).
// The K/V rows of two steps ahead are always in flight.
#include "blocks.hpp"
#include "common.hpp"

#include <cstdlib>

namespace nh {

constexpr int MAX_GROUPS = 8;

struct AttentionParams {
    const float *q;
    float *out;
    float *partial;      // [unit][section][group][width + 2] when sections > 1
    uint64_t q_sh, q_sb, q_sr, o_sh, o_sb, o_sr;
    const uint16_t *cache_k, *cache_v;
    uint32_t heads, kv_heads, groups, batch, rows, capacity, keys, sections;
    const uint32_t *cursor;
    float scale;
    uint32_t *refusal;
};

__device__ __forceinline__ void unpack8(const uint4 &raw, float (&out)[8]) {
    const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
        out[2 * j] = half_to_float((uint16_t)(words[j] & 0xffffu));
        out[2 * j + 1] = half_to_float((uint16_t)(words[j] >> 16));
    }
}

// exp(max(argument, -104)) (crates/neura-kernel/src/substrate.rs:110-116)
__device__ __forceinline__ float softmax_exp(float argument) { return expf(fmaxf(argument, -104.0f)); }

// sum over the LPK lanes that share a key: DPP adds inside a row of 16 lanes
template <int LPK>
__device__ __forceinline__ float key_sum(float v) {
    static_assert(LPK == 4 || LPK == 8 || LPK == 16 || LPK == 32, "lanes per key");
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, false));  // lane ^ 1
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, false));  // lane ^ 2
    if (LPK >= 8) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false));  // half mirror: the other quad of 8
    if (LPK >= 16) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, false));  // mirror: the other half of 16
    if (LPK >= 32) v += __shfl_xor(v, 16, 64);
    return v;
}

template <int WIDTH>
__global__ __launch_bounds__(256) void attention_kernel(AttentionParams p) {
    constexpr int LPK = WIDTH / 8;   // lanes per key
    constexpr int KPW = 64 / LPK;    // keys per wave step
    __shared__ float merged[4][MAX_GROUPS][WIDTH + 2];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t sub = lane / LPK, dl = lane % LPK;
    const uint32_t unit = blockIdx.x;  // (kv head, plane, row)
    const uint32_t row = unit % p.rows;
    const uint32_t b = (unit / p.rows) % p.batch, kvh = unit / p.rows / p.batch;
    const uint32_t section = blockIdx.y;
    const uint32_t G = p.groups;

    // A section is a fixed span of the window, whatever the cursor says: the K and V rows of its first two
    // steps go out before the cursor has even arrived (rows past the visible keys are fetched and dropped).
    const uint32_t chunk = (p.keys + p.sections - 1u) / p.sections;
    const uint32_t begin = min(p.keys, section * chunk);
    const uint64_t plane = ((uint64_t)kvh * p.batch + b) * p.capacity;
    const uint32_t step = 4u * KPW;
    uint32_t key = begin + wave * KPW + sub;
    uint4 kraw[2], vraw[2];
#pragma unroll
    for (int ahead = 0; ahead < 2; ahead++) {
        const uint32_t at_key = min(key + ahead * step, p.capacity - 1u);
        const uint64_t at = (plane + at_key) * WIDTH + dl * 8u;
        kraw[ahead] = *reinterpret_cast<const uint4 *>(p.cache_k + at);
        vraw[ahead] = *reinterpret_cast<const uint4 *>(p.cache_v + at);
    }

    uint32_t origin = p.cursor ? p.cursor[b] : 0u;
    if (origin + p.rows > p.keys) {  // refusal::ORIGIN (attention.rs:250-252)
        if (tid == 0) atomicMax(p.refusal, (uint32_t)REFUSAL_ORIGIN);
        origin = p.keys - p.rows;
    }
    const uint32_t visible = min(p.keys, origin + row + 1u);  // key `at` counts iff at <= origin + row
    const uint32_t last = min(visible, begin + chunk);

    float qr[MAX_GROUPS][8], acc[MAX_GROUPS][8], top[MAX_GROUPS], mass[MAX_GROUPS];
#pragma unroll
    for (int g = 0; g < MAX_GROUPS; g++) {
        top[g] = -INFINITY;
        mass[g] = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; j++) acc[g][j] = 0.0f, qr[g][j] = 0.0f;
        if (g < (int)G) {
            const float *src = p.q + (uint64_t)(kvh * G + g) * p.q_sh + (uint64_t)b * p.q_sb + (uint64_t)row * p.q_sr + dl * 8u;
#pragma unroll
            for (int j = 0; j < 8; j++) qr[g][j] = src[j];
        }
    }
    for (; key < last; key += 2u * step) {
#pragma unroll
        for (int phase = 0; phase < 2; phase++) {
            const uint32_t now = key + phase * step;
            float kf[8], vf[8];
            unpack8(kraw[phase], kf);
            unpack8(vraw[phase], vf);
            {  // the loads of two steps ahead reuse this phase's registers
                const uint32_t at_key = min(now + 2u * step, p.capacity - 1u);
                const uint64_t at = (plane + at_key) * WIDTH + dl * 8u;
                kraw[phase] = *reinterpret_cast<const uint4 *>(p.cache_k + at);
                vraw[phase] = *reinterpret_cast<const uint4 *>(p.cache_v + at);
            }
            if (now < last) {
#pragma unroll
                for (int g = 0; g < MAX_GROUPS; g++) {
                    if (g >= (int)G) break;
                    float score = 0.0f;
#pragma unroll
                    for (int j = 0; j < 8; j++) score = fmaf(qr[g][j], kf[j], score);
                    score = key_sum<LPK>(score) * p.scale;
                    float next = fmaxf(top[g], score);
                    float rescale = top[g] == -INFINITY ? 0.0f : softmax_exp(top[g] - next);
                    float weight = softmax_exp(score - next);
                    top[g] = next;
                    mass[g] = fmaf(mass[g], rescale, weight);
#pragma unroll
                    for (int j = 0; j < 8; j++) acc[g][j] = fmaf(acc[g][j], rescale, weight * vf[j]);
                }
            }
        }
    }
    // merge the KPW key streams of a wave: lanes with the same dl
#pragma unroll
    for (int g = 0; g < MAX_GROUPS; g++) {
        if (g >= (int)G) break;
#pragma unroll
        for (int offset = LPK; offset < 64; offset <<= 1) {
            float other_top = __shfl_xor(top[g], offset, 64);
            float other_mass = __shfl_xor(mass[g], offset, 64);
            float next = fmaxf(top[g], other_top);
            float mine = top[g] == -INFINITY ? 0.0f : softmax_exp(top[g] - next);
            float theirs = other_top == -INFINITY ? 0.0f : softmax_exp(other_top - next);
            mass[g] = mass[g] * mine + other_mass * theirs;
#pragma unroll
            for (int j = 0; j < 8; j++) acc[g][j] = acc[g][j] * mine + __shfl_xor(acc[g][j], offset, 64) * theirs;
            top[g] = next;
        }
        if (sub == 0) {
#pragma unroll
            for (int j = 0; j < 8; j++) merged[wave][g][dl * 8 + j] = acc[g][j];
            if (dl == 0) {
                merged[wave][g][WIDTH] = top[g];
                merged[wave][g][WIDTH + 1] = mass[g];
            }
        }
    }
    __syncthreads();
    // merge the four waves; thread -> (group, channel)
    for (uint32_t index = tid; index < G * WIDTH; index += 256) {
        uint32_t g = index / WIDTH, c = index % WIDTH;
        float largest = -INFINITY;
#pragma unroll
        for (int w = 0; w < 4; w++) largest = fmaxf(largest, merged[w][g][WIDTH]);
        float total = 0.0f, value = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            float held = merged[w][g][WIDTH];
            float weight = held == -INFINITY ? 0.0f : softmax_exp(held - largest);
            total += merged[w][g][WIDTH + 1] * weight;
            value += merged[w][g][c] * weight;
        }
        const uint32_t head = kvh * G + g;
        if (p.sections > 1) {
            float *dst = p.partial + (((uint64_t)unit * p.sections + section) * G + g) * (WIDTH + 2);
            dst[c] = value;
            if (c == 0) {
                dst[WIDTH] = largest;
                dst[WIDTH + 1] = total;
            }
        } else {
            float normalized = total > 0.0f ? 1.0f / total : 0.0f;
            p.out[(uint64_t)head * p.o_sh + (uint64_t)b * p.o_sb + (uint64_t)row * p.o_sr + c] = value * normalized;
        }
    }
}

// Fold of the sections of one (unit, query head): crates/neura-kernel/src/task/attention.rs:619-671.
// One workgroup per (unit, group, block of 32 channels).  Thread s first turns the statistics of
// section s into its weight; then thread (channel, stripe) sums its channel over every eighth
// section -- all of its loads in flight at once -- and the eight stripes meet in LDS.
__global__ __launch_bounds__(256) void attention_fold_kernel(AttentionParams p, uint32_t width) {
    __shared__ float weights[256], masses[256], held[256], stripes[8][32];
    const uint32_t G = p.groups, tid = threadIdx.x;
    const uint32_t blocks = (width + 31u) / 32u;
    const uint32_t cblock = blockIdx.x % blocks, ug = blockIdx.x / blocks;
    const uint32_t unit = ug / G, g = ug % G;
    const uint32_t row = unit % p.rows;
    const uint32_t b = (unit / p.rows) % p.batch, kvh = unit / p.rows / p.batch;
    const float *src = p.partial + ((uint64_t)unit * p.sections * G + g) * (width + 2);
    const uint64_t hop = (uint64_t)G * (width + 2);  // one section further
    float top = -INFINITY, mass = 0.0f;
    if (tid < p.sections) {
        top = src[tid * hop + width];
        mass = src[tid * hop + width + 1];
    }
    // the channel sums do not wait for the weights: fetch first
    const uint32_t c = cblock * 32u + (tid & 31u), stripe = tid >> 5;
    float values[32];
#pragma unroll
    for (int j = 0; j < 32; j++) {
        const uint32_t s = stripe + 8u * j;
        values[j] = (s < p.sections && c < width) ? src[s * hop + c] : 0.0f;
    }
    held[tid] = top;
    __syncthreads();
    for (uint32_t stride = 128; stride > 0; stride >>= 1) {
        if (tid < stride) held[tid] = fmaxf(held[tid], held[tid + stride]);
        __syncthreads();
    }
    const float largest = held[0];
    const float weight = top == -INFINITY ? 0.0f : softmax_exp(top - largest);
    weights[tid] = weight;
    masses[tid] = mass * weight;
    __syncthreads();
    float total = 0.0f;
    for (uint32_t s = 0; s < p.sections; s++) total += masses[s];
    const float normalized = total > 0.0f ? 1.0f / total : 0.0f;
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < 32; j++) {
        const uint32_t s = stripe + 8u * j;
        if (s < p.sections) sum = fmaf(values[j], weights[s], sum);
    }
    stripes[stripe][tid & 31u] = sum;
    __syncthreads();
    if (tid < 32 && c < width) {
        float value = ((stripes[0][tid] + stripes[1][tid]) + (stripes[2][tid] + stripes[3][tid])) +
                      ((stripes[4][tid] + stripes[5][tid]) + (stripes[6][tid] + stripes[7][tid]));
        p.out[(uint64_t)(kvh * G + g) * p.o_sh + (uint64_t)b * p.o_sb + (uint64_t)row * p.o_sr + c] = value * normalized;
    }
}

int32_t launch_attention(nh_device *d, const AttentionArgs &a) {
    AttentionParams p{};
    p.q = a.q, p.out = a.out;
    p.q_sh = a.q_sh, p.q_sb = a.q_sb, p.q_sr = a.q_sr, p.o_sh = a.o_sh, p.o_sb = a.o_sb, p.o_sr = a.o_sr;
    p.cache_k = a.cache_k, p.cache_v = a.cache_v;
    p.heads = a.heads, p.kv_heads = a.kv_heads, p.groups = a.heads / a.kv_heads;
    p.batch = a.batch, p.rows = a.rows, p.capacity = a.capacity, p.keys = a.keys;
    p.cursor = a.cursor, p.scale = a.scale, p.refusal = d->refusal;
    if (p.groups > (uint32_t)MAX_GROUPS) return fail(NH_E_ARGUMENT, "%u query heads share a key head where this kernel rides %d", p.groups, MAX_GROUPS);
    uint32_t units = a.kv_heads * a.batch * a.rows;
    if (!units) return NH_OK;
    // sections of the context: enough workgroups to fill the chip four times over, none thinner
    // than 64 keys (thinner sections cost more in the fold than they gain in the walk)
    const char *held = getenv("NEURA_HIP_ATTENTION_KEYS");
    const uint32_t thinnest = held && atoi(held) > 0 ? (uint32_t)atoi(held) : 64u;
    uint32_t wanted = ((uint32_t)d->compute_units * 4 + units - 1) / units;
    uint32_t most = (a.keys + thinnest - 1) / thinnest;
    p.sections = wanted < 1 ? 1 : (wanted > most ? most : wanted);
    if (p.sections > 256) p.sections = 256;
    if (p.sections > 1) {
        p.partial = static_cast<float *>(scratch(d, (size_t)p.sections * a.heads * a.batch * a.rows * (a.width + 2) * sizeof(float)));
        if (!p.partial) return NH_E_MEMORY;
    }
    dim3 grid(units, p.sections), block(256);
    switch (a.width) {
    case 32: hipLaunchKernelGGL(attention_kernel<32>, grid, block, 0, d->stream, p); break;
    case 64: hipLaunchKernelGGL(attention_kernel<64>, grid, block, 0, d->stream, p); break;
    case 128: hipLaunchKernelGGL(attention_kernel<128>, grid, block, 0, d->stream, p); break;
    case 256: hipLaunchKernelGGL(attention_kernel<256>, grid, block, 0, d->stream, p); break;
    default: return fail(NH_E_ARGUMENT, "a head of %u numbers fits none of the widths 32, 64, 128, 256 this kernel walks", a.width);
    }
    NH_HIP(hipGetLastError());
    if (p.sections > 1) {
        hipLaunchKernelGGL(attention_fold_kernel, dim3(units * p.groups * ((a.width + 31) / 32)), dim3(256), 0, d->stream, p, a.width);
        NH_HIP(hipGetLastError());
    }
    return NH_OK;
}

}  // namespace nh
