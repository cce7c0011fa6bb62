// Causal grouped-query attention over an fp16 K/V cache (flash-decoding form).
//
// One workgroup serves one (kv head, plane, query row, key section): the `groups` query
// heads that share the kv head ride along, so every K/V row is fetched once for all of them.
// A key row of `WIDTH` halves is read by WIDTH/8 lanes with one 128-bit load each; a wave
// therefore walks 64/(WIDTH/8) keys per step and the four waves of a workgroup interleave.
// Every lane keeps a running (max, sum, accumulator) for its own key stream; streams are
// merged with shuffles inside a wave, through LDS across waves, and across sections by a
// second kernel (crates/neura-kernel/src/task/attention.rs:619-671 does the same fold).
#include "blocks.hpp"
#include "common.hpp"

namespace nh {

constexpr int MAX_GROUPS = 8;

struct AttentionParams {
    const float *q;
    float *out;
    float *partial;  // [sections][heads][batch][rows][width + 2] when sections > 1
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

template <int WIDTH>
__global__ __launch_bounds__(256) void attention_kernel(AttentionParams p) {
    constexpr int LPK = WIDTH / 8;   // lanes per key
    constexpr int KPW = 64 / LPK;    // keys per wave step
    __shared__ float merged[4][MAX_GROUPS][WIDTH + 2];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t sub = lane / LPK, dl = lane % LPK;
    uint32_t unit = blockIdx.x;  // (kv head, plane, row)
    const uint32_t row = unit % p.rows;
    unit /= p.rows;
    const uint32_t b = unit % p.batch, kvh = unit / p.batch;
    const uint32_t section = blockIdx.y;
    const uint32_t G = p.groups;

    uint32_t origin = p.cursor ? p.cursor[b] : 0u;
    if (origin + p.rows > p.keys) {  // refusal::ORIGIN (attention.rs:250-252)
        if (tid == 0) atomicMax(p.refusal, (uint32_t)REFUSAL_ORIGIN);
        origin = p.keys - p.rows;
    }
    const uint32_t visible = min(p.keys, origin + row + 1u);  // key `at` counts iff at <= origin + row
    const uint32_t chunk = (visible + p.sections - 1u) / p.sections;
    const uint32_t first = min(visible, section * chunk), last = min(visible, first + chunk);

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
    const uint64_t plane = ((uint64_t)kvh * p.batch + b) * p.capacity;
    for (uint32_t key = first + wave * KPW + sub; key < last; key += 4u * KPW) {
        const uint64_t at = (plane + key) * WIDTH + dl * 8u;
        uint4 kraw = *reinterpret_cast<const uint4 *>(p.cache_k + at);
        uint4 vraw = *reinterpret_cast<const uint4 *>(p.cache_v + at);
        float kf[8], vf[8];
        unpack8(kraw, kf);
        unpack8(vraw, vf);
#pragma unroll
        for (int g = 0; g < MAX_GROUPS; g++) {
            if (g >= (int)G) break;
            float score = 0.0f;
#pragma unroll
            for (int j = 0; j < 8; j++) score = fmaf(qr[g][j], kf[j], score);
#pragma unroll
            for (int offset = LPK / 2; offset > 0; offset >>= 1) score += __shfl_xor(score, offset, 64);
            score *= p.scale;
            float next = fmaxf(top[g], score);
            float rescale = top[g] == -INFINITY ? 0.0f : softmax_exp(top[g] - next);
            float weight = softmax_exp(score - next);
            top[g] = next;
            mass[g] = mass[g] * rescale + weight;
#pragma unroll
            for (int j = 0; j < 8; j++) acc[g][j] = acc[g][j] * rescale + weight * vf[j];
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
            float *dst = p.partial + ((((uint64_t)section * p.heads + head) * p.batch + b) * p.rows + row) * (WIDTH + 2);
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

// combine the sections of one (head, plane, row): crates/neura-kernel/src/task/attention.rs:619-671
__global__ __launch_bounds__(256) void attention_fold_kernel(AttentionParams p, uint32_t width) {
    const uint32_t words = width + 2;
    const uint64_t vectors = (uint64_t)p.heads * p.batch * p.rows;
    for (uint64_t index = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; index < vectors * width;
         index += (uint64_t)gridDim.x * blockDim.x) {
        uint64_t vector = index / width;
        uint32_t c = (uint32_t)(index % width);
        float largest = -INFINITY;
        for (uint32_t s = 0; s < p.sections; s++) largest = fmaxf(largest, p.partial[(s * vectors + vector) * words + width]);
        float total = 0.0f, value = 0.0f;
        for (uint32_t s = 0; s < p.sections; s++) {
            const float *src = p.partial + (s * vectors + vector) * words;
            float weight = src[width] == -INFINITY ? 0.0f : softmax_exp(src[width] - largest);
            total += src[width + 1] * weight;
            value += src[c] * weight;
        }
        float normalized = total > 0.0f ? 1.0f / total : 0.0f;
        uint32_t row = (uint32_t)(vector % p.rows);
        uint32_t b = (uint32_t)((vector / p.rows) % p.batch);
        uint32_t head = (uint32_t)(vector / p.rows / p.batch);
        p.out[(uint64_t)head * p.o_sh + (uint64_t)b * p.o_sb + (uint64_t)row * p.o_sr + c] = value * normalized;
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
    // enough sections to put ~2 workgroups on every compute unit, none thinner than 64 keys
    uint32_t wanted = ((uint32_t)d->compute_units * 2 + units - 1) / units;
    uint32_t most = (a.keys + 63) / 64;
    p.sections = wanted < 1 ? 1 : (wanted > most ? most : wanted);
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
        uint64_t outputs = (uint64_t)a.heads * a.batch * a.rows * a.width;
        uint32_t blocks = (uint32_t)((outputs + 255) / 256 < 65535 ? (outputs + 255) / 256 : 65535);
        hipLaunchKernelGGL(attention_fold_kernel, dim3(blocks), dim3(256), 0, d->stream, p, a.width);
        NH_HIP(hipGetLastError());
    }
    return NH_OK;
}

}  // namespace nh
