// Sampled choice: temperature, the `keep` largest logits, a nucleus of cumulative mass, and a Gumbel-max draw among what is
// left (crates/neura-kernel/src/task/choice.rs:933-989 for one workgroup a row; :1045-1107 and :1270-1359 for the sectioned
// form followed here; crates/neura-generate/src/sampling.rs:69-94 for the temperature).
//
// A row of logits is cut into sections of 4096 columns.  One workgroup a section scales its logits by 1 / temperature,
// works out the section's largest value and softmax mass against it, sorts the section in LDS (bitonic, larger value
// first, lower column first among equals) and keeps its first 64.  One workgroup a row then sorts the kept candidates of
// all sections, folds the section masses against the row's largest value in section order, cuts the candidates at `keep`
// and at the nucleus, and takes the largest of value + noise(seed, column).
#include "common.hpp"

namespace nh {

namespace {

constexpr uint32_t SECTION = 4096, CANDIDATES = 64, NO_VALUE = 0xffffffffu;
constexpr float EXP_UNDERFLOW = -104.0f;  // crates/neura-kernel/src/substrate.rs:110-116

__device__ __forceinline__ float softmax_exp(float argument) { return expf(fmaxf(argument, EXP_UNDERFLOW)); }

// (value, index) ranks before (other_value, other_index): crates/neura-kernel/src/task/choice.rs:396-404
__device__ __forceinline__ bool ranks_before(float value, uint32_t index, float other_value, uint32_t other_index) {
    return value > other_value || (value == other_value && index < other_index);
}

// crates/neura-kernel/src/task/choice.rs:81-89 over element_key((0, 0, 0, column)) (substrate.rs:146-152): a row draws
// the numbers its own seed names whatever row it answers in
__device__ __forceinline__ float gumbel_noise(uint32_t seed, uint32_t column) {
    uint32_t hash = seed ^ ((column * 0x27d4eb2fu) * 0x9e3779b9u);
    hash ^= hash >> 16;
    hash *= 0x7feb352du;
    hash ^= hash >> 15;
    hash *= 0x846ca68bu;
    hash ^= hash >> 16;
    return -logf(-logf((float)(hash >> 8) * (1.0f / 16777216.0f)));
}

// sorts values[0 .. count) / indices[0 .. count) in LDS, count a power of two, best rank first
__device__ void sort_ranked(float *values, uint32_t *indices, uint32_t count) {
    for (uint32_t k = 2; k <= count; k <<= 1) {
        for (uint32_t j = k >> 1; j > 0; j >>= 1) {
            for (uint32_t t = threadIdx.x; t < count / 2; t += blockDim.x) {
                const uint32_t i = ((t & ~(j - 1u)) << 1) | (t & (j - 1u));  // bit j clear
                const uint32_t partner = i | j;
                const bool forward = (i & k) == 0;
                const float a = values[i], b = values[partner];
                const uint32_t ia = indices[i], ib = indices[partner];
                const bool swap = forward ? ranks_before(b, ib, a, ia) : ranks_before(a, ia, b, ib);
                if (swap) {
                    values[i] = b, values[partner] = a;
                    indices[i] = ib, indices[partner] = ia;
                }
            }
            __syncthreads();
        }
    }
}

__device__ float block_max(float value, float *room) {
    for (int offset = 32; offset > 0; offset >>= 1) value = fmaxf(value, __shfl_xor(value, offset, 64));
    if ((threadIdx.x & 63u) == 0) room[threadIdx.x >> 6] = value;
    __syncthreads();
    float out = room[0];
    for (uint32_t w = 1; w < blockDim.x / 64; w++) out = fmaxf(out, room[w]);
    __syncthreads();
    return out;
}

__device__ float block_sum(float value, float *room) {
    for (int offset = 32; offset > 0; offset >>= 1) value += __shfl_xor(value, offset, 64);
    if ((threadIdx.x & 63u) == 0) room[threadIdx.x >> 6] = value;
    __syncthreads();
    float out = room[0];
    for (uint32_t w = 1; w < blockDim.x / 64; w++) out += room[w];
    __syncthreads();
    return out;
}

__global__ __launch_bounds__(256) void sample_sections_kernel(const float *__restrict__ logits, uint32_t n, uint32_t sections,
                                                              const nh_draw *__restrict__ draws, float *__restrict__ kept_values,
                                                              uint32_t *__restrict__ kept_indices, float *__restrict__ stats) {
    __shared__ float values[SECTION];
    __shared__ uint32_t indices[SECTION];
    __shared__ float room[4];
    const uint32_t row = blockIdx.y, section = blockIdx.x;
    const uint32_t first = section * SECTION, count = min(n - first, SECTION);
    const float scale = __fdiv_rn(1.0f, draws[row].temperature);  // logits * recip(temperature), sampling.rs:82
    const float *src = logits + (size_t)row * n + first;
    float largest = -INFINITY;
    for (uint32_t i = threadIdx.x; i < SECTION; i += 256) {
        const bool held = i < count;
        const float value = held ? __fmul_rn(src[i], scale) : -INFINITY;
        values[i] = value;
        indices[i] = held ? first + i : NO_VALUE;
        largest = fmaxf(largest, value);
    }
    largest = block_max(largest, room);
    float mass = 0.0f;
    for (uint32_t i = threadIdx.x; i < count; i += 256) mass += softmax_exp(values[i] - largest);
    mass = block_sum(mass, room);
    sort_ranked(values, indices, SECTION);
    const size_t at = (size_t)row * sections + section;
    if (threadIdx.x < CANDIDATES) {
        kept_values[at * CANDIDATES + threadIdx.x] = values[threadIdx.x];
        kept_indices[at * CANDIDATES + threadIdx.x] = indices[threadIdx.x];
    }
    if (threadIdx.x == 0) stats[2 * at] = largest, stats[2 * at + 1] = mass;
}

__global__ __launch_bounds__(256) void sample_fold_kernel(const float *__restrict__ kept_values, const uint32_t *__restrict__ kept_indices,
                                                          const float *__restrict__ stats, uint32_t sections, uint32_t padded,
                                                          const nh_draw *__restrict__ draws, uint32_t *__restrict__ out) {
    __shared__ float values[SECTION];
    __shared__ uint32_t indices[SECTION];
    __shared__ float masses[CANDIDATES], weights[CANDIDATES];
    const uint32_t row = blockIdx.x, held = sections * CANDIDATES;
    for (uint32_t i = threadIdx.x; i < padded; i += 256) {
        values[i] = i < held ? kept_values[(size_t)row * held + i] : -INFINITY;
        indices[i] = i < held ? kept_indices[(size_t)row * held + i] : NO_VALUE;
    }
    __syncthreads();
    sort_ranked(values, indices, padded);
    const nh_draw draw = draws[row];
    // the row's largest value, and the masses of its sections against it, in section order (choice.rs:1305-1325)
    float row_max = -INFINITY;
    for (uint32_t s = 0; s < sections; s++) row_max = fmaxf(row_max, stats[2 * ((size_t)row * sections + s)]);
    if (threadIdx.x < CANDIDATES) {
        const uint32_t column = indices[threadIdx.x];
        masses[threadIdx.x] = softmax_exp(values[threadIdx.x] - row_max);
        weights[threadIdx.x] = column == NO_VALUE ? -INFINITY : values[threadIdx.x] + gumbel_noise(draw.seed, column);
    }
    __syncthreads();
    if (threadIdx.x != 0) return;
    float total = 0.0f;
    for (uint32_t s = 0; s < sections; s++) {
        const size_t at = 2 * ((size_t)row * sections + s);
        total = total + stats[at + 1] * softmax_exp(stats[at] - row_max);
    }
    uint32_t count = 0;
    while (count < draw.keep && count < CANDIDATES && indices[count] != NO_VALUE) count++;
    float mass = 0.0f;
    for (uint32_t c = 0; c < count; c++) mass = mass + masses[c];
    const float tail = total - mass, threshold = draw.cumulative * total;
    uint32_t boundary = count;
    float running = 0.0f;
    for (uint32_t c = 0; c < count; c++) {
        running = running + masses[c];
        if (running + tail >= threshold && c + 1 < boundary) boundary = c + 1;
    }
    float best = -INFINITY;
    uint32_t chosen = NO_VALUE;
    for (uint32_t c = 0; c < boundary; c++) {
        const float weight = weights[c];
        const uint32_t column = indices[c];
        // choice_precedes (choice.rs:46-51): the larger weight, the lower column among equals
        if (chosen == NO_VALUE || weight > best || (weight == best && column < chosen)) best = weight, chosen = column;
    }
    out[row] = chosen == NO_VALUE ? 0u : chosen;
}

}  // namespace

size_t sample_scratch_bytes(uint32_t rows, uint32_t n) {
    const size_t sections = (n + SECTION - 1) / SECTION;
    return (size_t)rows * sections * (CANDIDATES * 8 + 8);
}

// draws: device memory, one a row
int32_t launch_sample(nh_device *d, const float *logits, uint32_t rows, uint32_t n, const nh_draw *draws, uint32_t *out) {
    if (!rows) return NH_OK;
    const uint32_t sections = (n + SECTION - 1) / SECTION;
    if (!n || sections * CANDIDATES > SECTION)
        return fail(NH_E_ARGUMENT, "a sampled row holds between one and %u columns, not %u", SECTION / CANDIDATES * SECTION, n);
    uint8_t *held = static_cast<uint8_t *>(scratch(d, sample_scratch_bytes(rows, n)));
    if (!held) return NH_E_MEMORY;
    const size_t kept = (size_t)rows * sections * CANDIDATES;
    float *kept_values = reinterpret_cast<float *>(held);
    uint32_t *kept_indices = reinterpret_cast<uint32_t *>(held + kept * 4);
    float *stats = reinterpret_cast<float *>(held + kept * 8);
    hipLaunchKernelGGL(sample_sections_kernel, dim3(sections, rows), dim3(256), 0, d->stream, logits, n, sections, draws, kept_values, kept_indices,
                       stats);
    NH_HIP(hipGetLastError());
    uint32_t padded = CANDIDATES;
    while (padded < sections * CANDIDATES) padded <<= 1;
    hipLaunchKernelGGL(sample_fold_kernel, dim3(rows), dim3(256), 0, d->stream, kept_values, kept_indices, stats, sections, padded, draws, out);
    NH_HIP(hipGetLastError());
    return NH_OK;
}

// the refusals of crates/neura-generate/src/sampling.rs:16-29 (and of the kernels, choice.rs:991-1013)
int32_t check_draws(const nh_draw *draws, uint32_t rows) {
    for (uint32_t r = 0; r < rows; r++) {
        const nh_draw &draw = draws[r];
        if (!(draw.temperature > 0.0f) || !(draw.temperature <= 3.402823466e38f))
            return fail(NH_E_ARGUMENT, "a sampling temperature of %g spreads no logits", (double)draw.temperature);
        if (draw.keep < 1 || draw.keep > CANDIDATES)
            return fail(NH_E_ARGUMENT, "a sample keeps %u candidates where a row holds between one and %u", draw.keep, CANDIDATES);
        if (!(draw.cumulative > 0.0f) || !(draw.cumulative <= 1.0f))
            return fail(NH_E_ARGUMENT, "a cumulative mass of %g keeps no candidate or names more than every candidate", (double)draw.cumulative);
    }
    return NH_OK;
}

}  // namespace nh
