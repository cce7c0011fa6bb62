// Sampled choice: temperature, the `keep` largest logits, a nucleus of cumulative mass, and a Gumbel-max draw among what is
// left (crates/neura-kernel/src/task/choice.rs:933-989 for one workgroup a row; :1045-1107 and :1270-1359 for the sectioned
// form followed here; crates/neura-generate/src/sampling.rs:69-94 for the temperature).
//
// A row of logits is cut into sections of 2048 columns.  One workgroup a section scales its logits by 1 / temperature,
// works out the section's largest value and softmax mass against it, and keeps its 64 best candidates (larger value
// first, lower column first among equals): every wave sorts runs of 64, one candidate a lane, with a bitonic network of
// lane exchanges, and merges two sorted runs into the best 64 of both with one mirrored compare and six more exchanges --
// no run longer than 64 is ever sorted.  One workgroup a row merges the sections' runs the same way, folds the section
// masses against the row's largest value in section order, cuts the candidates at `keep` and at the nucleus, and takes the
// largest of value + noise(seed, column).
#include "common.hpp"

namespace nh {

namespace {

constexpr uint32_t SECTION = 2048, CANDIDATES = 64, NO_VALUE = 0xffffffffu, MOST_SECTIONS = 128;
constexpr float EXP_UNDERFLOW = -104.0f;  // crates/neura-kernel/src/substrate.rs:110-116

__device__ __forceinline__ float softmax_exp(float argument) { return expf(fmaxf(argument, EXP_UNDERFLOW)); }

// A candidate as one 64-bit key whose unsigned order is the rank of crates/neura-kernel/src/task/choice.rs:396-404: the
// larger value first, the lower column first among equal values.  High word: the value's bits made monotonic (-0 reads
// as +0, as the comparison of floats has it); low word: the column's complement.  A padding entry (-inf, no column)
// ranks after every column that holds -inf.
__device__ __forceinline__ uint64_t candidate_key(float value, uint32_t index) {
    const uint32_t bits = __builtin_bit_cast(uint32_t, value + 0.0f);
    const uint32_t order = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
    return ((uint64_t)order << 32) | (uint32_t)~index;
}
__device__ __forceinline__ float key_value(uint64_t key) {
    const uint32_t order = (uint32_t)(key >> 32);
    return __builtin_bit_cast(float, (order & 0x80000000u) ? (order & 0x7fffffffu) : ~order);
}
__device__ __forceinline__ uint32_t key_index(uint64_t key) { return ~(uint32_t)key; }

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

// the word lane ^ J holds: inside a row of 16 lanes through the data-parallel primitives (a few cycles), across rows
// through the LDS crossbar
template <uint32_t J>
__device__ __forceinline__ uint32_t from_lane_xor(uint32_t word, uint32_t lane) {
    const int held = (int)word;
    // (every lane is written: the first operand, what an unwritten lane would keep, is never seen)
    if (J == 1) return (uint32_t)__builtin_amdgcn_update_dpp(held, held, 0xB1, 0xf, 0xf, false);  // quad_perm [1, 0, 3, 2]
    if (J == 2) return (uint32_t)__builtin_amdgcn_update_dpp(held, held, 0x4E, 0xf, 0xf, false);  // quad_perm [2, 3, 0, 1]
    if (J == 4) {
        // a rotation of a row of 16 by 4 and by 12 lanes: one of the two reaches lane ^ 4, which one the lane's own
        // number sent the same way tells (a lane constant, worked out once)
        const int by4 = __builtin_amdgcn_update_dpp(held, held, 0x124, 0xf, 0xf, false);
        const int by12 = __builtin_amdgcn_update_dpp(held, held, 0x12C, 0xf, 0xf, false);
        const uint32_t source = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)lane, 0x124, 0xf, 0xf, false);
        return (uint32_t)(source == (lane ^ 4u) ? by4 : by12);
    }
    if (J == 8) return (uint32_t)__builtin_amdgcn_update_dpp(held, held, 0x128, 0xf, 0xf, false);  // row_ror:8
    if (J == 16) return (uint32_t)__builtin_amdgcn_ds_swizzle(held, 0x401F);                    // lane ^ 16
    return (uint32_t)__shfl_xor(held, 32, 64);
}

// One candidate a lane.  A compare-exchange with lane ^ J: in a forward pair the lower lane keeps the better candidate.
template <uint32_t J>
__device__ __forceinline__ void wave_exchange(uint64_t &key, uint32_t lane, bool forward) {
    const uint64_t other = ((uint64_t)from_lane_xor<J>((uint32_t)(key >> 32), lane) << 32) | from_lane_xor<J>((uint32_t)key, lane);
    // no branches: the lower lane of a forward pair (and the upper lane of a backward one) keeps the better of the two, the
    // other lane the worse (two equal keys are two padding entries: either will do)
    const bool wants_worse = ((lane & J) == 0) != forward;
    key = ((other > key) != wants_worse) ? other : key;
}

// the exchanges with lanes ^ J, ^ J/2, ... ^ 1 that turn bitonic runs of 2J into sorted ones
template <uint32_t J>
__device__ __forceinline__ void wave_clean(uint64_t &key, uint32_t lane, bool forward) {
    wave_exchange<J>(key, lane, forward);
    if constexpr (J > 1) wave_clean<J / 2>(key, lane, forward);
}

// sorts the 64 candidates of a wave best rank first (bitonic network)
__device__ __forceinline__ void wave_sort(uint64_t &key, uint32_t lane) {
    wave_clean<1>(key, lane, (lane & 2u) == 0);
    wave_clean<2>(key, lane, (lane & 4u) == 0);
    wave_clean<4>(key, lane, (lane & 8u) == 0);
    wave_clean<8>(key, lane, (lane & 16u) == 0);
    wave_clean<16>(key, lane, (lane & 32u) == 0);
    wave_clean<32>(key, lane, true);
}

// `key` and `other` each hold 64 candidates sorted over the lanes: the best 64 of the 128, sorted, end up in `key`.
// The better of a[i] and b[63 - i] is one of them, and those 64 form a bitonic run.
__device__ __forceinline__ void wave_merge(uint64_t &key, uint64_t other, uint32_t lane) {
    const uint64_t mirrored = ((uint64_t)(uint32_t)__shfl((int)(other >> 32), (int)(63u - lane), 64) << 32) |
                              (uint32_t)__shfl((int)(uint32_t)other, (int)(63u - lane), 64);
    key = mirrored > key ? mirrored : key;
    wave_clean<32>(key, lane, true);
}

// The waves of a workgroup each hold a sorted run: the best 64 of all runs end up in wave 0, through a tree of merges
// over LDS (log2(WAVES) barriers).  Every wave must call.
template <int WAVES>
__device__ __forceinline__ void block_merge(uint64_t &key, uint64_t (*keys)[CANDIDATES], uint32_t wave, uint32_t lane) {
#pragma unroll
    for (uint32_t stride = 1; stride < WAVES; stride <<= 1) {
        if ((wave & (2 * stride - 1)) == stride) keys[wave][lane] = key;
        __syncthreads();
        if ((wave & (2 * stride - 1)) == 0 && wave + stride < WAVES) wave_merge(key, keys[wave + stride][lane], lane);
    }
}

template <int WAVES>
__device__ float block_max(float value, float *room) {
    for (int offset = 32; offset > 0; offset >>= 1) value = fmaxf(value, __shfl_xor(value, offset, 64));
    if ((threadIdx.x & 63u) == 0) room[threadIdx.x >> 6] = value;
    __syncthreads();
    float out = room[0];
    for (uint32_t w = 1; w < WAVES; w++) out = fmaxf(out, room[w]);
    __syncthreads();
    return out;
}

template <int WAVES>
__device__ float block_sum(float value, float *room) {
    for (int offset = 32; offset > 0; offset >>= 1) value += __shfl_xor(value, offset, 64);
    if ((threadIdx.x & 63u) == 0) room[threadIdx.x >> 6] = value;
    __syncthreads();
    float out = room[0];
    for (uint32_t w = 1; w < WAVES; w++) out += room[w];
    __syncthreads();
    return out;
}

constexpr int SECTION_WAVES = 8;  // 512 threads: four columns a thread

__global__ __launch_bounds__(SECTION_WAVES * 64) void sample_sections_kernel(const float *__restrict__ logits, uint32_t n, uint32_t sections,
                                                                             const nh_draw *__restrict__ draws, uint64_t *__restrict__ kept,
                                                                             float *__restrict__ stats) {
    NH_FETCH(logits, n, sections, draws, kept, stats);
    __shared__ uint64_t keys[SECTION_WAVES][CANDIDATES];
    __shared__ float room[SECTION_WAVES];
    const uint32_t row = blockIdx.y, section = blockIdx.x, lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t first = section * SECTION, count = min(n - first, SECTION);
    const float scale = __fdiv_rn(1.0f, draws[row].temperature);  // logits * recip(temperature), sampling.rs:82
    const float *src = logits + (size_t)row * n + first;
    constexpr int PER = SECTION / (SECTION_WAVES * 64);
    float value[PER];
    uint64_t key[PER];
    float largest = -INFINITY;
#pragma unroll
    for (int e = 0; e < PER; e++) {
        const uint32_t i = threadIdx.x + e * SECTION_WAVES * 64;
        const bool held = i < count;
        value[e] = held ? __fmul_rn(src[i], scale) : -INFINITY;
        key[e] = candidate_key(value[e], held ? first + i : NO_VALUE);
        largest = fmaxf(largest, value[e]);
    }
    largest = block_max<SECTION_WAVES>(largest, room);
    float mass = 0.0f;
#pragma unroll
    for (int e = 0; e < PER; e++)
        if (threadIdx.x + e * SECTION_WAVES * 64 < count) mass += softmax_exp(value[e] - largest);
    mass = block_sum<SECTION_WAVES>(mass, room);
    // each wave sorts its four runs of 64 and keeps the best 64 of them; the waves' runs then merge pairwise
#pragma unroll
    for (int e = 0; e < PER; e++) wave_sort(key[e], lane);
#pragma unroll
    for (int e = 1; e < PER; e++) wave_merge(key[0], key[e], lane);
    block_merge<SECTION_WAVES>(key[0], keys, wave, lane);
    if (wave != 0) return;
    const size_t at = (size_t)row * sections + section;
    kept[at * CANDIDATES + lane] = key[0];
    if (lane == 0) stats[2 * at] = largest, stats[2 * at + 1] = mass;
}

constexpr int FOLD_WAVES = 16;

// the float lane `at` of the wave holds, `at` a compile-time constant: a scalar read, no LDS
__device__ __forceinline__ float lane_float(float held, int at) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, held), at));
}

__global__ __launch_bounds__(FOLD_WAVES * 64) void sample_fold_kernel(const uint64_t *__restrict__ kept, const float *__restrict__ stats,
                                                                      uint32_t sections, const nh_draw *__restrict__ draws,
                                                                      uint32_t *__restrict__ out) {
    __shared__ uint64_t keys[FOLD_WAVES][CANDIDATES];
    const uint32_t row = blockIdx.x, lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    // the sections' runs are sorted as they lie: every wave merges its share (all of it fetched before the first merge),
    // then the waves' results merge pairwise
    constexpr int SHARE = MOST_SECTIONS / FOLD_WAVES;
    uint64_t held[SHARE];
#pragma unroll
    for (int i = 0; i < SHARE; i++) {
        const uint32_t s = wave + FOLD_WAVES * i;
        held[i] = s < sections ? kept[((size_t)row * sections + s) * CANDIDATES + lane] : candidate_key(-INFINITY, NO_VALUE);
    }
    // the row's largest value, and the masses of its sections against it (choice.rs:1305-1325): two sections a lane
    float section_max[2], section_mass[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const uint32_t s = lane + 64u * h;
        section_max[h] = s < sections ? stats[2 * ((size_t)row * sections + s)] : -INFINITY;
        section_mass[h] = s < sections ? stats[2 * ((size_t)row * sections + s) + 1] : 0.0f;
    }
    const nh_draw draw = draws[row];
    uint64_t key = held[0];
#pragma unroll
    for (int i = 1; i < SHARE; i++)
        if (wave + FOLD_WAVES * i < sections) wave_merge(key, held[i], lane);
    block_merge<FOLD_WAVES>(key, keys, wave, lane);
    if (wave != 0) return;
    const float value = key_value(key);
    const uint32_t index = key_index(key);
    float row_max = fmaxf(section_max[0], section_max[1]);
    for (int offset = 32; offset > 0; offset >>= 1) row_max = fmaxf(row_max, __shfl_xor(row_max, offset, 64));
    const float term[2] = {section_mass[0] * softmax_exp(section_max[0] - row_max), section_mass[1] * softmax_exp(section_max[1] - row_max)};
    const float candidate_mass = softmax_exp(value - row_max);
    const float weight = index == NO_VALUE ? -INFINITY : value + gumbel_noise(draw.seed, index);
    // From here every lane walks the same scalars, read out of the lanes that hold them, in the reference's order:
    // the sections' masses added in section order, the candidates' in rank order (choice.rs:1318-1345).
    float total = 0.0f;
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
        for (int s = 0; s < 64; s++)
            if ((uint32_t)(s + 64 * h) < sections) total = total + lane_float(term[h], s);
    const uint32_t most = draw.keep < CANDIDATES ? draw.keep : CANDIDATES;
    const uint64_t valid = __ballot(index != NO_VALUE && lane < most);  // a prefix of the lanes: the run is sorted
    const uint32_t count = (uint32_t)__popcll(valid);
    float mass = 0.0f;
#pragma unroll
    for (int c = 0; c < 64; c++)
        if ((uint32_t)c < count) mass = mass + lane_float(candidate_mass, c);
    const float tail = total - mass, threshold = draw.cumulative * total;
    uint32_t boundary = count;
    float running = 0.0f;
#pragma unroll
    for (int c = 0; c < 64; c++)
        if ((uint32_t)c < count) {
            running = running + lane_float(candidate_mass, c);
            if (running + tail >= threshold && (uint32_t)c + 1 < boundary) boundary = (uint32_t)c + 1;
        }
    float best = -INFINITY;
    uint32_t chosen = NO_VALUE;
#pragma unroll
    for (int c = 0; c < 64; c++)
        if ((uint32_t)c < boundary) {
            const float held = lane_float(weight, c);
            const uint32_t column = (uint32_t)__builtin_amdgcn_readlane((int)index, c);
            // choice_precedes (choice.rs:46-51): the larger weight, the lower column among equals
            if (chosen == NO_VALUE || held > best || (held == best && column < chosen)) best = held, chosen = column;
        }
    if (lane == 0) out[row] = chosen == NO_VALUE ? 0u : chosen;
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
    if (!n || sections > MOST_SECTIONS) return fail(NH_E_ARGUMENT, "a sampled row holds between one and %u columns, not %u", MOST_SECTIONS * SECTION, n);
    uint8_t *held = static_cast<uint8_t *>(scratch(d, sample_scratch_bytes(rows, n)));
    if (!held) return NH_E_MEMORY;
    uint64_t *kept = reinterpret_cast<uint64_t *>(held);
    float *stats = reinterpret_cast<float *>(held + (size_t)rows * sections * CANDIDATES * 8);
    hipLaunchKernelGGL(sample_sections_kernel, dim3(sections, rows), dim3(SECTION_WAVES * 64), 0, d->stream, logits, n, sections, draws, kept, stats);
    NH_HIP(hipGetLastError());
    hipLaunchKernelGGL(sample_fold_kernel, dim3(rows), dim3(FOLD_WAVES * 64), 0, d->stream, kept, stats, sections, draws, out);
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
