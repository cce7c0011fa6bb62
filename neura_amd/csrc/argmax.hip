// Greedy choice: per row the largest value, the lowest index on ties
// (crates/neura-kernel/src/task/choice.rs:46-51, :355-368; sectioned + fold :331-353).
#include "common.hpp"

// The section partials of nh_argmax_static, the greedy choice for callers that cannot allocate, live in this array
// instead of the device scratch (which grows by hipMalloc).  Every GPU the library runs on holds its own copy at its own
// address until the process ends; in host code the name is only a handle for hipGetSymbolAddress, never an address a
// kernel could follow.  64 rows of 1024 sections of (value, index): 512 KiB.
constexpr uint32_t STATIC_ARGMAX_ROWS = 64;
constexpr size_t STATIC_ARGMAX_BYTES = (size_t)STATIC_ARGMAX_ROWS * 1024u * (sizeof(float) + sizeof(uint32_t));
static __device__ __align__(256) uint8_t scratch[STATIC_ARGMAX_BYTES];

namespace nh {

__device__ __forceinline__ bool precedes(float value, uint32_t index, float other_value, uint32_t other_index) {
    // true when (other_value, other_index) beats (value, index)
    return other_value > value || (other_value == value && other_index < index);
}

__device__ __forceinline__ void wave_choice(float &value, uint32_t &index) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        float other_value = __shfl_xor(value, offset, 64);
        uint32_t other_index = __shfl_xor(index, offset, 64);
        if (precedes(value, index, other_value, other_index)) value = other_value, index = other_index;
    }
}

__device__ void block_choice(float &value, uint32_t &index, float *values, uint32_t *indices) {
    wave_choice(value, index);
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    if (lane == 0) values[wave] = value, indices[wave] = index;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (uint32_t w = 1; w < blockDim.x / 64; w++)
            if (precedes(value, index, values[w], indices[w])) value = values[w], index = indices[w];
    }
}

__global__ __launch_bounds__(256) void argmax_sections_kernel(const float *__restrict__ values, uint32_t n, uint32_t sections,
                                                              float *__restrict__ best_values, uint32_t *__restrict__ best_indices) {
    NH_FETCH(values, n, sections, best_values, best_indices, gridDim.x);
    __shared__ float held_values[4];
    __shared__ uint32_t held_indices[4];
    const uint32_t row = blockIdx.y, section = blockIdx.x;
    const uint32_t chunk = (n + sections - 1) / sections;
    const uint32_t first = section * chunk, last = min(n, first + chunk);
    const float *src = values + (size_t)row * n;
    float value = -INFINITY;
    uint32_t index = first < n ? first : 0u;
    // eight values a thread at a time, all asked for before the first is compared (past the section its last value again,
    // dropped): a loop that compares each value as it arrives spends a memory round trip on every one
    for (uint32_t base = first; base < last; base += 2048u) {
        float held[8];
#pragma unroll
        for (int j = 0; j < 8; j++) held[j] = src[min(base + threadIdx.x + 256u * j, last - 1u)];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t i = base + threadIdx.x + 256u * j;
            if (i < last && precedes(value, index, held[j], i)) value = held[j], index = i;
        }
    }
    block_choice(value, index, held_values, held_indices);
    if (threadIdx.x == 0) {
        best_values[(size_t)row * sections + section] = value;
        best_indices[(size_t)row * sections + section] = index;
    }
}

// `published`, where given: the host's pinned words [rows + 1] -- every row's choice again, then the word at `refusal`
__global__ __launch_bounds__(256) void argmax_fold_kernel(const float *__restrict__ best_values, const uint32_t *__restrict__ best_indices,
                                                          uint32_t sections, uint32_t *__restrict__ out, uint32_t *__restrict__ published,
                                                          const uint32_t *__restrict__ refusal) {
    NH_FETCH(best_values, best_indices, sections, out, published, refusal);
    __shared__ float held_values[4];
    __shared__ uint32_t held_indices[4];
    const uint32_t row = blockIdx.x;
    const uint32_t refused = published && row == 0 && threadIdx.x == 0 ? *refusal : 0u;
    float value = -INFINITY;
    uint32_t index = 0xffffffffu;
    for (uint32_t s = threadIdx.x; s < sections; s += 256) {
        float held = best_values[(size_t)row * sections + s];
        uint32_t at = best_indices[(size_t)row * sections + s];
        if (index == 0xffffffffu || precedes(value, index, held, at)) value = held, index = at;
    }
    block_choice(value, index, held_values, held_indices);
    if (threadIdx.x == 0) {
        const uint32_t chosen = index == 0xffffffffu ? 0u : index;
        out[row] = chosen;
        if (published) {
            published[row] = chosen;
            if (row == 0) published[gridDim.x] = refused;
        }
    }
}

static uint32_t argmax_sections(uint32_t n) {
    uint32_t sections = (n + 2047) / 2048;
    if (sections < 1) sections = 1;
    if (sections > 1024) sections = 1024;
    return sections;
}

static int32_t launch_argmax_over(nh_device *d, const float *values, uint32_t rows, uint32_t n, uint32_t *out, uint8_t *held, uint32_t *published = nullptr,
                                  const uint32_t *refusal = nullptr) {
    const uint32_t sections = argmax_sections(n);
    float *best_values = reinterpret_cast<float *>(held);
    uint32_t *best_indices = reinterpret_cast<uint32_t *>(held + (size_t)rows * sections * sizeof(float));
    hipLaunchKernelGGL(argmax_sections_kernel, dim3(sections, rows), dim3(256), 0, d->stream, values, n, sections, best_values, best_indices);
    NH_HIP(hipGetLastError());
    hipLaunchKernelGGL(argmax_fold_kernel, dim3(rows), dim3(256), 0, d->stream, best_values, best_indices, sections, out, published, refusal);
    NH_HIP(hipGetLastError());
    return NH_OK;
}

int32_t launch_argmax(nh_device *d, const float *values, uint32_t rows, uint32_t n, uint32_t *out, uint32_t *published, const uint32_t *refusal) {
    if (!rows) return NH_OK;
    if (published && !refusal) return fail(NH_E_ARGUMENT, "choices published to the host go with the refusal word");
    const size_t bytes = (size_t)rows * argmax_sections(n) * (sizeof(float) + sizeof(uint32_t));
    uint8_t *held = static_cast<uint8_t *>(scratch(d, bytes));
    if (!held) return NH_E_MEMORY;
    return launch_argmax_over(d, values, rows, n, out, held, published, refusal);
}

// ---- the greedy choice for callers that cannot allocate ----------------------------------------------------------
// once per device, with that device current (nh_open calls it): where this device keeps its copy of the array
int32_t argmax_static_setup(nh_device *d) {
    void *address = nullptr;
    hipError_t found = hipGetSymbolAddress(&address, HIP_SYMBOL(::scratch));
    if (found != hipSuccess || !address) return hip_fail(found, "hipGetSymbolAddress(scratch)");
    d->static_scratch = static_cast<uint8_t *>(address);
    return NH_OK;
}

int32_t launch_argmax_static(nh_device *d, const float *values, uint32_t rows, uint32_t n, uint32_t *out) {
    if (!rows) return NH_OK;
    if (!d->static_scratch) return fail(NH_E_DEVICE, "device %d holds no address of the static scratch array", d->index);
    const size_t bytes = (size_t)rows * argmax_sections(n) * (sizeof(float) + sizeof(uint32_t));
    if (rows > STATIC_ARGMAX_ROWS || bytes > STATIC_ARGMAX_BYTES)
        return fail(NH_E_ARGUMENT, "a greedy choice over %u rows of %u needs %zu bytes of partials, and the static scratch holds %zu (at most %u rows)",
                    rows, n, bytes, STATIC_ARGMAX_BYTES, STATIC_ARGMAX_ROWS);
    // nothing in the array has to start at zero: the first kernel writes every partial the second one reads
    return launch_argmax_over(d, values, rows, n, out, d->static_scratch);
}

}  // namespace nh
