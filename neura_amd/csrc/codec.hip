// Element-wise readers: bit-exact dequantisation of raw ggml blocks, fp32 -> fp16 conversion
// and the embedding gather.  Compiled with -ffp-contract=off: the reference rounds every
// product before the next operation.
#include "blocks.hpp"
#include "common.hpp"

namespace nh {

template <int ELEMENT>
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t *__restrict__ src, uint64_t elements, float *__restrict__ dst) {
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < elements; i += (uint64_t)gridDim.x * blockDim.x) {
        dst[i] = stored_element<ELEMENT>(src, i);
    }
}

static uint32_t grid_for(nh_device *d, uint64_t items, uint32_t block) {
    uint64_t wanted = (items + block - 1) / block;
    uint64_t most = (uint64_t)d->compute_units * 16;
    return (uint32_t)(wanted < 1 ? 1 : (wanted > most ? most : wanted));
}

int32_t launch_dequant(nh_device *d, int32_t element, const void *src, uint64_t elements, float *dst) {
    if (!elements) return NH_OK;
    uint32_t grid = grid_for(d, elements, 256);
    const uint8_t *bytes = static_cast<const uint8_t *>(src);
    switch (element) {
    case NH_Q8_0: hipLaunchKernelGGL(dequant_kernel<NH_Q8_0>, dim3(grid), dim3(256), 0, d->stream, bytes, elements, dst); break;
    case NH_Q4_K: hipLaunchKernelGGL(dequant_kernel<NH_Q4_K>, dim3(grid), dim3(256), 0, d->stream, bytes, elements, dst); break;
    case NH_Q6_K: hipLaunchKernelGGL(dequant_kernel<NH_Q6_K>, dim3(grid), dim3(256), 0, d->stream, bytes, elements, dst); break;
    case NH_Q5_K: hipLaunchKernelGGL(dequant_kernel<NH_Q5_K>, dim3(grid), dim3(256), 0, d->stream, bytes, elements, dst); break;
    case NH_Q3_K: hipLaunchKernelGGL(dequant_kernel<NH_Q3_K>, dim3(grid), dim3(256), 0, d->stream, bytes, elements, dst); break;
    case NH_F16: hipLaunchKernelGGL(dequant_kernel<NH_F16>, dim3(grid), dim3(256), 0, d->stream, bytes, elements, dst); break;
    case NH_F32: hipLaunchKernelGGL(dequant_kernel<NH_F32>, dim3(grid), dim3(256), 0, d->stream, bytes, elements, dst); break;
    default: return fail(NH_E_ARGUMENT, "element %d carries no reader", element);
    }
    NH_HIP(hipGetLastError());
    return NH_OK;
}

__global__ __launch_bounds__(256) void convert_half_kernel(const float *__restrict__ src, uint64_t elements, uint16_t *__restrict__ dst) {
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < elements; i += (uint64_t)gridDim.x * blockDim.x)
        dst[i] = float_to_half(src[i]);
}

int32_t launch_convert_half(nh_device *d, const float *src, uint64_t elements, uint16_t *dst) {
    if (!elements) return NH_OK;
    hipLaunchKernelGGL(convert_half_kernel, dim3(grid_for(d, elements, 256)), dim3(256), 0, d->stream, src, elements, dst);
    NH_HIP(hipGetLastError());
    return NH_OK;
}

// The device's Q8_0 encoder (run_convert_q8_0, q8_0_quantum, q8_0_code,
// crates/neura-kernel/src/task/convert.rs:355-430): per block of 32 the quantum is the largest
// magnitude / 127, stored as a half, and every code is value * (1 / quantum) rounded half away
// from zero as trunc(scaled +- 0.5), clamped to +-127.  Elements past the end count as zero.
// Eight lanes share a block: each loads four numbers, the magnitude folds over the eight, and each
// stores its four codes as two 16-bit halves (a block starts on an even byte, not on a word).
// The bytes behind an odd number of blocks, up to the four-byte word, are zero.
__global__ __launch_bounds__(256) void pack_q8_0_kernel(const float *__restrict__ src, uint64_t elements, uint64_t blocks,
                                                        uint8_t *__restrict__ dst) {
    const uint64_t lanes = blocks * 8;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < (lanes + 63) / 64 * 64; i += (uint64_t)gridDim.x * blockDim.x) {
        const uint64_t block = i / 8, first = i * 4;
        float v[4];
        if (first + 4 <= elements && i < lanes) {
            const float4 held = *reinterpret_cast<const float4 *>(src + first);
            v[0] = held.x, v[1] = held.y, v[2] = held.z, v[3] = held.w;
        } else {
            for (int j = 0; j < 4; j++) v[j] = (i < lanes && first + j < elements) ? src[first + j] : 0.0f;
        }
        float size = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
        size = fmaxf(size, __shfl_xor(size, 1));
        size = fmaxf(size, __shfl_xor(size, 2));
        size = fmaxf(size, __shfl_xor(size, 4));
        if (i >= lanes) continue;
        const float quantum = __fdiv_rn(size, 127.0f);
        const float inverse = quantum != 0.0f ? __fdiv_rn(1.0f, quantum) : 0.0f;
        uint32_t word = 0;
        for (int j = 0; j < 4; j++) {
            const float scaled = __fmul_rn(v[j], inverse);
            const float rounded = truncf(__fadd_rn(scaled, scaled >= 0.0f ? 0.5f : -0.5f));
            const int code = (int)fminf(fmaxf(rounded, -127.0f), 127.0f);
            word |= ((uint32_t)code & 0xffu) << (8 * j);
        }
        uint16_t *field = reinterpret_cast<uint16_t *>(dst + block * 34);
        const uint32_t lane = (uint32_t)(i % 8);
        if (lane == 0) field[0] = float_to_half(quantum);
        field[1 + 2 * lane] = (uint16_t)word;
        field[2 + 2 * lane] = (uint16_t)(word >> 16);
        if (lane == 7 && block + 1 == blocks && (blocks & 1)) field[17] = 0;
    }
}

int32_t launch_pack_q8_0(nh_device *d, const float *src, uint64_t elements, uint8_t *dst) {
    if (!elements) return NH_OK;
    const uint64_t blocks = (elements + 31) / 32;
    hipLaunchKernelGGL(pack_q8_0_kernel, dim3(grid_for(d, blocks * 8, 256)), dim3(256), 0, d->stream, src, elements, blocks, dst);
    NH_HIP(hipGetLastError());
    return NH_OK;
}

// out[t][c] = dequant(table[token[t]])[c] * mask[t % batch]   (crates/neura-kernel/src/task/select.rs:29-49,
// examples/qwen/model.rs:94).  One thread per element: blockIdx.y walks the row in spans of 256.
template <int ELEMENT>
__global__ __launch_bounds__(256) void gather_kernel(const uint8_t *__restrict__ table, uint32_t vocab, uint32_t width, uint64_t row_bytes,
                                                     const uint32_t *__restrict__ tokens, uint32_t batch,
                                                     const uint8_t *__restrict__ mask, float *__restrict__ out, uint32_t *refusal) {
    NH_FETCH(table, vocab, width, row_bytes, tokens, batch, mask, out, refusal);
    uint32_t t = blockIdx.x;
    uint32_t token = tokens[t];
    float keep = (mask == nullptr || mask[t % batch]) ? 1.0f : 0.0f;
    if (token >= vocab) {
        if (threadIdx.x == 0 && blockIdx.y == 0) atomicMax(refusal, (uint32_t)REFUSAL_INDEX);
        for (uint32_t c = blockIdx.y * blockDim.x + threadIdx.x; c < width; c += gridDim.y * blockDim.x) out[(uint64_t)t * width + c] = 0.0f;
        return;
    }
    const uint8_t *row = table + (uint64_t)token * row_bytes;
    for (uint32_t c = blockIdx.y * blockDim.x + threadIdx.x; c < width; c += gridDim.y * blockDim.x) {
        out[(uint64_t)t * width + c] = stored_element<ELEMENT>(row, c) * keep;
    }
}

int32_t launch_gather(nh_device *d, int32_t element, const void *table, uint32_t vocab, uint32_t width, const uint32_t *tokens,
                      uint32_t count, uint32_t batch, const uint8_t *mask, float *out) {
    if (!count) return NH_OK;
    const uint8_t *bytes = static_cast<const uint8_t *>(table);
    uint64_t row_bytes = payload_bytes(element, width);
    uint32_t spans = (width + 255) / 256;
    const dim3 grid(count, spans < 64 ? spans : 64);
    switch (element) {
    case NH_Q8_0:
        hipLaunchKernelGGL(gather_kernel<NH_Q8_0>, grid, dim3(256), 0, d->stream, bytes, vocab, width, row_bytes, tokens, batch, mask,
                           out, d->refusal);
        break;
    case NH_Q4_K:
        hipLaunchKernelGGL(gather_kernel<NH_Q4_K>, grid, dim3(256), 0, d->stream, bytes, vocab, width, row_bytes, tokens, batch, mask,
                           out, d->refusal);
        break;
    case NH_Q6_K:
        hipLaunchKernelGGL(gather_kernel<NH_Q6_K>, grid, dim3(256), 0, d->stream, bytes, vocab, width, row_bytes, tokens, batch, mask,
                           out, d->refusal);
        break;
    case NH_Q5_K:
        hipLaunchKernelGGL(gather_kernel<NH_Q5_K>, grid, dim3(256), 0, d->stream, bytes, vocab, width, row_bytes, tokens, batch, mask,
                           out, d->refusal);
        break;
    case NH_Q3_K:
        hipLaunchKernelGGL(gather_kernel<NH_Q3_K>, grid, dim3(256), 0, d->stream, bytes, vocab, width, row_bytes, tokens, batch, mask,
                           out, d->refusal);
        break;
    case NH_F16:
        hipLaunchKernelGGL(gather_kernel<NH_F16>, grid, dim3(256), 0, d->stream, bytes, vocab, width, row_bytes, tokens, batch, mask,
                           out, d->refusal);
        break;
    case NH_F32:
        hipLaunchKernelGGL(gather_kernel<NH_F32>, grid, dim3(256), 0, d->stream, bytes, vocab, width, row_bytes, tokens, batch, mask,
                           out, d->refusal);
        break;
    default: return fail(NH_E_ARGUMENT, "element %d carries no reader", element);
    }
    NH_HIP(hipGetLastError());
    return NH_OK;
}

}  // namespace nh
