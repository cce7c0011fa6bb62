// Row operators around the products: RMSNorm, rotary embedding, fp16 cache append,
// SwiGLU and plane masking.
#include "blocks.hpp"
#include "common.hpp"

namespace nh {

// One workgroup per row; the sum of squares follows the reference's order (thread t adds
// columns t, t+256, ..., then a 256-wide tree: crates/neura-kernel/src/task/norm.rs:69-104,
// reduce.rs:21-38) so the scale is the same fp32 number.
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float *__restrict__ x, const float *__restrict__ residual,
                                                      const float *__restrict__ w, float eps, uint32_t C, float *__restrict__ out,
                                                      float *__restrict__ sum_out) {
    __shared__ float red[256];
    const uint32_t row = blockIdx.x, tid = threadIdx.x;
    const float *xr = x + (size_t)row * C;
    const float *rr = residual ? residual + (size_t)row * C : nullptr;
    float square = 0.0f;
    for (uint32_t c = tid; c < C; c += 256) {
        float value = rr ? __fadd_rn(xr[c], rr[c]) : xr[c];
        square = __fadd_rn(square, __fmul_rn(value, value));
    }
    red[tid] = square;
    __syncthreads();
    for (uint32_t stride = 128; stride > 0; stride >>= 1) {
        if (tid < stride) red[tid] = __fadd_rn(red[tid], red[tid + stride]);
        __syncthreads();
    }
    float scale = rms_scale_of(red[0], C, eps);
    for (uint32_t c = tid; c < C; c += 256) {
        float value = rr ? __fadd_rn(xr[c], rr[c]) : xr[c];
        if (sum_out) sum_out[(size_t)row * C + c] = value;
        float result = __fmul_rn(value, scale);
        if (w) result = __fmul_rn(result, w[c]);
        out[(size_t)row * C + c] = result;
    }
}

int32_t launch_rmsnorm(nh_device *d, const float *x, const float *residual, const float *w, float eps, uint32_t rows, uint32_t C,
                       float *out, float *sum_out) {
    if (!rows) return NH_OK;
    hipLaunchKernelGGL(rmsnorm_kernel, dim3(rows), dim3(256), 0, d->stream, x, residual, w, eps, C, out, sum_out);
    NH_HIP(hipGetLastError());
    return NH_OK;
}

// rotate-half (crates/neura-kernel/src/task/rope.rs:95-122); the angle is
// f32(position) * table[channel], the table holding pow(base, -2c/width) (rope.rs:48-50)
__device__ __forceinline__ void rotate(float low, float high, uint32_t position, float frequency, float &out_low, float &out_high) {
    float angle = __fmul_rn((float)position, frequency);
    float cosine = cosf(angle), sine = sinf(angle);
    out_low = low * cosine - high * sine;
    out_high = high * cosine + low * sine;
}

__global__ __launch_bounds__(256) void rope_kernel(const float *__restrict__ x, uint32_t planes, uint32_t batch, uint32_t rows,
                                                   uint32_t width, const uint32_t *__restrict__ cursor,
                                                   const float *__restrict__ table, float *__restrict__ out) {
    const uint32_t half = width / 2;
    const uint64_t pairs = (uint64_t)planes * batch * rows * half;
    for (uint64_t index = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; index < pairs; index += (uint64_t)gridDim.x * blockDim.x) {
        uint32_t c = (uint32_t)(index % half);
        uint64_t vector = index / half;  // (plane, b, row)
        uint32_t row = (uint32_t)(vector % rows);
        uint32_t b = (uint32_t)((vector / rows) % batch);
        const float *src = x + vector * width;
        float low, high;
        rotate(src[c], src[c + half], (cursor ? cursor[b] : 0u) + row, table[c], low, high);
        out[vector * width + c] = low;
        out[vector * width + c + half] = high;
    }
}

int32_t launch_rope(nh_device *d, const float *x, uint32_t planes, uint32_t batch, uint32_t rows, uint32_t width,
                    const uint32_t *cursor, float base, float *out) {
    const float *table = rope_frequencies(d, base, width);
    if (!table) return NH_E_DEVICE;
    uint64_t pairs = (uint64_t)planes * batch * rows * (width / 2);
    if (!pairs) return NH_OK;
    uint32_t grid = (uint32_t)((pairs + 255) / 256 < 65535 ? (pairs + 255) / 256 : 65535);
    hipLaunchKernelGGL(rope_kernel, dim3(grid), dim3(256), 0, d->stream, x, planes, batch, rows, width, cursor, table, out);
    NH_HIP(hipGetLastError());
    return NH_OK;
}

// cast to the states' element and scatter whole rows (crates/neura-decoder/src/cache.rs:311-351,
// crates/neura-kernel/src/task/scatter.rs:149-171); an inactive plane writes the scratch rows
template <int CE>
__global__ __launch_bounds__(256) void cache_write_kernel(const float *__restrict__ k, const float *__restrict__ v,
                                                          void *__restrict__ cache_k, void *__restrict__ cache_v,
                                                          uint32_t kv_heads, uint32_t batch, uint32_t rows, uint32_t width,
                                                          uint32_t capacity, uint32_t window, const uint32_t *__restrict__ cursor,
                                                          const uint8_t *__restrict__ mask, uint32_t *refusal, bool ring) {
    const uint64_t total = (uint64_t)kv_heads * batch * rows * width;
    for (uint64_t index = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; index < total; index += (uint64_t)gridDim.x * blockDim.x) {
        uint32_t c = (uint32_t)(index % width);
        uint64_t vector = index / width;
        uint32_t row = (uint32_t)(vector % rows);
        uint32_t b = (uint32_t)((vector / rows) % batch);
        uint32_t head = (uint32_t)(vector / rows / batch);
        bool active = mask == nullptr || mask[b];
        // a ring seats position p at p mod window (crates/neura-decoder/src/layout.rs:32-36)
        uint32_t seat = ring ? (cursor[b] + row) % window : cursor[b] + row;
        uint32_t slot = active ? seat : window + row;
        if (slot >= capacity) {
            atomicMax(refusal, (uint32_t)REFUSAL_ORIGIN);
            continue;
        }
        uint64_t at = (((uint64_t)head * batch + b) * capacity + slot) * width + c;
        cache_store<CE>(cache_k, at, k[index]);
        cache_store<CE>(cache_v, at, v[index]);
    }
}

int32_t launch_cache_write(nh_device *d, const float *k, const float *v, void *cache_k, void *cache_v, uint32_t kv_heads,
                           uint32_t batch, uint32_t rows, uint32_t width, uint32_t capacity, uint32_t window, const uint32_t *cursor,
                           const uint8_t *mask, bool ring, int32_t cache_element) {
    uint64_t total = (uint64_t)kv_heads * batch * rows * width;
    if (!total) return NH_OK;
    uint32_t grid = (uint32_t)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
#define NH_WRITE(CE) hipLaunchKernelGGL(cache_write_kernel<CE>, dim3(grid), dim3(256), 0, d->stream, k, v, cache_k, cache_v, kv_heads, batch, rows, width, \
                                        capacity, window, cursor, mask, d->refusal, ring)
    if (cache_element == NH_F32) NH_WRITE(NH_F32);
    else if (cache_element == NH_BF16) NH_WRITE(NH_BF16);
    else NH_WRITE(NH_F16);
#undef NH_WRITE
    NH_HIP(hipGetLastError());
    return NH_OK;
}

// one token of one plane: value + bias cast into the value state at the cursor (what cache_write_kernel does for
// a value row whose key went out with the product that rotated it)
template <int CE>
__global__ __launch_bounds__(256) void value_append_kernel(const float *__restrict__ v, const float *__restrict__ bias, void *__restrict__ cache_v,
                                                           uint32_t kv_heads, uint32_t width, uint32_t capacity, const uint32_t *__restrict__ cursor,
                                                           uint32_t *refusal, uint32_t ring) {
    NH_FETCH(v, bias, cache_v, kv_heads, width, capacity, cursor, refusal, ring, blockDim.x);
    const uint32_t index = blockIdx.x * blockDim.x + threadIdx.x;
    if (index >= kv_heads * width) return;
    const uint32_t slot = ring ? cursor[0] % ring : cursor[0];
    if (slot >= capacity) {
        atomicMax(refusal, (uint32_t)REFUSAL_ORIGIN);
        return;
    }
    const uint32_t head = index / width, c = index % width;
    const float value = bias ? v[index] + bias[index] : v[index];
    cache_store<CE>(cache_v, ((uint64_t)head * capacity + slot) * width + c, value);
}

int32_t launch_value_append(nh_device *d, const float *v, const float *bias, void *cache_v, uint32_t kv_heads, uint32_t width, uint32_t capacity,
                            const uint32_t *cursor, uint32_t ring, int32_t cache_element) {
    const uint32_t total = kv_heads * width;
    if (!total) return NH_OK;
#define NH_APPEND(CE) hipLaunchKernelGGL(value_append_kernel<CE>, dim3((total + 255) / 256), dim3(256), 0, d->stream, v, bias, cache_v, kv_heads, width, capacity, \
                                         cursor, d->refusal, ring)
    if (cache_element == NH_F32) NH_APPEND(NH_F32);
    else if (cache_element == NH_BF16) NH_APPEND(NH_BF16);
    else NH_APPEND(NH_F16);
#undef NH_APPEND
    NH_HIP(hipGetLastError());
    return NH_OK;
}

__global__ __launch_bounds__(256) void rope_angles_kernel(const float *__restrict__ table, uint32_t half, uint32_t positions,
                                                          float *__restrict__ cosines, float *__restrict__ sines) {
    const uint64_t total = (uint64_t)positions * half;
    for (uint64_t index = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; index < total; index += (uint64_t)gridDim.x * blockDim.x) {
        const float angle = __fmul_rn((float)(uint32_t)(index / half), table[index % half]);  // as rotate() forms it
        cosines[index] = cosf(angle);
        sines[index] = sinf(angle);
    }
}

int32_t launch_rope_angles(nh_device *d, float base, uint32_t width, uint32_t positions, float *cosines, float *sines) {
    const float *table = rope_frequencies(d, base, width);
    if (!table) return NH_E_DEVICE;
    const uint64_t total = (uint64_t)positions * (width / 2);
    if (!total) return NH_OK;
    uint32_t grid = (uint32_t)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
    hipLaunchKernelGGL(rope_angles_kernel, dim3(grid), dim3(256), 0, d->stream, table, width / 2, positions, cosines, sines);
    NH_HIP(hipGetLastError());
    return NH_OK;
}

// The decoder's fused form of the two kernels above on a token-major buffer
// qkv [T][(heads + 2 kv_heads) * width], t = row * batch + plane: q is roped in place, k is
// roped, k and v are cast to the states' element and appended to the caches.
// A token a blockIdx.y, its (vector, channel pair) items over blockIdx.x: no 64-bit division on the way to an item.  `cosines` /
// `sines` [positions][width / 2] (may be null): what rotate() would compute for (position, channel pair), tabulated by
// rope_angles_kernel with the same instructions, so a table entry is bit for bit the cosine and sine formed on the spot;
// positions past the table are formed on the spot.
template <int CE>
__global__ __launch_bounds__(256) void rope_append_kernel(float *__restrict__ qkv, uint32_t heads, uint32_t kv_heads, uint32_t width,
                                                          uint32_t batch, uint32_t rows, void *__restrict__ cache_k,
                                                          void *__restrict__ cache_v, uint32_t capacity, uint32_t window,
                                                          const uint32_t *__restrict__ cursor, const uint8_t *__restrict__ mask,
                                                          const float *__restrict__ table, uint32_t *refusal, bool ring,
                                                          const float *__restrict__ cosines, const float *__restrict__ sines, uint32_t positions) {
    NH_FETCH(qkv, heads, kv_heads, width, batch, rows, cache_k, cache_v, capacity, window, cursor, mask, table, refusal, cosines, sines, positions);
    const uint32_t half = width / 2;
    const uint32_t vectors = heads + 2 * kv_heads;  // per token: q heads, k heads, v heads
    const uint32_t stride = vectors * width;
    const uint32_t items = vectors * half, tokens = batch * rows;
    const uint32_t item = blockIdx.x * blockDim.x + threadIdx.x;
    if (item >= items) return;
    const uint32_t c = item % half, vector = item / half;
    for (uint32_t t = blockIdx.y; t < tokens; t += gridDim.y) {
        const uint32_t row = t / batch, b = t % batch;
        float *src = qkv + (size_t)t * stride + (size_t)vector * width;
        const uint32_t position = cursor[b] + row;
        const bool key = vector >= heads && vector < heads + kv_heads;
        float low = src[c], high = src[c + half];
        if (vector < heads || key) {
            if (cosines && position < positions) {
                const float cosine = cosines[(size_t)position * half + c], sine = sines[(size_t)position * half + c];
                const float turned_low = low * cosine - high * sine, turned_high = high * cosine + low * sine;
                low = turned_low, high = turned_high;
            } else {
                rotate(low, high, position, table[c], low, high);
            }
        }
        if (vector < heads) {
            src[c] = low;
            src[c + half] = high;
            continue;
        }
        const bool active = mask == nullptr || mask[b];
        const uint32_t slot = active ? (ring ? position % window : position) : window + row;
        if (slot >= capacity) {
            atomicMax(refusal, (uint32_t)REFUSAL_ORIGIN);
            continue;
        }
        const uint32_t head = key ? vector - heads : vector - heads - kv_heads;
        const uint64_t at = (((uint64_t)head * batch + b) * capacity + slot) * width;
        void *cache = key ? cache_k : cache_v;
        cache_store<CE>(cache, at + c, low);
        cache_store<CE>(cache, at + c + half, high);
    }
}

int32_t launch_rope_append(nh_device *d, float *qkv, uint32_t heads, uint32_t kv_heads, uint32_t width, uint32_t batch, uint32_t rows,
                           void *cache_k, void *cache_v, uint32_t capacity, uint32_t window, const uint32_t *cursor,
                           const uint8_t *mask, float base, bool ring, int32_t cache_element, const float *cosines, const float *sines,
                           uint32_t positions) {
    const float *table = rope_frequencies(d, base, width);
    if (!table) return NH_E_DEVICE;
    const uint32_t items = (heads + 2 * kv_heads) * (width / 2), tokens = batch * rows;
    if (!items || !tokens) return NH_OK;
    const dim3 grid((items + 255u) / 256u, tokens < 65535u ? tokens : 65535u);
#define NH_ROPE(CE) hipLaunchKernelGGL(rope_append_kernel<CE>, grid, dim3(256), 0, d->stream, qkv, heads, kv_heads, width, batch, rows, cache_k, \
                                       cache_v, capacity, window, cursor, mask, table, d->refusal, ring, cosines, sines, positions)
    if (cache_element == NH_F32) NH_ROPE(NH_F32);
    else if (cache_element == NH_BF16) NH_ROPE(NH_BF16);
    else NH_ROPE(NH_F16);
#undef NH_ROPE
    NH_HIP(hipGetLastError());
    return NH_OK;
}

// silu(gate) * up (examples/qwen/mlp.rs:33; crates/neura-pointwise/src/op.rs:163)
// dst[r][c] = src[r][c] + bias[c]: places the columns of one projection in a wider row, or adds a bias where it stands
__global__ __launch_bounds__(256) void columns_kernel(const float *__restrict__ src, uint32_t lds, const float *__restrict__ bias,
                                                      float *__restrict__ dst, uint32_t ldd, uint32_t rows, uint32_t n) {
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < (uint64_t)rows * n; i += (uint64_t)gridDim.x * blockDim.x) {
        const uint32_t r = (uint32_t)(i / n), c = (uint32_t)(i % n);
        const float value = src[(size_t)r * lds + c];
        dst[(size_t)r * ldd + c] = bias ? value + bias[c] : value;
    }
}

int32_t launch_columns(nh_device *d, const float *src, uint32_t lds, const float *bias, float *dst, uint32_t ldd, uint32_t rows, uint32_t n) {
    if (!rows || !n) return NH_OK;
    const uint64_t wanted = ((uint64_t)rows * n + 255) / 256, most = (uint64_t)d->compute_units * 8;
    hipLaunchKernelGGL(columns_kernel, dim3((uint32_t)(wanted < most ? wanted : most)), dim3(256), 0, d->stream, src, lds, bias, dst, ldd, rows, n);
    NH_HIP(hipGetLastError());
    return NH_OK;
}

__global__ __launch_bounds__(256) void silu_mul_kernel(const float *__restrict__ gate, const float *__restrict__ up, uint64_t n,
                                                       float *__restrict__ out) {
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (uint64_t)gridDim.x * blockDim.x) {
        float a = gate[i];
        out[i] = a * (1.0f / (1.0f + expf(-a))) * up[i];
    }
}

int32_t launch_silu_mul(nh_device *d, const float *gate, const float *up, uint64_t n, float *out) {
    if (!n) return NH_OK;
    uint32_t grid = (uint32_t)((n + 255) / 256 < 65535 ? (n + 255) / 256 : 65535);
    hipLaunchKernelGGL(silu_mul_kernel, dim3(grid), dim3(256), 0, d->stream, gate, up, n, out);
    NH_HIP(hipGetLastError());
    return NH_OK;
}

// hidden *= mask of its plane (examples/qwen/model.rs:100); rows are t = row * batch + plane
__global__ __launch_bounds__(256) void mask_rows_kernel(float *__restrict__ x, uint32_t rows, uint32_t batch, uint32_t width,
                                                        const uint8_t *__restrict__ mask) {
    const uint64_t total = (uint64_t)rows * batch * width;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (uint64_t)gridDim.x * blockDim.x) {
        uint32_t b = (uint32_t)((i / width) % batch);
        if (!mask[b]) x[i] = 0.0f;
    }
}

int32_t launch_mask_rows(nh_device *d, float *x, uint32_t rows, uint32_t batch, uint32_t width, const uint8_t *mask) {
    uint64_t total = (uint64_t)rows * batch * width;
    if (!total || !mask) return NH_OK;
    uint32_t grid = (uint32_t)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
    hipLaunchKernelGGL(mask_rows_kernel, dim3(grid), dim3(256), 0, d->stream, x, rows, batch, width, mask);
    NH_HIP(hipGetLastError());
    return NH_OK;
}

}  // namespace nh
