// Wide products (prefill): Y[m][n] = sum_k X[m][k] * W[n][k], W in raw GGUF blocks.
//
// Tile 64 (m) x 64 (n) x 32 (k) per 256-thread workgroup.  The weight tile is dequantised
// into LDS once per k step (one Q8_0 block / one Q4_K sub-block deep) and reused by all 64
// activation rows; each thread owns a 4 x 4 patch of the output in registers.
#include "blocks.hpp"
#include "common.hpp"

namespace nh {

constexpr int BM = 64, BN = 64, BK = 32;

template <int ELEMENT, bool X_HALF>
__global__ __launch_bounds__(256) void gemm_kernel(const uint8_t *__restrict__ W, uint32_t N, uint32_t K, uint32_t row_bytes,
                                                   const void *__restrict__ X, uint32_t M, float *Y, const float *residual,
                                                   uint32_t ldy) {
    __shared__ float xs[BK][BM + 4];
    __shared__ float ws[BK][BN + 4];
    const uint32_t tid = threadIdx.x;
    const uint32_t m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const uint32_t tx = tid % 16, ty = tid / 16;  // patch: rows m0 + ty*4.., columns n0 + tx*4..
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = 0.0f;

    for (uint32_t k0 = 0; k0 < K; k0 += BK) {
        // stage X: 64 rows x 32 k, thread -> (row = tid / 4, 8 consecutive k)
        {
            uint32_t r = tid / 4, kk = (tid % 4) * 8;
            uint32_t m = m0 + r;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                float value = 0.0f;
                if (m < M && k0 + kk + j < K) {
                    if (X_HALF)
                        value = half_to_float(static_cast<const uint16_t *>(X)[(size_t)m * K + k0 + kk + j]);
                    else
                        value = static_cast<const float *>(X)[(size_t)m * K + k0 + kk + j];
                }
                xs[kk + j][r] = value;
            }
        }
        // stage W: 64 rows x 32 k dequantised
        {
            uint32_t r = tid / 4, kk = (tid % 4) * 8;
            uint32_t n = n0 + r;
            const uint8_t *row = W + (size_t)(n < N ? n : 0) * row_bytes;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                float value = 0.0f;
                if (n < N && k0 + kk + j < K) {
                    if (ELEMENT == NH_Q8_0)
                        value = q8_0_element(row, k0 + kk + j);
                    else
                        value = q4_k_element(row, k0 + kk + j);
                }
                ws[kk + j][r] = value;
            }
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK; kk++) {
            float4 a = *reinterpret_cast<const float4 *>(&xs[kk][ty * 4]);
            float4 b = *reinterpret_cast<const float4 *>(&ws[kk][tx * 4]);
            const float av[4] = {a.x, a.y, a.z, a.w}, bv[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        uint32_t m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            uint32_t n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float value = acc[i][j];
            if (residual) value = residual[(size_t)m * ldy + n] + value;
            Y[(size_t)m * ldy + n] = value;
        }
    }
}

int32_t launch_gemm(nh_device *d, const GemmArgs &a) {
    if (!a.M || !a.N) return NH_OK;
    dim3 grid((a.N + BN - 1) / BN, (a.M + BM - 1) / BM), block(256);
    uint32_t row_bytes = (uint32_t)payload_bytes(a.element, a.K);
    const uint8_t *W = static_cast<const uint8_t *>(a.W);
    bool half = a.x_element == NH_F16;
#define NH_GEMM(E, H) hipLaunchKernelGGL((gemm_kernel<E, H>), grid, block, 0, d->stream, W, a.N, a.K, row_bytes, a.X, a.M, a.Y, a.residual, a.ldy)
    if (a.element == NH_Q8_0) {
        if (half) NH_GEMM(NH_Q8_0, true);
        else NH_GEMM(NH_Q8_0, false);
    } else if (a.element == NH_Q4_K) {
        if (half) NH_GEMM(NH_Q4_K, true);
        else NH_GEMM(NH_Q4_K, false);
    } else {
        return fail(NH_E_ARGUMENT, "element %d carries no wide product", a.element);
    }
#undef NH_GEMM
    NH_HIP(hipGetLastError());
    return NH_OK;
}

}  // namespace nh
