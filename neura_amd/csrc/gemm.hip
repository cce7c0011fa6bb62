// Wide products (prefill): Y[m][n] = sum_k X[m][k] * W[n][k], W in raw GGUF blocks.
//
// Tile 64 (m) x 64 (n) x 32 (k) per 256-thread workgroup.  The weight tile is dequantised
// into LDS once per k step (one Q8_0 block / one Q4_K sub-block deep) and reused by all 64
// activation rows; each thread owns a 4 x 4 patch of the output in registers.
#include "blocks.hpp"
#include "common.hpp"

#include <cstdlib>

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

// ------------------------------------------------------------------- Q4_K on MFMA --------
//
// Workgroup tile: 128 activation rows x 128 weight rows, walked 64 k at a time (one 64-element
// group of a super-block = sub-blocks 2g and 2g+1).  The 256 threads unpack the weight tile into
// LDS as halves holding code * sc -- an integer below 1024, exact in half precision -- so the
// matrix cores multiply exact integers by half-precision activations and add in fp32; after the
// four groups of a super-block the 64 x 64 result of each wave is weighed by d in fp32 and
// added to the running sums, and one more MFMA of depth 16 over (minimum, sub-block activation
// sum) pairs, weighed by dmin, takes the minimums off:
//     y = sum_blocks  d * sum_s sc_s * sum_k q_k x_k  -  dmin * sum_s m_s * sum_k x_k
// which is the reference's value (crates/neura-kernel/src/dot.rs:328-350, matmul.rs:1083-1221)
// regrouped per sub-block.  fp32 activations enter as two half rows each (the value rounded to
// half and the rounding residue times 2^11, after a power-of-two row scale), so 22 bits of
// every activation take part; half activations enter as they are.
//
// A nibble masked in place in a 16-bit lane is the half subnormal code * 2^-24 (or 2^-20);
// one packed half multiply by sc * 2^10 (or 2^6) turns it into the normal half code*sc*2^-14.

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int GT = 128;           // tile edge (rows of A' and rows of W)
constexpr int GK = 64;            // k per step
constexpr int GS = GK + 8;        // LDS row stride in halves: 144 B keeps 128-bit reads of 8 neighbouring rows on distinct banks

struct GemmQ4Params {
    const uint8_t *W;
    uint32_t N, K, row_bytes;
    const _Float16 *A;   // [rows][K] halves; with `split`, row 2m is the rounded value of activation row m and row 2m+1 its residue * 2^11
    uint32_t rows;       // rows of A
    float *Y;
    const float *residual;
    uint32_t ldy, M;
    int32_t split;
    const float *unscale;  // [M] with split: undoes the row scale
};

// fp32 activations -> scaled (value, residue) half rows
__global__ __launch_bounds__(256) void gemm_split_rows_kernel(const float *__restrict__ X, uint32_t K, _Float16 *__restrict__ A, float *__restrict__ unscale) {
    __shared__ uint32_t wave_top[4];
    const uint32_t m = blockIdx.x, tid = threadIdx.x;
    const float *x = X + (size_t)m * K;
    uint32_t top = 0;
    for (uint32_t k = tid; k < K; k += 256) top = max(top, __builtin_bit_cast(uint32_t, x[k]) & 0x7fffffffu);
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) top = max(top, (uint32_t)__shfl_xor((int)top, offset, 64));
    if ((tid & 63u) == 0) wave_top[tid >> 6] = top;
    __syncthreads();
    top = max(max(wave_top[0], wave_top[1]), max(wave_top[2], wave_top[3]));
    // a power of two that puts the largest magnitude in [2^13, 2^14)
    const uint32_t raw = top >> 23, exponent = min(max(raw, 27u), 254u);
    const float scale = __builtin_bit_cast(float, (267u - exponent) << 23);
    if (tid == 0) unscale[m] = raw == 255u ? __builtin_bit_cast(float, 0x7fc00000u) : __builtin_bit_cast(float, (exponent - 13u) << 23);
    _Float16 *hi = A + (size_t)(2 * m) * K, *lo = hi + K;
    for (uint32_t k = tid; k < K; k += 256) {
        const float t = x[k] * scale;
        const _Float16 h = (_Float16)t;
        hi[k] = h;
        lo[k] = (_Float16)((t - (float)h) * 2048.0f);
    }
}

__global__ __launch_bounds__(256, 2) void gemm_q4k_mfma_kernel(GemmQ4Params p) {
    __shared__ __attribute__((aligned(16))) _Float16 As[GT][GS];
    __shared__ __attribute__((aligned(16))) _Float16 Bs[GT][GS];
    __shared__ __attribute__((aligned(16))) float xs[GT][8];        // sub-block sums of the activation rows of this super-block, / 64
    __shared__ __attribute__((aligned(16))) _Float16 mns[GT][8];    // the eight minimums of every weight row
    __shared__ uint32_t dds[GT];                                    // (d, dmin) of every weight row
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t n0 = blockIdx.x * GT, m0 = blockIdx.y * GT;
    // staging role: one row of each tile, one half (32 k) of the step
    const uint32_t srow = tid >> 1, sh = tid & 1u;
    const uint8_t *wrow = p.W + (size_t)min(n0 + srow, p.N - 1u) * p.row_bytes;
    const _Float16 *arow = p.A + (size_t)min(m0 + srow, p.rows - 1u) * p.K + 32u * sh;
    // compute role: wave (wm, wn) owns rows 64 wm.. of A' and weight rows 64 wn..
    const uint32_t wm = wave >> 1, wn = wave & 1u, l32 = lane & 31u, part = lane >> 5;

    f32x16 acc[2][2], tmp[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f, tmp[i][j][e] = 0.0f;

    typedef const __attribute__((address_space(1))) u32x4 *global_uint4;
    u32x4 hdr, qs, av[4];
    auto fetch = [&](uint32_t step) {
        const uint32_t b = step >> 2, g = step & 3u;
        const uint8_t *block = wrow + (size_t)b * 144u;
        hdr = *(global_uint4)(uintptr_t)block;
        qs = *(global_uint4)(uintptr_t)(block + 16u + 32u * g + 16u * sh);
        const _Float16 *at = arow + (size_t)step * 64u;
#pragma unroll
        for (int i = 0; i < 4; i++) av[i] = *(global_uint4)(uintptr_t)(at + 8 * i);
    };
    const uint32_t steps = p.K / 64u;
    fetch(0);
    for (uint32_t step = 0; step < steps; step++) {
        const uint32_t g = step & 3u;
        __syncthreads();  // the previous step's operands have been read
        {
            // ---- weights: 16 bytes = 16 low nibbles (sub-block 2g) and 16 high nibbles (sub-block 2g+1)
            const uint32_t shift = 16u * (g & 1u);
            const uint32_t ya = (hdr.y >> shift) & 0xffffu, za = (hdr.z >> shift) & 0xffffu, wa = (hdr.w >> shift) & 0xffffu;
            uint32_t sc0, sc1, mn0, mn1;  // crates/neura-precision/src/ggml.rs:127-136
            if (g < 2) {
                sc0 = ya & 63u, sc1 = (ya >> 8) & 63u, mn0 = za & 63u, mn1 = (za >> 8) & 63u;
            } else {
                sc0 = (wa & 0x0fu) | (((ya >> 6) & 3u) << 4);
                sc1 = ((wa >> 8) & 0x0fu) | (((ya >> 14) & 3u) << 4);
                mn0 = ((wa >> 4) & 0x0fu) | (((za >> 6) & 3u) << 4);
                mn1 = ((wa >> 12) & 0x0fu) | (((za >> 14) & 3u) << 4);
            }
            const _Float16 s_low = (_Float16)(float)(sc0 << 10), s_high = (_Float16)(float)(sc1 << 6);
            const half2_t low_scale = {s_low, s_low}, high_scale = {s_high, s_high};
            const uint32_t words[4] = {qs.x, qs.y, qs.z, qs.w};
            uint32_t low[8], high[8];
#pragma unroll
            for (int w = 0; w < 4; w++) {
                const uint32_t even = words[w], odd = words[w] >> 8;
                // element order inside a word: 0, 2 then 1, 3 (the byte lanes); the activations are staged in the same order
                low[2 * w] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, even & 0x000f000fu) * low_scale);
                low[2 * w + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, odd & 0x000f000fu) * low_scale);
                high[2 * w] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, even & 0x00f000f0u) * high_scale);
                high[2 * w + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, odd & 0x00f000f0u) * high_scale);
            }
            uint4 *blow = reinterpret_cast<uint4 *>(&Bs[srow][16u * sh]), *bhigh = reinterpret_cast<uint4 *>(&Bs[srow][32u + 16u * sh]);
            blow[0] = make_uint4(low[0], low[1], low[2], low[3]);
            blow[1] = make_uint4(low[4], low[5], low[6], low[7]);
            bhigh[0] = make_uint4(high[0], high[1], high[2], high[3]);
            bhigh[1] = make_uint4(high[4], high[5], high[6], high[7]);
            if (sh == 0) {
                mns[srow][2 * g] = (_Float16)(float)mn0;
                mns[srow][2 * g + 1] = (_Float16)(float)mn1;
                if (g == 0) dds[srow] = hdr.x;
            }
            // ---- activations: 32 halves of sub-block 2g + sh, reordered like the weights; their sum for the minimums
            float total = 0.0f;
            const half2_t ones = {(_Float16)1.0f, (_Float16)1.0f};
            uint4 *adst = reinterpret_cast<uint4 *>(&As[srow][32u * sh]);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t d[4] = {av[i].x, av[i].y, av[i].z, av[i].w};
#pragma unroll
                for (int e = 0; e < 4; e++) total = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, d[e]), ones, total, false);
                adst[i] = make_uint4(__builtin_amdgcn_perm(d[1], d[0], 0x05040100u), __builtin_amdgcn_perm(d[1], d[0], 0x07060302u),
                                     __builtin_amdgcn_perm(d[3], d[2], 0x05040100u), __builtin_amdgcn_perm(d[3], d[2], 0x07060302u));
            }
            xs[srow][2 * g + sh] = total * 0.015625f;
        }
        __syncthreads();
        if (step + 1 < steps) fetch(step + 1);
        // ---- 64 x 64 x 64 per wave
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            half8_t a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; i++) a[i] = *reinterpret_cast<const half8_t *>(&As[64u * wm + 32u * i + l32][16u * kk + 8u * part]);
#pragma unroll
            for (int j = 0; j < 2; j++) b[j] = *reinterpret_cast<const half8_t *>(&Bs[64u * wn + 32u * j + l32][16u * kk + 8u * part]);
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) tmp[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], tmp[i][j], 0, 0, 0);
        }
        if (g == 3) {
            // ---- the super-block is complete: weigh by d, then take the minimums off
            float dscale[2], mscale[2];
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const half2_t dd = __builtin_bit_cast(half2_t, dds[64u * wn + 32u * j + l32]);
                dscale[j] = (float)dd.x * 16384.0f;  // the weights were staged * 2^-14
                mscale[j] = (float)dd.y * -64.0f;    // the sums were staged / 64
            }
            half8_t a2[2], b2[2];
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const float4 *sums = reinterpret_cast<const float4 *>(xs[64u * wm + 32u * i + l32]);
                const float4 s0 = sums[0], s1 = sums[1];
                const float v[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const _Float16 h = (_Float16)v[e];
                    a2[i][e] = part ? (_Float16)((v[e] - (float)h) * 2048.0f) : h;  // k 0..7: the sums; k 8..15: their residues * 2^11
                }
            }
#pragma unroll
            for (int j = 0; j < 2; j++) {
                b2[j] = *reinterpret_cast<const half8_t *>(mns[64u * wn + 32u * j + l32]);
                if (part) b2[j] = b2[j] * (_Float16)0.00048828125f;  // k 8..15: the minimums * 2^-11
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) {
#pragma unroll
                    for (int e = 0; e < 16; e++) acc[i][j][e] = fmaf(dscale[j], tmp[i][j][e], acc[i][j][e]);
                    f32x16 zero;
#pragma unroll
                    for (int e = 0; e < 16; e++) zero[e] = 0.0f;
                    const f32x16 mins = __builtin_amdgcn_mfma_f32_32x32x16_f16(a2[i], b2[j], zero, 0, 0, 0);
#pragma unroll
                    for (int e = 0; e < 16; e++) acc[i][j][e] = fmaf(mscale[j], mins[e], acc[i][j][e]), tmp[i][j][e] = 0.0f;
                }
        }
    }
    // ---- out: lane (l32, part) holds column n = l32 of a 32 x 32 block; register 4q + e is row 8q + 4 part + e
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint32_t n = n0 + 64u * wn + 32u * j + l32;
            if (n >= p.N) continue;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const uint32_t row = m0 + 64u * wm + 32u * i + 8u * q + 4u * part;  // first of four rows of A'
                if (p.split) {
#pragma unroll
                    for (int e = 0; e < 2; e++) {
                        const uint32_t m = (row >> 1) + e;
                        if (m >= p.M) continue;
                        float value = fmaf(acc[i][j][4 * q + 2 * e + 1], 0.00048828125f, acc[i][j][4 * q + 2 * e]) * p.unscale[m];
                        const size_t at = (size_t)m * p.ldy + n;
                        p.Y[at] = p.residual ? p.residual[at] + value : value;
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const uint32_t m = row + e;
                        if (m >= p.M) continue;
                        const size_t at = (size_t)m * p.ldy + n;
                        p.Y[at] = p.residual ? p.residual[at] + acc[i][j][4 * q + e] : acc[i][j][4 * q + e];
                    }
                }
            }
        }
}

static int32_t launch_gemm_q4k_mfma(nh_device *d, const GemmArgs &a) {
    GemmQ4Params p{};
    p.W = static_cast<const uint8_t *>(a.W);
    p.N = a.N;
    p.K = a.K;
    p.row_bytes = (uint32_t)payload_bytes(NH_Q4_K, a.K);
    p.Y = a.Y;
    p.residual = a.residual;
    p.ldy = a.ldy;
    p.M = a.M;
    if (a.x_element == NH_F16) {
        p.A = static_cast<const _Float16 *>(a.X);
        p.rows = a.M;
        p.split = 0;
    } else {
        // scratch: [2M][K] halves, then M row scales
        const size_t halves = (size_t)2 * a.M * a.K * sizeof(_Float16);
        uint8_t *room = static_cast<uint8_t *>(scratch(d, halves + (size_t)a.M * sizeof(float)));
        if (!room) return NH_E_MEMORY;
        _Float16 *A = reinterpret_cast<_Float16 *>(room);
        float *unscale = reinterpret_cast<float *>(room + halves);
        hipLaunchKernelGGL(gemm_split_rows_kernel, dim3(a.M), dim3(256), 0, d->stream, static_cast<const float *>(a.X), a.K, A, unscale);
        NH_HIP(hipGetLastError());
        p.A = A;
        p.rows = 2 * a.M;
        p.split = 1;
        p.unscale = unscale;
    }
    dim3 grid((a.N + GT - 1) / GT, (p.rows + GT - 1) / GT);
    hipLaunchKernelGGL(gemm_q4k_mfma_kernel, grid, dim3(256), 0, d->stream, p);
    NH_HIP(hipGetLastError());
    return NH_OK;
}

int32_t launch_gemm(nh_device *d, const GemmArgs &a) {
    if (!a.M || !a.N) return NH_OK;
    {
        const char *held = getenv("NEURA_HIP_GEMM_MFMA");
        const bool wanted = !(held && held[0] == '0');
        const bool aligned = ((uintptr_t)a.X & 15u) == 0 && ((uintptr_t)a.W & 15u) == 0;
        if (wanted && aligned && a.element == NH_Q4_K && a.K % 256u == 0) return launch_gemm_q4k_mfma(d, a);
    }
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
