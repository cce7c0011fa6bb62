// Wide products (prefill): Y[m][n] = sum_k X[m][k] * W[n][k], W in raw GGUF blocks.
//
// Tile 64 (m) x 64 (n) x 32 (k) per 256-thread workgroup.  The weight tile is dequantised
// into LDS once per k step (one Q8_0 block / one sub-block of a super-block format deep) and reused by all 64
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
                if (n < N && k0 + kk + j < K) value = stored_element<ELEMENT>(row, k0 + kk + j);
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
//
// Everything that does not depend on the weights is done once per activation row by a kernel
// of its own (gemm_pack_rows_kernel): the halves in the element order the unpacked nibbles come
// out in, and the sub-block sums the minimums are weighed by, already cut into the operand of
// their MFMA.  The tile loop is left with copies for the activations and four instructions
// per eight weights, and stages step s + 1 into the other half of LDS while the matrix cores
// walk step s: one barrier per step.

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int GT = 128;           // tile edge (rows of A' and rows of W)
constexpr int GK = 64;            // k per step
constexpr int GS = GK + 8;        // LDS row stride in halves: 144 B keeps 128-bit reads of 8 neighbouring rows on distinct banks

struct GemmQ4Params {
    const uint8_t *W;
    const uint8_t *W1, *W2;  // matrices stacked along N behind W: columns [end0, end1) and [end1, N); both ends are multiples of the tile
    uint32_t end0, end1;
    uint32_t N, K, row_bytes;
    const _Float16 *A;   // [rows][K] halves, every four k in the order 0, 2, 1, 3; with `split`, row 2m is the rounded value of
                         // activation row m and row 2m+1 its residue * 2^11
    const _Float16 *S;   // [rows][K / 256][16]: the eight sub-block sums / 64 of a super-block as halves, then their residues * 2^11
    uint32_t rows;       // rows of A
    float *Y;
    const float *residual;
    uint32_t ldy, M;
    int32_t split;
    const float *unscale;  // [M] with split: undoes the row scale
};

__device__ __forceinline__ void fetch_parameters(const GemmQ4Params &p) {
    NH_FETCH(p.W, p.W1, p.W2, p.end0, p.end1, p.N, p.K, p.row_bytes, p.A, p.S, p.rows, p.Y, p.residual, p.ldy, p.M, p.split, p.unscale);
}

// Four neighbouring numbers of a row (`hi`: as halves; `lo`, with SPLIT: their residues * 2^11) into the packed rows, and their
// share of the sub-block sums: eight neighbouring lanes hold the 32 numbers of a sub-block.
template <bool SPLIT>
__device__ __forceinline__ void pack_piece(const _Float16 (&hi)[4], const _Float16 (&lo)[4], uint32_t row, uint32_t k, uint32_t K, uint32_t nsb,
                                           _Float16 *__restrict__ A, _Float16 *__restrict__ S) {
    // the nibbles of four weight bytes unpack as bytes 0, 2, 1, 3
    const half4_t out_hi = {hi[0], hi[2], hi[1], hi[3]}, out_lo = {lo[0], lo[2], lo[1], lo[3]};
    *reinterpret_cast<half4_t *>(A + (size_t)row * K + k) = out_hi;
    if (SPLIT) *reinterpret_cast<half4_t *>(A + (size_t)(row + 1u) * K + k) = out_lo;
    // sums of the 32 halves of a sub-block: eight neighbouring lanes
    float sum_hi = ((float)hi[0] + (float)hi[1]) + ((float)hi[2] + (float)hi[3]);
    float sum_lo = ((float)lo[0] + (float)lo[1]) + ((float)lo[2] + (float)lo[3]);
#pragma unroll
    for (int offset = 1; offset < 8; offset <<= 1) {
        sum_hi += __shfl_xor(sum_hi, offset, 64);
        sum_lo += __shfl_xor(sum_lo, offset, 64);
    }
    if ((threadIdx.x & 7u) == 0) {
        const uint32_t sb = k >> 8, slot = (k >> 5) & 7u;
        {
            const float v = sum_hi * 0.015625f;
            const _Float16 h = (_Float16)v;
            _Float16 *dst = S + ((size_t)row * nsb + sb) * 16u;
            dst[slot] = h;
            dst[8u + slot] = (_Float16)((v - (float)h) * 2048.0f);
        }
        if (SPLIT) {
            const float v = sum_lo * 0.015625f;
            const _Float16 h = (_Float16)v;
            _Float16 *dst = S + ((size_t)(row + 1u) * nsb + sb) * 16u;
            dst[slot] = h;
            dst[8u + slot] = (_Float16)((v - (float)h) * 2048.0f);
        }
    }
}

// One workgroup per activation row: the row as MFMA-ready halves (and, for fp32 rows, its residue row and scale).
// PRELUDE: what a row is before it is packed -- 0: X as it lies; 1: X normalised (rmsnorm_kernel's arithmetic, so the same
// fp32 numbers: thread t adds the squares of columns t, t + 256, ..., then a 256-wide tree); 2: silu(gate) * X as
// silu_mul_kernel forms it.  `aux` is the norm's weight vector or the gate rows.
constexpr int PACK_PLAIN = 0, PACK_NORM = 1, PACK_SWIGLU = 2;
template <bool HALF_IN, int PRELUDE = PACK_PLAIN>
__global__ __launch_bounds__(256) void gemm_pack_rows_kernel(const void *__restrict__ X, uint32_t K, _Float16 *__restrict__ A,
                                                             _Float16 *__restrict__ S, float *__restrict__ unscale,
                                                             const float *__restrict__ aux = nullptr, float eps = 0.0f) {
    static_assert(!(HALF_IN && PRELUDE != PACK_PLAIN), "half rows are packed as they lie");
    __shared__ uint32_t wave_top[4];
    __shared__ float red[256];
    const uint32_t m = blockIdx.x, tid = threadIdx.x;
    const uint32_t nsb = (K + 255u) / 256u;
    float scale = 1.0f, norm = 1.0f;
    if (PRELUDE == PACK_NORM) {
        const float *xr = static_cast<const float *>(X) + (size_t)m * K;
        float square = 0.0f;
        for (uint32_t c = tid; c < K; c += 256) square = __fadd_rn(square, __fmul_rn(xr[c], xr[c]));
        red[tid] = square;
        __syncthreads();
        for (uint32_t stride = 128; stride > 0; stride >>= 1) {
            if (tid < stride) red[tid] = __fadd_rn(red[tid], red[tid + stride]);
            __syncthreads();
        }
        norm = rms_scale_of(red[0], K, eps);
    }
    // four neighbouring numbers of the row as the packing sees them
    auto fetch = [&](uint32_t k) -> float4 {
        float4 v = *reinterpret_cast<const float4 *>(static_cast<const float *>(X) + (size_t)m * K + k);
        if (PRELUDE == PACK_NORM) {
            const float4 w = *reinterpret_cast<const float4 *>(aux + k);
            v.x = __fmul_rn(__fmul_rn(v.x, norm), w.x), v.y = __fmul_rn(__fmul_rn(v.y, norm), w.y);
            v.z = __fmul_rn(__fmul_rn(v.z, norm), w.z), v.w = __fmul_rn(__fmul_rn(v.w, norm), w.w);
        } else if (PRELUDE == PACK_SWIGLU) {
            const float4 g = *reinterpret_cast<const float4 *>(aux + (size_t)m * K + k);
            v.x = g.x * (1.0f / (1.0f + expf(-g.x))) * v.x, v.y = g.y * (1.0f / (1.0f + expf(-g.y))) * v.y;
            v.z = g.z * (1.0f / (1.0f + expf(-g.z))) * v.z, v.w = g.w * (1.0f / (1.0f + expf(-g.w))) * v.w;
        }
        return v;
    };
    if (!HALF_IN) {
        uint32_t top = 0;
        for (uint32_t k = tid * 4u; k < K; k += 1024u) {
            const float4 v = fetch(k);
            top = max(max(top, __builtin_bit_cast(uint32_t, v.x) & 0x7fffffffu), __builtin_bit_cast(uint32_t, v.y) & 0x7fffffffu);
            top = max(max(top, __builtin_bit_cast(uint32_t, v.z) & 0x7fffffffu), __builtin_bit_cast(uint32_t, v.w) & 0x7fffffffu);
        }
#pragma unroll
        for (int offset = 32; offset > 0; offset >>= 1) top = max(top, (uint32_t)__shfl_xor((int)top, offset, 64));
        if ((tid & 63u) == 0) wave_top[tid >> 6] = top;
        __syncthreads();
        top = max(max(wave_top[0], wave_top[1]), max(wave_top[2], wave_top[3]));
        // a power of two that puts the largest magnitude in [2^13, 2^14)
        const uint32_t raw = top >> 23, exponent = min(max(raw, 27u), 254u);
        scale = __builtin_bit_cast(float, (267u - exponent) << 23);
        if (tid == 0) unscale[m] = raw == 255u ? __builtin_bit_cast(float, 0x7fc00000u) : __builtin_bit_cast(float, (exponent - 13u) << 23);
    }
    const uint32_t row = HALF_IN ? m : 2u * m;
    for (uint32_t k = tid * 4u; k < K; k += 1024u) {
        _Float16 hi[4], lo[4];
        if (HALF_IN) {
            const half4_t v = *reinterpret_cast<const half4_t *>(static_cast<const _Float16 *>(X) + (size_t)m * K + k);
#pragma unroll
            for (int e = 0; e < 4; e++) hi[e] = v[e], lo[e] = (_Float16)0.0f;
        } else {
            const float4 v = fetch(k);
            const float t[4] = {v.x * scale, v.y * scale, v.z * scale, v.w * scale};
#pragma unroll
            for (int e = 0; e < 4; e++) {
                hi[e] = (_Float16)t[e];
                lo[e] = (_Float16)((t[e] - (float)hi[e]) * 2048.0f);
            }
        }
        pack_piece<!HALF_IN>(hi, lo, row, k, K, nsb, A, S);
    }
}

// The same for fp32 rows, through LDS: the kernel above walks a row three times (the norm's squares, the largest magnitude,
// the packing) and meets every value as it arrives -- a memory round trip a value and walk, 22 in a row on a 3584-wide row
// with the norm, 37 on an 18944-wide gated one.  Here a row crosses memory once, four 16-byte loads a thread in flight at a
// time, and waits in LDS as the prelude left it: the squares are added from LDS in the same thread order, the packing reads
// LDS.  The same arithmetic on the same numbers: the packed rows are the kernel above's bit for bit.  K is a multiple of 4.
template <int PRELUDE>
__global__ __launch_bounds__(256) void gemm_pack_rows_staged_kernel(const float *__restrict__ X, uint32_t K, _Float16 *__restrict__ A,
                                                                    _Float16 *__restrict__ S, float *__restrict__ unscale,
                                                                    const float *__restrict__ aux, float eps) {
    extern __shared__ __attribute__((aligned(16))) float staged_row[];  // [K]
    __shared__ uint32_t wave_top[4];
    __shared__ float red[256];
    const uint32_t m = blockIdx.x, tid = threadIdx.x;
    const uint32_t nsb = (K + 255u) / 256u;
    const float *xr = X + (size_t)m * K;
    const float *other = PRELUDE == PACK_NORM ? aux : (PRELUDE == PACK_SWIGLU ? aux + (size_t)m * K : nullptr);
    float norm = 1.0f;
    if (PRELUDE == PACK_NORM) {
        for (uint32_t k0 = tid * 4u; k0 < K; k0 += 4096u) {
            float4 held[4];
#pragma unroll
            for (int j = 0; j < 4; j++) held[j] = *reinterpret_cast<const float4 *>(xr + min(k0 + 1024u * j, K - 4u));
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (k0 + 1024u * j < K) *reinterpret_cast<float4 *>(staged_row + k0 + 1024u * j) = held[j];
        }
        __syncthreads();
        float square = 0.0f;  // thread t adds the squares of columns t, t + 256, ... as rmsnorm_kernel does
        for (uint32_t c = tid; c < K; c += 256) square = __fadd_rn(square, __fmul_rn(staged_row[c], staged_row[c]));
        red[tid] = square;
        __syncthreads();
        for (uint32_t stride = 128; stride > 0; stride >>= 1) {
            if (tid < stride) red[tid] = __fadd_rn(red[tid], red[tid + stride]);
            __syncthreads();
        }
        norm = rms_scale_of(red[0], K, eps);
    }
    uint32_t top = 0;
    for (uint32_t k0 = tid * 4u; k0 < K; k0 += 4096u) {
        float4 held[4], with[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t k = min(k0 + 1024u * j, K - 4u);
            held[j] = PRELUDE == PACK_NORM ? *reinterpret_cast<const float4 *>(staged_row + k) : *reinterpret_cast<const float4 *>(xr + k);
            if (PRELUDE != PACK_PLAIN) with[j] = *reinterpret_cast<const float4 *>(other + k);
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (k0 + 1024u * j >= K) continue;
            float4 v = held[j];
            if (PRELUDE == PACK_NORM) {
                const float4 w = with[j];
                v.x = __fmul_rn(__fmul_rn(v.x, norm), w.x), v.y = __fmul_rn(__fmul_rn(v.y, norm), w.y);
                v.z = __fmul_rn(__fmul_rn(v.z, norm), w.z), v.w = __fmul_rn(__fmul_rn(v.w, norm), w.w);
            } else if (PRELUDE == PACK_SWIGLU) {
                const float4 g = with[j];
                v.x = g.x * (1.0f / (1.0f + expf(-g.x))) * v.x, v.y = g.y * (1.0f / (1.0f + expf(-g.y))) * v.y;
                v.z = g.z * (1.0f / (1.0f + expf(-g.z))) * v.z, v.w = g.w * (1.0f / (1.0f + expf(-g.w))) * v.w;
            }
            top = max(max(top, __builtin_bit_cast(uint32_t, v.x) & 0x7fffffffu), __builtin_bit_cast(uint32_t, v.y) & 0x7fffffffu);
            top = max(max(top, __builtin_bit_cast(uint32_t, v.z) & 0x7fffffffu), __builtin_bit_cast(uint32_t, v.w) & 0x7fffffffu);
            *reinterpret_cast<float4 *>(staged_row + k0 + 1024u * j) = v;  // the thread that packs these four wrote them
        }
    }
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) top = max(top, (uint32_t)__shfl_xor((int)top, offset, 64));
    if ((tid & 63u) == 0) wave_top[tid >> 6] = top;
    __syncthreads();
    top = max(max(wave_top[0], wave_top[1]), max(wave_top[2], wave_top[3]));
    // a power of two that puts the largest magnitude in [2^13, 2^14)
    const uint32_t raw = top >> 23, exponent = min(max(raw, 27u), 254u);
    const float scale = __builtin_bit_cast(float, (267u - exponent) << 23);
    if (tid == 0) unscale[m] = raw == 255u ? __builtin_bit_cast(float, 0x7fc00000u) : __builtin_bit_cast(float, (exponent - 13u) << 23);
    for (uint32_t k = tid * 4u; k < K; k += 1024u) {
        const float4 v = *reinterpret_cast<const float4 *>(staged_row + k);
        const float t[4] = {v.x * scale, v.y * scale, v.z * scale, v.w * scale};
        _Float16 hi[4], lo[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            hi[e] = (_Float16)t[e];
            lo[e] = (_Float16)((t[e] - (float)hi[e]) * 2048.0f);
        }
        pack_piece<true>(hi, lo, 2u * m, k, K, nsb, A, S);
    }
}

static bool pack_unstaged() {  // NEURA_HIP_PACK_STAGED=0: the packing that walks a row in memory
    const char *held = getenv("NEURA_HIP_PACK_STAGED");
    return held && held[0] == '0';
}
constexpr size_t PACK_STAGED_LDS_MOST = 152 * 1024;  // the widest row the staged packing holds: 38912 numbers
constexpr size_t GEMM_Q4K_LDS = sizeof(_Float16) * (2 * GT * GS + 2 * GT * GS + 2 * GT * 8) + sizeof(uint32_t) * 2 * GT;

// What the multiplier waves of a super-block wide product do (waves 0..3 of the workgroup; the stagers fill As, Bs, mns and dds).
// FLOORS: the weights have minimums (Q4_K, Q5_K), taken off with one more MFMA per four steps over (minimum, activation sum)
// pairs; SCALE is what the stagers divided the weights' operand by.  Four steps share one (d, dmin) in dds[(step / 4) & 1].
template <bool FLOORS>
__device__ __forceinline__ void gemm_multiply(const GemmQ4Params &p, _Float16 (*As)[GT][GS], _Float16 (*Bs)[GT][GS], _Float16 (*mns)[GT][8], uint32_t (*dds)[GT],
                                              const uint32_t wave, const uint32_t lane, const uint32_t n0, const uint32_t m0, const uint32_t steps, const float unscale_weights) {
    typedef const __attribute__((address_space(1))) u32x4 *global_uint4;
    // ---------------------------------------------------------------------- multipliers
    // wave (wm, wn) owns rows 64 wm.. of A' and weight rows 64 wn..
    const uint32_t wm = wave >> 1, wn = wave & 1u, l32 = lane & 31u, part = lane >> 5;
    const uint32_t nsb = p.K / 256u;
    const _Float16 *sums[2];
#pragma unroll
    for (int i = 0; i < 2; i++) sums[i] = p.S + (size_t)min(m0 + 64u * wm + 32u * i + l32, p.rows - 1u) * nsb * 16u + 8u * part;
    (void)sums;

    f32x16 acc[2][2], tmp[2][2], zero;
#pragma unroll
    for (int e = 0; e < 16; e++) zero[e] = 0.0f;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = zero, tmp[i][j] = zero;

    for (uint32_t first = 0; first < steps; first += 4) {
        const uint32_t sbuf = (first >> 2) & 1u;
        u32x4 sraw[2] = {u32x4{0u, 0u, 0u, 0u}, u32x4{0u, 0u, 0u, 0u}};
        if (FLOORS) {
#pragma unroll
            for (int i = 0; i < 2; i++) sraw[i] = *(global_uint4)(uintptr_t)(sums[i] + (size_t)(first >> 2) * 16u);  // wanted at the end of the super-block
        }
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const uint32_t buf = g & 1u;
            __syncthreads();  // the step is staged
            // ---- 64 x 64 x 64 per wave; the operands of the next 16 k are on their way while the matrix cores walk these
            half8_t a[2][2], b[2][2];
            auto operands = [&](int kk) {
#pragma unroll
                for (int i = 0; i < 2; i++) a[kk & 1][i] = *reinterpret_cast<const half8_t *>(&As[buf][64u * wm + 32u * i + l32][16u * kk + 8u * part]);
#pragma unroll
                for (int j = 0; j < 2; j++) b[kk & 1][j] = *reinterpret_cast<const half8_t *>(&Bs[buf][64u * wn + 32u * j + l32][16u * kk + 8u * part]);
            };
            operands(0);
#pragma unroll
            for (int kk = 0; kk < 4; kk++) {
                if (kk < 3) operands(kk + 1);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int j = 0; j < 2; j++)
                        tmp[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[kk & 1][i], b[kk & 1][j], (g == 0 && kk == 0) ? zero : tmp[i][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // ---- the super-block is complete: weigh by d, then take the minimums off
        float dscale[2], mscale[2];
        half8_t b2[2];
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const half2_t dd = __builtin_bit_cast(half2_t, dds[sbuf][64u * wn + 32u * j + l32]);
            dscale[j] = (float)dd.x * unscale_weights;
            mscale[j] = (float)dd.y * -64.0f;  // the sums were packed / 64
            if (FLOORS) {
                b2[j] = *reinterpret_cast<const half8_t *>(mns[sbuf][64u * wn + 32u * j + l32]);
                if (part) b2[j] = b2[j] * (_Float16)0.00048828125f;  // k 8..15: the minimums * 2^-11 against the residues * 2^11
            }
        }
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const half8_t a2 = __builtin_bit_cast(half8_t, sraw[i]);  // k 0..7: the sums; k 8..15: their residues
#pragma unroll
            for (int j = 0; j < 2; j++) {
#pragma unroll
                for (int e = 0; e < 16; e++) acc[i][j][e] = fmaf(dscale[j], tmp[i][j][e], acc[i][j][e]);
                if (FLOORS) {
                    const f32x16 mins = __builtin_amdgcn_mfma_f32_32x32x16_f16(a2, b2[j], zero, 0, 0, 0);
#pragma unroll
                    for (int e = 0; e < 16; e++) acc[i][j][e] = fmaf(mscale[j], mins[e], acc[i][j][e]);
                }
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

// The eight waves of a workgroup split the work by kind.  Waves 4..7 (the stagers) fetch raw blocks and packed
// activations four steps ahead into registers, unpack step s + 1 into LDS; waves 0..3 (the multipliers) do nothing
// but read operands and drive the matrix cores over step s.  One stager and one multiplier share each SIMD, so
// unpacking and memory latency hide behind the MFMAs instead of taking turns with them.
//
// FIFTH: Q5_K.  The header is Q4_K's; behind it come 32 bytes of fifth bits (bit 2g of byte l belongs to weight l of group g's
// low half, bit 2g + 1 to weight 32 + l) and then the nibbles.  A code of five bits times a scale of six stays below 2048, so
// the operand is as exact as Q4_K's: the fifth bit is set beside the nibble before the one multiplication.
template <bool FIFTH>
__device__ __forceinline__ void gemm_q45k_mfma(const GemmQ4Params &p) {
    constexpr uint32_t BLOCK = FIFTH ? 176u : 144u, NIBBLES = FIFTH ? 48u : 16u;
    extern __shared__ __attribute__((aligned(16))) uint8_t gemm_lds[];
    _Float16(*As)[GT][GS] = reinterpret_cast<_Float16(*)[GT][GS]>(gemm_lds);                                           // [2]
    _Float16(*Bs)[GT][GS] = reinterpret_cast<_Float16(*)[GT][GS]>(gemm_lds + sizeof(_Float16) * 2 * GT * GS);          // [2]
    _Float16(*mns)[GT][8] = reinterpret_cast<_Float16(*)[GT][8]>(gemm_lds + sizeof(_Float16) * 4 * GT * GS);           // [2] by super-block parity: the eight minimums of every weight row
    uint32_t(*dds)[GT] = reinterpret_cast<uint32_t(*)[GT]>(gemm_lds + sizeof(_Float16) * (4 * GT * GS + 2 * GT * 8));  // [2]: (d, dmin) of every weight row
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t n0 = blockIdx.x * GT, m0 = blockIdx.y * GT;
    const uint32_t steps = p.K / 64u;  // a multiple of 4: K is whole super-blocks
    typedef const __attribute__((address_space(1))) u32x4 *global_uint4;

    if (wave >= 4) {
        // ------------------------------------------------------------------ stagers
        // one row of each tile, one half (32 k) of the step
        const uint32_t tid = threadIdx.x - 256u;
        const uint32_t srow = tid >> 1, sh = tid & 1u;
        // a tile lies in one matrix: the boundaries between stacked matrices are multiples of the tile
        const uint32_t column = min(n0 + srow, p.N - 1u);
        const uint8_t *wrow = column < p.end0   ? p.W + (size_t)column * p.row_bytes
                              : column < p.end1 ? p.W1 + (size_t)(column - p.end0) * p.row_bytes
                                                : p.W2 + (size_t)(column - p.end1) * p.row_bytes;
        const _Float16 *arow = p.A + (size_t)min(m0 + srow, p.rows - 1u) * p.K + 32u * sh;
        u32x4 ahead, qs[4], av[4][4];  // the next super-block's header; groups and activations by slot = step % 4
        u32x4 fifth_ahead = {0u, 0u, 0u, 0u};  // Q5_K: the fifth bits of this thread's sixteen columns, next super-block
        const half2_t offset = {(_Float16)1024.0f, (_Float16)1024.0f}, powers = {(_Float16)1024.0f, (_Float16)64.0f};
        ahead = *(global_uint4)(uintptr_t)wrow;
        if (FIFTH) fifth_ahead = *(global_uint4)(uintptr_t)(wrow + 16u + 16u * sh);
#pragma unroll
        for (int g = 0; g < 4; g++) {  // steps 0..3 = super-block 0
            qs[g] = *(global_uint4)(uintptr_t)(wrow + NIBBLES + 32u * g + 16u * sh);
#pragma unroll
            for (int i = 0; i < 4; i++) av[g][i] = *(global_uint4)(uintptr_t)(arow + (size_t)g * 64u + 8 * i);
            __builtin_amdgcn_sched_barrier(0);  // slot 0 goes out first: the loop waits for the oldest slot only
        }
        for (uint32_t first = 0; first < steps; first += 4) {
            const u32x4 hdr = ahead, fifth = fifth_ahead;
            const uint32_t next = min((first >> 2) + 1u, (steps >> 2) - 1u);
            ahead = *(global_uint4)(uintptr_t)(wrow + (size_t)next * BLOCK);
            if (FIFTH) fifth_ahead = *(global_uint4)(uintptr_t)(wrow + (size_t)next * BLOCK + 16u + 16u * sh);
            const uint32_t fifth_words[4] = {fifth.x, fifth.y, fifth.z, fifth.w};
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const uint32_t buf = g & 1u, sbuf = (first >> 2) & 1u;
                // 6-bit fields of sub-blocks 2g, 2g+1 (crates/neura-precision/src/ggml.rs:127-136); 0x6400 | v is the half 1024 + v
                const uint32_t shift = 16u * (g & 1u);
                const uint32_t ya = (hdr.y >> shift) & 0xffffu, wa = (hdr.w >> shift) & 0xffffu;
                const uint32_t sc = g < 2 ? (ya & 0x3f3fu) : ((wa & 0x0f0fu) | ((ya >> 2) & 0x3030u));
                const uint32_t both = __builtin_amdgcn_perm(0u, sc, 0x0c010c00u) | 0x64006400u;  // (1024 + sc0, 1024 + sc1)
                const half2_t scales = (__builtin_bit_cast(half2_t, both) - offset) * powers;     // (sc0 * 2^10, sc1 * 2^6)
                const half2_t low_scale = {scales.x, scales.x}, high_scale = {scales.y, scales.y};
                const uint32_t words[4] = {qs[g].x, qs[g].y, qs[g].z, qs[g].w};
                uint32_t low[8], high[8];
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    const uint32_t even = words[w], odd = words[w] >> 8;
                    // element order inside a word: 0, 2 then 1, 3 (the byte lanes); the activations were packed in the same order
                    uint32_t low_even = even & 0x000f000fu, low_odd = odd & 0x000f000fu, high_even = even & 0x00f000f0u, high_odd = odd & 0x00f000f0u;
                    if (FIFTH) {
                        // bit 2g of a byte to bit 4 of its lane (beside the low nibble), bit 2g + 1 to bit 8 (beside the high nibble's four)
                        const uint32_t bits = fifth_words[w] >> (2 * g);
                        low_even |= (bits & 0x00010001u) << 4, low_odd |= ((bits >> 8) & 0x00010001u) << 4;
                        high_even |= (bits & 0x00020002u) << 7, high_odd |= ((bits >> 8) & 0x00020002u) << 7;
                    }
                    low[2 * w] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, low_even) * low_scale);
                    low[2 * w + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, low_odd) * low_scale);
                    high[2 * w] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, high_even) * high_scale);
                    high[2 * w + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, high_odd) * high_scale);
                }
                u32x4 *blow = reinterpret_cast<u32x4 *>(&Bs[buf][srow][16u * sh]), *bhigh = reinterpret_cast<u32x4 *>(&Bs[buf][srow][32u + 16u * sh]);
                blow[0] = u32x4{low[0], low[1], low[2], low[3]};
                blow[1] = u32x4{low[4], low[5], low[6], low[7]};
                bhigh[0] = u32x4{high[0], high[1], high[2], high[3]};
                bhigh[1] = u32x4{high[4], high[5], high[6], high[7]};
                if (g == 0 && sh == 0) {
                    // the eight minimums of the super-block, as halves
                    const uint32_t lo4 = hdr.z & 0x3f3f3f3fu;                                         // m0..m3
                    const uint32_t hi4 = ((hdr.w >> 4) & 0x0f0f0f0fu) | ((hdr.z >> 2) & 0x30303030u);  // m4..m7
                    const half2_t m01 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, lo4, 0x0c010c00u) | 0x64006400u) - offset;
                    const half2_t m23 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, lo4, 0x0c030c02u) | 0x64006400u) - offset;
                    const half2_t m45 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, hi4, 0x0c010c00u) | 0x64006400u) - offset;
                    const half2_t m67 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, hi4, 0x0c030c02u) | 0x64006400u) - offset;
                    *reinterpret_cast<u32x4 *>(mns[sbuf][srow]) = u32x4{__builtin_bit_cast(uint32_t, m01), __builtin_bit_cast(uint32_t, m23),
                                                                        __builtin_bit_cast(uint32_t, m45), __builtin_bit_cast(uint32_t, m67)};
                    dds[sbuf][srow] = hdr.x;
                }
                u32x4 *adst = reinterpret_cast<u32x4 *>(&As[buf][srow][32u * sh]);
#pragma unroll
                for (int i = 0; i < 4; i++) adst[i] = av[g][i];
                // the slot is free: the same group of the next super-block goes out.  Past the end the last super-block is
                // fetched again and dropped: with the same loads in every round the waits count exactly how many are newer
                {
                    const uint8_t *block = wrow + (size_t)next * BLOCK;
                    qs[g] = *(global_uint4)(uintptr_t)(block + NIBBLES + 32u * g + 16u * sh);
                    const _Float16 *at = arow + (size_t)(4u * next + g) * 64u;
#pragma unroll
                    for (int i = 0; i < 4; i++) av[g][i] = *(global_uint4)(uintptr_t)(at + 8 * i);
                }
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();  // step is staged; the multipliers are done with the step before it
            }
        }
        return;
    }

    gemm_multiply<true>(p, As, Bs, mns, dds, wave, lane, n0, m0, steps, 16384.0f);  // the weights were staged * 2^-14
}

__global__ __launch_bounds__(512) void gemm_q4k_mfma_kernel(GemmQ4Params p) {
    fetch_parameters(p);
    gemm_q45k_mfma<false>(p);
}
__global__ __launch_bounds__(512) void gemm_q5k_mfma_kernel(GemmQ4Params p) {
    fetch_parameters(p);
    gemm_q45k_mfma<true>(p);
}

// ------------------------------------------------------------------- Q4_K, weights through registers --------
//
// LDS is what bounds the kernel above (it takes a workgroup's writes at 64 B a clock and serves its reads at 128: a step moves
// 32 KB in and 64 KB out, twice the time its MFMAs take).  Here the weights never touch it: eight multiplier waves own
// 64 x 32 of the 128 x 128 tile each, and lane (l32, part) of one loads, unpacks and feeds the matrix cores the weights of ITS
// row 32 wn + l32 -- per 64-k step one 16-byte load (bytes 16 part .. of the step's 32: the low nibbles are k = 16 part .. + 15,
// the high nibbles k = 32 + 16 part ..), whose four 8-weight pieces are the B operands of the step's four MFMA depths; the
// activation operand of depth kk is read from the matching 16-byte chunk of the staged row (chunk (kk >> 1) * 4 + 2 part +
// (kk & 1)), so the k order inside a step is the weights', not the natural one, and nothing has to move.  The header of a
// lane's row is in its registers, so d, dmin and the minimums need no LDS either.  Two multipliers share a SIMD (one unpacks
// while the other's MFMAs run) beside one of the four stagers, which only copy packed activation rows: whole 128-byte
// lines, eight lanes a row.  A stage of LDS is a whole super-block of k (256 columns of the 128 rows, 66 KB; two stages), so
// the twelve waves meet at one barrier a super-block, not one a step.
constexpr int GSB = 256 + 8;  // LDS row stride of a stage in halves: 528 B keeps 128-bit reads of 8 neighbouring rows on distinct banks
constexpr size_t GEMM_Q4K_REGB_LDS = sizeof(_Float16) * 2 * GT * GSB;

__global__ __launch_bounds__(768) void gemm_q4k_regb_mfma_kernel(GemmQ4Params p) {
    fetch_parameters(p);
    extern __shared__ __attribute__((aligned(16))) uint8_t gemm_lds[];
    _Float16(*As)[GT][GSB] = reinterpret_cast<_Float16(*)[GT][GSB]>(gemm_lds);  // [2]
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t n0 = blockIdx.x * GT, m0 = blockIdx.y * GT;
    const uint32_t steps = p.K / 64u;  // a multiple of 4: K is whole super-blocks
    const uint32_t nsb = steps >> 2;
    typedef const __attribute__((address_space(1))) u32x4 *global_uint4;

    if (wave >= 8) {
        // ------------------------------------------------------------------ stagers: rows abase + 32 j, 16-byte chunks achunk + 8 c
        const uint32_t tid = threadIdx.x - 512u;
        const uint32_t abase = tid >> 3, achunk = tid & 7u;
        const _Float16 *asrc[4];
#pragma unroll
        for (int j = 0; j < 4; j++) asrc[j] = p.A + (size_t)min(m0 + abase + 32u * j, p.rows - 1u) * p.K + 8u * achunk;
        u32x4 av[4][4];  // the super-block on its way: [64-k step][row]
        auto fetch = [&](uint32_t sb) {
            const size_t at = (size_t)min(sb, nsb - 1u) * 256u;  // past the end the last super-block again, dropped
#pragma unroll
            for (int c = 0; c < 4; c++)
#pragma unroll
                for (int j = 0; j < 4; j++) av[c][j] = *(global_uint4)(uintptr_t)(asrc[j] + at + 64u * c);
        };
        fetch(0);
        for (uint32_t sb = 0; sb < nsb; sb++) {
            const uint32_t buf = sb & 1u;
#pragma unroll
            for (int c = 0; c < 4; c++)
#pragma unroll
                for (int j = 0; j < 4; j++) *reinterpret_cast<u32x4 *>(&As[buf][abase + 32u * j][64u * c + 8u * achunk]) = av[c][j];
            fetch(sb + 1u);
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();  // the super-block is staged; the multipliers are done with the one before it
        }
        return;
    }

    // ---------------------------------------------------------------------- multipliers
    const uint32_t wm = wave >> 2, wn = wave & 3u, l32 = lane & 31u, part = lane >> 5;
    // a tile lies in one matrix: the boundaries between stacked matrices are multiples of the tile
    const uint32_t column = min(n0 + 32u * wn + l32, p.N - 1u);
    const uint8_t *wrow = column < p.end0   ? p.W + (size_t)column * p.row_bytes
                          : column < p.end1 ? p.W1 + (size_t)(column - p.end0) * p.row_bytes
                                            : p.W2 + (size_t)(column - p.end1) * p.row_bytes;
    const _Float16 *sums[2];
#pragma unroll
    for (int i = 0; i < 2; i++) sums[i] = p.S + (size_t)min(m0 + 64u * wm + 32u * i + l32, p.rows - 1u) * nsb * 16u + 8u * part;
    const half2_t offset = {(_Float16)1024.0f, (_Float16)1024.0f}, powers = {(_Float16)1024.0f, (_Float16)64.0f};

    f32x16 acc[2], tmp[2], zero;
#pragma unroll
    for (int e = 0; e < 16; e++) zero[e] = 0.0f;
    acc[0] = acc[1] = tmp[0] = tmp[1] = zero;

    // the lane's weights: a super-block's header and its four 16-byte runs, one super-block ahead
    u32x4 ahead, qs[4];
    ahead = *(global_uint4)(uintptr_t)wrow;
#pragma unroll
    for (int g = 0; g < 4; g++) qs[g] = *(global_uint4)(uintptr_t)(wrow + 16u + 32u * g + 16u * part);
    for (uint32_t first = 0; first < steps; first += 4) {
        const u32x4 hdr = ahead;
        const uint32_t next = min((first >> 2) + 1u, nsb - 1u);  // past the end the last super-block again, dropped
        ahead = *(global_uint4)(uintptr_t)(wrow + (size_t)next * 144u);
        u32x4 sraw[2];
#pragma unroll
        for (int i = 0; i < 2; i++) sraw[i] = *(global_uint4)(uintptr_t)(sums[i] + (size_t)(first >> 2) * 16u);  // wanted at the end of the super-block
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const uint32_t sbuf = (first >> 2) & 1u;
            // 6-bit fields of sub-blocks 2g, 2g+1 (crates/neura-precision/src/ggml.rs:127-136); 0x6400 | v is the half 1024 + v
            const uint32_t shift = 16u * (g & 1u);
            const uint32_t ya = (hdr.y >> shift) & 0xffffu, wa = (hdr.w >> shift) & 0xffffu;
            const uint32_t sc = g < 2 ? (ya & 0x3f3fu) : ((wa & 0x0f0fu) | ((ya >> 2) & 0x3030u));
            const uint32_t both = __builtin_amdgcn_perm(0u, sc, 0x0c010c00u) | 0x64006400u;  // (1024 + sc0, 1024 + sc1)
            const half2_t scales = (__builtin_bit_cast(half2_t, both) - offset) * powers;     // (sc0 * 2^10, sc1 * 2^6)
            const half2_t low_scale = {scales.x, scales.x}, high_scale = {scales.y, scales.y};
            const uint32_t words[4] = {qs[g].x, qs[g].y, qs[g].z, qs[g].w};
            // the slot is free once its words are copied out: the same run of the next super-block goes out
            qs[g] = *(global_uint4)(uintptr_t)(wrow + (size_t)next * 144u + 16u + 32u * g + 16u * part);
            if (g == 0) __syncthreads();  // the super-block's activations are staged
            const _Float16 *arow0 = &As[sbuf][64u * wm + l32][64u * g], *arow1 = &As[sbuf][64u * wm + 32u + l32][64u * g];
#pragma unroll
            for (int kk = 0; kk < 4; kk++) {
                // depth kk: words 2 (kk & 1), + 1 of the run, low nibbles for kk < 2; element order inside a word: 0, 2 then 1, 3
                // (the byte lanes), the order the activations were packed in
                uint32_t b[4];
#pragma unroll
                for (int w = 0; w < 2; w++) {
                    const uint32_t even = words[2 * (kk & 1) + w], odd = even >> 8;
                    if (kk < 2) {
                        b[2 * w] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, even & 0x000f000fu) * low_scale);
                        b[2 * w + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, odd & 0x000f000fu) * low_scale);
                    } else {
                        b[2 * w] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, even & 0x00f000f0u) * high_scale);
                        b[2 * w + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, odd & 0x00f000f0u) * high_scale);
                    }
                }
                const half8_t weights = __builtin_bit_cast(half8_t, u32x4{b[0], b[1], b[2], b[3]});
                const uint32_t chunk = 8u * ((kk >> 1) * 4u + 2u * part + (kk & 1));  // where those eight k lie in the staged row
                const half8_t a0 = *reinterpret_cast<const half8_t *>(arow0 + chunk), a1 = *reinterpret_cast<const half8_t *>(arow1 + chunk);
                tmp[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a0, weights, (g == 0 && kk == 0) ? zero : tmp[0], 0, 0, 0);
                tmp[1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a1, weights, (g == 0 && kk == 0) ? zero : tmp[1], 0, 0, 0);
            }
        }
        // ---- the super-block is complete: weigh by d, then take the minimums off (the eight minimums as halves, k 8..15 * 2^-11
        // against the sums' residues * 2^11)
        const half2_t dd = __builtin_bit_cast(half2_t, hdr.x);
        const float dscale = (float)dd.x * 16384.0f;  // the weights were unpacked * 2^-14
        const float mscale = (float)dd.y * -64.0f;    // the sums were packed / 64
        const uint32_t lo4 = hdr.z & 0x3f3f3f3fu;                                         // m0..m3
        const uint32_t hi4 = ((hdr.w >> 4) & 0x0f0f0f0fu) | ((hdr.z >> 2) & 0x30303030u);  // m4..m7
        half2_t m01 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, lo4, 0x0c010c00u) | 0x64006400u) - offset;
        half2_t m23 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, lo4, 0x0c030c02u) | 0x64006400u) - offset;
        half2_t m45 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, hi4, 0x0c010c00u) | 0x64006400u) - offset;
        half2_t m67 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, hi4, 0x0c030c02u) | 0x64006400u) - offset;
        if (part) {
            const half2_t down = {(_Float16)0.00048828125f, (_Float16)0.00048828125f};
            m01 = m01 * down, m23 = m23 * down, m45 = m45 * down, m67 = m67 * down;
        }
        const half8_t b2 = __builtin_bit_cast(half8_t, u32x4{__builtin_bit_cast(uint32_t, m01), __builtin_bit_cast(uint32_t, m23),
                                                             __builtin_bit_cast(uint32_t, m45), __builtin_bit_cast(uint32_t, m67)});
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const f32x16 mins = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, sraw[i]), b2, zero, 0, 0, 0);
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][e] = fmaf(dscale, tmp[i][e], acc[i][e]);
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][e] = fmaf(mscale, mins[e], acc[i][e]);
        }
    }
    // ---- out: lane (l32, part) holds column n = l32 of a 32 x 32 block; register 4q + e is row 8q + 4 part + e
    const uint32_t n = n0 + 32u * wn + l32;
    if (n >= p.N) return;
#pragma unroll
    for (int i = 0; i < 2; i++) {
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t row = m0 + 64u * wm + 32u * i + 8u * q + 4u * part;  // first of four rows of A'
            if (p.split) {
#pragma unroll
                for (int e = 0; e < 2; e++) {
                    const uint32_t m = (row >> 1) + e;
                    if (m >= p.M) continue;
                    float value = fmaf(acc[i][4 * q + 2 * e + 1], 0.00048828125f, acc[i][4 * q + 2 * e]) * p.unscale[m];
                    const size_t at = (size_t)m * p.ldy + n;
                    p.Y[at] = p.residual ? p.residual[at] + value : value;
                }
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const uint32_t m = row + e;
                    if (m >= p.M) continue;
                    const size_t at = (size_t)m * p.ldy + n;
                    p.Y[at] = p.residual ? p.residual[at] + acc[i][4 * q + e] : acc[i][4 * q + e];
                }
            }
        }
    }
}

// ------------------------------------------------------------------- Q8_0 on MFMA --------
//
// The same tiles, the same packed activation rows and the same division of the waves.  A step of 64 k is two blocks: a
// stager owns one row and one block of the step, reads the nine words that cover its 34 bytes from the 4-byte boundary
// below it (a block starts on a half word as often as not; crates/neura-kernel/src/dot.rs:197-264 reads it the same way),
// and unpacks the 32 codes into LDS as the halves they are -- a signed byte b is the low byte of the half 1024 + 128 + b
// once its top bit is flipped, so one byte shuffle, one xor and one packed subtraction make two exact halves.  The block's
// scale cannot ride in the operand (a half times a byte is no half), so the multipliers close a sum after every block:
// two MFMAs of depth 16 into a fresh accumulator, then acc += d * sum in fp32 (run_weight_q8_0,
// crates/neura-kernel/src/task/matmul.rs:309-318, weighs a block the same way).  The weighing of one block runs on the
// vector unit while the matrix cores walk the next: the second block of a step is weighed behind the first MFMAs of the
// step after it.  K is a multiple of 64; steps are walked four at a time, the ones past the end as zero codes and zero
// scales, so every round issues the same loads and the waits count them exactly.
typedef uint32_t u32x4_loose __attribute__((ext_vector_type(4), aligned(4)));
constexpr size_t GEMM_Q8_LDS = sizeof(_Float16) * (4 * GT * GS) + sizeof(float) * 2 * 2 * GT;

__global__ __launch_bounds__(512) void gemm_q8_0_mfma_kernel(GemmQ4Params p) {
    fetch_parameters(p);
    extern __shared__ __attribute__((aligned(16))) uint8_t gemm_lds[];
    _Float16(*As)[GT][GS] = reinterpret_cast<_Float16(*)[GT][GS]>(gemm_lds);                                   // [2]
    _Float16(*Bs)[GT][GS] = reinterpret_cast<_Float16(*)[GT][GS]>(gemm_lds + sizeof(_Float16) * 2 * GT * GS);  // [2]
    float(*dds)[2][GT] = reinterpret_cast<float(*)[2][GT]>(gemm_lds + sizeof(_Float16) * 4 * GT * GS);         // [2][block of the step]: d of every weight row
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t n0 = blockIdx.x * GT, m0 = blockIdx.y * GT;
    const uint32_t steps = p.K / 64u, walked = (steps + 3u) & ~3u;
    typedef const __attribute__((address_space(1))) u32x4 *global_uint4;
    typedef const __attribute__((address_space(1))) u32x4_loose *global_loose4;

    if (wave >= 4) {
        // ------------------------------------------------------------------ stagers
        const uint32_t tid = threadIdx.x - 256u;
        const uint32_t srow = tid >> 1, sh = tid & 1u;
        const uint32_t column = min(n0 + srow, p.N - 1u);
        const uint8_t *wrow = column < p.end0   ? p.W + (size_t)column * p.row_bytes
                              : column < p.end1 ? p.W1 + (size_t)(column - p.end0) * p.row_bytes
                                                : p.W2 + (size_t)(column - p.end1) * p.row_bytes;
        const _Float16 *arow = p.A + (size_t)min(m0 + srow, p.rows - 1u) * p.K + 32u * sh;
        u32x4 qa[4], qb[4], av[4][4];  // by slot = step % 4
        uint32_t qc[4];
        auto fetch = [&](int g, uint32_t step) {
            const uint32_t s = min(step, steps - 1u);  // past the end the last step is fetched again and dropped
            const uintptr_t at = (uintptr_t)(wrow + (size_t)(2u * s + sh) * 34u), low = at & ~(uintptr_t)3;
            qa[g] = *(global_loose4)low;
            qb[g] = *(global_loose4)(low + 16u);
            // a block on a word boundary ends two bytes into the ninth word: those two only are read (the last block of a
            // tensor ends where its allocation may)
            if (at & 2u) qc[g] = *(const __attribute__((address_space(1))) uint32_t *)(low + 32u);
            else qc[g] = *(const __attribute__((address_space(1))) uint16_t *)(low + 32u);
#pragma unroll
            for (int i = 0; i < 4; i++) av[g][i] = *(global_uint4)(uintptr_t)(arow + (size_t)s * 64u + 8 * i);
        };
#pragma unroll
        for (int g = 0; g < 4; g++) {
            fetch(g, (uint32_t)g);
            __builtin_amdgcn_sched_barrier(0);  // slot 0 goes out first: the loop waits for the oldest slot only
        }
        const half2_t offset = {(_Float16)1152.0f, (_Float16)1152.0f};
        for (uint32_t first = 0; first < walked; first += 4) {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const uint32_t buf = g & 1u, step = first + g;
                const bool odd = ((uintptr_t)(wrow + (size_t)(2u * min(step, steps - 1u) + sh) * 34u) & 2u) != 0;
                const uint32_t live = step < steps ? 0xffffffffu : 0u;
                const uint32_t words[9] = {qa[g].x, qa[g].y, qa[g].z, qa[g].w, qb[g].x, qb[g].y, qb[g].z, qb[g].w, qc[g]};
                const uint32_t scale_bits = (odd ? words[0] >> 16 : words[0] & 0xffffu) & live;
                uint32_t out[16];
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const uint32_t codes = (odd ? words[j + 1] : __funnelshift_r(words[j], words[j + 1], 16)) & live;
                    // element order inside a word: 0, 2 then 1, 3, the order the activations were packed in
                    const uint32_t even = __builtin_amdgcn_perm(0u, codes, 0x0c020c00u) ^ 0x64806480u;
                    const uint32_t uneven = __builtin_amdgcn_perm(0u, codes, 0x0c030c01u) ^ 0x64806480u;
                    out[2 * j] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, even) - offset);
                    out[2 * j + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, uneven) - offset);
                }
                u32x4 *bdst = reinterpret_cast<u32x4 *>(&Bs[buf][srow][32u * sh]);
#pragma unroll
                for (int i = 0; i < 4; i++) bdst[i] = u32x4{out[4 * i], out[4 * i + 1], out[4 * i + 2], out[4 * i + 3]};
                dds[buf][sh][srow] = (float)__builtin_bit_cast(_Float16, (uint16_t)scale_bits);
                u32x4 *adst = reinterpret_cast<u32x4 *>(&As[buf][srow][32u * sh]);
#pragma unroll
                for (int i = 0; i < 4; i++) adst[i] = av[g][i];
                fetch(g, step + 4u);  // the slot is free: the same slot of the next round goes out
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();  // step is staged; the multipliers are done with the step before it
            }
        }
        return;
    }

    // ---------------------------------------------------------------------- multipliers
    const uint32_t wm = wave >> 1, wn = wave & 1u, l32 = lane & 31u, part = lane >> 5;
    f32x16 acc[2][2], tmp[2][2][2], zero;
#pragma unroll
    for (int e = 0; e < 16; e++) zero[e] = 0.0f;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = zero, tmp[0][i][j] = zero, tmp[1][i][j] = zero;
    float late[2] = {0.0f, 0.0f};  // the scales of the block whose sums wait in tmp[1]

    auto weigh = [&](int h, const float *scales) {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int e = 0; e < 16; e++) acc[i][j][e] = fmaf(scales[j], tmp[h][i][j][e], acc[i][j][e]);
    };

    for (uint32_t step = 0; step < walked; step++) {
        const uint32_t buf = step & 1u;
        __syncthreads();  // the step is staged
        float early[2], next[2];
#pragma unroll
        for (int j = 0; j < 2; j++) early[j] = dds[buf][0][64u * wn + 32u * j + l32], next[j] = dds[buf][1][64u * wn + 32u * j + l32];
        half8_t a[2][2], b[2][2];
        auto operands = [&](int kk) {
#pragma unroll
            for (int i = 0; i < 2; i++) a[kk & 1][i] = *reinterpret_cast<const half8_t *>(&As[buf][64u * wm + 32u * i + l32][16u * kk + 8u * part]);
#pragma unroll
            for (int j = 0; j < 2; j++) b[kk & 1][j] = *reinterpret_cast<const half8_t *>(&Bs[buf][64u * wn + 32u * j + l32][16u * kk + 8u * part]);
        };
        operands(0);
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            if (kk < 3) operands(kk + 1);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
                    tmp[kk >> 1][i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[kk & 1][i], b[kk & 1][j], (kk & 1) ? tmp[kk >> 1][i][j] : zero, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            // the sums the matrix cores are not writing are weighed meanwhile: the block before this step's first behind
            // its first MFMAs, this step's first behind the MFMAs of its second
            if (kk == 0) weigh(1, late);
            if (kk == 2) weigh(0, early);
            if (kk == 0 || kk == 2) __builtin_amdgcn_sched_barrier(0);
        }
        late[0] = next[0], late[1] = next[1];
    }
    weigh(1, late);
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

// ------------------------------------------------------------------- Q6_K on MFMA --------
//
// A Q6_K weight is d * sc * (q - 32) with q of six bits and sc a signed byte a 16 weights (crates/neura-precision/src/ggml.rs,
// the Q6_K reader): sc * (q - 32) reaches +-4064, past the integers a half holds exactly.  The byte splits as
// sc = 16 * (sc >> 4) + (sc & 15), and (q - 32) * (sc & 15) (below 512) and 16 * (q - 32) * (sc >> 4) (a nine-bit integer times
// 16) are both exact halves: the weights enter as two operand planes and the matrix cores add the two products in fp32, so
// tmp holds exactly sum a * sc * (q - 32) however the scales fall.  A step is 32 k: its 64 operand columns are plane one
// then plane two of those 32 weights, against the step's 32 activations written twice; four steps (half a super-block)
// are weighed by d together.  The same tiles, packed activation rows, division of the waves and multipliers as the Q4_K
// kernel; there are no minimums.  Blocks are 210 bytes and start on any half word: a stager reads each 16-byte run it
// needs as the four aligned words below it and the half word above, and shifts the five into place.
struct Q6Raw {
    u32x4 ql[4], qh[2], sc;          // this thread's runs of the low nibbles, of the high bit pairs, and the 16 scales
    uint32_t qle[4], qhe[2], sce, d;  // the half word above each run; d
};

__global__ __launch_bounds__(512) void gemm_q6k_mfma_kernel(GemmQ4Params p) {
    fetch_parameters(p);
    extern __shared__ __attribute__((aligned(16))) uint8_t gemm_lds[];
    _Float16(*As)[GT][GS] = reinterpret_cast<_Float16(*)[GT][GS]>(gemm_lds);
    _Float16(*Bs)[GT][GS] = reinterpret_cast<_Float16(*)[GT][GS]>(gemm_lds + sizeof(_Float16) * 2 * GT * GS);
    _Float16(*mns)[GT][8] = reinterpret_cast<_Float16(*)[GT][8]>(gemm_lds + sizeof(_Float16) * 4 * GT * GS);  // unused: no minimums
    uint32_t(*dds)[GT] = reinterpret_cast<uint32_t(*)[GT]>(gemm_lds + sizeof(_Float16) * (4 * GT * GS + 2 * GT * 8));
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t n0 = blockIdx.x * GT, m0 = blockIdx.y * GT;
    const uint32_t steps = p.K / 32u;  // a multiple of 8: K is whole super-blocks
    typedef const __attribute__((address_space(1))) u32x4 *global_uint4;
    typedef const __attribute__((address_space(1))) uint16_t *global_half_word;

    if (wave >= 4) {
        // ------------------------------------------------------------------ stagers
        // one row of each tile, one half (16 k: one scale) of the step
        const uint32_t tid = threadIdx.x - 256u;
        const uint32_t srow = tid >> 1, sh = tid & 1u;
        const uint32_t column = min(n0 + srow, p.N - 1u);
        const uint8_t *wrow = column < p.end0   ? p.W + (size_t)column * p.row_bytes
                              : column < p.end1 ? p.W1 + (size_t)(column - p.end0) * p.row_bytes
                                                : p.W2 + (size_t)(column - p.end1) * p.row_bytes;
        const _Float16 *arow = p.A + (size_t)min(m0 + srow, p.rows - 1u) * p.K + 16u * sh;
        const uint32_t nsb = steps >> 3;
        // 16 bytes from `at` (any half word) as the aligned 16 below and the half word at + 14
        auto run = [&](const uint8_t *at, u32x4 &low, uint32_t &above) {
            low = *(global_uint4)((uintptr_t)at & ~(uintptr_t)3);
            above = *(global_half_word)(uintptr_t)(at + 14u);
        };
        auto fetch = [&](Q6Raw &raw, uint32_t sb) {
            const uint8_t *block = wrow + (size_t)min(sb, nsb - 1u) * 210u;  // past the end the last super-block again, dropped
#pragma unroll
            for (int r = 0; r < 4; r++) run(block + 64u * (r >> 1) + 32u * (r & 1) + 16u * sh, raw.ql[r], raw.qle[r]);
#pragma unroll
            for (int n = 0; n < 2; n++) run(block + 128u + 32u * n + 16u * sh, raw.qh[n], raw.qhe[n]);
            run(block + 192u, raw.sc, raw.sce);
            raw.d = *(global_half_word)(uintptr_t)(block + 208u);
        };
        // the run as it lies: nothing to do on a word boundary, else every word takes its upper half from the next
        auto placed = [](const u32x4 &low, uint32_t above, uint32_t shift) -> u32x4 {
            return u32x4{__builtin_amdgcn_alignbit(low.y, low.x, shift), __builtin_amdgcn_alignbit(low.z, low.y, shift),
                         __builtin_amdgcn_alignbit(low.w, low.z, shift), __builtin_amdgcn_alignbit(above, low.w, shift)};
        };
        u32x4 av[4][2];  // activations by slot = step % 4
        auto fetch_activations = [&](int slot, uint32_t step) {
            const _Float16 *at = arow + (size_t)min(step, steps - 1u) * 32u;
#pragma unroll
            for (int i = 0; i < 2; i++) av[slot][i] = *(global_uint4)(uintptr_t)(at + 8 * i);
        };
        const half2_t bias = {(_Float16)1056.0f, (_Float16)1056.0f};  // 0x6400 | q is the half 1024 + q; the weight is q - 32
        Q6Raw raws[2];
        fetch(raws[0], 0);
        __builtin_amdgcn_sched_barrier(0);  // the first super-block goes out first: the loop waits for the oldest loads only
#pragma unroll
        for (int slot = 0; slot < 4; slot++) fetch_activations(slot, slot);
        fetch(raws[1], 1);
        __builtin_amdgcn_sched_barrier(0);
        auto super_block = [&](Q6Raw &raw, const uint32_t sb) {
            const uint32_t shift = (uint32_t)((uintptr_t)(wrow + (size_t)sb * 210u) & 2u) * 8u;  // 0 or 16: where the block starts in its word
            const u32x4 scales = placed(raw.sc, raw.sce, shift);
            const uint32_t scale_words[4] = {scales.x, scales.y, scales.z, scales.w};
            u32x4 high_pairs = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int s = 0; s < 8; s++) {
                const uint32_t buf = s & 1u, sbuf = (s >> 2) & 1u;  // steps are whole super-blocks: step 8 sb + s has parity s & 1
                const int n = s >> 2, quarter = s & 3;
                if (quarter == 0) high_pairs = placed(raw.qh[n], raw.qhe[n], shift);
                // group 2 s + sh of the super-block: scale byte 2 (s & 1) + sh of word s / 2
                const int sc = __builtin_amdgcn_sbfe((int)scale_words[s >> 1], 16u * (s & 1) + 8u * sh, 8u);
                const _Float16 fine = (_Float16)(float)(sc & 15), coarse = (_Float16)(float)(16 * (sc >> 4));
                const half2_t fine2 = {fine, fine}, coarse2 = {coarse, coarse};
                const u32x4 nibbles = placed(raw.ql[2 * n + (quarter & 1)], raw.qle[2 * n + (quarter & 1)], shift);
                const uint32_t nibble_words[4] = {nibbles.x, nibbles.y, nibbles.z, nibbles.w};
                const uint32_t pair_words[4] = {high_pairs.x, high_pairs.y, high_pairs.z, high_pairs.w};
                uint32_t one[8], two[8];
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    const uint32_t low4 = (quarter >= 2 ? nibble_words[w] >> 4 : nibble_words[w]) & 0x0f0f0f0fu;
                    const uint32_t q4 = low4 | (((pair_words[w] >> (2 * quarter)) & 0x03030303u) << 4);  // four weights' six bits, one a byte
                    // element order inside a word: 0, 2 then 1, 3, as the activations were packed
                    const half2_t even = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, q4, 0x0c020c00u) | 0x64006400u) - bias;
                    const half2_t odd = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, q4, 0x0c030c01u) | 0x64006400u) - bias;
                    one[2 * w] = __builtin_bit_cast(uint32_t, even * fine2), one[2 * w + 1] = __builtin_bit_cast(uint32_t, odd * fine2);
                    two[2 * w] = __builtin_bit_cast(uint32_t, even * coarse2), two[2 * w + 1] = __builtin_bit_cast(uint32_t, odd * coarse2);
                }
                u32x4 *first = reinterpret_cast<u32x4 *>(&Bs[buf][srow][16u * sh]), *second = reinterpret_cast<u32x4 *>(&Bs[buf][srow][32u + 16u * sh]);
                first[0] = u32x4{one[0], one[1], one[2], one[3]};
                first[1] = u32x4{one[4], one[5], one[6], one[7]};
                second[0] = u32x4{two[0], two[1], two[2], two[3]};
                second[1] = u32x4{two[4], two[5], two[6], two[7]};
                if (quarter == 0 && sh == 0) dds[sbuf][srow] = raw.d;  // (d, no dmin) of these four steps
                u32x4 *once = reinterpret_cast<u32x4 *>(&As[buf][srow][16u * sh]), *again = reinterpret_cast<u32x4 *>(&As[buf][srow][32u + 16u * sh]);
#pragma unroll
                for (int i = 0; i < 2; i++) once[i] = av[s & 3][i], again[i] = av[s & 3][i];
                fetch_activations(s & 3, 8u * sb + (uint32_t)s + 4u);
                if (s == 7) fetch(raw, sb + 2u);  // these registers are free: the super-block after the next
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();  // step is staged; the multipliers are done with the step before it
            }
        };
        uint32_t sb = 0;
        for (; sb + 2u <= nsb; sb += 2u) {
            super_block(raws[0], sb);
            super_block(raws[1], sb + 1u);
        }
        if (sb < nsb) super_block(raws[0], sb);
        return;
    }
    gemm_multiply<false>(p, As, Bs, mns, dds, wave, lane, n0, m0, steps, 1.0f);
}

// ------------------------------------------------------------------- Q3_K on MFMA --------
//
// A Q3_K weight is d * (sc - 32) * c with c in -4..3 (two bits less 4 unless the third bit is set) and sc of six bits a 16
// weights (crates/neura-precision/src/ggml.rs:224-229, 291-306): (sc - 32) * c stays within +-128 and is an exact half, so the
// weights are one operand plane, a step is 64 k as in the Q4_K kernel (a stager's 32 weights are two scale groups), a
// super-block's four steps are weighed by d together, and there are no minimums.  Blocks are 110 bytes and start on any
// half word; they are read as the Q6_K kernel reads its own.
struct Q3Raw {
    u32x4 hm[2], qs[4], sc;           // the third bits of the 32 columns, the bit pairs of both halves, bytes 94..109 (scales, d)
    uint32_t hme[2], qse[4], sce;     // the half word above each run
};

__global__ __launch_bounds__(512) void gemm_q3k_mfma_kernel(GemmQ4Params p) {
    fetch_parameters(p);
    extern __shared__ __attribute__((aligned(16))) uint8_t gemm_lds[];
    _Float16(*As)[GT][GS] = reinterpret_cast<_Float16(*)[GT][GS]>(gemm_lds);
    _Float16(*Bs)[GT][GS] = reinterpret_cast<_Float16(*)[GT][GS]>(gemm_lds + sizeof(_Float16) * 2 * GT * GS);
    _Float16(*mns)[GT][8] = reinterpret_cast<_Float16(*)[GT][8]>(gemm_lds + sizeof(_Float16) * 4 * GT * GS);  // unused: no minimums
    uint32_t(*dds)[GT] = reinterpret_cast<uint32_t(*)[GT]>(gemm_lds + sizeof(_Float16) * (4 * GT * GS + 2 * GT * 8));
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t n0 = blockIdx.x * GT, m0 = blockIdx.y * GT;
    const uint32_t steps = p.K / 64u;  // a multiple of 4: K is whole super-blocks
    typedef const __attribute__((address_space(1))) u32x4 *global_uint4;
    typedef const __attribute__((address_space(1))) uint16_t *global_half_word;

    if (wave >= 4) {
        // ------------------------------------------------------------------ stagers
        // one row of each tile, one half (32 k: two scales) of the step
        const uint32_t tid = threadIdx.x - 256u;
        const uint32_t srow = tid >> 1, sh = tid & 1u;
        const uint32_t column = min(n0 + srow, p.N - 1u);
        const uint8_t *wrow = column < p.end0   ? p.W + (size_t)column * p.row_bytes
                              : column < p.end1 ? p.W1 + (size_t)(column - p.end0) * p.row_bytes
                                                : p.W2 + (size_t)(column - p.end1) * p.row_bytes;
        const _Float16 *arow = p.A + (size_t)min(m0 + srow, p.rows - 1u) * p.K + 32u * sh;
        const uint32_t nsb = steps >> 2;
        auto run = [&](const uint8_t *at, u32x4 &low, uint32_t &above) {
            low = *(global_uint4)((uintptr_t)at & ~(uintptr_t)3);
            above = *(global_half_word)(uintptr_t)(at + 14u);
        };
        auto fetch = [&](Q3Raw &raw, uint32_t sb) {
            const uint8_t *block = wrow + (size_t)min(sb, nsb - 1u) * 110u;  // past the end the last super-block again, dropped
#pragma unroll
            for (int r = 0; r < 2; r++) run(block + 16u * r, raw.hm[r], raw.hme[r]);
#pragma unroll
            for (int r = 0; r < 4; r++) run(block + 32u + 16u * r, raw.qs[r], raw.qse[r]);
            run(block + 94u, raw.sc, raw.sce);
        };
        auto placed = [](const u32x4 &low, uint32_t above, uint32_t shift) -> u32x4 {
            return u32x4{__builtin_amdgcn_alignbit(low.y, low.x, shift), __builtin_amdgcn_alignbit(low.z, low.y, shift),
                         __builtin_amdgcn_alignbit(low.w, low.z, shift), __builtin_amdgcn_alignbit(above, low.w, shift)};
        };
        u32x4 av[4][4];  // activations by slot = step % 4
        auto fetch_activations = [&](int slot, uint32_t step) {
            const _Float16 *at = arow + (size_t)min(step, steps - 1u) * 64u;
#pragma unroll
            for (int i = 0; i < 4; i++) av[slot][i] = *(global_uint4)(uintptr_t)(at + 8 * i);
        };
        const half2_t scale_bias = {(_Float16)1056.0f, (_Float16)1056.0f};  // 0x6400 | v is the half 1024 + v; a scale is stored 32 too large
        const half2_t code_bias = {(_Float16)1028.0f, (_Float16)1028.0f};   // and a code 4 too large
        Q3Raw raws[2];
        fetch(raws[0], 0);
        __builtin_amdgcn_sched_barrier(0);  // the first super-block goes out first: the loop waits for the oldest loads only
#pragma unroll
        for (int slot = 0; slot < 4; slot++) fetch_activations(slot, slot);
        fetch(raws[1], 1);
        __builtin_amdgcn_sched_barrier(0);
        auto super_block = [&](Q3Raw &raw, const uint32_t sb) {
            const uint32_t shift = (uint32_t)((uintptr_t)(wrow + (size_t)sb * 110u) & 2u) * 8u;  // 0 or 16: where the block starts in its word
            const u32x4 tail = placed(raw.sc, raw.sce, shift ^ 16u);  // bytes 94..109: this run starts on the other half of a word
            // bytes 96..107: the scales' nibbles (two words) and their top bit pairs (one)
            const uint32_t nibble_words[2] = {__builtin_amdgcn_alignbit(tail.y, tail.x, 16u), __builtin_amdgcn_alignbit(tail.z, tail.y, 16u)};
            const uint32_t tops = __builtin_amdgcn_alignbit(tail.w, tail.z, 16u);
            const u32x4 third0 = placed(raw.hm[0], raw.hme[0], shift), third1 = placed(raw.hm[1], raw.hme[1], shift);
            const uint32_t third_words[8] = {third0.x, third0.y, third0.z, third0.w, third1.x, third1.y, third1.z, third1.w};
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const uint32_t buf = g & 1u, sbuf = sb & 1u;
                const int n = g >> 1;
                // scales 4 g + 2 sh and the one after: nibble 2 sh + t of word g & 1 (low nibbles for the first eight scales), top
                // bits from byte 2 sh + t of the third word at 2 g
                const uint32_t two = (nibble_words[g & 1] >> (16u * sh)) & 0xffffu, top = (tops >> (16u * sh)) & 0xffffu;
                const uint32_t pair = ((g < 2 ? two : two >> 4) & 0x0f0fu) | (((top >> (2 * g)) & 0x0303u) << 4);
                const half2_t scales = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, pair, 0x0c010c00u) | 0x64006400u) - scale_bias;
                const half2_t first_scale = {scales.x, scales.x}, second_scale = {scales.y, scales.y};
                const u32x4 pairs0 = placed(raw.qs[2 * n], raw.qse[2 * n], shift), pairs1 = placed(raw.qs[2 * n + 1], raw.qse[2 * n + 1], shift);
                const uint32_t pair_words[8] = {pairs0.x, pairs0.y, pairs0.z, pairs0.w, pairs1.x, pairs1.y, pairs1.z, pairs1.w};
                const uint32_t j = 2u * (g & 1) + sh;  // which bit pair of a byte, and with 4 n which third bit
                uint32_t out[16];
#pragma unroll
                for (int w = 0; w < 8; w++) {
                    const uint32_t v = ((pair_words[w] >> (2u * j)) & 0x03030303u) | (((third_words[w] >> (4u * n + j)) & 0x01010101u) << 2);  // code + 4, one a byte
                    // element order inside a word: 0, 2 then 1, 3, as the activations were packed
                    const half2_t even = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, v, 0x0c020c00u) | 0x64006400u) - code_bias;
                    const half2_t odd = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, v, 0x0c030c01u) | 0x64006400u) - code_bias;
                    const half2_t scale = w < 4 ? first_scale : second_scale;
                    out[2 * w] = __builtin_bit_cast(uint32_t, even * scale), out[2 * w + 1] = __builtin_bit_cast(uint32_t, odd * scale);
                }
                u32x4 *to = reinterpret_cast<u32x4 *>(&Bs[buf][srow][32u * sh]);
#pragma unroll
                for (int i = 0; i < 4; i++) to[i] = u32x4{out[4 * i], out[4 * i + 1], out[4 * i + 2], out[4 * i + 3]};
                if (g == 0 && sh == 0) dds[sbuf][srow] = tail.w >> 16;  // (d, no dmin)
                u32x4 *adst = reinterpret_cast<u32x4 *>(&As[buf][srow][32u * sh]);
#pragma unroll
                for (int i = 0; i < 4; i++) adst[i] = av[g][i];
                fetch_activations(g, 4u * sb + (uint32_t)g + 4u);
                if (g == 3) fetch(raw, sb + 2u);  // these registers are free: the super-block after the next
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();  // step is staged; the multipliers are done with the step before it
            }
        };
        uint32_t sb = 0;
        for (; sb + 2u <= nsb; sb += 2u) {
            super_block(raws[0], sb);
            super_block(raws[1], sb + 1u);
        }
        if (sb < nsb) super_block(raws[0], sb);
        return;
    }
    gemm_multiply<false>(p, As, Bs, mns, dds, wave, lane, n0, m0, steps, 1.0f);
}

// bytes of device scratch a Q4_K wide product over M activation rows of K numbers packs into
size_t gemm_q4k_scratch_bytes(uint32_t M, uint32_t K, bool half_rows) {
    const size_t rows = half_rows ? M : (size_t)2 * M;
    return rows * K * sizeof(_Float16) + rows * ((K + 255u) / 256u) * 16u * sizeof(_Float16) + (size_t)M * sizeof(float);
}

static int32_t launch_gemm_mfma(nh_device *d, const GemmArgs &a) {
    GemmQ4Params p{};
    p.W = static_cast<const uint8_t *>(a.W);
    p.W1 = static_cast<const uint8_t *>(a.W_more[0]), p.W2 = static_cast<const uint8_t *>(a.W_more[1]);
    p.end0 = p.W1 ? a.end[0] : a.N, p.end1 = p.W2 ? a.end[1] : a.N;
    if ((p.W1 && (p.end0 % GT || p.end0 > a.N)) || (p.W2 && (!p.W1 || p.end1 % GT || p.end1 < p.end0 || p.end1 > a.N)))
        return fail(NH_E_ARGUMENT, "matrices stacked at columns %u and %u of %u do not fall on tiles of %d", a.end[0], a.end[1], a.N, GT);
    p.N = a.N;
    p.K = a.K;
    p.row_bytes = (uint32_t)payload_bytes(a.element, a.K);
    p.Y = a.Y;
    p.residual = a.residual;
    p.ldy = a.ldy;
    p.M = a.M;
    const bool half_rows = a.x_element == NH_F16;
    p.rows = half_rows ? a.M : 2 * a.M;
    p.split = half_rows ? 0 : 1;
    // scratch: [rows][K] halves, [rows][K / 256][16] sums, M row scales
    const size_t halves = (size_t)p.rows * a.K * sizeof(_Float16), sums = (size_t)p.rows * ((a.K + 255u) / 256u) * 16u * sizeof(_Float16);
    uint8_t *room = static_cast<uint8_t *>(scratch(d, gemm_q4k_scratch_bytes(a.M, a.K, half_rows)));
    if (!room) return NH_E_MEMORY;
    _Float16 *A = reinterpret_cast<_Float16 *>(room), *S = reinterpret_cast<_Float16 *>(room + halves);
    float *unscale = reinterpret_cast<float *>(room + halves + sums);
    if ((a.norm_w || a.gate) && (half_rows || (a.norm_w && a.gate) || ((uintptr_t)(a.norm_w ? a.norm_w : a.gate) & 15u)))
        return fail(NH_E_ARGUMENT, "a wide product normalises or gates fp32 rows read from 16-byte aligned addresses, one of the two");
    if (a.packed) {
        // what the launch before left in the scratch is this launch's operand
    } else if (half_rows) {
        hipLaunchKernelGGL(gemm_pack_rows_kernel<true>, dim3(a.M), dim3(256), 0, d->stream, a.X, a.K, A, S, unscale, nullptr, 0.0f);
    } else if (a.K % 4u == 0 && a.K >= 4u && (size_t)a.K * sizeof(float) <= PACK_STAGED_LDS_MOST && !pack_unstaged()) {
        // a row of fp32 numbers crosses memory once and waits in LDS
        const size_t lds = (size_t)a.K * sizeof(float);
        static bool roomy = false;
        if (!roomy) {
            NH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_pack_rows_staged_kernel<PACK_PLAIN>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)PACK_STAGED_LDS_MOST));
            NH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_pack_rows_staged_kernel<PACK_NORM>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)PACK_STAGED_LDS_MOST));
            NH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_pack_rows_staged_kernel<PACK_SWIGLU>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)PACK_STAGED_LDS_MOST));
            roomy = true;
        }
        const float *rows = static_cast<const float *>(a.X);
        if (a.norm_w) hipLaunchKernelGGL(gemm_pack_rows_staged_kernel<PACK_NORM>, dim3(a.M), dim3(256), lds, d->stream, rows, a.K, A, S, unscale, a.norm_w, a.eps);
        else if (a.gate) hipLaunchKernelGGL(gemm_pack_rows_staged_kernel<PACK_SWIGLU>, dim3(a.M), dim3(256), lds, d->stream, rows, a.K, A, S, unscale, a.gate, 0.0f);
        else hipLaunchKernelGGL(gemm_pack_rows_staged_kernel<PACK_PLAIN>, dim3(a.M), dim3(256), lds, d->stream, rows, a.K, A, S, unscale, static_cast<const float *>(nullptr), 0.0f);
    } else if (a.norm_w) {
        hipLaunchKernelGGL((gemm_pack_rows_kernel<false, PACK_NORM>), dim3(a.M), dim3(256), 0, d->stream, a.X, a.K, A, S, unscale, a.norm_w, a.eps);
    } else if (a.gate) {
        hipLaunchKernelGGL((gemm_pack_rows_kernel<false, PACK_SWIGLU>), dim3(a.M), dim3(256), 0, d->stream, a.X, a.K, A, S, unscale, a.gate, 0.0f);
    } else {
        hipLaunchKernelGGL(gemm_pack_rows_kernel<false>, dim3(a.M), dim3(256), 0, d->stream, a.X, a.K, A, S, unscale, nullptr, 0.0f);
    }
    NH_HIP(hipGetLastError());
    p.A = A, p.S = S, p.unscale = unscale;
    static bool sized = false;
    if (!sized) {
        NH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_q4k_mfma_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)GEMM_Q4K_LDS));
        NH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_q8_0_mfma_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)GEMM_Q8_LDS));
        NH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_q4k_regb_mfma_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)GEMM_Q4K_REGB_LDS));
        NH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_q6k_mfma_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)GEMM_Q4K_LDS));
        NH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_q5k_mfma_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)GEMM_Q4K_LDS));
        NH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_q3k_mfma_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)GEMM_Q4K_LDS));
        sized = true;
    }
    dim3 grid((a.N + GT - 1) / GT, (p.rows + GT - 1) / GT);
    if (a.element == NH_Q8_0) hipLaunchKernelGGL(gemm_q8_0_mfma_kernel, grid, dim3(512), GEMM_Q8_LDS, d->stream, p);
    else if (a.element == NH_Q6_K) hipLaunchKernelGGL(gemm_q6k_mfma_kernel, grid, dim3(512), GEMM_Q4K_LDS, d->stream, p);
    else if (a.element == NH_Q5_K) hipLaunchKernelGGL(gemm_q5k_mfma_kernel, grid, dim3(512), GEMM_Q4K_LDS, d->stream, p);
    else if (a.element == NH_Q3_K) hipLaunchKernelGGL(gemm_q3k_mfma_kernel, grid, dim3(512), GEMM_Q4K_LDS, d->stream, p);
    else if (const char *held = getenv("NEURA_HIP_GEMM_REGB"); held && held[0] == '0')  // the form that unpacks the weights into LDS
        hipLaunchKernelGGL(gemm_q4k_mfma_kernel, grid, dim3(512), GEMM_Q4K_LDS, d->stream, p);
    else hipLaunchKernelGGL(gemm_q4k_regb_mfma_kernel, grid, dim3(768), GEMM_Q4K_REGB_LDS, d->stream, p);
    NH_HIP(hipGetLastError());
    return NH_OK;
}

// the matrix-core forms take Q4_K, Q5_K, Q6_K and Q3_K rows of whole super-blocks and Q8_0 rows of whole pairs of blocks, read
// from 16-byte aligned addresses (a Q8_0, Q6_K or Q3_K matrix from a 4-byte one; its rows may start on any half word)
static bool mfma_takes(int32_t element, uint32_t K, const void *X, const void *W) {
    const char *held = getenv("NEURA_HIP_GEMM_MFMA");
    const bool wanted = !(held && held[0] == '0');
    const bool aligned = ((uintptr_t)X & 15u) == 0 && ((uintptr_t)W & (element == NH_Q4_K || element == NH_Q5_K ? 15u : 3u)) == 0;
    return wanted && aligned && K > 0 &&
           (((element == NH_Q4_K || element == NH_Q5_K || element == NH_Q6_K || element == NH_Q3_K) && K % 256u == 0) || (element == NH_Q8_0 && K % 64u == 0));
}

bool gemm_stacks(int32_t element, uint32_t K, const void *X, const void *W0, const void *W1, const void *W2, uint32_t end0, uint32_t end1) {
    if (!mfma_takes(element, K, X, W0)) return false;
    const uintptr_t loose = element == NH_Q4_K || element == NH_Q5_K ? 15u : 3u;
    if (W1 && (((uintptr_t)W1 & loose) || end0 % GT)) return false;
    if (W2 && (((uintptr_t)W2 & loose) || end1 % GT || !W1)) return false;
    return true;
}

int32_t launch_gemm(nh_device *d, const GemmArgs &a) {
    if (!a.M || !a.N) return NH_OK;
    if (mfma_takes(a.element, a.K, a.X, a.W)) return launch_gemm_mfma(d, a);
    if (a.W_more[0] || a.W_more[1] || a.packed || a.norm_w || a.gate)
        return fail(NH_E_ARGUMENT, "this wide product stacks no matrices, reuses no packed activations and packs rows as they lie (ask gemm_stacks first)");
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
    } else if (a.element == NH_Q6_K) {
        if (half) NH_GEMM(NH_Q6_K, true);
        else NH_GEMM(NH_Q6_K, false);
    } else if (a.element == NH_Q5_K) {
        if (half) NH_GEMM(NH_Q5_K, true);
        else NH_GEMM(NH_Q5_K, false);
    } else if (a.element == NH_Q3_K) {
        if (half) NH_GEMM(NH_Q3_K, true);
        else NH_GEMM(NH_Q3_K, false);
    } else {
        return fail(NH_E_ARGUMENT, "element %d carries no wide product", a.element);
    }
#undef NH_GEMM
    NH_HIP(hipGetLastError());
    return NH_OK;
}

}  // namespace nh
