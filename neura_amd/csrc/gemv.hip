// Narrow products (1..8 activation rows) over raw GGUF blocks: y[r][n] = sum_k x[r][k] * W[n][k].
//
// Which Q4_K form a product reaches with no switch set (launch_gemv asks them in this order; the 16-row tile product and
// the four-rows-to-an-MFMA kernel live in gemv_tile16.hip):
//
//   gemv_q4k_rows4_kernel      3 or 4 activation rows whose digit planes fit LDS (K up to about 10240), matrices that end on 16-row tiles
//                              (batch 3 and 4: q|k|v, attn_output, gate|up, the head)
//   gemv_q4k_tile16_kernel     1 row, any K of whole super-blocks, matrices that end on 16-row tiles: every product of a
//                              batch-1 decode step of the 0.5B .. 7B shapes; 2 rows the same (ffn_down's 18944 columns
//                              included); 3 and 4 rows where the kernel above refuses and the digits still fit LDS
//                              (with FIFTH the same for one row of Q5_K; gemv_q6k_tile16_kernel is its sibling for one row of Q6_K or Q3_K)
//   gemv_q4k_f16_kernel        5 to 8 rows, K <= 4096, at least 4 x 256 tiles of 16 rows (gate|up and the head at batch 5-8)
//   gemv_q4k_mfma32_kernel     5 to 8 rows otherwise (q|k|v -- with the rotation and the cache append in its epilogue where five to
//                              eight planes step one token each --, attn_output; ffn_down in K slices with gemv_fold_kernel), matrices
//                              that end on 32-row tiles; 3 and 4 rows of short (<= 8192 rows) or very tall (>= 65536) matrices that the
//                              two kernels on top refused
//   gemv_q4k_mfma_kernel       what is left with matrices on 16-row tiles and either several rows or K > 4096: ffn_down at
//                              batch 3 and 4 (K = 18944 does not fit the LDS of the forms above at four rows)
//   gemv_q4k_decode_kernel     1 row, K <= 4096, matrices that do NOT end on 16-row tiles or activations off a 16-byte
//                              boundary (odd vocabularies and widths: the small decoders of the tests); the vector form
//   gemv_q4k_kernel            the same refusals with K > 4096 or 2 to 4 rows: the LDS-tile vector form
//
// NEURA_HIP_TILE16=0, NEURA_HIP_ROWS4=0, NEURA_HIP_MFMA=0|2, NEURA_HIP_MFMA32=0|2 and NEURA_HIP_F16_TILES=0|2 push a product
// down (or up) this list so that the tests can hold the forms to each other on the same shapes.
//
// The vector form, Q4_K: a super-block is 144 B = a 16 B header (d, dmin, 12 scale bytes) + 128 B of nibbles.
// One lane owns one 64-element group of one super-block: it loads the header and its 32
// nibble bytes with three 128-bit loads, keeps its 64 activations in registers for the whole
// kernel and walks the output rows, so every weight byte is read from HBM exactly once and
// the activations never leave the register file.  A wave covers up to 16 super-blocks
// (4096 k); deeper rows are cut into slices whose partial sums a second kernel folds.
//
// Q8_0: 34 B blocks leave rows only 2-byte aligned, so a workgroup copies whole row slices
// into LDS with aligned 128-bit loads and each lane then reads its own block from LDS.
#include "blocks.hpp"
#include "common.hpp"
#include "gemv_shared.hpp"

#include <cstdlib>

namespace nh {

// skewed LDS index of activation i: 4 floats of padding per 64 keep 128-bit reads of
// neighbouring lanes on different banks
__device__ __forceinline__ uint32_t skew64(uint32_t i) { return i + (i >> 6) * 4; }
__device__ __forceinline__ uint32_t skew32(uint32_t i) { return i + (i >> 5) * 4; }

// 1 / sqrt(mean(x^2) + eps) of one activation row, to every thread.  Thread t adds columns t, t+256, ...
// as the reference's norm kernel does (crates/neura-kernel/src/task/norm.rs:69-83); the 256 partial
// sums are then joined inside each wave by shuffles and across waves through LDS with one barrier,
// not by the reference's eight-level tree (reduce.rs:21-38): a different order of the same fp32 adds.
__device__ float rms_scale(const float *__restrict__ x, uint32_t K, float eps, float *red) {
    float square = 0.0f;
    if (threadIdx.x < 256) {  // larger workgroups leave the sum to their first 256 threads
        for (uint32_t c = threadIdx.x; c < K; c += 256) {
            float value = x[c];
            square = __fadd_rn(square, __fmul_rn(value, value));
        }
    }
    square = wave_sum(square);
    if ((threadIdx.x & 63u) == 0 && threadIdx.x < 256) red[threadIdx.x >> 6] = square;
    __syncthreads();
    const float total = (red[0] + red[1]) + (red[2] + red[3]);
    __syncthreads();  // red is reused by the next row
    return rms_scale_of(total, K, eps);
}

// Stages x[k0 .. k0 + kn) of one activation row into LDS at dst[skew(i)], RMS-normalised over the whole row and
// weighed when norm_w is given.  With 256 threads and at most 32 values per thread every load goes out before the
// first value is used and the row is read once: a loop that handles each value as it arrives spends one memory
// round trip per value (6 us on a 3584-wide row).  Deeper slices take the looped form.
template <int PER, typename Skew>
__device__ __forceinline__ void stage_row_at_once(const float *__restrict__ x, uint32_t K, uint32_t k0, uint32_t kn, const float *__restrict__ norm_w,
                                                  float eps, float *dst, float *red, Skew skew) {
    const uint32_t tid = threadIdx.x;
    float held[PER], weight[PER];
    // every load is issued whatever its column (past the slice it reads the slice's last value, dropped below): loads
    // under a condition wait for one another
#pragma unroll
    for (int j = 0; j < PER; j++) held[j] = x[k0 + min(tid + 256u * j, kn - 1u)];
    if (norm_w) {
#pragma unroll
        for (int j = 0; j < PER; j++) weight[j] = norm_w[k0 + min(tid + 256u * j, kn - 1u)];
    }
#pragma unroll
    for (int j = 0; j < PER; j++)
        if (tid + 256u * j >= kn) held[j] = 0.0f;
    if (norm_w) {
        float square = 0.0f;  // thread t adds columns t, t + 256, ... in order (crates/neura-kernel/src/task/norm.rs:69-83)
#pragma unroll
        for (int j = 0; j < PER; j++) square = __fadd_rn(square, __fmul_rn(held[j], held[j]));
        square = wave_sum(square);
        if ((tid & 63u) == 0) red[tid >> 6] = square;
        __syncthreads();
        const float scale = rms_scale_of((red[0] + red[1]) + (red[2] + red[3]), K, eps);
        __syncthreads();  // red is reused by the next row
#pragma unroll
        for (int j = 0; j < PER; j++) held[j] = __fmul_rn(__fmul_rn(held[j], scale), weight[j]);
    }
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const uint32_t c = tid + 256u * j;
        if (c < kn) dst[skew(c)] = held[j];
    }
}

// MOST: the values a thread holds at most (a kernel pays for its widest form in registers whether or not a launch takes it)
template <int MOST = 16, typename Skew>
__device__ __forceinline__ void stage_row(const float *__restrict__ x, uint32_t K, uint32_t k0, uint32_t kn, const float *__restrict__ norm_w,
                                          float eps, float *dst, float *red, Skew skew) {
    const uint32_t tid = threadIdx.x;
    const bool at_once = blockDim.x == 256 && kn > 0 && (!norm_w || (k0 == 0 && kn == K));
    if (at_once && kn <= 1024u) {  // no more loads than the slice needs, to the next power of two
        stage_row_at_once<4>(x, K, k0, kn, norm_w, eps, dst, red, skew);
    } else if (MOST >= 8 && at_once && kn <= 2048u) {
        stage_row_at_once<MOST >= 8 ? 8 : 4>(x, K, k0, kn, norm_w, eps, dst, red, skew);
    } else if (MOST >= 16 && at_once && kn <= 4096u) {
        stage_row_at_once<MOST >= 16 ? 16 : 4>(x, K, k0, kn, norm_w, eps, dst, red, skew);
    } else if (MOST >= 32 && at_once && kn <= 8192u) {
        stage_row_at_once<MOST >= 32 ? 32 : 4>(x, K, k0, kn, norm_w, eps, dst, red, skew);
    } else {
        float scale = 1.0f;
        if (norm_w) scale = rms_scale(x, K, eps, red);
        for (uint32_t i = tid; i < kn; i += blockDim.x) {
            float value = x[k0 + i];
            if (norm_w) value = __fmul_rn(__fmul_rn(value, scale), norm_w[k0 + i]);
            dst[skew(i)] = value;
        }
    }
}

// logical row i of a pass -> output row.  With swiglu, even i walk the gate rows and odd i the
// up rows so that one lane group ends up holding both halves of an output.
__device__ __forceinline__ uint32_t weight_row(uint32_t i, uint32_t N, int32_t swiglu) {
    return swiglu ? ((i & 1u) ? N / 2 + (i >> 1) : (i >> 1)) : i;
}

// first byte of output row n and the end of the matrix that holds it.  Written with selects
// over scalars: indexing the parameter arrays by a per-lane segment would turn into loads
// from the kernel argument block and serialise the weight loads behind them.
__device__ __forceinline__ const uint8_t *row_start(const GemvParams &p, uint32_t n, const uint8_t *&matrix_end) {
    const uint8_t *w0 = p.W[0], *w1 = p.W[1], *w2 = p.W[2];
    const uint32_t e0 = p.end[0], e1 = p.end[1], e2 = p.end[2];
    const bool first = n < e0, second = n < e1;
    const uint8_t *base = first ? w0 : (second ? w1 : w2);
    const uint32_t before = first ? 0u : (second ? e0 : e1);
    const uint32_t rows = first ? e0 : (second ? e1 - e0 : e2 - e1);
    matrix_end = base + (size_t)rows * p.row_bytes;
    return base + (size_t)(n - before) * p.row_bytes;
}

template <int R, int RB>
__device__ __forceinline__ void publish(const GemvParams &p, uint32_t first, uint32_t split, float (&acc)[R][RB]) {
    if (p.splits > 1) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            uint32_t i = first + r;
            if (i >= p.N) continue;
            uint32_t n = weight_row(i, p.N, p.swiglu);
#pragma unroll
            for (int b = 0; b < RB; b++) p.partial[((size_t)split * RB + b) * p.N + n] = acc[r][b];
        }
        return;
    }
    if (p.swiglu) {
#pragma unroll
        for (int r = 0; r + 1 < R; r += 2) {
            uint32_t i = first + r;
            if (i + 1 >= p.N) continue;
#pragma unroll
            for (int b = 0; b < RB; b++) p.y[(size_t)b * (p.N / 2) + (i >> 1)] = silu(acc[r][b]) * acc[r + 1][b];
        }
        return;
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        uint32_t n = first + r;
        if (n >= p.N) continue;
#pragma unroll
        for (int b = 0; b < RB; b++) {
            float value = acc[r][b];
            if (p.residual) value = p.residual[(size_t)b * p.N + n] + value;
            p.y[(size_t)b * p.N + n] = value;
        }
    }
}

// ---------------------------------------------------------------------------- Q4_K -------


// Sum over the 32 low-nibble and the 32 high-nibble weights of 8 words against xl / xh.
// A nibble masked in place inside a 16-bit lane IS a half-precision subnormal: bits 0..3 read
// as code * 2^-24 and bits 4..7 as code * 2^-20, both exact.  The mixed-precision multiply-add
// (v_fma_mix_f32) widens the half operand on the fly, so a nibble costs one mask per pair and
// one multiply-add; the powers of two are folded into the block scales by the caller.
template <typename V4>
__device__ __forceinline__ void nibble_dots(const V4 &qa, const V4 &qb, const float (&xl)[32], const float (&xh)[32], float &low,
                                            float &high) {
    const uint32_t words[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
    float l = 0.0f, h = 0.0f;
#pragma unroll
    for (int w = 0; w < 8; w++) {
        const uint32_t even = words[w], odd = words[w] >> 8;  // bytes (0, 2) and bytes (1, 3) in the 16-bit lanes
        const half2_t l02 = __builtin_bit_cast(half2_t, even & 0x000f000fu);
        const half2_t h02 = __builtin_bit_cast(half2_t, even & 0x00f000f0u);
        const half2_t l13 = __builtin_bit_cast(half2_t, odd & 0x000f000fu);
        const half2_t h13 = __builtin_bit_cast(half2_t, odd & 0x00f000f0u);
        l = fmaf((float)l02.x, xl[4 * w + 0], l);
        l = fmaf((float)l13.x, xl[4 * w + 1], l);
        l = fmaf((float)l02.y, xl[4 * w + 2], l);
        l = fmaf((float)l13.y, xl[4 * w + 3], l);
        h = fmaf((float)h02.x, xh[4 * w + 0], h);
        h = fmaf((float)h13.x, xh[4 * w + 1], h);
        h = fmaf((float)h02.y, xh[4 * w + 2], h);
        h = fmaf((float)h13.y, xh[4 * w + 3], h);
    }
    low = l;   // scaled by 2^-24: the caller folds 2^24 into xl or the block scale
    high = h;  // scaled by 2^-20
}

// the two (scale, min) pairs of group g (sub-blocks 2g and 2g+1) from a block header
__device__ __forceinline__ void group_scales(const uint4 &hdr, uint32_t g, float &d0, float &d1, float &m0, float &m1) {
    float d = half_to_float((uint16_t)(hdr.x & 0xffffu));
    float dmin = half_to_float((uint16_t)(hdr.x >> 16));
    uint32_t shift = 16u * (g & 1u);
    uint32_t ya = (hdr.y >> shift) & 0xffffu, za = (hdr.z >> shift) & 0xffffu, wa = (hdr.w >> shift) & 0xffffu;
    uint32_t sc0, sc1, mn0, mn1;
    if (g < 2) {
        sc0 = ya & 63u;
        sc1 = (ya >> 8) & 63u;
        mn0 = za & 63u;
        mn1 = (za >> 8) & 63u;
    } else {
        sc0 = (wa & 0x0fu) | (((ya >> 6) & 3u) << 4);
        sc1 = ((wa >> 8) & 0x0fu) | (((ya >> 14) & 3u) << 4);
        mn0 = ((wa >> 4) & 0x0fu) | (((za >> 6) & 3u) << 4);
        mn1 = ((wa >> 12) & 0x0fu) | (((za >> 14) & 3u) << 4);
    }
    d0 = d * (float)sc0;
    d1 = d * (float)sc1;
    m0 = dmin * (float)mn0;
    m1 = dmin * (float)mn1;
}

// Sums R per-lane partials over the G lanes of a row group.  The first log2(R) steps fold two
// rows into one register (each lane keeps the row its own index selects), so R rows cost
// R - 1 + log2(G / R) exchanges instead of R log2(G); steps inside a row of 16 lanes are DPP
// adds, only the steps across 16 and 32 lanes go through the LDS crossbar.  On return lane u
// (u < R, u = lane % G) of every group holds the total of row u.
template <int R, int G>
__device__ __forceinline__ float fold_rows(float (&acc)[R], uint32_t lane) {
    static_assert(R == 2 || R == 4, "rows per pass");
    static_assert(G == 16 || G == 32 || G == 64, "lanes per row group");
    float v;
    const bool odd = lane & 1u;
    if (R == 4) {
        const bool upper = lane & 2u;
        float keep01 = odd ? acc[1] : acc[0], send01 = odd ? acc[0] : acc[1];
        float keep23 = odd ? acc[3] : acc[2], send23 = odd ? acc[2] : acc[3];
        float v01 = keep01 + dpp<DPP_QUAD_XOR1>(send01);
        float v23 = keep23 + dpp<DPP_QUAD_XOR1>(send23);
        float keep = upper ? v23 : v01, send = upper ? v01 : v23;
        v = keep + dpp<DPP_QUAD_XOR2>(send);
    } else {
        float keep = odd ? acc[1] : acc[0], send = odd ? acc[0] : acc[1];
        v = keep + dpp<DPP_QUAD_XOR1>(send);
        v += dpp<DPP_QUAD_XOR2>(v);
    }
    v += dpp<DPP_ROW_ROR4>(v);  // rotations inside a row of 16 lanes keep lane % 4
    v += dpp<DPP_ROW_ROR8>(v);
    if (G >= 32) v += __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));  // lane ^ 16
    if (G >= 64) v += __shfl_xor(v, 32, 64);
    return v;
}

// The epilogue of a q|k|v product that folds the rotation in: lane u < R of a lane group holds logical row i = first + u, and
// logical rows 2t, 2t + 1 are channels c and c + width/2 of one head (crates/neura-kernel/src/task/rope.rs:95-122).  The
// projection's bias, if it has one, comes before the rotation; q rows go to y, k rows rotated and v rows as they are to the
// caches as halves, at the cursor (at cursor mod span in a ring).  Every lane of the wave calls it.
template <int R>
__device__ __forceinline__ void rotate_and_store(const GemvParams &p, float total, uint32_t i, uint32_t u) {
    const uint32_t half = p.rope_width >> 1, pair = min(i, p.N - 1u) >> 1, c = pair % half;
    const uint32_t n = (pair / half) * p.rope_width + c + (i & 1u) * half;
    if (u < R && i < p.N) {
        const float *b0 = p.bias[0], *b1 = p.bias[1], *b2 = p.bias[2];
        const uint32_t e0 = p.end[0], e1 = p.end[1];
        const float *bias = n < e0 ? b0 : (n < e1 ? b1 : b2);
        const uint32_t before = n < e0 ? 0u : (n < e1 ? e0 : e1);
        if (bias) total += bias[n - before];
    }
    const float other = dpp<DPP_QUAD_XOR1>(total);
    if (u < R && i < p.N) {
        const uint32_t position = p.rope_cursor[0];
        float value = total;
        if (n < p.rope_k_rows) {
            // cos and sin of f32(position) * pow(base, -2c/width), tabulated once per model by the rotation's own kernel
            const float cosine = p.rope_cosines[(size_t)min(position, p.rope_positions - 1u) * half + c];
            const float sine = p.rope_sines[(size_t)min(position, p.rope_positions - 1u) * half + c];
            value = (i & 1u) ? total * cosine + other * sine : total * cosine - other * sine;
        }
        if (n < p.rope_q_rows) {
            p.y[n] = value;
        } else if (position >= p.rope_positions || (!p.rope_ring && position >= p.rope_capacity)) {
            atomicMax(p.refusal, (uint32_t)REFUSAL_ORIGIN);
        } else {
            const bool key = n < p.rope_k_rows;
            const uint32_t within = n - (key ? p.rope_q_rows : p.rope_k_rows);  // head * width + channel
            const uint32_t head = within / p.rope_width, channel = within % p.rope_width;
            uint16_t *cache = key ? p.rope_k : p.rope_v;
            const uint32_t slot = p.rope_ring ? position % p.rope_ring : position;  // a ring seats position p at p mod its span
            state_store(cache, p.rope_element, ((uint64_t)head * p.rope_capacity + slot) * p.rope_width + channel, value);
        }
    }
}

// One pass of the decode kernel over R rows: the raw blocks a lane owns.
template <int R>
struct DecodeTile {
    u32x4 hdr[R], qa[R], qb[R];
};

// Decode path (one activation row).  G = lanes per output row (64: one row group per wave
// pass, the hot case; 32 / 16: short rows, several row groups side by side in a wave).
//
// A lane owns one 64-element group of one super-block for the whole kernel and keeps its 64
// activations in registers.  Every integer field is consumed as a half-precision subnormal by
// mixed-precision multiply-adds (nibbles: * 2^-24 / 2^-20, undone by scaling the activations
// once; scales: * 2^-24, undone once per pass), so a weight costs 1.6 vector instructions.
template <int R, int G, bool PIPE, int NW, bool ROPE = false>
__global__ __launch_bounds__(NW * 64) void gemv_q4k_decode_kernel(GemvParams p) {
    extern __shared__ float xs[];  // skew64(slice)
    __shared__ float red[256];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t split = blockIdx.y;
    const uint32_t blk0 = split * p.blocks_per_split;
    const uint32_t nb = min(p.blocks_per_split, p.nblk - blk0);
    const uint32_t k0 = blk0 * 256u, kn = nb * 256u;

    constexpr uint32_t RS = 64u / G;
    constexpr uint32_t rows_per_pass = R * RS;
    const uint32_t u = lane & (G - 1u), rs = lane / G;
    const bool active = u < nb * 4u;
    const uint32_t unit = active ? u : 0u;  // an idle lane re-reads unit 0 against zero activations
    const uint32_t g = unit & 3u;
    const uint32_t lane_offset = (blk0 + (unit >> 2)) * 144u + g * 32u;
    const ScaleLane lane_scales = scale_lane(g);

    auto load = [&](DecodeTile<R> &t, uint32_t rg) {
        const uint32_t first = rg * rows_per_pass + rs * R;  // first logical row of this lane group (a multiple of R)
        // R rows of one matrix: rows never straddle a matrix (every end is a multiple of R)
        const uint8_t *base[R];
        if (p.swiglu) {
            const uint32_t pair = min(first, p.N - R) >> 1;  // logical rows 2q, 2q+1 = gate row q, up row q
#pragma unroll
            for (int r = 0; r < R; r++) base[r] = ((r & 1) ? p.W[1] : p.W[0]) + (size_t)(pair + (r >> 1)) * p.row_bytes;
        } else {
            // with the rotation folded in, logical rows 2t, 2t+1 are channels t and t + width/2 of one head
            const uint32_t logical = min(first, p.N - R);
            const uint32_t half = p.rope_width >> 1, pair = logical >> 1;
            const uint32_t n = ROPE ? (pair / half) * p.rope_width + pair % half : logical;
            const uint32_t hop = ROPE ? half : 1u;
            const bool in0 = n < p.end[0], in1 = n < p.end[1];
            const uint8_t *matrix = in0 ? p.W[0] : (in1 ? p.W[1] : p.W[2]);
            const uint32_t before = in0 ? 0u : (in1 ? p.end[0] : p.end[1]);
#pragma unroll
            for (int r = 0; r < R; r++) base[r] = matrix + (size_t)(n - before + r * hop) * p.row_bytes;
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            typedef const __attribute__((address_space(1))) u32x4 *global_uint4;  // the arena is global memory
            const uint8_t *at = base[r] + lane_offset;
            t.hdr[r] = *(global_uint4)(uintptr_t)(at - g * 32u);
            t.qa[r] = *(global_uint4)(uintptr_t)(at + 16u);
            t.qb[r] = *(global_uint4)(uintptr_t)(at + 32u);
        }
    };

    const uint32_t stride = gridDim.x * NW;
    uint32_t rg = blockIdx.x * NW + wave;
    DecodeTile<R> ta, tb;
    if (rg < p.row_groups) load(ta, rg);  // in flight while the activations are staged

    stage_row(p.x, p.K, k0, kn, p.norm_w, p.eps, xs, red, [](uint32_t i) { return skew64(i); });
    __syncthreads();

    float xl[32], xh[32];
    float xsl = 0.0f, xsh = 0.0f;  // plain sums of this lane's activations (for the block minimums)
    {
        const float4 *src = reinterpret_cast<const float4 *>(xs + skew64(unit * 64u));
        const float keep = active ? 1.0f : 0.0f;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            // sum and scale each chunk as it arrives: raw and scaled copies never coexist
            float4 a = src[j], c = src[8 + j];
            xsl += (a.x + a.y) + (a.z + a.w);
            xsh += (c.x + c.y) + (c.z + c.w);
            const float sl = keep * 16777216.0f, sh = keep * 1048576.0f;  // nibbles arrive * 2^-24 / * 2^-20
            xl[4 * j] = a.x * sl, xl[4 * j + 1] = a.y * sl, xl[4 * j + 2] = a.z * sl, xl[4 * j + 3] = a.w * sl;
            xh[4 * j] = c.x * sh, xh[4 * j + 1] = c.y * sh, xh[4 * j + 2] = c.z * sh, xh[4 * j + 3] = c.w * sh;
        }
        xsl *= keep, xsh *= keep;
    }

    auto compute = [&](const DecodeTile<R> &t, uint32_t rg) {
        const uint32_t first = rg * rows_per_pass + rs * R;
        float acc[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            float low, high;
            nibble_dots(t.qa[r], t.qb[r], xl, xh, low, high);
            half2_t sc, mn;
            scale_pairs(t.hdr[r], lane_scales, sc, mn);
            const half2_t dd = __builtin_bit_cast(half2_t, t.hdr[r].x);  // (d, dmin)
            const float weighed = fmaf((float)sc.y, high, (float)sc.x * low);
            const float floor_ = fmaf((float)mn.y, xsh, (float)mn.x * xsl);
            acc[r] = fmaf((float)dd.x, weighed, -((float)dd.y * floor_));
        }
        float total = fold_rows<R, G>(acc, lane) * 16777216.0f;  // the scales arrived * 2^-24
        const uint32_t i = first + u;                             // lane u < R holds row first + u
        if (p.splits > 1) {
            if (u < R && i < p.N) p.partial[(size_t)split * p.N + weight_row(i, p.N, p.swiglu)] = total;
        } else if (p.swiglu) {
            float up = dpp<DPP_QUAD_XOR1>(total);
            if (u < R && !(u & 1u) && i + 1 < p.N) p.y[i >> 1] = silu(total) * up;
        } else if (ROPE) {
            rotate_and_store<R>(p, total, i, u);
        } else if (u < R && i < p.N) {
            p.y[i] = p.residual ? p.residual[i] + total : total;
        }
    };

    if (PIPE) {
        while (rg < p.row_groups) {
            uint32_t next = rg + stride;
            if (next < p.row_groups) load(tb, next);
            compute(ta, rg);
            rg = next;
            if (rg >= p.row_groups) break;
            next = rg + stride;
            if (next < p.row_groups) load(ta, next);
            compute(tb, rg);
            rg = next;
        }
    } else {
        while (rg < p.row_groups) {
            compute(ta, rg);
            rg += stride;
            __builtin_amdgcn_sched_barrier(0);  // the next loads reuse this tile's registers: keep them behind the arithmetic
            if (rg < p.row_groups) load(ta, rg);
        }
    }
}

// General narrow product: RB activation rows (2 or 4) staged in LDS and re-read per row group.
template <int R, int RB>
__global__ __launch_bounds__(256) void gemv_q4k_kernel(GemvParams p) {
    fetch_parameters(p);
    extern __shared__ float xs[];  // [RB][skew64(slice)]
    __shared__ float red[256];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t split = blockIdx.y;
    const uint32_t blk0 = split * p.blocks_per_split;
    const uint32_t nb = min(p.blocks_per_split, p.nblk - blk0);
    const uint32_t k0 = blk0 * 256u, kn = nb * 256u;
    const uint32_t xstride = skew64(p.blocks_per_split * 256u);

#pragma unroll
    for (int b = 0; b < RB; b++)
        stage_row(p.x + (size_t)b * p.K, p.K, k0, kn, p.norm_w, p.eps, xs + b * xstride, red, [](uint32_t i) { return skew64(i); });
    __syncthreads();

    const uint32_t G = p.group;  // lanes per output row
    const uint32_t u = lane & (G - 1u), rs = lane / G, RS = 64u / G;
    const bool active = u < nb * 4u;
    const uint32_t blk = active ? (u >> 2) : 0u, g = u & 3u;
    float xl[32], xh[32];

    const uint32_t rows_per_pass = R * RS;
    for (uint32_t rg = blockIdx.x * 4u + wave; rg < p.row_groups; rg += gridDim.x * 4u) {
        const uint32_t first = rg * rows_per_pass + rs * R;  // first logical row of this lane group
        uint4 hdr[R], qa[R], qb[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            uint32_t i = first + r;
            uint32_t n = weight_row(i < p.N ? i : 0u, p.N, p.swiglu);
            const uint8_t *matrix_end;
            const uint8_t *base = row_start(p, n, matrix_end) + (size_t)(blk0 + blk) * 144u;
            hdr[r] = *reinterpret_cast<const uint4 *>(base);
            qa[r] = *reinterpret_cast<const uint4 *>(base + 16u + g * 32u);
            qb[r] = *reinterpret_cast<const uint4 *>(base + 32u + g * 32u);
        }
        float acc[R][RB];
#pragma unroll
        for (int b = 0; b < RB; b++) {
            const float4 *src = reinterpret_cast<const float4 *>(xs + b * xstride + skew64((blk * 4u + g) * 64u));
            float xsl = 0.0f, xsh = 0.0f;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                float4 a = active ? src[j] : make_float4(0.f, 0.f, 0.f, 0.f);
                float4 c = active ? src[8 + j] : make_float4(0.f, 0.f, 0.f, 0.f);
                xl[4 * j] = a.x, xl[4 * j + 1] = a.y, xl[4 * j + 2] = a.z, xl[4 * j + 3] = a.w;
                xh[4 * j] = c.x, xh[4 * j + 1] = c.y, xh[4 * j + 2] = c.z, xh[4 * j + 3] = c.w;
            }
#pragma unroll
            for (int j = 0; j < 32; j++) xsl += xl[j], xsh += xh[j];
#pragma unroll
            for (int r = 0; r < R; r++) {
                float d0, d1, m0, m1, low, high;
                group_scales(hdr[r], g, d0, d1, m0, m1);
                nibble_dots(qa[r], qb[r], xl, xh, low, high);
                acc[r][b] = (d0 * (low * 16777216.0f) + d1 * (high * 1048576.0f)) - (m0 * xsl + m1 * xsh);
            }
        }
        // sum over the G lanes of the group
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int b = 0; b < RB; b++) {
                float v = acc[r][b];
                for (uint32_t offset = G >> 1; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, 64);
                acc[r][b] = v;
            }
        if (u == 0) publish<R, RB>(p, first, split, acc);
    }
}

// ---------------------------------------------------------------------------- Q8_0 -------

template <int R, int RB>
__global__ __launch_bounds__(256) void gemv_q8_0_kernel(GemvParams p) {
    fetch_parameters(p);
    extern __shared__ float shared[];  // xs [RB][skew32(slice)] then the staged weight tile
    __shared__ float red[256];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t split = blockIdx.y;
    const uint32_t blk0 = split * p.blocks_per_split;
    const uint32_t nb = min(p.blocks_per_split, p.nblk - blk0);
    const uint32_t k0 = blk0 * 32u, kn = nb * 32u;
    const uint32_t xstride = skew32(p.blocks_per_split * 32u);
    float *xs = shared;
    uint8_t *tile = reinterpret_cast<uint8_t *>(shared + RB * xstride);  // 16-byte aligned: xstride is a multiple of 4
    const uint32_t lrow = p.chunks_per_row * 16u;

#pragma unroll
    for (int b = 0; b < RB; b++)
        stage_row(p.x + (size_t)b * p.K, p.K, k0, kn, p.norm_w, p.eps, xs + b * xstride, red, [](uint32_t i) { return skew32(i); });
    __syncthreads();

    const uint32_t G = p.group;
    const uint32_t u = lane & (G - 1u), rs = lane / G, RS = 64u / G;
    const bool active = u < nb;

    float xr[32];
    float xsum = 0.0f;
    if (RB == 1) {
        const float4 *src = reinterpret_cast<const float4 *>(xs + skew32((active ? u : 0u) * 32u));
#pragma unroll
        for (int j = 0; j < 8; j++) {
            float4 a = active ? src[j] : make_float4(0.f, 0.f, 0.f, 0.f);
            xr[4 * j] = a.x, xr[4 * j + 1] = a.y, xr[4 * j + 2] = a.z, xr[4 * j + 3] = a.w;
        }
#pragma unroll
        for (int j = 0; j < 32; j++) xsum += xr[j];
    }

    const uint32_t rows_per_wave = R * RS, rows_per_tile = rows_per_wave * 4u;
    const uint32_t slice_bytes = nb * 34u;
    const uint32_t tiles = (p.row_groups + 3u) / 4u;  // row_groups counts wave passes
    for (uint32_t t = blockIdx.x; t < tiles; t += gridDim.x) {
        const uint32_t tile_first = t * rows_per_tile;
        __syncthreads();  // the previous tile is no longer read
        for (uint32_t c = tid; c < rows_per_tile * p.chunks_per_row; c += 256) {
            uint32_t local = c / p.chunks_per_row, chunk = c % p.chunks_per_row;
            uint32_t i = tile_first + local;
            if (i >= p.N) continue;
            uint32_t n = weight_row(i, p.N, p.swiglu);
            const uint8_t *w_end;
            const uint8_t *start = row_start(p, n, w_end) + (size_t)blk0 * 34u;
            const uint8_t *aligned = start - ((uintptr_t)start & 15u);
            uint32_t lead = (uint32_t)((uintptr_t)start & 15u);
            if (chunk * 16u >= lead + slice_bytes) continue;
            const uint8_t *src = aligned + chunk * 16u;
            uint4 held;
            if (src + 16 <= w_end) {
                held = *reinterpret_cast<const uint4 *>(src);
            } else {  // the last bytes of the tensor: never read past its end
                uint8_t bytes[16];
#pragma unroll
                for (int j = 0; j < 16; j++) bytes[j] = (src + j < w_end) ? src[j] : (uint8_t)0;
                held = *reinterpret_cast<uint4 *>(bytes);
            }
            *reinterpret_cast<uint4 *>(tile + local * lrow + chunk * 16u) = held;
        }
        __syncthreads();

        const uint32_t local_first = wave * rows_per_wave + rs * R;
        const uint32_t first = tile_first + local_first;
        float acc[R][RB];
        uint32_t quants[R][8];
        float scales[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            uint32_t i = first + r;
            uint32_t n = weight_row(i < p.N ? i : 0u, p.N, p.swiglu);
            const uint8_t *matrix_end;
            uint32_t lead = (uint32_t)((uintptr_t)(row_start(p, n, matrix_end) + (size_t)blk0 * 34u) & 15u);
            uint32_t at = (local_first + r) * lrow + lead + (active ? u : 0u) * 34u;  // byte offset of the block in the tile
            bool held = active && i < p.N;
            scales[r] = held ? half_to_float(*reinterpret_cast<const uint16_t *>(tile + at)) : 0.0f;
            uint32_t payload = at + 2u;
            const uint32_t *words = reinterpret_cast<const uint32_t *>(tile + (payload & ~3u));
            uint32_t shift = (payload & 3u) * 8u;  // 0 or 16
            uint32_t raw[9];
#pragma unroll
            for (int j = 0; j < 9; j++) raw[j] = held ? words[j] : 0u;
#pragma unroll
            for (int j = 0; j < 8; j++) quants[r][j] = __funnelshift_r(raw[j], raw[j + 1], shift) ^ 0x80808080u;  // q + 128
        }
#pragma unroll
        for (int b = 0; b < RB; b++) {
            if (RB > 1) {
                const float4 *src = reinterpret_cast<const float4 *>(xs + b * xstride + skew32((active ? u : 0u) * 32u));
                xsum = 0.0f;
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    float4 a = active ? src[j] : make_float4(0.f, 0.f, 0.f, 0.f);
                    xr[4 * j] = a.x, xr[4 * j + 1] = a.y, xr[4 * j + 2] = a.z, xr[4 * j + 3] = a.w;
                }
#pragma unroll
                for (int j = 0; j < 32; j++) xsum += xr[j];
            }
#pragma unroll
            for (int r = 0; r < R; r++) {
                float total = 0.0f;
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    uint32_t w = quants[r][j];
                    total = fmaf(xr[4 * j + 0], (float)(w & 0xffu), total);
                    total = fmaf(xr[4 * j + 1], (float)((w >> 8) & 0xffu), total);
                    total = fmaf(xr[4 * j + 2], (float)((w >> 16) & 0xffu), total);
                    total = fmaf(xr[4 * j + 3], (float)(w >> 24), total);
                }
                acc[r][b] = scales[r] * (total - 128.0f * xsum);
            }
        }
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int b = 0; b < RB; b++) {
                float v = acc[r][b];
                for (uint32_t offset = G >> 1; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, 64);
                acc[r][b] = v;
            }
        if (u == 0) publish<R, RB>(p, first, split, acc);
    }
}

// The activation row of the product behind a decode attention, merged from the sums the attention left a section of the keys
// each (SectionSums; crates/neura-kernel/src/task/attention.rs:619-671 is the merge): element (head, channel) is the sections'
// channel sums weighed by e^(section's largest score - the largest of all) over the masses weighed the same way.  Every load
// a thread needs -- the statistics of two (head, section) pairs, sixteen channel sums of each of its four elements -- is asked
// for before the first is used (sections past the last read the last again and are dropped).  The statistics cross in LDS:
// the thread of a pair turns its section's largest score into the section's weight, the thread of an element then reads
// sixteen weights and masses.  `width` is a power of two (the decode attention's 64 or 128).
template <typename Skew>
__device__ __forceinline__ void stage_merged(const float *__restrict__ partial, uint32_t sections, uint32_t G, uint32_t width, uint32_t K, float *xs, Skew skew) {
    constexpr uint32_t MOST = MERGED_SECTIONS_MOST, HEADS_MOST = 32;
    __shared__ __attribute__((aligned(16))) float tops[HEADS_MOST * MOST], masses[HEADS_MOST * MOST], weights[HEADS_MOST * MOST];
    const uint32_t tid = threadIdx.x, shift = 31u - __builtin_clz(width), heads = K >> shift, hop = G * (width + 2u);
    const uint32_t by_groups = 65536u / G + 1u;  // x / G = x * by_groups >> 16 for the few heads here
    auto sums_of = [&](uint32_t head) {
        const uint32_t unit = head * by_groups >> 16;
        return partial + ((uint64_t)unit * sections * G + (head - unit * G)) * (width + 2u);
    };
    // seat tid + 256 j of the statistics: head seat / MOST, section seat % MOST; a seat past the heads or the sections holds
    // no score and no mass (its loads read the last head's, the last section's, and are dropped)
    float top[2], mass[2];
    bool seated[2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const uint32_t seat = tid + 256u * j, head = seat / MOST, section = seat % MOST;
        seated[j] = head < heads && section < sections;
        const float *stats = sums_of(min(head, heads - 1u)) + min(section, sections - 1u) * hop + width;
        top[j] = stats[0], mass[j] = stats[1];
    }
    for (uint32_t base = 0; base < K; base += 1024u) {
        float values[4][MOST];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const uint32_t i = min(base + tid + 256u * e, K - 1u);
            const float *column = sums_of(i >> shift) + (i & (width - 1u));
#pragma unroll
            for (uint32_t s = 0; s < MOST; s++) values[e][s] = column[min(s, sections - 1u) * hop];
        }
        if (base == 0) {
#pragma unroll
            for (int j = 0; j < 2; j++) tops[tid + 256u * j] = seated[j] ? top[j] : -INFINITY, masses[tid + 256u * j] = seated[j] ? mass[j] : 0.0f;
            __syncthreads();
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const float4 *row = reinterpret_cast<const float4 *>(tops + ((tid + 256u * j) & ~(MOST - 1u)));
                float largest = -INFINITY;
#pragma unroll
                for (uint32_t q = 0; q < MOST / 4u; q++) largest = fmaxf(fmaxf(largest, fmaxf(row[q].x, row[q].y)), fmaxf(row[q].z, row[q].w));
                weights[tid + 256u * j] = !seated[j] || top[j] == -INFINITY ? 0.0f : softmax_exp(top[j] - largest);
            }
            __syncthreads();
        }
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const uint32_t i = base + tid + 256u * e;
            if (i >= K) continue;
            const float4 *head_weights = reinterpret_cast<const float4 *>(weights + (i >> shift) * MOST);
            const float4 *head_masses = reinterpret_cast<const float4 *>(masses + (i >> shift) * MOST);
            float total = 0.0f, sum = 0.0f;
#pragma unroll
            for (uint32_t q = 0; q < MOST / 4u; q++) {
                const float4 w = head_weights[q], m = head_masses[q];
                total = fmaf(m.x, w.x, total), total = fmaf(m.y, w.y, total), total = fmaf(m.z, w.z, total), total = fmaf(m.w, w.w, total);
                sum = fmaf(values[e][4 * q], w.x, sum), sum = fmaf(values[e][4 * q + 1], w.y, sum);
                sum = fmaf(values[e][4 * q + 2], w.z, sum), sum = fmaf(values[e][4 * q + 3], w.w, sum);
            }
            xs[skew(i)] = total > 0.0f ? sum * (1.0f / total) : 0.0f;
        }
    }
}

// Q8_0, one activation row, rows of at most 64 blocks (K <= 2048): the shape of the Q4_K decode kernel.  A lane owns one
// block column for the whole kernel and keeps its 32 activations in registers; the 34 bytes of a block sit on a 2-byte
// boundary, so a lane reads the nine words that cover it from the 4-byte boundary below it (the reference's own reading,
// crates/neura-kernel/src/dot.rs:197-264) and realigns by 16 bits where the block starts on a half word.  No LDS tile and no
// barrier between the rows: the first pass's words are on their way while the activations are staged.
typedef uint32_t u32x4_loose __attribute__((ext_vector_type(4), aligned(4)));

template <int R>
struct Q8Tile {
    u32x4 a[R], b[R];
    uint32_t c[R];
    uint32_t odd[R];  // 2 where the row's block starts on a half word, else 0
};

// DEEP (rows of 65 to 256 blocks, K <= 8192): the four waves of a workgroup walk the same rows, wave w the blocks 64 w ..
// 64 w + 63, and meet in LDS once a pass.
// The leading arguments are what the first weight loads and the activations' need: plain words the hardware hands to a wave in
// scalar registers as it starts (Q8_LEAD packs them: the rotation's width rides above the blocks a row, the SwiGLU flag above
// N); they take the place of the same members of the parameter block, whose other members are loaded as they come to use.
#define Q8_LEAD(p) (p).W[0], (p).W[1], (p).W[2], (p).x, (p).row_bytes, (p).nblk | ((p).rope_width << 16), (p).row_groups, (p).N | ((p).swiglu ? 0x80000000u : 0u), (p).end[0], (p).end[1], (p)
// MERGE: the activation row is merged from a decode attention's section sums (x points at them) as it is staged.
template <int R, int G, bool DEEP = false, bool ROPE = false, bool MERGE = false>
__global__ __launch_bounds__(256) void gemv_q8_0_decode_kernel(const uint8_t *lead_w0, const uint8_t *lead_w1, const uint8_t *lead_w2, const float *lead_x,
                                                               uint32_t lead_row_bytes, uint32_t lead_nblk_width, uint32_t lead_row_groups, uint32_t lead_n_swiglu,
                                                               uint32_t lead_end0, uint32_t lead_end1, GemvParams rest) {
    GemvParams p = rest;
    p.W[0] = lead_w0, p.W[1] = lead_w1, p.W[2] = lead_w2, p.x = lead_x, p.row_bytes = lead_row_bytes, p.row_groups = lead_row_groups;
    p.nblk = lead_nblk_width & 0xffffu, p.rope_width = lead_nblk_width >> 16, p.K = 32u * (lead_nblk_width & 0xffffu);
    p.N = lead_n_swiglu & 0x7fffffffu, p.swiglu = (int32_t)(lead_n_swiglu >> 31), p.end[0] = lead_end0, p.end[1] = lead_end1;
    static_assert(!DEEP || G == 64, "a deep row fills every wave");
    static_assert(!ROPE || (R == 2 && !DEEP), "the rotation pairs the two rows of a pass");
    extern __shared__ float xs[];  // skew32(K)
    __shared__ float red[256];
    __shared__ float part[2][4][R];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    constexpr uint32_t RS = 64u / G, rows_per_pass = R * RS;
    const uint32_t u = lane & (G - 1u), rs = lane / G;
    const uint32_t block = DEEP ? 64u * wave + u : u;
    const bool active = block < p.nblk;
    const uint32_t unit = active ? block : 0u;  // an idle lane re-reads block 0 against zero activations

    auto load = [&](Q8Tile<R> &t, uint32_t rg) {
        const uint32_t first = rg * rows_per_pass + rs * R;  // first logical row of this lane group (a multiple of R)
        const uint8_t *base[R];
        if (p.swiglu) {
            const uint32_t pair = min(first, p.N - R) >> 1;  // logical rows 2q, 2q+1 = gate row q, up row q
#pragma unroll
            for (int r = 0; r < R; r++) base[r] = ((r & 1) ? p.W[1] : p.W[0]) + (size_t)(pair + (r >> 1)) * p.row_bytes;
        } else {
            // R rows of one matrix: every matrix end is a multiple of R.  With the rotation folded in, logical rows 2t, 2t+1
            // are channels t and t + width/2 of one head
            const uint32_t logical = min(first, p.N - R);
            const uint32_t half = p.rope_width >> 1, pair = logical >> 1;
            const uint32_t n = ROPE ? (pair / half) * p.rope_width + pair % half : logical;
            const uint32_t hop = ROPE ? half : 1u;
            const bool in0 = n < p.end[0], in1 = n < p.end[1];
            const uint8_t *matrix = in0 ? p.W[0] : (in1 ? p.W[1] : p.W[2]);
            const uint32_t before = in0 ? 0u : (in1 ? p.end[0] : p.end[1]);
#pragma unroll
            for (int r = 0; r < R; r++) base[r] = matrix + (size_t)(n - before + r * hop) * p.row_bytes;
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uintptr_t at = (uintptr_t)(base[r] + unit * 34u);
            const uintptr_t low = at & ~(uintptr_t)3;
            t.odd[r] = (uint32_t)(at & 2u);
            t.a[r] = *(const __attribute__((address_space(1))) u32x4_loose *)low;
            t.b[r] = *(const __attribute__((address_space(1))) u32x4_loose *)(low + 16u);
            // a block on a word boundary ends two bytes into the ninth word: those two only are read (the last block of a
            // tensor ends where its allocation may)
            if (at & 2u) t.c[r] = *(const __attribute__((address_space(1))) uint32_t *)(low + 32u);
            else t.c[r] = *(const __attribute__((address_space(1))) uint16_t *)(low + 32u);
        }
    };

    const uint32_t stride = DEEP ? gridDim.x : gridDim.x * 4u;
    uint32_t rg = DEEP ? blockIdx.x : blockIdx.x * 4u + wave;
    uint32_t parity = 0;
    Q8Tile<R> held;
    if (rg < p.row_groups) load(held, rg);  // in flight while the activations are staged

    if constexpr (MERGE) stage_merged(p.x, p.merge_sections, p.merge_groups, p.merge_width, p.K, xs, [](uint32_t i) { return skew32(i); });
    else stage_row<DEEP ? 32 : 8>(p.x, p.K, 0u, p.K, p.norm_w, p.eps, xs, red, [](uint32_t i) { return skew32(i); });  // rows of 256 blocks, or of 64
    __syncthreads();

    float xr[32];
    float xsum = 0.0f;
    {
        const float4 *src = reinterpret_cast<const float4 *>(xs + skew32(unit * 32u));
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const float4 a = active ? src[j] : make_float4(0.f, 0.f, 0.f, 0.f);
            xr[4 * j] = a.x, xr[4 * j + 1] = a.y, xr[4 * j + 2] = a.z, xr[4 * j + 3] = a.w;
        }
#pragma unroll
        for (int j = 0; j < 32; j++) xsum += xr[j];
    }

    while (rg < p.row_groups) {
        const uint32_t first = rg * rows_per_pass + rs * R;
        float acc[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint32_t words[9] = {held.a[r].x, held.a[r].y, held.a[r].z, held.a[r].w, held.b[r].x, held.b[r].y, held.b[r].z, held.b[r].w, held.c[r]};
            const bool odd = held.odd[r] != 0u;
            // the scale is the half at the block's first two bytes, the 32 codes follow it
            const float scale = half_to_float((uint16_t)(odd ? words[0] >> 16 : words[0] & 0xffffu));
            float total = 0.0f;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const uint32_t w = (odd ? words[j + 1] : __funnelshift_r(words[j], words[j + 1], 16)) ^ 0x80808080u;  // q + 128
                total = fmaf(xr[4 * j + 0], (float)(w & 0xffu), total);
                total = fmaf(xr[4 * j + 1], (float)((w >> 8) & 0xffu), total);
                total = fmaf(xr[4 * j + 2], (float)((w >> 16) & 0xffu), total);
                total = fmaf(xr[4 * j + 3], (float)(w >> 24), total);
            }
            acc[r] = scale * (total - 128.0f * xsum);
        }
        rg += stride;
        __builtin_amdgcn_sched_barrier(0);  // the next loads reuse this tile's registers: keep them behind the arithmetic
        float sum = fold_rows<R, G>(acc, lane);  // lane u < R holds row first + u
        if (rg < p.row_groups) load(held, rg);
        if (DEEP) {
            if (u < R) part[parity][wave][u] = sum;
            __syncthreads();  // every wave walks the same passes
            if (u < R) sum = (part[parity][0][u] + part[parity][1][u]) + (part[parity][2][u] + part[parity][3][u]);
            parity ^= 1u;
            if (wave != 0) continue;
        }
        const uint32_t i = first + u;
        if (p.swiglu) {
            const float up = dpp<DPP_QUAD_XOR1>(sum);
            if (u < R && !(u & 1u) && i + 1 < p.N) p.y[i >> 1] = silu(sum) * up;
        } else if (ROPE) {
            rotate_and_store<R>(p, sum, i, u);
        } else if (u < R && i < p.N) {
            p.y[i] = p.residual ? p.residual[i] + sum : sum;
        }
    }
}

// ------------------------------------------------------------ Q6_K, Q5_K, Q3_K -------
//
// 210-, 176- and 110-byte super-blocks; the first and the last leave rows on 2-byte boundaries.  A wave copies the two
// rows it is about to walk into LDS with aligned 128-bit loads -- a row is contiguous, the copy fully coalesced -- and its
// lanes pick the fields out of LDS.  A lane takes 32 weights of a super-block: eight neighbouring elements
// (8j .. 8j + 7) of each of the four 32-element runs of one half.  In all three formats those share one or two 8-byte
// pieces of low bits and one of high bits, and each run has one scale for the eight:
//   Q6_K (crates/neura-precision/src/ggml.rs:394-407, crates/neura-kernel/src/dot.rs:663-797): (d * scale) * (code - 32)
//   Q5_K (ggml.rs:321-335, dot.rs:621-661): d * sc * code - dmin * m
//   Q3_K (ggml.rs:291-306, dot.rs:544-581): (d * (scale - 32)) * (code - 4), the third bit being the code's top bit
// Every run contributes weight * (sum(x * code) - offset * sum(x)) - minimum * sum(x): the stored codes convert to fp32
// with one instruction each, and sum(x) per eight activations is worked out once per workgroup.  The sums run in lane
// order, not in the reference's run order.
__device__ __forceinline__ uint32_t byte_of(uint32_t word, uint32_t at) { return (word >> (8u * at)) & 0xffu; }

template <int ELEMENT>
struct Staged;

template <>
struct Staged<NH_Q6_K> {
    static constexpr uint32_t BYTES = 210u;
    static constexpr float OFFSET = 32.0f;
    static constexpr bool FLOORS = false;
    // codes[g][h]: elements 8j + 4h .. + 3 of run g, one code a byte
    template <typename Word>
    static __device__ __forceinline__ void unit(const uint8_t *block, Word word, uint32_t half, uint32_t j, uint32_t (&codes)[4][2], float (&weight)[4],
                                                float (&floor)[4]) {
        const float d = half_to_float(*reinterpret_cast<const uint16_t *>(block + 208u));
        const uint32_t scales[2] = {word(192u + half * 8u), word(196u + half * 8u)};  // run g, elements 16c ..: byte 2g + c
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint32_t lows = word(half * 64u + 8u * j + 4u * h), highs = word(half * 64u + 32u + 8u * j + 4u * h);
            const uint32_t pairs = word(128u + half * 32u + 8u * j + 4u * h);
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const uint32_t nibbles = ((g & 1) ? highs : lows) >> (g >= 2 ? 4 : 0);
                codes[g][h] = (nibbles & 0x0f0f0f0fu) | (((pairs >> (2 * g)) & 0x03030303u) << 4);
            }
        }
#pragma unroll
        for (int g = 0; g < 4; g++) {
            weight[g] = d * (float)(int8_t)byte_of(scales[g >> 1], 2u * (g & 1) + (j >> 1));
            floor[g] = 0.0f;
        }
    }
};

template <>
struct Staged<NH_Q5_K> {
    static constexpr uint32_t BYTES = 176u;
    static constexpr float OFFSET = 0.0f;
    static constexpr bool FLOORS = true;
    template <typename Word>
    static __device__ __forceinline__ void unit(const uint8_t *block, Word word, uint32_t half, uint32_t j, uint32_t (&codes)[4][2], float (&weight)[4],
                                                float (&floor)[4]) {
        // runs 0..3 of a half are sub-blocks 4 half + t: nibble group 2 half + t / 2, low nibbles for even t
        const uint32_t header = word(0u);
        const float d = half_to_float((uint16_t)header), dmin = half_to_float((uint16_t)(header >> 16));
        const uint32_t s0 = word(4u), s1 = word(8u), s2 = word(12u);  // the twelve scale bytes (ggml.rs:127-136)
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint32_t first = word(48u + half * 64u + 8u * j + 4u * h), second = word(48u + half * 64u + 32u + 8u * j + 4u * h);
            const uint32_t fifths = word(16u + 8u * j + 4u * h);
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const uint32_t nibbles = ((t & 2) ? second : first) >> ((t & 1) ? 4 : 0);
                codes[t][h] = (nibbles & 0x0f0f0f0fu) | (((fifths >> (4u * half + t)) & 0x01010101u) << 4);
            }
        }
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const uint32_t a = byte_of(s0, t), b = byte_of(s1, t), c = byte_of(s2, t);
            const uint32_t sc = half ? ((c & 15u) | ((a >> 6) << 4)) : (a & 63u);
            const uint32_t mn = half ? ((c >> 4) | ((b >> 6) << 4)) : (b & 63u);
            weight[t] = d * (float)sc;
            floor[t] = dmin * (float)mn;
        }
    }
};

template <>
struct Staged<NH_Q3_K> {
    static constexpr uint32_t BYTES = 110u;
    static constexpr float OFFSET = 4.0f;
    static constexpr bool FLOORS = false;
    template <typename Word>
    static __device__ __forceinline__ void unit(const uint8_t *block, Word word, uint32_t half, uint32_t j, uint32_t (&codes)[4][2], float (&weight)[4],
                                                float (&floor)[4]) {
        const float d = half_to_float(*reinterpret_cast<const uint16_t *>(block + 108u));
        const uint32_t lows[2] = {word(96u), word(100u)}, highs = word(104u);  // six-bit scales (ggml.rs:224-229)
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint32_t pairs = word(32u + half * 32u + 8u * j + 4u * h), thirds = word(8u * j + 4u * h);
#pragma unroll
            for (int t = 0; t < 4; t++) codes[t][h] = ((pairs >> (2 * t)) & 0x03030303u) | (((thirds >> (4u * half + t)) & 0x01010101u) << 2);
        }
#pragma unroll
        for (int t = 0; t < 4; t++) {
            // scale 8 half + 2t + c, c = 1 for elements 16 .. 31 of the run: a nibble of byte 2t + c, two bits of byte 8 + (2t + c) % 4
            const uint32_t at = 2u * (t & 1) + (j >> 1);
            const uint32_t low = byte_of(lows[t >> 1], at);
            const uint32_t nibble = half ? (low >> 4) : (low & 15u);
            const uint32_t top = (byte_of(highs, at) >> (2u * (2u * half + (t >> 1)))) & 3u;
            weight[t] = d * ((float)(nibble | (top << 4)) - 32.0f);
            floor[t] = 0.0f;
        }
    }
};

__device__ __forceinline__ uint32_t skew128(uint32_t i) { return i + (i >> 7) * 4; }

// sixteen bytes from `at`, those at and past `end` read as zero without being touched.  Out of line: only the last rows of a
// tensor come here, and the byte loads would otherwise sit in every caller's loop.
__device__ __noinline__ u32x4 piece_before(const uint8_t *at, const uint8_t *end) {
    uint32_t words[4] = {0u, 0u, 0u, 0u};
    for (uint32_t j = 0; j < 16u; j++)
        if (at + j < end) words[j >> 2] |= (uint32_t)at[j] << (8u * (j & 3u));
    u32x4 held = {words[0], words[1], words[2], words[3]};
    return held;
}

template <int ELEMENT, int RB>
__global__ __launch_bounds__(256) void gemv_staged_kernel(GEMV_LEAD_PARAMETERS) {
    GEMV_TAKE_LEAD;
    typedef Staged<ELEMENT> Format;
    extern __shared__ float xs[];  // [RB][slice]; the sums per eight activations; then the raw row slices, two per wave
    __shared__ float red[256];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t split = blockIdx.y;
    const uint32_t blk0 = split * p.blocks_per_split;
    const uint32_t nb = min(p.blocks_per_split, p.nblk - blk0);
    const uint32_t k0 = blk0 * 256u, kn = nb * 256u;
    const uint32_t append_cursor = RB == 1 && p.append_value ? p.rope_cursor[0] : 0u;  // asked for here, wanted at the very end
    // the 16-byte pieces of the two rows `first`, `first + 1` this lane copies: fetched one pair of rows ahead, so the copy
    // of the next pair is in flight while this pair is multiplied (a slice is at most 16 blocks: four pieces a lane and row)
    typedef const __attribute__((address_space(1))) u32x4 *global_uint4;
    u32x4 ahead[2][4];
    uint32_t ahead_lead[2] = {0u, 0u};
    auto fetch = [&](uint32_t first) {
#pragma unroll
        for (int r = 0; r < 2; r++) {
            const uint32_t i = min(first + r, p.N - 1u);
            const uint8_t *matrix_end;
            const uint8_t *src = row_start(p, weight_row(i, p.N, p.swiglu), matrix_end) + (size_t)blk0 * Format::BYTES;
            ahead_lead[r] = (uint32_t)((uintptr_t)src & 15u);
            const uint8_t *from = src - ahead_lead[r];
            const uint32_t bytes = ahead_lead[r] + nb * Format::BYTES;
            const uint32_t pieces = (bytes + 15u) / 16u;
            if (from + 16u * pieces <= matrix_end) {  // the same for every lane of the wave
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const uint32_t c = lane + 64u * k;
                    u32x4 held = {0u, 0u, 0u, 0u};
                    if (c < pieces) held = *(global_uint4)(uintptr_t)(from + 16u * c);
                    ahead[r][k] = held;
                }
            } else {  // the last bytes of the tensor: never read past its end
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const uint32_t c = lane + 64u * k;
                    u32x4 held = {0u, 0u, 0u, 0u};
                    if (c < pieces) held = piece_before(from + 16u * c, matrix_end);
                    ahead[r][k] = held;
                }
            }
        }
    };
    const uint32_t stride = 2u * gridDim.x * 4u;
    uint32_t first = 2u * (blockIdx.x * 4u + wave);
    if (first < p.N) fetch(first);  // on its way while the activations are staged
    // halves of 128 activations sit 16 bytes apart: the lanes of a wave read eight of them at once
    const uint32_t xstride = skew128(p.blocks_per_split * 256u);
    for (uint32_t b = 0; b < RB; b++) {
        stage_row(p.x + (size_t)b * p.K, p.K, k0, kn, p.norm_w, p.eps, xs + b * xstride, red, [](uint32_t i) { return skew128(i); });
    }
    __syncthreads();
    // what the codes' offset (or a run's minimum) multiplies, once for all rows: per unit and run the sum of the eight
    // activations, times the offset where the format has one
    float *const sums = xs + RB * xstride;
    const uint32_t sstride = p.blocks_per_split * 32u;
    for (uint32_t b = 0; b < RB; b++)
        for (uint32_t q = tid; q < nb * 32u; q += 256u) {
            const uint32_t u = q >> 2, g = q & 3u;
            const float4 *at = reinterpret_cast<const float4 *>(xs + b * xstride + skew128((u >> 2) * 128u) + g * 32u + 8u * (u & 3u));
            const float4 lo = at[0], hi = at[1];
            const float total = ((lo.x + lo.y) + (lo.z + lo.w)) + ((hi.x + hi.y) + (hi.z + hi.w));
            sums[b * sstride + q] = Format::FLOORS ? total : -Format::OFFSET * total;
        }
    __syncthreads();
    const uint32_t raw_stride = p.chunks_per_row * 16u;  // bytes of one staged row slice
    uint8_t *const mine = reinterpret_cast<uint8_t *>(sums + RB * sstride) + (size_t)wave * 2u * raw_stride;
    const uint32_t units = nb * 8u;

    for (; first < p.N; first += stride) {
        uint32_t lead[2];
#pragma unroll
        for (int r = 0; r < 2; r++) {
            lead[r] = ahead_lead[r];
#pragma unroll
            for (int k = 0; k < 4; k++)
                if ((lane + 64u * k) < p.chunks_per_row) *reinterpret_cast<u32x4 *>(mine + r * raw_stride + 16u * (lane + 64u * k)) = ahead[r][k];
        }
        if (first + stride < p.N) fetch(first + stride);
        __builtin_amdgcn_wave_barrier();  // LDS serves a wave's accesses in order: the reads below see these writes

        float acc[2][RB];
#pragma unroll
        for (int r = 0; r < 2; r++)
#pragma unroll
            for (int b = 0; b < RB; b++) acc[r][b] = 0.0f;
        for (uint32_t u = lane; u < units; u += 64u) {
            const uint32_t blk = u >> 3, half = (u >> 2) & 1u, j = u & 3u;
            float4 xv[RB][4][2];
            float base[RB][4];
#pragma unroll
            for (int b = 0; b < RB; b++) {
                const float4 held = *reinterpret_cast<const float4 *>(sums + b * sstride + 4u * u);
                base[b][0] = held.x, base[b][1] = held.y, base[b][2] = held.z, base[b][3] = held.w;
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const float4 *at = reinterpret_cast<const float4 *>(xs + b * xstride + skew128(blk * 256u + half * 128u) + g * 32u + 8u * j);
                    xv[b][g][0] = at[0], xv[b][g][1] = at[1];
                }
            }
#pragma unroll
            for (int r = 0; r < 2; r++) {
                const uint8_t *block = mine + r * raw_stride + lead[r] + blk * Format::BYTES;
                // a block sits on a 2-byte boundary: its words are cut out of the aligned words around them (LDS serves a
                // misaligned read at a fraction of its rate)
                const uint32_t off = Format::BYTES % 4u ? (uint32_t)(uintptr_t)block & 3u : 0u;
                const uint32_t *words = reinterpret_cast<const uint32_t *>(block - off);
                auto word = [&](uint32_t at) {
                    if (Format::BYTES % 4u == 0) return words[at / 4u];
                    return __builtin_amdgcn_alignbit(words[at / 4u + 1u], words[at / 4u], off * 8u);
                };
                uint32_t codes[4][2];
                float weight[4], floor[4];
                Format::unit(block, word, half, j, codes, weight, floor);
#pragma unroll
                for (int g = 0; g < 4; g++) {
#pragma unroll
                    for (int b = 0; b < RB; b++) {
                        // the codes go to fp32 as they are stored, one conversion each; their offset came with the sum
                        float dot = Format::FLOORS ? 0.0f : base[b][g];
#pragma unroll
                        for (int h = 0; h < 2; h++) {
                            const uint32_t c = codes[g][h];
                            dot = fmaf(xv[b][g][h].x, (float)(c & 0xffu), dot);
                            dot = fmaf(xv[b][g][h].y, (float)((c >> 8) & 0xffu), dot);
                            dot = fmaf(xv[b][g][h].z, (float)((c >> 16) & 0xffu), dot);
                            dot = fmaf(xv[b][g][h].w, (float)(c >> 24), dot);
                        }
                        acc[r][b] = fmaf(weight[g], dot, acc[r][b]);
                        if (Format::FLOORS) acc[r][b] = fmaf(-floor[g], base[b][g], acc[r][b]);
                    }
                }
            }
        }
#pragma unroll
        for (int r = 0; r < 2; r++)
#pragma unroll
            for (int b = 0; b < RB; b++) acc[r][b] = wave_sum(acc[r][b]);
        if (lane == 0) publish<2, RB>(p, first, split, acc);
        if (RB == 1 && p.append_value && lane < 2 && first + lane < p.N) {
            // a value projection of one token: its rows (+ bias) go into the value state at the cursor as halves, as
            // value_append_kernel would cast them
            const uint32_t n = first + lane;
            const float sum = lane ? acc[1][0] : acc[0][0];
            const float value = p.bias[0] ? sum + p.bias[0][n] : sum;
            const uint32_t slot = p.rope_ring ? append_cursor % p.rope_ring : append_cursor;
            if (slot >= p.rope_capacity) atomicMax(p.refusal, (uint32_t)REFUSAL_ORIGIN);
            else state_store(p.rope_v, p.rope_element, ((uint64_t)(n / p.rope_width) * p.rope_capacity + slot) * p.rope_width + n % p.rope_width, value);
        }
        __builtin_amdgcn_wave_barrier();  // the next rows overwrite the staged ones
    }
}

// ------------------------------------------------------------------- Q4_K on MFMA --------
//
// The same product with the multiply-adds on the matrix cores, in exact integer arithmetic.
// A wave owns a tile of 16 output rows; lane (r, g) = (lane % 16, lane / 16) loads the header
// and the 32 nibble bytes of 64-element group g of one super-block of row r.
// v_mfma_i32_4x4x4_16B_i8 runs sixteen independent 4x4x4 products, one per four neighbouring
// lanes: lane j of a quad supplies column j of B (four weights of its own row and group, one per
// byte) and row j of A (four activations of column j), and receives C[0..3][j] -- the dot
// products of its own weights with four activation columns.  Sums never mix groups, and the
// lane that holds a partial sum also holds the block header that scales it.
//
// Unpacking is two masks and a shift per 8 weights: word & 0x0f0f0f0f is four weights of
// sub-block 2g, (word >> 4) & 0x0f0f0f0f four of sub-block 2g+1, each already one per byte.
// The activations are staged once per workgroup in LDS as integers: a row slice is scaled by a
// power of two so its largest magnitude lies in [2^29, 2^30), rounded to an integer, and cut
// into four signed base-256 digits (the four columns of the A operand), so every activation
// within 2^-6 of the row's largest keeps its whole fp32 mantissa and every product and sum on the matrix cores is exact.
// Per super-block, lane and activation row: 8 MFMAs over the low nibbles and 8 over the high
// nibbles; the eight integer sums are joined in fp32, weighed by d*sc, and the minimums take the
// integer sum of the sub-block's activations: d*sc*sum(q*x) - dmin*m*sum(x), the reference's
// value (crates/neura-kernel/src/dot.rs:583-619) regrouped per sub-block.

typedef int i32x4 __attribute__((ext_vector_type(4)));

struct MfmaParams {
    const uint8_t *W[3];
    uint32_t end[3];
    const float *x;
    float *y;
    const float *residual;
    const float *norm_w;
    float *partial;
    uint32_t N, K, row_bytes;
    uint32_t nblk, slice_blocks, splits;
    uint32_t rows;   // activation rows of this launch, 1..4
    uint32_t tiles;  // 16-row tiles
    int32_t swiglu;
    float eps;
    // the rotation folded into a q|k|v product of several planes, one token each (gemv_q4k_mfma32_kernel<.., ROPE>): activation
    // row b is plane b, whose token sits at rope_cursor[b]
    const float *rope_cosines, *rope_sines, *bias[3];
    const uint32_t *rope_cursor;
    uint16_t *rope_k, *rope_v;
    uint32_t *refusal;
    uint32_t rope_width, rope_q_rows, rope_k_rows, rope_capacity, rope_positions, rope_ring;
    int32_t rope_element;
};

// What a wave of the matrix-core products needs before its first loads, as leading plain arguments the hardware hands over in
// scalar registers when it starts the wave (the activation rows ride above the blocks a row, the K slices above the blocks a
// slice); they take the place of the same members of the parameter block, whose other members are loaded as they come to use.
#define MFMA_LEAD_PARAMETERS                                                                                                                          \
    const uint8_t *lead_w0, const uint8_t *lead_w1, const uint8_t *lead_w2, const float *lead_x, uint32_t lead_row_bytes, uint32_t lead_nblk_rows,      \
        uint32_t lead_slice_splits, uint32_t lead_tiles, uint32_t lead_end0, uint32_t lead_end1, MfmaParams rest
#define MFMA_LEAD(p)                                                                                                                                   \
    (p).W[0], (p).W[1], (p).W[2], (p).x, (p).row_bytes, (p).nblk | ((p).rows << 16), (p).slice_blocks | ((p).splits << 16), (p).tiles, (p).end[0], (p).end[1], (p)
#define MFMA_TAKE_LEAD                                                                                                                                 \
    MfmaParams p = rest;                                                                                                                               \
    p.W[0] = lead_w0, p.W[1] = lead_w1, p.W[2] = lead_w2, p.x = lead_x, p.row_bytes = lead_row_bytes, p.tiles = lead_tiles;                             \
    p.nblk = lead_nblk_rows & 0xffffu, p.rows = lead_nblk_rows >> 16, p.K = 256u * (lead_nblk_rows & 0xffffu);                                          \
    p.slice_blocks = lead_slice_splits & 0xffffu, p.splits = lead_slice_splits >> 16, p.end[0] = lead_end0, p.end[1] = lead_end1

struct MfmaUnit {
    u32x4 hdr, qa, qb;
};


// KS waves share one tile (each takes every KS-th super-block of the slice); NW waves per
// workgroup; P activation rows; D super-blocks in flight per wave (the loads run ahead of the
// arithmetic across tile boundaries, and the first ones are issued before the activations are staged).

// Digit planes of four elements: plane[0] holds their most significant digits (element e in byte e), plane[3] the least.
__device__ __forceinline__ void digit_planes(uint32_t d0, uint32_t d1, uint32_t d2, uint32_t d3, uint32_t (&plane)[4]) {
    const uint32_t lo01 = __builtin_amdgcn_perm(d1, d0, 0x05010400u), hi01 = __builtin_amdgcn_perm(d1, d0, 0x07030602u);
    const uint32_t lo23 = __builtin_amdgcn_perm(d3, d2, 0x05010400u), hi23 = __builtin_amdgcn_perm(d3, d2, 0x07030602u);
    plane[3] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
    plane[2] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
    plane[1] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
    plane[0] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
}

template <int KS, int NW, int P, int D>
__global__ __launch_bounds__(NW * 64) void gemv_q4k_mfma_kernel(MFMA_LEAD_PARAMETERS) {
    MFMA_TAKE_LEAD;
    extern __shared__ uint32_t xop[];  // [block][16 steps][4 groups][4 P digit columns] of 4 bytes; then sums; then tile partials
    __shared__ float red[256];
    __shared__ uint32_t wave_top[NW];
    __shared__ float unscale[P];
    constexpr uint32_t NT = NW * 64, TPW = NW / KS, NCW = 4 * P;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t split = blockIdx.y;
    const uint32_t blk0 = split * p.slice_blocks;
    const uint32_t nb = min(p.slice_blocks, p.nblk - blk0);
    const uint32_t k0 = blk0 * 256u, kn = nb * 256u;
    float *xsum = reinterpret_cast<float *>(xop + (size_t)p.slice_blocks * 64u * NCW);  // [block][group][P][2 sub-blocks]
    float *part = xsum + (size_t)p.slice_blocks * 8u * P;                               // [2][TPW][KS][P][16]

    const uint32_t r = lane & 15u, g = lane >> 4;
    const uint32_t ks = KS == 1 ? 0u : wave % KS, tslot = wave / KS;
    const uint32_t stride = gridDim.x * TPW;
    typedef const __attribute__((address_space(1))) u32x4 *global_uint4;
    // first byte this lane reads of super-block 0 of the slice in `tile`
    // selects over scalars: indexing the parameter arrays by a computed segment would copy them to scratch memory
    const uint8_t *const w0 = p.W[0], *const w1 = p.W[1], *const w2 = p.W[2];
    const uint32_t end0 = p.end[0], end1 = p.end[1];
    const uint8_t *const swiglu_base = r < 8u ? w0 : w1;
    const bool gated = p.swiglu != 0;
    const uint32_t row_bytes = p.row_bytes;
    // captured by value: a by-reference closure would select between the addresses of w0, w1, w2 in memory
    auto lane_row = [w0, w1, w2, end0, end1, swiglu_base, gated, row_bytes, blk0, g, r](uint32_t tile) -> const uint8_t * {
        const uint8_t *rowp;
        if (gated) {
            rowp = swiglu_base + (size_t)(tile * 8u + (r & 7u)) * row_bytes;
        } else {
            const uint32_t n0 = tile * 16u;
            const bool in0 = n0 < end0, in1 = n0 < end1;
            const uint8_t *matrix = in0 ? w0 : (in1 ? w1 : w2);
            const uint32_t before = in0 ? 0u : (in1 ? end0 : end1);
            rowp = matrix + (size_t)(n0 - before + r) * row_bytes;
        }
        return rowp + (size_t)blk0 * 144u + g * 32u;
    };
    // The loads run D super-blocks ahead of the arithmetic: (ahead_base, ahead_b) is the next one to fetch.  Every fetch
    // issues its three loads, whatever is left: past the last super-block of this wave the last one is fetched again and
    // never used.  A fetch that could be skipped would make the compiler, which counts the loads in flight along every
    // path, wait for the newest load before each use of the oldest, and the ring would hide nothing.
    MfmaUnit ring[D];
    uint32_t ahead_base = blockIdx.x * TPW, ahead_b = ks;
    const uint8_t *ahead_row = lane_row(min(ahead_base + tslot, p.tiles - 1u));
    auto fetch = [&](MfmaUnit &u) {
        const uint8_t *at = ahead_row + (size_t)ahead_b * 144u;
        u.hdr = *(global_uint4)(uintptr_t)(at - g * 32u);
        u.qa = *(global_uint4)(uintptr_t)(at + 16u);
        u.qb = *(global_uint4)(uintptr_t)(at + 32u);
        if (ahead_b + KS < nb) {
            ahead_b += KS;
        } else if (ahead_base + stride + tslot < p.tiles) {
            ahead_b = ks;
            ahead_base += stride;
            ahead_row = lane_row(ahead_base + tslot);
        }
    };
#pragma unroll
    for (int i = 0; i < D; i++) fetch(ring[i]);

    // ---- activations -> integer digits in operand order
    // A thread takes chunks of 8 activations (8 consecutive chunks = one 64-element group).  When the slice is at most
    // four chunks per thread, every load goes out before the first value is used and the row is read once; a deeper
    // slice is walked twice (largest magnitude, then digits) with its loads one after the other.
    const uint32_t chunks = nb * 32u;
    const bool resident = chunks <= 4u * NT && (!p.norm_w || p.K == kn);
    for (uint32_t row = 0; row < P; row++) {
        const float *xr = p.x + (size_t)min(row, p.rows - 1u) * p.K;
        float t[4][8];
        float rms = 1.0f;
        uint32_t top = 0;  // largest magnitude as bits: infinities and NaNs sort above every finite value
        if (resident) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t q = tid + NT * j;
                float4 a = make_float4(0.f, 0.f, 0.f, 0.f), b = a;
                if (q < chunks) a = *reinterpret_cast<const float4 *>(xr + k0 + 8u * q), b = *reinterpret_cast<const float4 *>(xr + k0 + 8u * q + 4u);
                t[j][0] = a.x, t[j][1] = a.y, t[j][2] = a.z, t[j][3] = a.w, t[j][4] = b.x, t[j][5] = b.y, t[j][6] = b.z, t[j][7] = b.w;
            }
            if (p.norm_w) {
                // the whole row is in registers: sum of squares (thread order differs from the reference's strided sum), then scale and weight
                float4 wa[4], wb[4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const uint32_t q = tid + NT * j;
                    wa[j] = wb[j] = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (q < chunks) wa[j] = *reinterpret_cast<const float4 *>(p.norm_w + 8u * q), wb[j] = *reinterpret_cast<const float4 *>(p.norm_w + 8u * q + 4u);
                }
                float square = 0.0f;
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int i = 0; i < 8; i++) square = __fadd_rn(square, __fmul_rn(t[j][i], t[j][i]));
                square = wave_sum(square);
                if (lane == 0) red[wave] = square;
                __syncthreads();
                float total = 0.0f;
#pragma unroll
                for (int w = 0; w < NW; w++) total += red[w];
                __syncthreads();
                rms = rms_scale_of(total, p.K, p.eps);
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const float w[8] = {wa[j].x, wa[j].y, wa[j].z, wa[j].w, wb[j].x, wb[j].y, wb[j].z, wb[j].w};
#pragma unroll
                    for (int i = 0; i < 8; i++) t[j][i] = __fmul_rn(__fmul_rn(t[j][i], rms), w[i]);
                }
            }
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int i = 0; i < 8; i++) top = max(top, __builtin_bit_cast(uint32_t, t[j][i]) & 0x7fffffffu);
        } else {
            if (p.norm_w) rms = rms_scale(xr, p.K, p.eps, red);
            for (uint32_t i = tid; i < kn; i += NT) {
                float value = xr[k0 + i];
                if (p.norm_w) value = __fmul_rn(__fmul_rn(value, rms), p.norm_w[k0 + i]);
                top = max(top, __builtin_bit_cast(uint32_t, value) & 0x7fffffffu);
            }
        }
#pragma unroll
        for (int offset = 32; offset > 0; offset >>= 1) top = max(top, (uint32_t)__shfl_xor((int)top, offset, 64));
        if (lane == 0) wave_top[wave] = top;
        __syncthreads();
        top = 0;
#pragma unroll
        for (int w = 0; w < NW; w++) top = max(top, wave_top[w]);
        __syncthreads();  // the next row overwrites wave_top
        // a power of two that puts the largest magnitude in [2^29, 2^30)
        const uint32_t raw_exponent = top >> 23;
        const uint32_t exponent = min(max(raw_exponent, 30u), 254u);
        const float scale = __builtin_bit_cast(float, (283u - exponent) << 23);
        if (tid == 0) unscale[row] = raw_exponent == 255u ? __builtin_bit_cast(float, 0x7fc00000u) : __builtin_bit_cast(float, (exponent - 29u) << 23);
        // one chunk: four signed base-256 digits of each rounded activation, most significant first, one byte per element
        auto stage = [&](uint32_t q, bool held, const float (&v)[8]) {
            float total = 0.0f;
            uint32_t word[2][4];
#pragma unroll
            for (int h = 0; h < 2; h++) {
                uint32_t digits[4];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float rounded = rintf(v[4 * h + i] * scale);
                    total += rounded;
                    digits[i] = signed_digits((int)rounded);
                }
                digit_planes(digits[0], digits[1], digits[2], digits[3], word[h]);
            }
            // sum of the 32 activations of this chunk's sub-block: 4 chunks = 4 neighbouring lanes
            total += dpp<DPP_QUAD_XOR1>(total);
            total += dpp<DPP_QUAD_XOR2>(total);
            if (held) {
                // chunk q = elements 8m..8m+7 of half `upper` of group g: nibble words 2m, 2m+1 of that half
                const uint32_t b = q >> 5, g = (q >> 3) & 3u, upper = (q >> 2) & 1u, step = 8u * upper + 2u * (q & 3u);
                uint4 *slot = reinterpret_cast<uint4 *>(xop + ((size_t)(b * 16u + step) * 4u + g) * NCW + 4u * row);
                slot[0] = make_uint4(word[0][0], word[0][1], word[0][2], word[0][3]);
                slot[NCW] = make_uint4(word[1][0], word[1][1], word[1][2], word[1][3]);  // the next step: 4 groups * NCW words further
                if ((q & 3u) == 0) xsum[((size_t)(b * 4u + g) * P + row) * 2u + upper] = total;
            }
        };
        if (resident) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if (NT * j >= chunks) break;  // uniform over the workgroup
                stage(tid + NT * j, tid + NT * j < chunks, t[j]);
            }
        } else {
            for (uint32_t first = 0; first < chunks; first += NT) {
                const uint32_t q = first + tid;
                const bool held = q < chunks;
                float v[8];
                if (held) {
                    const float4 a = *reinterpret_cast<const float4 *>(xr + k0 + 8u * q), b = *reinterpret_cast<const float4 *>(xr + k0 + 8u * q + 4u);
                    v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w, v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
                    if (p.norm_w) {
                        const float4 wa = *reinterpret_cast<const float4 *>(p.norm_w + k0 + 8u * q), wb = *reinterpret_cast<const float4 *>(p.norm_w + k0 + 8u * q + 4u);
                        const float w[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
#pragma unroll
                        for (int i = 0; i < 8; i++) v[i] = __fmul_rn(__fmul_rn(v[i], rms), w[i]);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 8; i++) v[i] = 0.0f;
                }
                stage(q, held, v);
            }
        }
    }
    __syncthreads();

    const ScaleLane lane_scales = scale_lane(g);
    // lane i of a quad supplies digit column i of an activation row
    const uint32_t *xlane = xop + (size_t)g * NCW + (lane & 3u);
    const float2 *slane = reinterpret_cast<const float2 *>(xsum) + (size_t)g * P;

    float acc[P];
#pragma unroll
    for (int pass = 0; pass < P; pass++) acc[pass] = 0.0f;
    auto compute = [&](const MfmaUnit &u, uint32_t b) {
        const uint32_t *xb = xlane + (size_t)b * 64u * NCW;
        const uint32_t words[8] = {u.qa.x, u.qa.y, u.qa.z, u.qa.w, u.qb.x, u.qb.y, u.qb.z, u.qb.w};
        i32x4 cl[P], ch[P];
#pragma unroll
        for (int pass = 0; pass < P; pass++) cl[pass] = ch[pass] = i32x4{0, 0, 0, 0};
#pragma unroll
        for (int w = 0; w < 8; w++) {
            const int low = (int)(words[w] & 0x0f0f0f0fu), high = (int)((words[w] >> 4) & 0x0f0f0f0fu);
#pragma unroll
            for (int pass = 0; pass < P; pass++) {
                const int xl = (int)xb[(size_t)w * 4u * NCW + 4 * pass], xh = (int)xb[(size_t)(8 + w) * 4u * NCW + 4 * pass];
                cl[pass] = __builtin_amdgcn_mfma_i32_4x4x4i8(xl, low, cl[pass], 0, 0, 0);
                ch[pass] = __builtin_amdgcn_mfma_i32_4x4x4i8(xh, high, ch[pass], 0, 0, 0);
            }
        }
        half2_t sc, mn;
        scale_pairs(u.hdr, lane_scales, sc, mn);                  // integers as half subnormals: value * 2^-24
        const half2_t dd = __builtin_bit_cast(half2_t, u.hdr.x);  // (d, dmin)
        const float d24 = (float)dd.x * 16777216.0f, m24 = (float)dd.y * 16777216.0f;
        const float s0 = d24 * (float)sc.x, s1 = d24 * (float)sc.y, m0 = m24 * (float)mn.x, m1 = m24 * (float)mn.y;
#pragma unroll
        for (int pass = 0; pass < P; pass++) {
            const float fl = fmaf(fmaf(fmaf((float)cl[pass][0], 256.0f, (float)cl[pass][1]), 256.0f, (float)cl[pass][2]), 256.0f, (float)cl[pass][3]);
            const float fh = fmaf(fmaf(fmaf((float)ch[pass][0], 256.0f, (float)ch[pass][1]), 256.0f, (float)ch[pass][2]), 256.0f, (float)ch[pass][3]);
            const float2 sums = slane[(size_t)b * 4u * P + pass];
            acc[pass] += fmaf(s0, fl, s1 * fh) - fmaf(m0, sums.x, m1 * sums.y);
        }
    };

    // one tile of this workgroup's round is finished by this wave: publish it (with its K partners) and start the next
    uint32_t parity = 0, base = blockIdx.x * TPW, b = ks;
    while (base < p.tiles) {
#pragma unroll
        for (int slot = 0; slot < D; slot++) {
            if (base >= p.tiles) break;
            const uint32_t tile = base + tslot;
            const bool live = tile < p.tiles;
            compute(ring[slot], b);  // a wave past the last tile multiplies what it fetched again; nothing of it is published
            fetch(ring[slot]);
            b += KS;
            if (b < nb) continue;
                // lane (r, g) holds group g's share of output row r for every activation row; the four groups are summed across lanes
                float value[P];
        #pragma unroll
                for (int j = 0; j < P; j++) {
                    float v = acc[j];
                    v += __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));  // lane ^ 16
                    v += __shfl_xor(v, 32, 64);
                    value[j] = v * unscale[j];
                }
                auto publish_one = [&](uint32_t t, uint32_t rr, uint32_t brow, float total, float up) {
                    // (t, rr): tile and row inside it; `up` is the up-projection partner when swiglu folds here
                    if (p.splits > 1) {
                        const uint32_t n = p.swiglu ? (rr < 8u ? t * 8u + rr : p.N / 2 + t * 8u + (rr - 8u)) : t * 16u + rr;
                        p.partial[((size_t)split * p.rows + brow) * p.N + n] = total;
                    } else if (p.swiglu) {
                        if (rr < 8u) p.y[(size_t)brow * (p.N / 2) + t * 8u + rr] = silu(total) * up;
                    } else {
                        const size_t at = (size_t)brow * p.N + t * 16u + rr;
                        p.y[at] = p.residual ? p.residual[at] + total : total;
                    }
                };
                if (KS == 1) {
        #pragma unroll
                    for (int j = 0; j < P; j++) {
                        const float up = dpp<DPP_ROW_ROR8>(value[j]);
                        if (live && g == 0 && (uint32_t)j < p.rows) publish_one(tile, r, (uint32_t)j, value[j], up);
                    }
                } else {
                    float *mine = part + ((size_t)(parity * TPW + tslot) * KS + ks) * P * 16u;
        #pragma unroll
                    for (int j = 0; j < P; j++)
                        if (g == 0) mine[j * 16u + r] = live ? value[j] : 0.0f;
                    __syncthreads();
                    for (uint32_t o = tid; o < TPW * p.rows * 16u; o += NT) {
                        const uint32_t rr = o & 15u, brow = (o >> 4) % p.rows, ts = (o >> 4) / p.rows;
                        const float *from = part + (size_t)(parity * TPW + ts) * KS * P * 16u + brow * 16u;
                        float total = 0.0f, up = 0.0f;
        #pragma unroll
                        for (int k = 0; k < KS; k++) total += from[(size_t)k * P * 16u + rr];
                        if (p.swiglu && p.splits == 1 && rr < 8u) {
        #pragma unroll
                            for (int k = 0; k < KS; k++) up += from[(size_t)k * P * 16u + rr + 8u];
                        }
                        if (base + ts < p.tiles) publish_one(base + ts, rr, brow, total, up);
                    }
                }
            // the next tile of this wave
#pragma unroll
            for (int pass = 0; pass < P; pass++) acc[pass] = 0.0f;
            b = ks;
            base += stride;
            parity ^= 1u;
        }
    }
}

// The Q4_K product on 32 x 32 x 32 integer MFMAs (v_mfma_i32_32x32x32_i8): weights are the B operand -- lane (n, q) =
// (lane % 32, lane / 32) supplies 16 nibbles of row n, one per byte, straight from its 16-byte load of half a group --
// and the digit planes of up to eight activation rows are the A operand (row m = 4 * activation row + plane, read from
// LDS as they were staged).  C comes back with lane n holding the sums of ITS OWN weight row against every plane: no
// sum ever crosses lanes, the lane that holds a sum holds the header that scales it, and one instruction multiplies
// 1024 weights by eight activation rows.  Against the vector kernel that is about half the vector instructions per
// weight for one activation row, and eight rows cost little more than one.  Digits are scaled per sub-block of 32
// (no pass over the row).  Four waves share a tile of 32 rows, each walking every fourth super-block; their partial
// sums meet lane by lane in LDS.  J: row pairs of C in use (activation rows 2j + q), NW: waves per workgroup.
typedef int i32x16 __attribute__((ext_vector_type(16)));

struct Tile32Unit {
    u32x4 hdr, g[4];
};

// ROPE: a q|k|v product of several planes, one token each, with the rotation, the biases and the cache append in its epilogue
// (crates/neura-kernel/src/task/rope.rs:95-122, crates/neura-decoder/src/cache.rs:347-348).  A tile then holds sixteen
// channels c.. of a head in its rows 0..15 and their partners c + width/2.. in its rows 16..31, so the lane 16 further holds the
// number a rotated output needs beside its own; q rows go to y, k rows rotated and v rows as they are into the states at the
// plane's cursor, as rope_append_kernel would leave them (the same table of cosines and sines, the same three roundings).
template <int J, int NW, int KS, bool ROPE = false>
__global__ __launch_bounds__(NW * 64, NW == 16 ? 4 : 3) void gemv_q4k_mfma32_kernel(MFMA_LEAD_PARAMETERS) {  // second bound: waves per SIMD
    MFMA_TAKE_LEAD;
    static_assert(!ROPE || J == 4, "the rotation is folded into the product of five to eight planes");

    constexpr uint32_t M8 = 8 * J, R2 = 2 * J, TPW = NW / KS, NT = NW * 64;
    constexpr bool STAGED = J == 1;  // raw blocks through LDS; with eight activation rows the digits leave no room for them
    extern __shared__ __attribute__((aligned(16))) uint32_t staged[];  // digits [block][sub-block][q][M8] of 16 bytes
    __shared__ float red[256];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // rows too deep to stage whole are cut into K slices (blockIdx.y), whose partial sums a second kernel folds
    const uint32_t split = blockIdx.y, blk0 = split * p.slice_blocks;
    const uint32_t nb = min(p.slice_blocks, p.nblk - blk0);
    const uint32_t k0 = blk0 * 256u;
    float2 *const sums = reinterpret_cast<float2 *>(staged + (size_t)nb * 64u * M8);  // [block][sub-block][R2]: (unscale, sub-block sum * unscale)
    float *const part = reinterpret_cast<float *>(sums + (size_t)nb * 8u * R2);        // [2][TPW][KS][J][64]
    u32x4 *const raw = reinterpret_cast<u32x4 *>(part + (size_t)2 * TPW * KS * J * 64u) + (size_t)wave * 288u;  // per wave: one super-block of the tile, raw
    typedef const __attribute__((address_space(1))) u32x4 *global_uint4;

    // ---- activations -> digit planes, 16 elements (half a sub-block) per thread; a row takes at most 256 threads
    // (K <= 4096), so a workgroup of sixteen waves stages four rows side by side
    constexpr uint32_t GROUPS = NT / 256u;
    const uint32_t chunks = nb * 16u;
    const uint32_t rg = tid >> 8, t = tid & 255u;
    // a thread's sixteen numbers of row `row0 + rg`, asked for whatever the row and the chunk (past them the last row's, the
    // last chunk's, dropped by the caller): the next rows' are on their way while these rows become digits
    auto fetch_rows = [&](uint32_t row0, float4 (&into)[4]) {
        const float *xr = p.x + (size_t)min(row0 + rg, p.rows - 1u) * p.K + k0 + 16u * min(t, chunks - 1u);
#pragma unroll
        for (int c = 0; c < 4; c++) into[c] = *reinterpret_cast<const float4 *>(xr + 4u * c);
    };
    float4 ahead[4], w[4];
    fetch_rows(0u, ahead);
    if (p.norm_w) {
#pragma unroll
        for (int c = 0; c < 4; c++) w[c] = *reinterpret_cast<const float4 *>(p.norm_w + k0 + 16u * min(t, chunks - 1u) + 4u * c);
    }
#pragma unroll
    for (uint32_t row0 = 0; row0 < R2; row0 += GROUPS) {
        const uint32_t row = row0 + rg;  // groups past the staged rows only keep the barriers company
        const bool real = row < p.rows;
        {
            const bool held = t < chunks && row < R2;
            float v[16];
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const float4 a = held && real ? ahead[c] : make_float4(0.f, 0.f, 0.f, 0.f);
                v[4 * c] = a.x, v[4 * c + 1] = a.y, v[4 * c + 2] = a.z, v[4 * c + 3] = a.w;
            }
            if (row0 + GROUPS < R2) fetch_rows(row0 + GROUPS, ahead);
            if (p.norm_w) {
                // the whole row is in registers across its 256 threads
                float square = 0.0f;
#pragma unroll
                for (int i = 0; i < 16; i++) square = __fadd_rn(square, __fmul_rn(v[i], v[i]));
                square = wave_sum(square);
                if (lane == 0) red[wave] = square;
                __syncthreads();
                const float total = (red[4u * rg] + red[4u * rg + 1u]) + (red[4u * rg + 2u] + red[4u * rg + 3u]);
                __syncthreads();  // red is reused by the next rows
                const float rms = rms_scale_of(total, p.K, p.eps);
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    v[4 * c] = __fmul_rn(__fmul_rn(v[4 * c], rms), w[c].x), v[4 * c + 1] = __fmul_rn(__fmul_rn(v[4 * c + 1], rms), w[c].y);
                    v[4 * c + 2] = __fmul_rn(__fmul_rn(v[4 * c + 2], rms), w[c].z), v[4 * c + 3] = __fmul_rn(__fmul_rn(v[4 * c + 3], rms), w[c].w);
                }
            }
            uint32_t top = 0;  // largest magnitude as bits: infinities and NaNs sort above every finite value
#pragma unroll
            for (int i = 0; i < 16; i++) top = max(top, __builtin_bit_cast(uint32_t, v[i]) & 0x7fffffffu);
            top = max(top, (uint32_t)dpp_int<DPP_QUAD_XOR1>((int)top));  // the other half of the sub-block
            const uint32_t raw_exponent = top >> 23;
            const uint32_t exponent = min(max(raw_exponent, 30u), 254u);
            const float scale = __builtin_bit_cast(float, (283u - exponent) << 23);
            const float unscale = raw_exponent == 255u ? __builtin_bit_cast(float, 0x7fc00000u) : __builtin_bit_cast(float, (exponent - 29u) << 23);
            float total = 0.0f;
            uint32_t plane[4][4];
#pragma unroll
            for (int c = 0; c < 4; c++) {
                uint32_t each[4], out[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float rounded = rintf(v[4 * c + e] * scale);
                    total += rounded;
                    each[e] = signed_digits((int)rounded);
                }
                digit_planes(each[0], each[1], each[2], each[3], out);
#pragma unroll
                for (int d = 0; d < 4; d++) plane[d][c] = out[d];
            }
            total += dpp<DPP_QUAD_XOR1>(total);
            if (held) {
                const uint32_t sub = t >> 1, q = t & 1u;  // sub-block of the row (block * 8 + sub-block), half of it
                u32x4 *at = reinterpret_cast<u32x4 *>(staged) + ((size_t)sub * 2u + q) * M8 + 4u * row;
#pragma unroll
                for (int d = 0; d < 4; d++) at[d] = real ? u32x4{plane[d][0], plane[d][1], plane[d][2], plane[d][3]} : u32x4{0u, 0u, 0u, 0u};
                if (q == 0) sums[(size_t)sub * R2 + row] = real ? make_float2(unscale, total * unscale) : make_float2(0.0f, 0.0f);
            }
        }
    }
    __syncthreads();

    // ---- tiles of 32 weight rows
    const uint32_t n = lane & 31u, q = lane >> 5;
    const uint32_t ts = wave / KS, ks = wave % KS;
    const uint32_t count = ks < nb ? (nb - ks + KS - 1u) / KS : 0u;  // super-blocks ks, ks + KS, ...
    const uint32_t last_step = count ? count - 1u : 0u;
    const uint8_t *const w0 = p.W[0], *const w1 = p.W[1], *const w2 = p.W[2];
    const uint32_t end0 = p.end[0], end1 = p.end[1];
    const bool gated = p.swiglu != 0;
    const u32x4 *const a_lane = reinterpret_cast<const u32x4 *>(staged) + (size_t)q * M8 + (lane & 31u);
    const bool a_held = (lane & 31u) < M8;
    uint32_t parity = 0;
    for (uint32_t base = blockIdx.x * TPW; base < p.tiles; base += gridDim.x * TPW) {
        const uint32_t tile = base + ts;
        const bool live = tile < p.tiles;
        const uint32_t at_tile = live ? tile : p.tiles - 1u;
        // first byte of row `r` of the tile
        const uint32_t r0 = at_tile * 32u;
        const bool in0 = r0 < end0, in1 = r0 < end1;
        const uint8_t *const plain_base = (in0 ? w0 : (in1 ? w1 : w2)) + (size_t)(r0 - (in0 ? 0u : (in1 ? end0 : end1))) * p.row_bytes;
        // ROPE: the tile's first output row -- channel c0 of a head -- and what its rows 16..31 lie further (half a head)
        const uint32_t rope_tiles_a_head = ROPE ? rest.rope_width / 32u : 1u, rope_half = ROPE ? rest.rope_width / 2u : 0u;
        const uint32_t rope_first = ROPE ? (at_tile / rope_tiles_a_head) * rest.rope_width + (at_tile % rope_tiles_a_head) * 16u : 0u;
        // (a head never straddles two matrices: the tile's first row names the matrix of all its rows)
        const uint8_t *const rope_base = (rope_first < end0 ? w0 : (rope_first < end1 ? w1 : w2)) +
                                         (size_t)(rope_first - (rope_first < end0 ? 0u : (rope_first < end1 ? end0 : end1))) * p.row_bytes;
        auto row_base = [&](uint32_t r) -> const uint8_t * {
            if (gated) return (r < 16u ? w0 : w1) + (size_t)(at_tile * 16u + (r & 15u)) * p.row_bytes;
            if constexpr (ROPE) return rope_base + (size_t)((r & 15u) + (r >= 16u ? rope_half : 0u)) * p.row_bytes;
            return plain_base + (size_t)r * p.row_bytes;
        };
        // A super-block of the tile is 32 rows x 144 bytes = 288 pieces of 16 bytes.  Lane l fetches pieces l, l + 64, ...: nine
        // neighbouring lanes read one row's block end to end (a load instruction touches 15 cache lines where one lane per
        // row would touch 32), and the pieces go through LDS to the lanes that multiply them.
        const uint8_t *src[5];
#pragma unroll
        for (int i = 0; i < 5; i++) {
            if (STAGED) {
                const uint32_t c = lane + 64u * i < 288u ? lane + 64u * i : lane;  // the last 32 pieces do not exist: fetched twice, dropped
                src[i] = row_base(c / 9u) + (size_t)blk0 * 144u + (c % 9u) * 16u;
            } else {
                src[i] = row_base(n) + (size_t)blk0 * 144u + (i == 0 ? 0u : 16u + 32u * (i - 1) + 16u * q);  // this lane's own header and half groups
            }
        }
        u32x4 ahead[5];
        auto fetch = [&](uint32_t step) {
            // past the wave's last super-block the last one is fetched again: the waits count on every step issuing its loads
            const size_t off = (size_t)min(ks + KS * min(step, last_step), nb - 1u) * 144u;
#pragma unroll
            for (int i = 0; i < 5; i++) ahead[i] = *(global_uint4)(uintptr_t)(src[i] + off);
        };
        float acc[J];
#pragma unroll
        for (int j = 0; j < J; j++) acc[j] = 0.0f;
        fetch(0);
        for (uint32_t step = 0; step < count; step++) {
            const uint32_t b = min(ks + KS * step, nb - 1u);
            Tile32Unit u;
            if (STAGED) {
#pragma unroll
                for (int i = 0; i < 5; i++)
                    if (i < 4 || lane < 32u) raw[lane + 64u * i] = ahead[i];
                fetch(step + 1u);
                __builtin_amdgcn_wave_barrier();  // LDS serves a wave's accesses in order: the reads below see these writes
                u.hdr = raw[n * 9u];
#pragma unroll
                for (int g = 0; g < 4; g++) u.g[g] = raw[n * 9u + 1u + 2u * g + q];
            } else {
                u.hdr = ahead[0];
#pragma unroll
                for (int g = 0; g < 4; g++) u.g[g] = ahead[1 + g];
                fetch(step + 1u);
            }
            // the eight 6-bit scales and minimums (crates/neura-precision/src/ggml.rs:127-136), four to a word
            const uint32_t sc_lo = u.hdr.y & 0x3f3f3f3fu, sc_hi = (u.hdr.w & 0x0f0f0f0fu) | ((u.hdr.y >> 2) & 0x30303030u);
            const uint32_t mn_lo = u.hdr.z & 0x3f3f3f3fu, mn_hi = ((u.hdr.w >> 4) & 0x0f0f0f0fu) | ((u.hdr.z >> 2) & 0x30303030u);
            const half2_t dd = __builtin_bit_cast(half2_t, u.hdr.x);  // (d, dmin)
            const float d = (float)dd.x, dmin = (float)dd.y;
#pragma unroll
            for (int s = 0; s < 8; s++) {
                const u32x4 words = u.g[s >> 1];
                const u32x4 nibbles = ((s & 1) ? (words >> 4) : words) & 0x0f0f0f0fu;
                u32x4 digits = {0u, 0u, 0u, 0u};
                if (a_held) digits = a_lane[((size_t)b * 8u + s) * 2u * M8];
                i32x16 zero;
#pragma unroll
                for (int e = 0; e < 16; e++) zero[e] = 0;
                const i32x16 c = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, digits), __builtin_bit_cast(i32x4, nibbles), zero, 0, 0, 0);
                const uint32_t sc_word = s < 4 ? sc_lo : sc_hi, mn_word = s < 4 ? mn_lo : mn_hi;
                const float weigh = d * (float)((sc_word >> (8 * (s & 3))) & 0xffu), floor_ = dmin * (float)((mn_word >> (8 * (s & 3))) & 0xffu);
#pragma unroll
                for (int j = 0; j < J; j++) {
                    const float joined = fmaf(fmaf(fmaf((float)c[4 * j], 256.0f, (float)c[4 * j + 1]), 256.0f, (float)c[4 * j + 2]), 256.0f, (float)c[4 * j + 3]);
                    const float2 xs = sums[((size_t)b * 8u + s) * R2 + 2u * j + q];
                    acc[j] += fmaf(weigh * xs.x, joined, -(floor_ * xs.y));
                }
                if (s & 1) __builtin_amdgcn_sched_barrier(0);  // two sub-blocks' sums live at a time, not eight
            }
            __builtin_amdgcn_wave_barrier();  // the next super-block overwrites the raw pieces
        }
        // ---- the four waves of the tile meet lane by lane
        float *mine = part + ((size_t)(parity * TPW + ts) * KS + ks) * J * 64u;
#pragma unroll
        for (int j = 0; j < J; j++) mine[j * 64 + lane] = acc[j];
        __syncthreads();
        // (the first J waves of the tile take a pair of activation rows each: one wave's reads of the tile's parts do not queue
        // behind another pair's, nor the rotation's loads; the sums and their order are the same)
        static_assert(KS >= J, "a wave of the tile for every pair of activation rows");
        if (ks < (uint32_t)J) {
            const float *from = part + (size_t)(parity * TPW + ts) * KS * J * 64u;
            for (int once = 0; once < 1; once++) {  // (a loop for its `continue`s)
                const uint32_t j = ks;
                float total = 0.0f;
#pragma unroll
                for (int k = 0; k < KS; k++) total += from[(size_t)k * J * 64u + j * 64u + lane];
                const uint32_t arow = 2u * j + q;
                if constexpr (ROPE) {
                    // (what the rotation needs is read from the kernel's own argument block, `rest`: a member of the local copy
                    // chosen by a number would put the whole copy into scratch memory)
                    const uint32_t row_n = rope_first + (n & 15u) + (n >= 16u ? rope_half : 0u);  // the output row among q|k|v's
                    const uint32_t c = (at_tile % rope_tiles_a_head) * 16u + (n & 15u);           // its channel pair
                    const bool first0 = rope_first < end0, first1 = rope_first < end1;            // the tile's matrix: one for all its rows
                    const float *bias = first0 ? rest.bias[0] : (first1 ? rest.bias[1] : rest.bias[2]);
                    if (bias) total += bias[row_n - (first0 ? 0u : (first1 ? end0 : end1))];
                    const float other = __shfl_xor(total, 16, 64);
                    if (!live || arow >= p.rows) continue;
                    const uint32_t position = rest.rope_cursor[arow];
                    float value = total;
                    if (row_n < rest.rope_k_rows) {
                        const size_t at = (size_t)min(position, rest.rope_positions - 1u) * rope_half + c;
                        const float cosine = rest.rope_cosines[at], sine = rest.rope_sines[at];
                        value = n >= 16u ? total * cosine + other * sine : total * cosine - other * sine;
                    }
                    if (row_n < rest.rope_q_rows) {
                        rest.y[(size_t)arow * rest.N + row_n] = value;
                    } else if (position >= rest.rope_positions || (!rest.rope_ring && position >= rest.rope_capacity)) {
                        atomicMax(rest.refusal, (uint32_t)REFUSAL_ORIGIN);
                    } else {
                        const bool key = row_n < rest.rope_k_rows;
                        const uint32_t within = row_n - (key ? rest.rope_q_rows : rest.rope_k_rows);  // head * width + channel
                        const uint32_t head = within / rest.rope_width, channel = within % rest.rope_width;
                        const uint32_t slot = rest.rope_ring ? position % rest.rope_ring : position;  // a ring seats position p at p mod its span
                        state_store(key ? rest.rope_k : rest.rope_v, rest.rope_element, (((uint64_t)head * p.rows + arow) * rest.rope_capacity + slot) * rest.rope_width + channel,
                                    value);
                    }
                    continue;
                }
                const float up = __shfl_xor(total, 16, 64);
                if (!live || arow >= p.rows) continue;
                if (p.splits > 1) {
                    const uint32_t column = gated ? (n < 16u ? tile * 16u + n : p.N / 2 + tile * 16u + (n - 16u)) : tile * 32u + n;
                    p.partial[((size_t)split * p.rows + arow) * p.N + column] = total;
                } else if (gated) {
                    if (n < 16u) p.y[(size_t)arow * (p.N / 2) + tile * 16u + n] = silu(total) * up;
                } else {
                    const size_t at = (size_t)arow * p.N + tile * 32u + n;
                    p.y[at] = p.residual ? p.residual[at] + total : total;
                }
            }
        }
        parity ^= 1u;
    }
}


// ------------------------------------------------- several activation rows on half-precision matrix cores ------
//
// Two to eight activation rows against 16-row tiles on v_mfma_f32_16x16x32_f16.  The weights are the B operand as exact
// normal halves code * sc * 2^-14 (a nibble masked in place in a 16-bit lane is the half subnormal code * 2^-24 or
// code * 2^-20; one packed multiply by sc * 2^10 or sc * 2^6 makes it normal), so the scale of a sub-block rides in
// the operand and a whole super-block accumulates on the matrix cores before anything is weighed: four instructions per
// eight weights and eight multiply-adds per super-block and lane, where the integer tiles convert and join digit sums
// per sub-block.  An fp32 activation enters as two half rows (the value rounded to half after a power-of-two row scale,
// and the rounding residue * 2^11): A row m < 8 is activation row m, A row 8 + m its residue, 22 bits of each take part.
// The minimums come off with one more MFMA per super-block over (minimum, sub-block sum) pairs, as in the wide product.
//
// Operand slots: one MFMA takes 32 k.  Lane (n, kq) = (lane % 16, lane / 16) loads, per super-block, its row's header and
// the 16 bytes at 16 + 64 j + 16 kq (j = 0, 1): half a 64-element group g = 2j + kq / 2, whose 16 low nibbles are elements
// 16 (kq & 1) .. + 15 of sub-block 2g and whose high nibbles are the same elements of sub-block 2g + 1.  MFMA (j, i),
// i = 2h + half, multiplies, in lane kq's eight slots, elements 16 (kq & 1) + 8 half + {0, 2, 1, 3, 4, 6, 5, 7} of
// sub-block 2g + h -- the order the masks leave them in -- and the activations are staged in LDS in that same order, so a
// lane's A operand is one 16-byte read.  Sub-blocks mix inside an MFMA; only d and dmin wait for the super-block's end.
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

constexpr uint32_t F16_BLOCK_PIECES = 8u * 4u * 16u + 2u * 16u;  // 16-byte pieces of LDS per staged super-block: operands, then sums
constexpr uint32_t F16_TWO_SETS_BLOCKS = 14;  // up to so many staged super-blocks leave LDS room for two sets of the waves' partial sums

template <int NW, int KS>
__global__ __launch_bounds__(NW * 64) void gemv_q4k_f16_kernel(MFMA_LEAD_PARAMETERS) {
    MFMA_TAKE_LEAD;
    constexpr uint32_t TPW = NW / KS, NT = NW * 64;
    static_assert(NT == 1024, "eight row groups of 128 threads stage the activations");
    extern __shared__ __attribute__((aligned(16))) uint32_t staged[];  // [block][F16_BLOCK_PIECES] pieces
    __shared__ float red[NW];
    __shared__ uint32_t tops[8];
    __shared__ float unscale[8];
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t split = blockIdx.y, blk0 = split * p.slice_blocks;
    const uint32_t nb = min(p.slice_blocks, p.nblk - blk0);
    const uint32_t k0 = blk0 * 256u, kn = nb * 256u;
    u32x4 *const pieces = reinterpret_cast<u32x4 *>(staged);
    float *const part = reinterpret_cast<float *>(pieces + (size_t)nb * F16_BLOCK_PIECES);  // [TPW][KS][4][64]
    typedef const __attribute__((address_space(1))) u32x4 *global_uint4;

    // ---- activations -> half planes in operand order: row r by threads 128 r .. 128 r + 127, eight neighbours a thread
    {
        const uint32_t r = tid >> 7, t = tid & 127u;
        const bool real = r < p.rows;
        const float *xr = p.x + (size_t)min(r, p.rows - 1u) * p.K + k0;
        float v[4][8];
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const uint32_t k = 8u * t + 1024u * c;
            float4 a = make_float4(0.f, 0.f, 0.f, 0.f), b = a;
            if (real && k < kn) a = *reinterpret_cast<const float4 *>(xr + k), b = *reinterpret_cast<const float4 *>(xr + k + 4u);
            v[c][0] = a.x, v[c][1] = a.y, v[c][2] = a.z, v[c][3] = a.w, v[c][4] = b.x, v[c][5] = b.y, v[c][6] = b.z, v[c][7] = b.w;
        }
        if (p.norm_w) {  // one slice holds the whole row (the launcher sees to it)
            float square = 0.0f;
#pragma unroll
            for (int c = 0; c < 4; c++)
#pragma unroll
                for (int i = 0; i < 8; i++) square = __fadd_rn(square, __fmul_rn(v[c][i], v[c][i]));
            square = wave_sum(square);
            if (lane == 0) red[wave] = square;
            __syncthreads();
            const float rms = rms_scale_of(red[2u * r] + red[2u * r + 1u], p.K, p.eps);
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const uint32_t k = 8u * t + 1024u * c;
                float4 a = make_float4(0.f, 0.f, 0.f, 0.f), b = a;
                if (k < kn) a = *reinterpret_cast<const float4 *>(p.norm_w + k0 + k), b = *reinterpret_cast<const float4 *>(p.norm_w + k0 + k + 4u);
                const float w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
                for (int i = 0; i < 8; i++) v[c][i] = __fmul_rn(__fmul_rn(v[c][i], rms), w[i]);
            }
        }
        uint32_t top = 0;  // largest magnitude as bits: infinities and NaNs sort above every finite value
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
            for (int i = 0; i < 8; i++) top = max(top, __builtin_bit_cast(uint32_t, v[c][i]) & 0x7fffffffu);
#pragma unroll
        for (int offset = 32; offset > 0; offset >>= 1) top = max(top, (uint32_t)__shfl_xor((int)top, offset, 64));
        if (tid < 8) tops[tid] = 0u;
        __syncthreads();
        if (lane == 0) atomicMax(&tops[r], top);
        __syncthreads();
        top = tops[r];
        // a power of two that puts the row's largest magnitude in [2^13, 2^14)
        const uint32_t raw = top >> 23, exponent = min(max(raw, 27u), 254u);
        const float scale = __builtin_bit_cast(float, (267u - exponent) << 23);
        if (t == 0) unscale[r] = raw == 255u ? __builtin_bit_cast(float, 0x7fc00000u) : __builtin_bit_cast(float, (exponent - 13u) << 23);
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const uint32_t k = 8u * t + 1024u * c;
            _Float16 hi[8], lo[8];
            float sum_hi = 0.0f, sum_lo = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const float scaled = v[c][i] * scale;
                hi[i] = (_Float16)scaled;
                lo[i] = (_Float16)((scaled - (float)hi[i]) * 2048.0f);
                sum_hi += (float)hi[i], sum_lo += (float)lo[i];
            }
            // the 32 halves of a sub-block: four neighbouring threads
            sum_hi += dpp<DPP_QUAD_XOR1>(sum_hi), sum_lo += dpp<DPP_QUAD_XOR1>(sum_lo);
            sum_hi += dpp<DPP_QUAD_XOR2>(sum_hi), sum_lo += dpp<DPP_QUAD_XOR2>(sum_lo);
            if (k < kn) {
                const uint32_t b = k >> 8, g = (k >> 6) & 3u, h = (k >> 5) & 1u, e = k & 31u;
                const uint32_t kq = 2u * (g & 1u) + (e >> 4), jj = 4u * (g >> 1) + 2u * h + ((e >> 3) & 1u);
                u32x4 *at = pieces + (size_t)b * F16_BLOCK_PIECES + (jj * 4u + kq) * 16u;
                typedef _Float16 half2v __attribute__((ext_vector_type(2)));
                auto pair = [](_Float16 a, _Float16 c) { return __builtin_bit_cast(uint32_t, half2v{a, c}); };
                // slots 0..7 take elements 0, 2, 1, 3, 4, 6, 5, 7
                at[r] = u32x4{pair(hi[0], hi[2]), pair(hi[1], hi[3]), pair(hi[4], hi[6]), pair(hi[5], hi[7])};
                at[8u + r] = u32x4{pair(lo[0], lo[2]), pair(lo[1], lo[3]), pair(lo[4], lo[6]), pair(lo[5], lo[7])};
                if ((t & 3u) == 0) {
                    // sums / 64 as a half and its residue * 2^11: slots s (kq = 0) and s (kq = 1) of the minimums' operand
                    const uint32_t sub = (k >> 5) & 7u;
                    _Float16 *sums = reinterpret_cast<_Float16 *>(pieces + (size_t)b * F16_BLOCK_PIECES + 8u * 4u * 16u);
                    const float a = sum_hi * 0.015625f, c2 = sum_lo * 0.015625f;
                    const _Float16 ah = (_Float16)a, ch = (_Float16)c2;
                    sums[(0u * 16u + r) * 8u + sub] = ah, sums[(1u * 16u + r) * 8u + sub] = (_Float16)((a - (float)ah) * 2048.0f);
                    sums[(0u * 16u + 8u + r) * 8u + sub] = ch, sums[(1u * 16u + 8u + r) * 8u + sub] = (_Float16)((c2 - (float)ch) * 2048.0f);
                }
            }
        }
    }
    __syncthreads();

    // ---- tiles of 16 weight rows
    const uint32_t n = lane & 15u, kq = lane >> 4;
    const uint32_t ts = wave / KS, ks = wave % KS;
    const uint32_t count = ks < nb ? (nb - ks + KS - 1u) / KS : 0u;  // super-blocks ks, ks + KS, ...
    const uint32_t last_step = count ? count - 1u : 0u;
    const uint8_t *const w0 = p.W[0], *const w1 = p.W[1], *const w2 = p.W[2];
    const uint32_t end0 = p.end[0], end1 = p.end[1];
    const bool gated = p.swiglu != 0;
    const half2_t offset = {(_Float16)1024.0f, (_Float16)1024.0f}, powers = {(_Float16)1024.0f, (_Float16)64.0f};
    const uint32_t shift = 16u * (kq >> 1);  // the group's pair of 6-bit fields inside its scale words
    // Rounds of tiles: in round i the workgroup's tile slot ts takes tile (blockIdx.x + i * gridDim.x) * TPW + ts.  A wave's loads
    // run two super-blocks ahead across rounds (the first blocks of the next tile are on their way while this tile's sums meet),
    // and every fetch issues its three loads: past the last round the last block again, dropped.
    const uint32_t rounds = (p.tiles > blockIdx.x * TPW) ? (p.tiles - blockIdx.x * TPW + gridDim.x * TPW - 1u) / (gridDim.x * TPW) : 0u;
    const uint32_t first_round = blockIdx.x, hop = gridDim.x, tiles = p.tiles, row_bytes = p.row_bytes;
    auto tile_of = [first_round, hop, ts](uint32_t round) __attribute__((always_inline)) -> uint32_t { return (first_round + round * hop) * TPW + ts; };
    // written with selects over scalars captured by value: nothing here may end up indexed
    const int64_t to_w1 = w1 - w0, to_w2 = w2 - w0;
    auto row_of = [w0, to_w1, to_w2, end0, end1, gated, n, tiles, row_bytes, blk0, tile_of](uint32_t round) __attribute__((always_inline)) -> const uint8_t * {
        const uint32_t at_tile = min(tile_of(round), tiles - 1u);
        const uint32_t r0 = at_tile * 16u;
        const bool in0 = r0 < end0, in1 = r0 < end1;
        const int64_t offset = gated ? (n < 8u ? (int64_t)0 : to_w1) + (int64_t)(at_tile * 8u + (n & 7u)) * row_bytes
                                     : (in0 ? (int64_t)0 : (in1 ? to_w1 : to_w2)) + (int64_t)(r0 - (in0 ? 0u : (in1 ? end0 : end1)) + n) * row_bytes;
        return w0 + offset + (size_t)blk0 * 144u;
    };
    const uint32_t walked = max(count, 1u);  // a wave with no super-block of its own still keeps the ring's rhythm
    uint32_t ahead_round = 0, ahead_step = 0;
    const uint8_t *ahead_row = row_of(0);
    u32x4 even[3], odd[3];
    auto fetch = [&](u32x4 (&ahead)[3]) __attribute__((always_inline)) {
        const uint8_t *block = ahead_row + (size_t)min(ks + KS * min(ahead_step, last_step), nb - 1u) * 144u;
        ahead[0] = *(global_uint4)(uintptr_t)block;
        ahead[1] = *(global_uint4)(uintptr_t)(block + 16u + 16u * kq);
        ahead[2] = *(global_uint4)(uintptr_t)(block + 80u + 16u * kq);
        if (++ahead_step >= walked) {
            ahead_step = 0;
            if (ahead_round + 1u < rounds) ahead_row = row_of(++ahead_round);
        }
    };
    // Two sets of partial sums where the operands leave room (up to fourteen super-blocks staged: what the launcher asked LDS
    // for says so): a tile's parts are read while the next tile's are written, and no wave waits for the readers.  Sixteen
    // super-blocks of operands leave room for one set, and a barrier behind the readers.
    const bool two_sets = nb <= F16_TWO_SETS_BLOCKS;
    uint32_t parity = 0;
    {
        f32x4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
        uint32_t tile = 0;
        bool live = false;
        auto take = [&](const u32x4 (&ahead)[3], uint32_t step) __attribute__((always_inline)) {
            const uint32_t b = min(ks + KS * step, nb - 1u);
            const u32x4 hdr = ahead[0], q0 = ahead[1], q1 = ahead[2];
            const u32x4 *a_block = pieces + (size_t)b * F16_BLOCK_PIECES + kq * 16u + n;
            f32x4_t tmp = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int j = 0; j < 2; j++) {
                // 6-bit scales of sub-blocks 2g, 2g + 1, g = 2j + kq / 2 (crates/neura-precision/src/ggml.rs:127-136); 0x6400 | v is the half 1024 + v
                const uint32_t ya = (hdr.y >> shift) & 0xffffu, wa = (hdr.w >> shift) & 0xffffu;
                const uint32_t sc = j == 0 ? (ya & 0x3f3fu) : ((wa & 0x0f0fu) | ((ya >> 2) & 0x3030u));
                const uint32_t both = __builtin_amdgcn_perm(0u, sc, 0x0c010c00u) | 0x64006400u;
                const half2_t scales = (__builtin_bit_cast(half2_t, both) - offset) * powers;  // (sc0 * 2^10, sc1 * 2^6)
                const half2_t low_scale = {scales.x, scales.x}, high_scale = {scales.y, scales.y};
                // the four operands of the activations are asked for before the weights are unpacked: the unpacking hides LDS
                u32x4 rows[4];
#pragma unroll
                for (int i = 0; i < 4; i++) rows[i] = a_block[(4u * j + i) * 64u];
                __builtin_amdgcn_sched_barrier(0);
                const u32x4 q = j == 0 ? q0 : q1;
                const uint32_t words[4] = {q.x, q.y, q.z, q.w};
                uint32_t low[8], high[8];
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    const uint32_t even = words[w], odd = words[w] >> 8;
                    low[2 * w] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, even & 0x000f000fu) * low_scale);
                    low[2 * w + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, odd & 0x000f000fu) * low_scale);
                    high[2 * w] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, even & 0x00f000f0u) * high_scale);
                    high[2 * w + 1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, odd & 0x00f000f0u) * high_scale);
                }
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t *from = (i < 2 ? low : high) + 4 * (i & 1);
                    const half8_t weights = __builtin_bit_cast(half8_t, u32x4{from[0], from[1], from[2], from[3]});
                    tmp = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, rows[i]), weights, tmp, 0, 0, 0);
                }
            }
            // ---- the super-block is complete: weigh by d, take the minimums off
            u32x4 mins = {0u, 0u, 0u, 0u}, sums = {0u, 0u, 0u, 0u};
            if (kq < 2u) {
                const uint32_t lo4 = hdr.z & 0x3f3f3f3fu;                                         // m0..m3
                const uint32_t hi4 = ((hdr.w >> 4) & 0x0f0f0f0fu) | ((hdr.z >> 2) & 0x30303030u);  // m4..m7
                half2_t m01 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, lo4, 0x0c010c00u) | 0x64006400u) - offset;
                half2_t m23 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, lo4, 0x0c030c02u) | 0x64006400u) - offset;
                half2_t m45 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, hi4, 0x0c010c00u) | 0x64006400u) - offset;
                half2_t m67 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(0u, hi4, 0x0c030c02u) | 0x64006400u) - offset;
                if (kq == 1u) {  // the minimums * 2^-11 against the residues * 2^11
                    const half2_t down = {(_Float16)0.00048828125f, (_Float16)0.00048828125f};
                    m01 = m01 * down, m23 = m23 * down, m45 = m45 * down, m67 = m67 * down;
                }
                mins = u32x4{__builtin_bit_cast(uint32_t, m01), __builtin_bit_cast(uint32_t, m23), __builtin_bit_cast(uint32_t, m45),
                             __builtin_bit_cast(uint32_t, m67)};
                sums = pieces[(size_t)b * F16_BLOCK_PIECES + 8u * 4u * 16u + kq * 16u + n];
            }
            const f32x4_t zero = {0.0f, 0.0f, 0.0f, 0.0f};
            const f32x4_t floors = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, sums), __builtin_bit_cast(half8_t, mins), zero, 0, 0, 0);
            const half2_t dd = __builtin_bit_cast(half2_t, hdr.x);  // (d, dmin)
            const float dscale = (float)dd.x * 16384.0f;  // the weights were staged * 2^-14
            const float mscale = (float)dd.y * -64.0f;    // the sums were staged / 64
#pragma unroll
            for (int e = 0; e < 4; e++) acc[e] = fmaf(mscale, floors[e], fmaf(dscale, tmp[e], acc[e]));
        };
        auto tile_end = [&]() __attribute__((always_inline)) {
        // ---- the waves of the tile meet lane by lane
        float *mine = part + (((size_t)parity * TPW + ts) * KS + ks) * 4u * 64u;
#pragma unroll
        for (int e = 0; e < 4; e++) mine[e * 64 + lane] = acc[e];
        __syncthreads();
        // (the first four waves of the tile take one of the four C registers each -- a wave's reads of the tile's parts do not
        // queue behind another register's, and every wave waits for them at the barrier below; the sums and their order are the same)
        static_assert(KS >= 4, "a wave of the tile for every C register");
        if (ks < 4u) {
            const float *from = part + ((size_t)parity * TPW + ts) * KS * 4u * 64u;
            for (int once = 0; once < 1; once++) {  // (a loop for its `continue`)
                const uint32_t e = ks;
                float total = 0.0f;
#pragma unroll
                for (int k = 0; k < KS; k++) total += from[(size_t)k * 4u * 64u + e * 64u + lane];
                // C row 4 kq + e: activation row 4 kq + e for kq < 2, its residue plane for kq >= 2 (32 lanes on)
                const float residue = __shfl_xor(total, 32, 64);
                const uint32_t arow = 4u * (kq & 1u) + e;
                float value = fmaf(residue, 0.00048828125f, total) * unscale[arow];
                const float up = __shfl_xor(value, 8, 64);
                if (!live || kq >= 2u || arow >= p.rows) continue;
                if (p.splits > 1) {
                    const uint32_t column = gated ? (n < 8u ? tile * 8u + n : p.N / 2 + tile * 8u + (n - 8u)) : tile * 16u + n;
                    p.partial[((size_t)split * p.rows + arow) * p.N + column] = value;
                } else if (gated) {
                    if (n < 8u) p.y[(size_t)arow * (p.N / 2) + tile * 8u + n] = silu(value) * up;
                } else {
                    const size_t at = (size_t)arow * p.N + tile * 16u + n;
                    p.y[at] = p.residual ? p.residual[at] + value : value;
                }
            }
        }
            if (two_sets) parity ^= 1u;  // (a wave gets no further than the next tile's barrier before the readers are done)
            else __syncthreads();        // the next tile's partial sums take the same places
#pragma unroll
            for (int e = 0; e < 4; e++) acc[e] = 0.0f;
        };
        fetch(even);
        fetch(odd);
        // every wave walks whole pairs of steps; a tile ends wherever its last step falls, and the steps past the last round
        // multiply what was fetched again and publish nothing
        uint32_t round = 0, step = 0;
        tile = tile_of(0), live = rounds > 0 && tile < p.tiles;
        const uint32_t steps = rounds * walked;
        auto unit = [&](u32x4 (&held)[3]) __attribute__((always_inline)) {
            if (count) take(held, step);
            fetch(held);
            if (++step >= walked) {
                if (round < rounds) tile_end();
                step = 0, round++;
                tile = tile_of(round), live = round < rounds && tile < p.tiles;
            }
        };
        for (uint32_t s0 = 0; s0 < steps; s0 += 2u) {
            unit(even);
            unit(odd);
        }
    }
}

// ------------------------------------------------------------------------- fold ----------

// sums the slice partials in slice order and applies the epilogue
// (crates/neura-kernel/src/task/matmul.rs:1318-1333)
__global__ __launch_bounds__(256) void gemv_fold_kernel(const float *__restrict__ partial, uint32_t splits, uint32_t rows, uint32_t N,
                                                        const float *__restrict__ residual, int32_t swiglu, float *__restrict__ y) {
    NH_FETCH(partial, splits, rows, N, residual, swiglu, y, blockDim.x);
    uint32_t outputs = swiglu ? N / 2 : N;
    for (uint32_t index = blockIdx.x * blockDim.x + threadIdx.x; index < rows * outputs; index += gridDim.x * blockDim.x) {
        uint32_t b = index / outputs, n = index % outputs;
        // eight slices at a time, every load asked for before the first is added (past the last slice the last again,
        // dropped): the sum still runs in slice order
        auto sum_of = [&](uint32_t column) {
            float total = 0.0f;
            for (uint32_t s0 = 0; s0 < splits; s0 += 8u) {
                float held[8];
#pragma unroll
                for (int j = 0; j < 8; j++) held[j] = partial[((size_t)min(s0 + j, splits - 1u) * rows + b) * N + column];
#pragma unroll
                for (int j = 0; j < 8; j++)
                    if (s0 + j < splits) total += held[j];
            }
            return total;
        };
        float total = sum_of(n);
        if (swiglu) {
            const float up = sum_of(N / 2 + n);
            total = silu(total) * up;
        } else if (residual) {
            total = residual[(size_t)b * N + n] + total;
        }
        y[(size_t)b * outputs + n] = total;
    }
}

// ------------------------------------------------------------------------- host ----------

static uint32_t pow2_at_least(uint32_t v, uint32_t floor) {
    uint32_t p = floor;
    while (p < v) p <<= 1;
    return p;
}


template <int RB>
static int32_t launch_rows(nh_device *d, const GemvArgs &a, const float *x, float *y, const float *residual) {
    GemvParams p{};
    for (int s = 0; s < 3; s++) {
        p.W[s] = static_cast<const uint8_t *>(a.W[s] ? a.W[s] : a.W[0]);
        p.end[s] = a.end[s];
    }
    p.x = x;
    if (a.merge) p.x = a.merge->partial, p.merge_sections = a.merge->sections, p.merge_groups = a.merge->groups, p.merge_width = a.merge->width;
    p.y = y;
    p.residual = residual;
    p.norm_w = a.norm_w;
    p.N = a.N;
    p.K = a.K;
    p.swiglu = a.swiglu;
    p.eps = a.eps;
    if (a.rope) {
        p.rope_cosines = a.rope->cosines, p.rope_sines = a.rope->sines, p.rope_cursor = a.rope->cursor, p.rope_k = a.rope->cache_k, p.rope_v = a.rope->cache_v;
        p.rope_width = a.rope->width, p.rope_q_rows = a.rope->q_rows, p.rope_k_rows = a.rope->k_rows, p.rope_capacity = a.rope->capacity;
        p.rope_positions = a.rope->positions, p.rope_ring = a.rope->ring, p.rope_element = a.rope->element;
        p.refusal = d->refusal;
        for (int s = 0; s < 3; s++) p.bias[s] = a.bias[s];
    } else if (a.bias[0] || a.bias[1] || a.bias[2]) {
        return fail(NH_E_ARGUMENT, "a product adds a bias only where it folds the rotation in");
    }
    p.row_bytes = (uint32_t)payload_bytes(a.element, a.K);
    const bool q4 = a.element == NH_Q4_K;
    p.nblk = a.K / (q4 ? 256u : 32u);
    // one lane per 64 (Q4_K) or 32 (Q8_0) elements; a slice fills at most one wave
    uint32_t units_per_block = q4 ? 4u : 1u;
    uint32_t most_blocks = q4 ? (RB >= 4 ? 8u : 16u) : 64u;
    p.splits = (p.nblk + most_blocks - 1) / most_blocks;
    p.blocks_per_split = (p.nblk + p.splits - 1) / p.splits;
    p.splits = (p.nblk + p.blocks_per_split - 1) / p.blocks_per_split;
    p.group = pow2_at_least(p.blocks_per_split * units_per_block, 16u);
    uint32_t RS = 64u / p.group;
    if (p.splits > 1) {
        p.partial = static_cast<float *>(scratch(d, (size_t)p.splits * RB * a.N * sizeof(float)));
        if (!p.partial) return NH_E_MEMORY;
    }
    // rows per lane group and pass: four rows amortise the cross-lane sum and keep more bytes
    // in flight per wave, two rows give twice the waves; tall matrices take four
    int R = (a.N >= 16384u && RB == 1) ? 4 : 2;
    if (RB >= 4) R = 2;
    // the decode kernel walks R rows of ONE matrix per lane group: every matrix boundary must be a
    // multiple of R (with swiglu the halves interleave, so N/2 must be a multiple of R/2)
    auto whole = [&](int rows) {
        if (a.swiglu) return a.N % (uint32_t)rows == 0 && a.end[0] == a.N / 2;
        return a.end[0] % (uint32_t)rows == 0 && a.end[1] % (uint32_t)rows == 0 && a.N % (uint32_t)rows == 0;
    };
    if (R == 4 && !whole(4)) R = 2;
    const bool fast = whole(R) && a.N >= (uint32_t)R && (uint64_t)a.N * p.row_bytes < (1ull << 32);
    uint32_t rows_per_pass = (uint32_t)R * RS;
    p.row_groups = (a.N + rows_per_pass - 1) / rows_per_pass;
    uint32_t blocks_x;
    size_t lds;
    if (q4) {
        blocks_x = (p.row_groups + 3) / 4;
        // one resident round of workgroups: 3 per compute unit at four rows (136 registers), 4 at two
        uint32_t most = (uint32_t)d->compute_units * (R == 4 ? 3u : 4u) / p.splits;
        if (most < 1) most = 1;
        if (blocks_x > most) blocks_x = most;
        uint32_t slice = p.blocks_per_split * 256u;
        lds = (size_t)RB * (slice + slice / 64 * 4) * sizeof(float);
    } else {
        uint32_t slice_bytes = p.blocks_per_split * 34u;
        p.chunks_per_row = (15u + slice_bytes + 15u) / 16u;
        uint32_t tiles = (p.row_groups + 3) / 4;
        blocks_x = tiles;
        uint32_t most = (uint32_t)d->compute_units * 4u / p.splits;
        if (most < 1) most = 1;
        if (blocks_x > most) blocks_x = most;
        uint32_t slice = p.blocks_per_split * 32u;
        lds = (size_t)RB * (slice + slice / 32 * 4) * sizeof(float) + (size_t)rows_per_pass * 4 * p.chunks_per_row * 16 + 16;
    }
    if (lds > 64 * 1024) return fail(NH_E_ARGUMENT, "a product of depth %u stages %zu bytes where a workgroup holds 65536", a.K, lds);
    dim3 grid(blocks_x, p.splits), block(256);
    profile_mark(d);
#define NH_LAUNCH(KERNEL, RR) hipLaunchKernelGGL((KERNEL<RR, RB>), grid, block, lds, d->stream, p)
#define NH_DECODE(RR, GG) hipLaunchKernelGGL((gemv_q4k_decode_kernel<RR, GG, false, 4>), grid, block, lds, d->stream, p)
    const bool q8_direct = !q4 && RB == 1 && fast && p.nblk <= 256u;
    if (a.merge && !(q8_direct && R == 2 && p.nblk <= 64u && !a.rope))
        return fail(NH_E_ARGUMENT, "this product merges no attention sections (ask gemv_merges_sections first)");
    if (a.rope && !(q4 && RB == 1 && fast && R == 2 && p.splits == 1) && !(q8_direct && R == 2 && p.nblk <= 64u))
        return fail(NH_E_ARGUMENT, "this product cannot fold the rotation in (ask gemv_fuses_rope first)");
    if (q4 && RB == 1 && fast && a.rope) {
        if (p.group == 64) hipLaunchKernelGGL((gemv_q4k_decode_kernel<2, 64, false, 4, true>), grid, block, lds, d->stream, p);
        else if (p.group == 32) hipLaunchKernelGGL((gemv_q4k_decode_kernel<2, 32, false, 4, true>), grid, block, lds, d->stream, p);
        else hipLaunchKernelGGL((gemv_q4k_decode_kernel<2, 16, false, 4, true>), grid, block, lds, d->stream, p);
    } else if (q4 && RB == 1 && fast) {
        if (R == 4) {
            if (p.group == 64) NH_DECODE(4, 64);
            else if (p.group == 32) NH_DECODE(4, 32);
            else NH_DECODE(4, 16);
        } else {
            if (p.group == 64) NH_DECODE(2, 64);
            else if (p.group == 32) NH_DECODE(2, 32);
            else NH_DECODE(2, 16);
        }
    } else if (q4) {
        if (R == 4) NH_LAUNCH(gemv_q4k_kernel, 4);
        else NH_LAUNCH(gemv_q4k_kernel, 2);
    } else if (q8_direct) {
        // one activation row, a row of blocks inside one wave (or, deeper, inside the four waves of a workgroup): the words of
        // a block straight from memory, no LDS tile, no K slices and no fold
        const bool deep = p.nblk > 64u;
        if (deep) p.group = 64, RS = 1;
        p.splits = 1, p.blocks_per_split = p.nblk;
        const uint32_t passes = (a.N + (uint32_t)R * RS - 1) / ((uint32_t)R * RS);
        p.row_groups = passes;
        uint32_t wgs = deep ? passes : (passes + 3) / 4;
        const uint32_t resident = (uint32_t)d->compute_units * 4u;
        if (wgs > resident) wgs = resident;
        const size_t staged = (size_t)(a.K + a.K / 32u * 4u) * sizeof(float);
        const dim3 wide(wgs);
#define NH_Q8(RR, GG) hipLaunchKernelGGL((gemv_q8_0_decode_kernel<RR, GG>), wide, block, staged, d->stream, Q8_LEAD(p))
        if (a.rope) {
            if (p.group == 64) hipLaunchKernelGGL((gemv_q8_0_decode_kernel<2, 64, false, true>), wide, block, staged, d->stream, Q8_LEAD(p));
            else if (p.group == 32) hipLaunchKernelGGL((gemv_q8_0_decode_kernel<2, 32, false, true>), wide, block, staged, d->stream, Q8_LEAD(p));
            else hipLaunchKernelGGL((gemv_q8_0_decode_kernel<2, 16, false, true>), wide, block, staged, d->stream, Q8_LEAD(p));
        } else if (a.merge) {
            if (p.group == 64) hipLaunchKernelGGL((gemv_q8_0_decode_kernel<2, 64, false, false, true>), wide, block, staged, d->stream, Q8_LEAD(p));
            else if (p.group == 32) hipLaunchKernelGGL((gemv_q8_0_decode_kernel<2, 32, false, false, true>), wide, block, staged, d->stream, Q8_LEAD(p));
            else hipLaunchKernelGGL((gemv_q8_0_decode_kernel<2, 16, false, false, true>), wide, block, staged, d->stream, Q8_LEAD(p));
        } else if (deep) {
            if (R == 4) hipLaunchKernelGGL((gemv_q8_0_decode_kernel<4, 64, true>), wide, block, staged, d->stream, Q8_LEAD(p));
            else hipLaunchKernelGGL((gemv_q8_0_decode_kernel<2, 64, true>), wide, block, staged, d->stream, Q8_LEAD(p));
        } else if (R == 4) {
            if (p.group == 64) NH_Q8(4, 64);
            else if (p.group == 32) NH_Q8(4, 32);
            else NH_Q8(4, 16);
        } else {
            if (p.group == 64) NH_Q8(2, 64);
            else if (p.group == 32) NH_Q8(2, 32);
            else NH_Q8(2, 16);
        }
#undef NH_Q8
    } else {
        if (R == 4) NH_LAUNCH(gemv_q8_0_kernel, 4);
        else NH_LAUNCH(gemv_q8_0_kernel, 2);
    }
#undef NH_LAUNCH
#undef NH_DECODE
    NH_HIP(hipGetLastError());
    if (p.splits > 1) {
        uint32_t outputs = (a.swiglu ? a.N / 2 : a.N) * RB;
        hipLaunchKernelGGL(gemv_fold_kernel, dim3((outputs + 255) / 256), dim3(256), 0, d->stream, p.partial, p.splits, (uint32_t)RB, a.N,
                           residual, a.swiglu, y);
        NH_HIP(hipGetLastError());
    }
    profile_mark(d);
    if (d->profile) d->profile_bytes += (uint64_t)a.N * p.row_bytes;
    return NH_OK;
}

// The MFMA kernel takes a product when every matrix boundary falls on a 16-row tile and the
// activations can be read with 128-bit loads.
static bool mfma_takes(const GemvArgs &a) {
    // 2: always; 1: where it measured faster than the vector kernels -- several activation rows (they ride on
    // the same unpacked weights) or rows deeper than one wave spans (no second launch to fold slices); 0: never
    const int mode = env_int("NEURA_HIP_MFMA", 1);
    if (a.element != NH_Q4_K || mode == 0) return false;
    if (mode == 1 && a.rows == 1 && a.K <= 4096) return false;
    if (a.N < 16 || a.N % 16 != 0) return false;
    if (a.swiglu) {
        if (a.end[0] != a.N / 2 || (a.N / 2) % 8 != 0) return false;
    } else if (a.end[0] % 16 != 0 || a.end[1] % 16 != 0) {
        return false;
    }
    if (((uintptr_t)a.x & 15u) || (a.norm_w && ((uintptr_t)a.norm_w & 15u))) return false;
    return true;
}

template <int KS, int NW, int P, int D>
static hipError_t launch_mfma_instance(nh_device *d, const MfmaParams &p, uint32_t blocks_x, size_t lds) {
    static bool widened = false;  // past 64 KiB of dynamic LDS a kernel has to be told once
    if (lds > 64 * 1024 && !widened) {
        hipError_t status = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_q4k_mfma_kernel<KS, NW, P, D>),
                                                hipFuncAttributeMaxDynamicSharedMemorySize, 156 * 1024);  // the static arrays take the rest of the 160 KiB
        if (status != hipSuccess) return status;
        widened = true;
    }
    hipLaunchKernelGGL((gemv_q4k_mfma_kernel<KS, NW, P, D>), dim3(blocks_x, p.splits), dim3(NW * 64), lds, d->stream, MFMA_LEAD(p));
    return hipGetLastError();
}

template <int KS, int NW>
static hipError_t launch_mfma_kernel(nh_device *d, const MfmaParams &p, uint32_t P, uint32_t blocks_x, size_t lds) {
    if (P == 1) {
        // sixteen waves leave 128 registers a lane: two super-blocks in flight fit, four would spill
        if (NW == 16) return launch_mfma_instance<KS, NW, 1, 2>(d, p, blocks_x, lds);
        return launch_mfma_instance<KS, NW, 1, 4>(d, p, blocks_x, lds);
    }
    if (P == 2) return launch_mfma_instance<KS, NW, 2, 2>(d, p, blocks_x, lds);
    return launch_mfma_instance<KS, NW, 4, 2>(d, p, blocks_x, lds);
}

// LDS bytes of the staged activations of `blocks` super-blocks for P activation rows: digits + sums
static size_t mfma_staged(uint32_t blocks, uint32_t P) { return (size_t)blocks * (1024u + 32u) * P; }

static int32_t launch_mfma(nh_device *d, const GemvArgs &a) {
    const uint32_t outputs = a.swiglu ? a.N / 2 : a.N;
    const uint32_t nblk = a.K / 256u;
    const size_t room = 140 * 1024;  // a gfx950 workgroup may take all 160 KiB of a compute unit; tile partials and static arrays need the rest
    for (uint32_t done = 0; done < a.rows;) {
        // activation rows per launch: 4, 2 or 1 (the kernel's instantiations); rows too deep to stage whole are cut into K slices
        uint32_t left = a.rows - done, P = left >= 3 ? 4u : left;
        MfmaParams p{};
        for (int s = 0; s < 3; s++) {
            p.W[s] = static_cast<const uint8_t *>(a.W[s] ? a.W[s] : a.W[0]);
            p.end[s] = a.end[s];
        }
        p.rows = min(P, left);
        p.x = a.x + (size_t)done * a.K;
        p.y = a.y + (size_t)done * outputs;
        p.residual = a.residual ? a.residual + (size_t)done * a.N : nullptr;
        p.norm_w = a.norm_w;
        p.N = a.N;
        p.K = a.K;
        p.row_bytes = nblk * 144u;
        p.nblk = nblk;
        p.swiglu = a.swiglu;
        p.eps = a.eps;
        p.tiles = a.N / 16u;
        p.splits = (uint32_t)((mfma_staged(nblk, P) + room - 1) / room);
        p.slice_blocks = (nblk + p.splits - 1) / p.splits;
        p.splits = (nblk + p.slice_blocks - 1) / p.slice_blocks;
        if (p.splits > 1) {
            p.partial = static_cast<float *>(scratch(d, (size_t)p.splits * p.rows * a.N * sizeof(float)));
            if (!p.partial) return NH_E_MEMORY;
        }
        // waves that share a tile: enough of them to fill the device when the matrix is short
        const uint32_t slots = (uint32_t)d->compute_units * 16u;
        uint32_t ks = 1;
        while (ks < 16 && p.tiles * p.splits * ks < slots && ks * 2 <= p.slice_blocks) ks *= 2;
        if (P > 1 && ks > 8) ks = 8;  // sixteen-wave workgroups leave 128 registers a lane, too few for several activation rows
        // waves per workgroup: four measured best (larger workgroups stage the activations less often but stream slower)
        uint32_t nw = 4;
        if (nw < ks) nw = ks;
        const uint32_t tiles_per_group = nw / ks;
        const size_t staged = mfma_staged(p.slice_blocks, P);
        const size_t lds = staged + (ks > 1 ? (size_t)2 * nw * P * 64u : 0);
        uint32_t blocks_x = (p.tiles + tiles_per_group - 1) / tiles_per_group;
        // resident waves per compute unit, by register use: 4 per SIMD (one or two activation rows), 3 for four
        uint32_t resident = (P == 4 ? 12u : 16u) / nw;
        const uint32_t by_lds = (uint32_t)((160 * 1024) / (lds + 1536));
        if (resident > by_lds) resident = by_lds;
        uint32_t most = (uint32_t)d->compute_units * (resident ? resident : 1u) / p.splits;
        if (most < 1) most = 1;
        if (blocks_x > most) blocks_x = most;
        profile_mark(d);
        hipError_t launched;
#define NH_MFMA_CASE(KK, WW) if (ks == KK && nw == WW) launched = launch_mfma_kernel<KK, WW>(d, p, P, blocks_x, lds); else
        NH_MFMA_CASE(1, 4) NH_MFMA_CASE(2, 4) NH_MFMA_CASE(4, 4)
        NH_MFMA_CASE(1, 8) NH_MFMA_CASE(2, 8) NH_MFMA_CASE(4, 8) NH_MFMA_CASE(8, 8)
        NH_MFMA_CASE(1, 16) NH_MFMA_CASE(2, 16) NH_MFMA_CASE(4, 16) NH_MFMA_CASE(8, 16)
        launched = launch_mfma_kernel<16, 16>(d, p, P, blocks_x, lds);
#undef NH_MFMA_CASE
        NH_HIP(launched);
        if (p.splits > 1) {
            hipLaunchKernelGGL(gemv_fold_kernel, dim3((outputs * p.rows + 255) / 256), dim3(256), 0, d->stream, p.partial, p.splits, p.rows, a.N,
                               p.residual, a.swiglu, p.y);
            NH_HIP(hipGetLastError());
        }
        profile_mark(d);
        if (d->profile) d->profile_bytes += (uint64_t)a.N * p.row_bytes;
        done += p.rows;
    }
    return NH_OK;
}

// mirrors the conditions under which launch_rows<1> takes the decode kernel with two rows per pass
static bool mfma32_takes(const nh_device *d, const GemvArgs &a);

bool gemv_fuses_rope(const GemvArgs &a, const RopeFusion &rope) {
    if (env_int("NEURA_HIP_FUSE_ROPE", 1) == 0) return false;
    if (a.rows >= 5 && a.rows <= 8) {  // one token of each of five to eight planes: the 32-row integer tiles
        GemvArgs folded = a;
        folded.rope = &rope;
        return !((uintptr_t)rope.cosines & 3u) && rope.positions > 0 && mfma32_takes(nullptr, folded);
    }
    if (a.rows != 1 || a.swiglu || a.residual) return false;
    {
        GemvArgs folded = a;
        folded.rope = &rope;
        if (tile16_takes(folded) || q6k_tile16_takes(folded)) return true;
    }
    if (a.element == NH_Q8_0) {
        // the direct Q8_0 decode kernel, a row of blocks inside one wave
        if (a.K % 32u != 0 || a.K > 2048u ) return false;
        if (a.N >= 16384u || a.N < 2u || (uint64_t)a.N * (a.K / 32u * 34u) >= (1ull << 32)) return false;
        if (a.end[0] % 2u || a.end[1] % 2u || a.N % 2u) return false;
    } else {
        if (a.element != NH_Q4_K || a.K % 256u != 0 || a.K > 4096u) return false;
        if (a.N >= 16384u || a.N < 2u || (uint64_t)a.N * (a.K / 256u * 144u) >= (1ull << 32)) return false;
    }
    if (env_int("NEURA_HIP_MFMA", 1) == 2) return false;
    const uint32_t width = rope.width;
    if (width < 2 || (width & (width - 1u)) != 0) return false;
    if (rope.q_rows % width || rope.k_rows % width || a.N % width || rope.q_rows > rope.k_rows || rope.k_rows > a.N) return false;
    // a head never straddles two matrices
    return a.end[0] % width == 0 && a.end[1] % width == 0 && a.end[2] == a.N;
}

// LDS of the 32-row tile kernel: digits, (unscale, sum) pairs, two rounds of partial sums, a raw super-block per wave
static size_t mfma32_lds(uint32_t nblk, uint32_t J, uint32_t NW) {
    return (size_t)nblk * 64u * 8u * J * 4u + (size_t)nblk * 8u * 2u * J * 8u + (size_t)2 * NW * J * 64u * 4u + (J == 1 ? (size_t)NW * 288u * 16u : 0u);
}

// whether the 32-row tile kernel serves this product: NEURA_HIP_MFMA32 = 0 never, 2 wherever it can, 1 (default) where
// it measured faster -- several activation rows, or one row against a tall matrix
static bool mfma32_takes(const nh_device *d, const GemvArgs &a) {
    const int mode = env_int("NEURA_HIP_MFMA32", 1);
    if (mode == 0 || a.element != NH_Q4_K || a.K % 256u != 0 || a.rows > 8) return false;
    if (a.rope) {
        // five to eight planes of one token each, rows of one K slice, heads of whole 32-row tiles that never straddle two matrices
        const uint32_t width = a.rope->width;
        if (a.rows < 5 || a.K > 3584u || a.swiglu || a.residual || width < 32u || width % 32u || a.N % width || a.end[0] % width || a.end[1] % width ||
            a.end[2] != a.N || a.rope->q_rows % width || a.rope->k_rows % width || a.rope->q_rows > a.rope->k_rows || a.rope->k_rows > a.N)
            return false;
    }
    // deeper rows go in K slices with a fold behind them: worth it from five activation rows on, and never with a fused norm
    if (a.K > 4096u && (a.norm_w || (mode != 2 && a.rows < 5))) return false;
    if (a.swiglu) {
        if (a.N % 2u || a.end[0] != a.N / 2 || (a.N / 2) % 16u != 0) return false;
    } else if (a.N % 32u != 0 || a.end[0] % 32u != 0 || a.end[1] % 32u != 0) {
        return false;
    }
    if (((uintptr_t)a.x & 15u) || (a.norm_w && ((uintptr_t)a.norm_w & 15u))) return false;
    const uint32_t J = a.rows <= 2 ? 1u : 4u;
    if (a.K <= 4096u && mfma32_lds(a.K / 256u, J, 16u) > 156u * 1024u) return false;  // eight rows of 4096 activations leave no room
    if (mode == 2) return true;
    // measured on the 7B shapes against the vector and 4 x 4 x 4 kernels: two rows win everywhere, five to eight rows
    // win everywhere, three and four rows (which pay for eight) win on short and on very tall matrices only; one row
    // never does (the vector kernel keeps its activations in registers)
    if (a.rows == 2 || a.rows >= 5) return true;
    return a.rows >= 3 && (a.N >= 65536u || a.N <= 8192u);
}

template <int J, int NW, int KS, bool ROPE = false>
static int32_t launch_mfma32_instance(nh_device *d, const MfmaParams &p, size_t lds) {
    static bool widened = false;  // past 64 KiB of dynamic LDS a kernel has to be told once
    if (lds > 64 * 1024 && !widened) {
        NH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_q4k_mfma32_kernel<J, NW, KS, ROPE>), hipFuncAttributeMaxDynamicSharedMemorySize, 158 * 1024));
        widened = true;
    }
    // one resident round of workgroups, as many as LDS and registers let a compute unit hold
    uint32_t resident = (uint32_t)((159 * 1024) / (lds + 1280));
    const uint32_t by_waves = NW == 16 ? 1u : 12u / NW;
    if (resident > by_waves) resident = by_waves;
    if (resident < 1) resident = 1;
    uint32_t blocks_x = (p.tiles + NW / KS - 1) / (NW / KS);
    uint32_t most = (uint32_t)d->compute_units * resident / p.splits;
    if (most < 1) most = 1;
    if (blocks_x > most) blocks_x = most;
    hipLaunchKernelGGL((gemv_q4k_mfma32_kernel<J, NW, KS, ROPE>), dim3(blocks_x, p.splits), dim3(NW * 64), lds, d->stream, MFMA_LEAD(p));
    NH_HIP(hipGetLastError());
    return NH_OK;
}

static int32_t launch_mfma32(nh_device *d, const GemvArgs &a) {
    MfmaParams p{};
    for (int s = 0; s < 3; s++) {
        p.W[s] = static_cast<const uint8_t *>(a.W[s] ? a.W[s] : a.W[0]);
        p.end[s] = a.end[s];
    }
    p.x = a.x, p.y = a.y, p.residual = a.residual, p.norm_w = a.norm_w;
    p.N = a.N, p.K = a.K, p.nblk = a.K / 256u, p.row_bytes = p.nblk * 144u, p.rows = a.rows;
    p.swiglu = a.swiglu, p.eps = a.eps;
    p.tiles = a.N / 32u;
    if (a.rope) {
        p.rope_cosines = a.rope->cosines, p.rope_sines = a.rope->sines, p.rope_cursor = a.rope->cursor, p.rope_k = a.rope->cache_k, p.rope_v = a.rope->cache_v;
        p.rope_width = a.rope->width, p.rope_q_rows = a.rope->q_rows, p.rope_k_rows = a.rope->k_rows, p.rope_capacity = a.rope->capacity;
        p.rope_positions = a.rope->positions, p.rope_ring = a.rope->ring, p.rope_element = a.rope->element;
        p.refusal = d->refusal;
        for (int s = 0; s < 3; s++) p.bias[s] = a.bias[s];
    }
    const uint32_t J = a.rows <= 2 ? 1u : 4u;  // a two-pair form spilled at 128 registers; three and four rows take the four-pair one
    // K slices: at most 14 super-blocks with eight staged rows (the digits of 3584 activations x 8 rows fill 112 KiB), 16 otherwise
    const uint32_t most_blocks = J == 4 ? 14u : 16u;
    p.splits = (p.nblk + most_blocks - 1) / most_blocks;
    p.slice_blocks = (p.nblk + p.splits - 1) / p.splits;
    p.splits = (p.nblk + p.slice_blocks - 1) / p.slice_blocks;
    if (p.splits > 1) {
        p.partial = static_cast<float *>(scratch(d, (size_t)p.splits * p.rows * a.N * sizeof(float)));
        if (!p.partial) return NH_E_MEMORY;
    }
    profile_mark(d);
    int32_t status;
    // with eight staged rows, a matrix of few tiles deals each tile's super-blocks to sixteen waves instead of four
    // (ffn_down of the 7B shape at eight rows, 112 tiles in six slices, is among the few: 22.0 -> 21.0 us)
    const bool few = p.tiles * p.splits < 3u * (uint32_t)d->compute_units;
    if (a.rope) status = few ? launch_mfma32_instance<4, 16, 16, true>(d, p, mfma32_lds(p.slice_blocks, 4, 16)) : launch_mfma32_instance<4, 16, 4, true>(d, p, mfma32_lds(p.slice_blocks, 4, 16));
    else if (J == 1) status = launch_mfma32_instance<1, 4, 4>(d, p, mfma32_lds(p.slice_blocks, 1, 4));
    else if (few) status = launch_mfma32_instance<4, 16, 16>(d, p, mfma32_lds(p.slice_blocks, 4, 16));
    else status = launch_mfma32_instance<4, 16, 4>(d, p, mfma32_lds(p.slice_blocks, 4, 16));
    if (status != NH_OK) return status;
    if (p.splits > 1) {
        const uint32_t outputs = a.swiglu ? a.N / 2 : a.N;
        hipLaunchKernelGGL(gemv_fold_kernel, dim3((outputs * p.rows + 255) / 256), dim3(256), 0, d->stream, p.partial, p.splits, p.rows, a.N,
                           p.residual, a.swiglu, p.y);
        NH_HIP(hipGetLastError());
    }
    profile_mark(d);
    if (d->profile) d->profile_bytes += (uint64_t)a.N * p.row_bytes;
    return NH_OK;
}

// whether the half-precision tile kernel serves this product: NEURA_HIP_F16_TILES = 0 never, 2 wherever it can (two to eight
// activation rows), 1 (default) where it measured faster than the integer tiles on the 7B shapes -- five to eight rows
// against a matrix of enough tiles to give every wave several super-blocks (gate|up 36.6 against 42 us, the head 91 against
// 110, ffn_down 29 against 27 with its fold; q|k|v and the output projection, one super-block a wave, are slower: 16.2 and
// 12.5 against 11.4 and 11.2)
static size_t f16_tiles_lds(uint32_t blocks, uint32_t NW) {
    return (size_t)blocks * F16_BLOCK_PIECES * 16u + (size_t)(blocks <= F16_TWO_SETS_BLOCKS ? 2u : 1u) * NW * 4u * 64u * sizeof(float);
}
static bool f16_tiles_take(const nh_device *d, const GemvArgs &a) {
    const int mode = env_int("NEURA_HIP_F16_TILES", 1);
    if (mode == 0 || a.element != NH_Q4_K || a.rope || a.K % 256u != 0 || a.rows < 2 || a.rows > 8) return false;
    if (mode != 2 && (a.rows < 5 || a.K > 4096u || a.N / 16u < 4u * (uint32_t)d->compute_units)) return false;
    if (a.K > 4096u && a.norm_w) return false;  // a fused norm wants the whole row in one slice
    if (a.swiglu) {
        if (a.N % 2u || a.end[0] != a.N / 2 || (a.N / 2) % 8u != 0) return false;
    } else if (a.N % 16u != 0 || a.end[0] % 16u != 0 || a.end[1] % 16u != 0) {
        return false;
    }
    for (int s = 0; s < 3; s++)
        if (a.W[s] && ((uintptr_t)a.W[s] & 15u)) return false;
    return !(((uintptr_t)a.x & 15u) || (a.norm_w && ((uintptr_t)a.norm_w & 15u)));
}

template <int NW, int KS>
static int32_t launch_f16_tiles_instance(nh_device *d, const MfmaParams &p, size_t lds) {
    static bool widened = false;  // past 64 KiB of dynamic LDS a kernel has to be told once
    if (lds > 64 * 1024 && !widened) {
        NH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_q4k_f16_kernel<NW, KS>), hipFuncAttributeMaxDynamicSharedMemorySize, 158 * 1024));
        widened = true;
    }
    uint32_t resident = (uint32_t)((159 * 1024) / (lds + 1280));
    if (resident > 1) resident = 1;  // sixteen waves a workgroup
    if (resident < 1) resident = 1;
    uint32_t blocks_x = (p.tiles + NW / KS - 1) / (NW / KS);
    uint32_t most = (uint32_t)d->compute_units * resident / p.splits;
    if (most < 1) most = 1;
    if (blocks_x > most) blocks_x = most;
    hipLaunchKernelGGL((gemv_q4k_f16_kernel<NW, KS>), dim3(blocks_x, p.splits), dim3(NW * 64), lds, d->stream, MFMA_LEAD(p));
    NH_HIP(hipGetLastError());
    return NH_OK;
}

static int32_t launch_f16_tiles(nh_device *d, const GemvArgs &a) {
    MfmaParams p{};
    for (int s = 0; s < 3; s++) {
        p.W[s] = static_cast<const uint8_t *>(a.W[s] ? a.W[s] : a.W[0]);
        p.end[s] = a.end[s];
    }
    p.x = a.x, p.y = a.y, p.residual = a.residual, p.norm_w = a.norm_w;
    p.N = a.N, p.K = a.K, p.nblk = a.K / 256u, p.row_bytes = p.nblk * 144u, p.rows = a.rows;
    p.swiglu = a.swiglu, p.eps = a.eps;
    p.tiles = a.N / 16u;
    // K slices: 16 super-blocks stage in 136 KiB
    const uint32_t most_blocks = 16u;
    p.splits = (p.nblk + most_blocks - 1) / most_blocks;
    p.slice_blocks = (p.nblk + p.splits - 1) / p.splits;
    p.splits = (p.nblk + p.slice_blocks - 1) / p.slice_blocks;
    if (p.splits > 1) {
        p.partial = static_cast<float *>(scratch(d, (size_t)p.splits * p.rows * a.N * sizeof(float)));
        if (!p.partial) return NH_E_MEMORY;
    }
    profile_mark(d);
    // sixteen waves a tile: a workgroup walks one tile at a time, so the tiles deal evenly over the compute units (with four waves
    // a tile and four tiles a round, gate|up's 2368 tiles were 2.3 rounds a workgroup, walked as three: batch 8 2.90 -> 2.78 ms a step)
    const size_t lds = f16_tiles_lds(p.slice_blocks, 16);
    int32_t status = launch_f16_tiles_instance<16, 16>(d, p, lds);
    if (status != NH_OK) return status;
    if (p.splits > 1) {
        const uint32_t outputs = a.swiglu ? a.N / 2 : a.N;
        hipLaunchKernelGGL(gemv_fold_kernel, dim3((outputs * p.rows + 255) / 256), dim3(256), 0, d->stream, p.partial, p.splits, p.rows, a.N,
                           p.residual, a.swiglu, p.y);
        NH_HIP(hipGetLastError());
    }
    profile_mark(d);
    if (d->profile) d->profile_bytes += (uint64_t)a.N * p.row_bytes;
    return NH_OK;
}

// Q6_K, Q5_K, Q3_K: one, two or four activation rows a launch (their slices and the raw rows share LDS: three workgroups a compute unit)
template <int ELEMENT, int RB>
static int32_t launch_staged_rows(nh_device *d, const GemvArgs &a, const float *x, float *y, const float *residual) {
    GemvParams p{};
    for (int s = 0; s < 3; s++) {
        p.W[s] = static_cast<const uint8_t *>(a.W[s] ? a.W[s] : a.W[0]);
        p.end[s] = a.end[s];
    }
    p.x = x, p.y = y, p.residual = residual, p.norm_w = a.norm_w;
    p.N = a.N, p.K = a.K, p.swiglu = a.swiglu, p.eps = a.eps;
    p.row_bytes = (uint32_t)payload_bytes(ELEMENT, a.K);
    p.nblk = a.K / 256u;
    if (a.append_value) {
        if (RB != 1 || a.swiglu || residual || p.nblk > 16u || !a.append_value->width || a.N % a.append_value->width)
            return fail(NH_E_ARGUMENT, "this product appends no value rows (one row, one K slice, whole heads, no other epilogue)");
        p.append_value = 1u, p.rope_v = a.append_value->cache_v, p.rope_cursor = a.append_value->cursor, p.rope_width = a.append_value->width;
        p.rope_capacity = a.append_value->capacity, p.rope_ring = a.append_value->ring, p.rope_element = a.append_value->element, p.bias[0] = a.bias[0], p.refusal = d->refusal;
    }
    // K slices of sixteen super-blocks at most; of eight with four activation rows, whose slices take the room of two rows' twice over
    const uint32_t most_blocks = RB == 4 ? 8u : 16u;
    p.splits = (p.nblk + most_blocks - 1) / most_blocks;
    p.blocks_per_split = (p.nblk + p.splits - 1) / p.splits;
    p.splits = (p.nblk + p.blocks_per_split - 1) / p.blocks_per_split;
    if (p.splits > 1) {
        p.partial = static_cast<float *>(scratch(d, (size_t)p.splits * RB * a.N * sizeof(float)));
        if (!p.partial) return NH_E_MEMORY;
    }
    p.chunks_per_row = (15u + p.blocks_per_split * Staged<ELEMENT>::BYTES + 15u) / 16u + 1u;  // a lead, the blocks, and the word past the last field
    // activation slices (8 floats of skew a block), their sums per eight, the raw rows
    const size_t lds = (size_t)RB * p.blocks_per_split * (264u + 32u) * sizeof(float) + (size_t)8 * p.chunks_per_row * 16u;
    uint32_t blocks_x = (a.N + 7u) / 8u;
    // three workgroups a compute unit: their LDS (about 41 KiB each at 14 blocks) and registers fit, and a fourth measured slower
    uint32_t most = (uint32_t)d->compute_units * 3u / p.splits;
    if (most < 1) most = 1;
    if (blocks_x > most) blocks_x = most;
    profile_mark(d);
    if (lds > 64u * 1024u) {
        static bool widened = false;  // past 64 KiB of dynamic LDS a kernel has to be told once
        if (!widened) {
            NH_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_staged_kernel<ELEMENT, RB>), hipFuncAttributeMaxDynamicSharedMemorySize, 158 * 1024));
            widened = true;
        }
    }
    hipLaunchKernelGGL((gemv_staged_kernel<ELEMENT, RB>), dim3(blocks_x, p.splits), dim3(256), lds, d->stream, GEMV_LEAD(p));
    NH_HIP(hipGetLastError());
    if (p.splits > 1) {
        uint32_t outputs = (a.swiglu ? a.N / 2 : a.N) * RB;
        hipLaunchKernelGGL(gemv_fold_kernel, dim3((outputs + 255) / 256), dim3(256), 0, d->stream, p.partial, p.splits, (uint32_t)RB, a.N,
                           residual, a.swiglu, y);
        NH_HIP(hipGetLastError());
    }
    profile_mark(d);
    if (d->profile) d->profile_bytes += (uint64_t)a.N * p.row_bytes;
    return NH_OK;
}

// What the Q8_0 decode kernel of two rows a lane group takes (launch_rows<1> sends such a product there), and the merge's own
// bounds: whole heads, no more of them than the statistics' corner of LDS holds.
bool gemv_merges_sections(const GemvArgs &a, uint32_t width) {
    if (!env_int("NEURA_HIP_MERGE_IN_PRODUCT", 1) || a.element != NH_Q8_0 || a.rows != 1 || a.rope || a.swiglu || a.norm_w || a.digits_in || a.digits_out) return false;
    if (!width || (width & (width - 1u)) || a.K % 32u || a.K / 32u > 64u || a.K % width || a.K / width > 32u) return false;
    if (a.N < 2u || a.N >= 16384u || a.N % 2u || a.end[0] % 2u || a.end[1] % 2u) return false;
    return (uint64_t)a.N * payload_bytes(a.element, a.K) < (1ull << 32);
}

// Whether a product with `append_value` set casts its rows into the value state itself: one row of a K-quant on the 16-row
// tiles, or on the staged kernel where a row is one K slice.
bool gemv_appends_value(const GemvArgs &a) {
    if (!a.append_value || a.rows != 1 || a.rope || a.swiglu || a.residual) return false;
    if (tile16_takes(a) || q6k_tile16_takes(a)) return true;
    return staged_super_block(a.element) && a.K <= 4096u && a.append_value->width && a.N % a.append_value->width == 0;
}

int32_t launch_gemv(nh_device *d, const GemvArgs &a) {
    if (!a.rope && !a.append_value && (a.bias[0] || a.bias[1] || a.bias[2]))
        return fail(NH_E_ARGUMENT, "a product adds a bias only where it folds the rotation in or appends value rows");
    if (a.append_value && !gemv_appends_value(a))
        return fail(NH_E_ARGUMENT, "this product does not append its rows to the value state (ask gemv_appends_value first)");
    if (a.merge && (!gemv_merges_sections(a, a.merge->width) || a.merge->sections < 2u || a.merge->sections > MERGED_SECTIONS_MOST || !a.merge->groups ||
                    (a.K / a.merge->width) % a.merge->groups))
        return fail(NH_E_ARGUMENT, "this product merges no attention sections (ask gemv_merges_sections first)");
    if (a.merge) return launch_rows<1>(d, a, a.x, a.y, a.residual);
    if (rows4_takes(a)) return launch_rows4(d, a);
    if (tile16_takes(a)) return launch_tile16(d, a);
    if (q6k_tile16_takes(a)) return launch_q6k_tile16(d, a);
    if (a.digits_out || a.digits_in) return fail(NH_E_ARGUMENT, "this product hands over no digit planes (ask gemv_hands_digits first)");
    if (a.rope && a.rows != 1) {  // several planes: the 32-row integer tiles or nothing
        if (!mfma32_takes(d, a)) return fail(NH_E_ARGUMENT, "this product cannot fold the rotation in (ask gemv_fuses_rope first)");
        return launch_mfma32(d, a);
    }
    if (a.rope && mfma_takes(a)) return fail(NH_E_ARGUMENT, "this product cannot fold the rotation in (ask gemv_fuses_rope first)");
    if (f16_tiles_take(d, a)) return launch_f16_tiles(d, a);
    if (mfma32_takes(d, a)) return launch_mfma32(d, a);
    if (mfma_takes(a)) return launch_mfma(d, a);
    // activation rows are taken four, two or one at a time
    uint32_t outputs = a.swiglu ? a.N / 2 : a.N;
    uint32_t done = 0;
    if (staged_super_block(a.element)) {
        if (a.swiglu && (a.N % 2u || a.end[0] != a.N / 2)) return fail(NH_E_ARGUMENT, "a swiglu product halves %u rows", a.N);
        while (done < a.rows) {
            const float *x = a.x + (size_t)done * a.K;
            float *y = a.y + (size_t)done * outputs;
            const float *residual = a.residual ? a.residual + (size_t)done * a.N : nullptr;
            const bool pair = a.rows - done >= 2;
            const bool four = a.rows - done >= 4;  // (the Q4_K_M mix at eight planes: 5.77 -> 5.46 ms a step against two rows a pass)
            int32_t status;
            if (a.element == NH_Q6_K)
                status = four ? launch_staged_rows<NH_Q6_K, 4>(d, a, x, y, residual)
                         : pair ? launch_staged_rows<NH_Q6_K, 2>(d, a, x, y, residual) : launch_staged_rows<NH_Q6_K, 1>(d, a, x, y, residual);
            else if (a.element == NH_Q5_K)
                status = four ? launch_staged_rows<NH_Q5_K, 4>(d, a, x, y, residual)
                         : pair ? launch_staged_rows<NH_Q5_K, 2>(d, a, x, y, residual) : launch_staged_rows<NH_Q5_K, 1>(d, a, x, y, residual);
            else
                status = four ? launch_staged_rows<NH_Q3_K, 4>(d, a, x, y, residual)
                         : pair ? launch_staged_rows<NH_Q3_K, 2>(d, a, x, y, residual) : launch_staged_rows<NH_Q3_K, 1>(d, a, x, y, residual);
            if (status != NH_OK) return status;
            done += four ? 4 : (pair ? 2 : 1);
        }
        return NH_OK;
    }
    while (done < a.rows) {
        uint32_t left = a.rows - done;
        const float *x = a.x + (size_t)done * a.K;
        float *y = a.y + (size_t)done * outputs;
        const float *residual = a.residual ? a.residual + (size_t)done * a.N : nullptr;
        int32_t status;
        if (left >= 4) {
            status = launch_rows<4>(d, a, x, y, residual);
            done += 4;
        } else if (left >= 2) {
            status = launch_rows<2>(d, a, x, y, residual);
            done += 2;
        } else {
            status = launch_rows<1>(d, a, x, y, residual);
            done += 1;
        }
        if (status != NH_OK) return status;
    }
    return NH_OK;
}

}  // namespace nh
