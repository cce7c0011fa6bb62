// Narrow products (1..8 activation rows) over raw GGUF blocks: y[r][n] = sum_k x[r][k] * W[n][k].
//
// Q4_K: a super-block is 144 B = a 16 B header (d, dmin, 12 scale bytes) + 128 B of nibbles.
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

#include <cstdlib>

namespace nh {

struct GemvParams {
    const uint8_t *W[3];  // up to three matrices stacked along N (q|k|v, or gate|up with swiglu)
    uint32_t end[3];      // first output row past each matrix
    const float *x;
    float *y;
    const float *residual;
    const float *norm_w;
    float *partial;
    uint32_t N, K, row_bytes;
    uint32_t nblk;              // blocks per row
    uint32_t blocks_per_split;  // blocks of one K slice
    uint32_t splits;
    uint32_t group;             // lanes that share one output row: 16, 32 or 64
    uint32_t row_groups;        // passes over the rows
    uint32_t chunks_per_row;    // Q8_0: 16-byte chunks of a staged row slice
    int32_t swiglu;
    float eps;
};

// skewed LDS index of activation i: 4 floats of padding per 64 keep 128-bit reads of
// neighbouring lanes on different banks
__device__ __forceinline__ uint32_t skew64(uint32_t i) { return i + (i >> 6) * 4; }
__device__ __forceinline__ uint32_t skew32(uint32_t i) { return i + (i >> 5) * 4; }

// sum of squares of one activation row in the order of the reference's norm kernel
// (crates/neura-kernel/src/task/norm.rs:69-83 + reduce.rs:21-38): thread t adds columns
// t, t+256, ...; then a 256-wide tree.  Returns 1/sqrt(mean + eps) to every thread.
__device__ float rms_scale(const float *__restrict__ x, uint32_t K, float eps, float *red) {
    if (threadIdx.x < 256) {  // larger workgroups leave the sum to their first 256 threads
        float square = 0.0f;
        for (uint32_t c = threadIdx.x; c < K; c += 256) {
            float value = x[c];
            square = __fadd_rn(square, __fmul_rn(value, value));
        }
        red[threadIdx.x] = square;
    }
    __syncthreads();
    for (uint32_t stride = 128; stride > 0; stride >>= 1) {
        if (threadIdx.x < stride) red[threadIdx.x] = __fadd_rn(red[threadIdx.x], red[threadIdx.x + stride]);
        __syncthreads();
    }
    float total = red[0];
    __syncthreads();
    return rms_scale_of(total, K, eps);
}

__device__ __forceinline__ float silu(float a) { return a * (1.0f / (1.0f + expf(-a))); }

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

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

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

// ---- cross-lane sums without LDS round trips ---------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
constexpr int DPP_QUAD_XOR1 = 0xB1;  // quad_perm [1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;  // quad_perm [2,3,0,1]
constexpr int DPP_ROW_ROR4 = 0x124, DPP_ROW_ROR8 = 0x128;

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

// Per-lane constants of the branch-free scale decode (they depend on the lane's group only).
struct ScaleLane {
    uint32_t pick;    // byte selector: the two bytes of this group from the low or the high scale word
    uint32_t pick_q;  // byte selector: the two bytes that carry the top bits (groups 2, 3)
    uint32_t mask_p, mask_q;
    uint32_t shift_m;  // 4 for groups 2, 3: their minimums sit in the high nibbles
};

__device__ __forceinline__ ScaleLane scale_lane(uint32_t g) {
    const uint32_t j = 2u * (g & 1u);
    ScaleLane s;
    s.pick_q = 0x0c000c00u | j | ((j + 1u) << 16);
    s.pick = g < 2 ? s.pick_q : (0x0c000c00u | (4u + j) | ((5u + j) << 16));
    s.mask_p = g < 2 ? 0x003f003fu : 0x000f000fu;
    s.mask_q = g < 2 ? 0u : 0x00300030u;
    s.shift_m = g < 2 ? 0u : 4u;
    return s;
}

// The 6-bit scales (sc) and minimums (mn) of sub-blocks 2g, 2g+1 as pairs of half-precision
// subnormals (value * 2^-24 in each 16-bit lane), straight from the header words:
// crates/neura-precision/src/ggml.rs:127-136 without a branch or an int -> float conversion.
__device__ __forceinline__ void scale_pairs(const u32x4 &hdr, const ScaleLane &s, half2_t &sc, half2_t &mn) {
    const uint32_t p_sc = __builtin_amdgcn_perm(hdr.w, hdr.y, s.pick), q_sc = __builtin_amdgcn_perm(hdr.w, hdr.y, s.pick_q);
    const uint32_t p_mn = __builtin_amdgcn_perm(hdr.w, hdr.z, s.pick) >> s.shift_m, q_mn = __builtin_amdgcn_perm(hdr.w, hdr.z, s.pick_q);
    sc = __builtin_bit_cast(half2_t, (p_sc & s.mask_p) | ((q_sc >> 2) & s.mask_q));
    mn = __builtin_bit_cast(half2_t, (p_mn & s.mask_p) | ((q_mn >> 2) & s.mask_q));
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
template <int R, int G, bool PIPE, int NW>
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
            const uint32_t n = min(first, p.N - R);
            const bool in0 = n < p.end[0], in1 = n < p.end[1];
            const uint8_t *matrix = in0 ? p.W[0] : (in1 ? p.W[1] : p.W[2]);
            const uint32_t before = in0 ? 0u : (in1 ? p.end[0] : p.end[1]);
#pragma unroll
            for (int r = 0; r < R; r++) base[r] = matrix + (size_t)(n - before + r) * p.row_bytes;
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

    {
        float scale = 1.0f;
        if (p.norm_w) scale = rms_scale(p.x, p.K, p.eps, red);
        for (uint32_t i = tid; i < kn; i += NW * 64) {
            float value = p.x[k0 + i];
            if (p.norm_w) value = __fmul_rn(__fmul_rn(value, scale), p.norm_w[k0 + i]);
            xs[skew64(i)] = value;
        }
    }
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
    extern __shared__ float xs[];  // [RB][skew64(slice)]
    __shared__ float red[256];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t split = blockIdx.y;
    const uint32_t blk0 = split * p.blocks_per_split;
    const uint32_t nb = min(p.blocks_per_split, p.nblk - blk0);
    const uint32_t k0 = blk0 * 256u, kn = nb * 256u;
    const uint32_t xstride = skew64(p.blocks_per_split * 256u);

#pragma unroll
    for (int b = 0; b < RB; b++) {
        const float *xb = p.x + (size_t)b * p.K;
        float scale = 1.0f;
        if (p.norm_w) scale = rms_scale(xb, p.K, p.eps, red);
        for (uint32_t i = tid; i < kn; i += 256) {
            float value = xb[k0 + i];
            if (p.norm_w) value = __fmul_rn(__fmul_rn(value, scale), p.norm_w[k0 + i]);
            xs[b * xstride + skew64(i)] = value;
        }
    }
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
    for (int b = 0; b < RB; b++) {
        const float *xb = p.x + (size_t)b * p.K;
        float scale = 1.0f;
        if (p.norm_w) scale = rms_scale(xb, p.K, p.eps, red);
        for (uint32_t i = tid; i < kn; i += 256) {
            float value = xb[k0 + i];
            if (p.norm_w) value = __fmul_rn(__fmul_rn(value, scale), p.norm_w[k0 + i]);
            xs[b * xstride + skew32(i)] = value;
        }
    }
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

// ------------------------------------------------------------------------- fold ----------

// sums the slice partials in slice order and applies the epilogue
// (crates/neura-kernel/src/task/matmul.rs:1318-1333)
__global__ __launch_bounds__(256) void gemv_fold_kernel(const float *__restrict__ partial, uint32_t splits, uint32_t rows, uint32_t N,
                                                        const float *__restrict__ residual, int32_t swiglu, float *__restrict__ y) {
    uint32_t outputs = swiglu ? N / 2 : N;
    for (uint32_t index = blockIdx.x * blockDim.x + threadIdx.x; index < rows * outputs; index += gridDim.x * blockDim.x) {
        uint32_t b = index / outputs, n = index % outputs;
        float total = 0.0f;
        for (uint32_t s = 0; s < splits; s++) total += partial[((size_t)s * rows + b) * N + n];
        if (swiglu) {
            float up = 0.0f;
            for (uint32_t s = 0; s < splits; s++) up += partial[((size_t)s * rows + b) * N + N / 2 + n];
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

static int env_int(const char *name, int fallback) {
    const char *held = getenv(name);
    return held && *held ? atoi(held) : fallback;
}

template <int RB>
static int32_t launch_rows(nh_device *d, const GemvArgs &a, const float *x, float *y, const float *residual) {
    GemvParams p{};
    for (int s = 0; s < 3; s++) {
        p.W[s] = static_cast<const uint8_t *>(a.W[s] ? a.W[s] : a.W[0]);
        p.end[s] = a.end[s];
    }
    p.x = x;
    p.y = y;
    p.residual = residual;
    p.norm_w = a.norm_w;
    p.N = a.N;
    p.K = a.K;
    p.swiglu = a.swiglu;
    p.eps = a.eps;
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
    R = env_int("NEURA_HIP_GEMV_ROWS", R);
    if (R != 2 && R != 4) R = 2;
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
        uint32_t most = (uint32_t)d->compute_units * (uint32_t)env_int("NEURA_HIP_GEMV_WGS", R == 4 ? 3 : 4) / p.splits;
        if (most < 1) most = 1;
        if (blocks_x > most) blocks_x = most;
        uint32_t slice = p.blocks_per_split * 256u;
        lds = (size_t)RB * (slice + slice / 64 * 4) * sizeof(float);
    } else {
        uint32_t slice_bytes = p.blocks_per_split * 34u;
        p.chunks_per_row = (15u + slice_bytes + 15u) / 16u;
        uint32_t tiles = (p.row_groups + 3) / 4;
        blocks_x = tiles;
        uint32_t most = (uint32_t)d->compute_units * (uint32_t)env_int("NEURA_HIP_GEMV_WGS", 4) / p.splits;
        if (most < 1) most = 1;
        if (blocks_x > most) blocks_x = most;
        uint32_t slice = p.blocks_per_split * 32u;
        lds = (size_t)RB * (slice + slice / 32 * 4) * sizeof(float) + (size_t)rows_per_pass * 4 * p.chunks_per_row * 16 + 16;
    }
    if (lds > 64 * 1024) return fail(NH_E_ARGUMENT, "a product of depth %u stages %zu bytes where a workgroup holds 65536", a.K, lds);
    dim3 grid(blocks_x, p.splits), block(256);
    const bool pipe = env_int("NEURA_HIP_GEMV_PIPE", 0) != 0;
    const int nw = env_int("NEURA_HIP_GEMV_WAVES", 4);
    profile_mark(d);
#define NH_LAUNCH(KERNEL, RR) hipLaunchKernelGGL((KERNEL<RR, RB>), grid, block, lds, d->stream, p)
#define NH_DECODE(RR, GG)                                                                                              \
    do {                                                                                                               \
        if (pipe) hipLaunchKernelGGL((gemv_q4k_decode_kernel<RR, GG, true, 4>), grid, block, lds, d->stream, p);       \
        else if (nw == 16) hipLaunchKernelGGL((gemv_q4k_decode_kernel<RR, GG, false, 16>), dim3((blocks_x + 3) / 4, p.splits), dim3(1024), lds, d->stream, p); \
        else if (nw == 8) hipLaunchKernelGGL((gemv_q4k_decode_kernel<RR, GG, false, 8>), dim3((blocks_x + 1) / 2, p.splits), dim3(512), lds, d->stream, p); \
        else hipLaunchKernelGGL((gemv_q4k_decode_kernel<RR, GG, false, 4>), grid, block, lds, d->stream, p);           \
    } while (0)
    if (q4 && RB == 1 && fast) {
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

int32_t launch_gemv(nh_device *d, const GemvArgs &a) {
    // activation rows are taken four, two or one at a time
    uint32_t outputs = a.swiglu ? a.N / 2 : a.N;
    uint32_t done = 0;
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
