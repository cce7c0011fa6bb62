// What the narrow-product kernels of gemv.hip and gemv_tile16.hip share: the kernel parameters, the branch-free decode of
// the Q4_K block scales, lane exchanges and the rotation's epilogue.
#pragma once
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
    uint32_t tile_rows;         // 16-row tile kernel, plain epilogue: weight rows a tile holds (12..16)
    uint32_t rows;              // 16-row tile kernel: activation rows of x (1..8)
    uint32_t chunks_per_row;    // Q8_0: 16-byte chunks of a staged row slice
    int32_t swiglu;
    float eps;
    // rotation folded into the product (decode kernel only): see RopeFusion
    const float *rope_cosines, *rope_sines;  // [position][width / 2]
    const uint32_t *rope_cursor;
    uint16_t *rope_k, *rope_v;
    uint32_t rope_width, rope_q_rows, rope_k_rows, rope_capacity, rope_positions, rope_ring;
    int32_t rope_element;  // what the states hold: NH_F16 (0 is NH_F32: launchers always name it), NH_BF16 or NH_F32
    uint32_t *refusal;
    const float *bias[3];  // per stacked matrix or nullptr (decode kernel with the rotation folded in only)
    // 16-row tile kernel: activations handed from one product to the next as the digit planes the matrix cores take
    // (gemv_digit_bytes() of them): written by a SwiGLU epilogue in place of y, read by a plain product in place of x
    uint8_t *digits_out;
    const uint8_t *digits_in;
    // Q8_0 decode kernel: x is the unmerged section sums of a decode attention (SectionSums), merged as the row is staged
    uint32_t merge_sections, merge_groups, merge_width;
    // staged K-quant kernel, one row: the outputs (+ bias[0]) also go into the value state rope_v at rope_cursor as halves
    uint32_t append_value;
    // 16-row tile kernel: what is handed to another product carries tag words (gemv_tile16.hip): `tick` is the device word a
    // step's first kernel moves on, tag_in / tag_out the numbers (1..127) of the seams this product reads and writes across,
    // pairs_out where a plain product of a chained launch leaves its outputs as (value, tag) pairs beside y
    const uint32_t *tick;
    uint32_t tag_in, tag_out;
    uint2 *pairs_out;
    uint32_t late_from;  // handed planes behind a seam: the first super-block whose chunks the product before writes in its last round
};

// the parameters a product reads before its first vector load, and the rotation's where it is folded in
__device__ __forceinline__ void fetch_parameters(const GemvParams &p, bool rope = false) {
    NH_FETCH(p.W[0], p.W[1], p.W[2], p.end[0], p.end[1], p.end[2], p.x, p.y, p.residual, p.norm_w, p.partial, p.N, p.K, p.row_bytes, p.nblk,
             p.blocks_per_split, p.splits, p.group, p.row_groups, p.tile_rows, p.rows, p.chunks_per_row, p.swiglu, p.eps, p.rope_width, p.digits_in,
             p.digits_out);
    if (rope)
        NH_FETCH(p.rope_cosines, p.rope_sines, p.rope_cursor, p.rope_k, p.rope_v, p.rope_q_rows, p.rope_k_rows, p.rope_capacity, p.rope_positions, p.rope_ring,
                 p.rope_element, p.bias[0], p.bias[1], p.bias[2], p.refusal);
}

// What a wave of a K-quant product needs before its first loads, as leading plain arguments the hardware hands over in scalar
// registers when it starts the wave (the activation rows and a tile's rows ride above the super-blocks a row, the SwiGLU flag
// above N); they take the place of the same members of the parameter block, whose other members are loaded as they come to use.
#define GEMV_LEAD_PARAMETERS                                                                                                                          \
    const uint8_t *lead_w0, const uint8_t *lead_w1, const uint8_t *lead_w2, const float *lead_x, uint32_t lead_row_bytes, uint32_t lead_nblk_rows,      \
        uint32_t lead_row_groups, uint32_t lead_n_swiglu, uint32_t lead_end0, uint32_t lead_end1, GemvParams rest
#define GEMV_LEAD(p)                                                                                                                                   \
    (p).W[0], (p).W[1], (p).W[2], (p).x, (p).row_bytes, (p).nblk | ((p).rows << 16) | ((p).tile_rows << 24), (p).row_groups,                           \
        (p).N | ((p).swiglu ? 0x80000000u : 0u), (p).end[0], (p).end[1], (p)
#define GEMV_TAKE_LEAD                                                                                                                                 \
    GemvParams p = rest;                                                                                                                               \
    p.W[0] = lead_w0, p.W[1] = lead_w1, p.W[2] = lead_w2, p.x = lead_x, p.row_bytes = lead_row_bytes, p.row_groups = lead_row_groups;                   \
    p.nblk = lead_nblk_rows & 0xffffu, p.rows = (lead_nblk_rows >> 16) & 0xffu, p.tile_rows = lead_nblk_rows >> 24, p.K = 256u * (lead_nblk_rows & 0xffffu); \
    p.N = lead_n_swiglu & 0x7fffffffu, p.swiglu = (int32_t)(lead_n_swiglu >> 31), p.end[0] = lead_end0, p.end[1] = lead_end1

__device__ __forceinline__ float silu(float a) { return a * (1.0f / (1.0f + expf(-a))); }

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// ---- cross-lane sums without LDS round trips ---------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
constexpr int DPP_QUAD_XOR1 = 0xB1;  // quad_perm [1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;  // quad_perm [2,3,0,1]
constexpr int DPP_ROW_ROR4 = 0x124, DPP_ROW_ROR8 = 0x128;

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

// one number into a key or value state of `element` (crates/neura-decoder/src/cache.rs:347-348 casts as it appends)
__device__ __forceinline__ void state_store(uint16_t *state, int32_t element, uint64_t at, float value) {
    if (element == NH_F32) reinterpret_cast<float *>(state)[at] = value;
    else state[at] = element == NH_BF16 ? float_to_bfloat16(value) : float_to_half(value);
}

// One rotated output of a q|k|v product that folds the rotation in: `total` is output row n (channel c of its head's first
// half, or c + width/2 when `second`), the lane 8 further round its row of 16 holds the partner channel.  The projection's
// bias, if it has one, comes before the rotation; q rows go to y, k rows rotated and v rows as they are to the caches as
// halves, at the cursor (at cursor mod span in a ring).  Lanes 0..15 of a wave call it together
// (crates/neura-kernel/src/task/rope.rs:95-122).  What it reads from memory can be fetched ahead with rope_operands().
struct RopeOperands {
    float bias, cosine, sine;
};

__device__ __forceinline__ RopeOperands rope_operands(const GemvParams &p, uint32_t n, uint32_t c, uint32_t position) {
    const uint32_t half = p.rope_width >> 1;
    const float *b0 = p.bias[0], *b1 = p.bias[1], *b2 = p.bias[2];
    const uint32_t e0 = p.end[0], e1 = p.end[1];
    const float *bias = n < e0 ? b0 : (n < e1 ? b1 : b2);
    const uint32_t before = n < e0 ? 0u : (n < e1 ? e0 : e1);
    RopeOperands held{0.0f, 1.0f, 0.0f};
    if (bias) held.bias = bias[n - before];
    if (n < p.rope_k_rows) {
        // cos and sin of f32(position) * pow(base, -2c/width), tabulated once per model by the rotation's own kernel
        held.cosine = p.rope_cosines[(size_t)min(position, p.rope_positions - 1u) * half + c];
        held.sine = p.rope_sines[(size_t)min(position, p.rope_positions - 1u) * half + c];
    }
    return held;
}

__device__ __forceinline__ void rope_store(const GemvParams &p, float total, uint32_t n, bool second, uint32_t position, const RopeOperands &held) {
    {
        const float *b0 = p.bias[0], *b1 = p.bias[1], *b2 = p.bias[2];
        const float *bias = n < p.end[0] ? b0 : (n < p.end[1] ? b1 : b2);
        if (bias) total += held.bias;
    }
    const float other = dpp<DPP_ROW_ROR8>(total);
    float value = total;
    if (n < p.rope_k_rows) value = second ? total * held.cosine + other * held.sine : total * held.cosine - other * held.sine;
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

template <int CTRL>
__device__ __forceinline__ int dpp_int(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, false);
}

// The four signed base-256 digits of an integer below 2^30 in magnitude, one per byte, least significant in byte 0:
// adding 128 at the three low byte positions makes every low byte the digit plus 128 (the carries are the ones the
// signed digits need), and flipping bit 7 takes the 128 off again.
__device__ __forceinline__ uint32_t signed_digits(int whole) { return ((uint32_t)whole + 0x00808080u) ^ 0x00808080u; }

// Sixteen outputs of a product as a chunk of the next product's activations: lanes 0..15 of a wave, each holding one output, turn
// them into three signed base-256 digit planes below a power-of-two scale of their own (the chunk's largest magnitude lands in
// [2^21, 2^22)) and return the word each writes of the chunk's 64-byte piece:
//   words 0..3 plane 0 | 4..6 plane 1, first twelve | 7 tag || 8 plane 1, last four | 9..11 plane 2, first twelve |
//   12 plane 2, last four | 13, 14 the (sum, scale) pair | 15 tag
// (the tag words end the piece's two 32-byte sectors: a reader behind a seam of one launch knows by them that a sector has arrived).
__device__ __forceinline__ uint32_t handed_piece_word(float value, uint32_t r, uint32_t tag) {
    uint32_t top = __builtin_bit_cast(uint32_t, value) & 0x7fffffffu;
    top = max(top, (uint32_t)dpp_int<DPP_QUAD_XOR1>((int)top));
    top = max(top, (uint32_t)dpp_int<DPP_QUAD_XOR2>((int)top));
    top = max(top, (uint32_t)dpp_int<DPP_ROW_ROR4>((int)top));
    top = max(top, (uint32_t)dpp_int<DPP_ROW_ROR8>((int)top));
    const uint32_t raw = top >> 23;
    const uint32_t exponent = min(max(raw, 22u), 254u);
    const float scale = __builtin_bit_cast(float, (275u - exponent) << 23);
    const float unscale = raw == 255u ? __builtin_bit_cast(float, 0x7fc00000u) : __builtin_bit_cast(float, (exponent - 21u) << 23);
    const float rounded = rintf(value * scale);
    float chunk_sum = rounded;
    chunk_sum += dpp<DPP_QUAD_XOR1>(chunk_sum);
    chunk_sum += dpp<DPP_QUAD_XOR2>(chunk_sum);
    chunk_sum += dpp<DPP_ROW_ROR4>(chunk_sum);
    chunk_sum += dpp<DPP_ROW_ROR8>(chunk_sum);
    const int dg = (int)signed_digits((int)rounded);
    const uint32_t plane = r < 4u ? 0u : (r < 9u ? 1u : 2u);
    const int first = (int)(r < 4u ? 4u * r : (r < 7u ? 4u * (r - 4u) : (r == 8u || r == 12u ? 12u : 4u * (r - 9u)))) & 15;
    const uint32_t d0 = (uint32_t)__shfl(dg, first, 16), d1 = (uint32_t)__shfl(dg, first + 1, 16);
    const uint32_t d2 = (uint32_t)__shfl(dg, first + 2, 16), d3 = (uint32_t)__shfl(dg, first + 3, 16);
    const uint32_t shift = 16u - 8u * plane;
    uint32_t word = ((d0 >> shift) & 0xffu) | (((d1 >> shift) & 0xffu) << 8) | (((d2 >> shift) & 0xffu) << 16) | (((d3 >> shift) & 0xffu) << 24);
    if (r == 13u) word = __builtin_bit_cast(uint32_t, chunk_sum * unscale);
    if (r == 14u) word = __builtin_bit_cast(uint32_t, unscale);
    if (r == 7u || r == 15u) word = tag;
    return word;
}

inline int env_int(const char *name, int fallback) {
    const char *held = getenv(name);
    return held && *held ? atoi(held) : fallback;
}

// Activations as the 16x16x64 integer MFMA takes them (gemv_tile16.hip, gemv_q6k_tile16.hip): per super-block of 256, sixteen
// chunks of 16 activations, each three signed base-256 digit planes of 16 bytes; where a chunk has a scale of its own, a
// (sum, scale) pair of floats beside it; in memory (handed from one product to the next) a chunk is one 64-byte piece
constexpr uint32_t TILE16_BLOCK_DIGITS = 768;
constexpr uint32_t TILE16_BLOCK_PAIRS = 128;
constexpr uint32_t TILE16_BLOCK_HANDED = 1024;

// the 16-row tile kernel (gemv_tile16.hip): whether it serves this product, and its launch
bool tile16_takes(const GemvArgs &args);
int32_t launch_tile16(nh_device *d, const GemvArgs &args);
// the same for two to eight activation rows, four rows to an MFMA
bool rows4_takes(const GemvArgs &args);
int32_t launch_rows4(nh_device *d, const GemvArgs &args);
// one activation row against a Q6_K matrix on the same tiles (gemv_q6k_tile16.hip)
bool q6k_tile16_takes(const GemvArgs &args);
int32_t launch_q6k_tile16(nh_device *d, const GemvArgs &args);
struct Q6kLaunch {  // what a launch of it is made of: the parameter block, waves a workgroup, workgroups, LDS
    GemvParams p;
    uint32_t waves, grid;
    size_t lds;
};
Q6kLaunch q6k_tile16_plan(nh_device *d, const GemvArgs &args);

}  // namespace nh
