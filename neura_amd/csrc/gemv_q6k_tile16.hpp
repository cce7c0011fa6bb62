// The Q6_K and Q3_K products of one activation row on 16-row tiles of the 16x16x64 integer MFMA: the product as a device function (the
// kernel of its own is in gemv_q6k_tile16.hip; gemv_tile16.hip runs it beside a Q4_K product in one launch).
#pragma once
#include "gemv_shared.hpp"

namespace nh {

// ---------------------------------------------------------------------------------------------------------------------
// One activation row against a Q6_K matrix (crates/neura-kernel/src/dot.rs:663-797 weighs the same numbers 32 at a time).
//
// A Q6_K super-block is 210 bytes: 128 bytes of low nibbles, 64 of high bit pairs, sixteen signed 8-bit scales -- one per
// 16 weights -- and a half d.  A 16-weight scale group is exactly one lane's K slice of v_mfma_i32_16x16x64_i8, so the tiles of
// the Q4_K product carry over: lane (r, q) = (lane % 16, lane / 16), h = q / 2, j = q % 2, takes of row r the 16 nibble bytes
// 64 h + 16 j .., the 16 bytes 32 further, the 16 bytes of bit pairs 32 h + 16 j .. and the eight scales of half h, and puts
// four B operands together from them with three instructions a word:
//     codes 128 h + 32 g + 16 j .. + 15   g = 0: low nibbles of the first piece  | bit pairs << 4      g = 1: of the second | << 2
//                                          g = 2: high nibbles of the first      | bit pairs as they lie   g = 3: of the second | >> 2
// -- the unsigned codes 0..63 as they are stored: the offset of 32 comes off against the activations' sums.  The activations are
// the A operand as in the Q4_K product: row m = 4 * slice + plane holds one of three signed base-256 digit planes of the chunk
// of 16 activations slice `slice` meets (chunk 8 h + 2 g + j of the super-block, which is also its scale's index), so C hands
// lane (r, q) the three plane sums of ITS OWN sixteen weights.  A chunk carries a (sum, scale) pair beside its planes, and what
// fp32 adds up is  d * sum over g of sc[g] * (scale[g] * planes[g] - 32 * sum[g]).
//
// Blocks of 210 bytes start on any half word, and a 16-byte load that starts off a 4-byte boundary runs at 60 % of the rate of
// one that starts on it (measured on this kernel's own pattern: 3.6 TB/s against 5.3-5.9).  So every load starts at the 4-byte
// boundary below what it wants -- two bytes early where the block sits on an odd half word -- and the pieces are shifted into
// place with v_alignbit: the two bytes a piece then lacks at its end are the first half word of the piece 16 bytes further,
// which a neighbouring lane of the same row holds (lane + 16 or lane - 16; the last piece of bit pairs ends in the scales'
// load), and cross with three lane exchanges a step.  The scales travel as 12 bytes from 192 + 8 h (so that no fetched word
// goes unread: a register the compiler sees no use for is one it reuses while the load is in flight); the upper lanes' end
// in d, which a fourth exchange hands to the lower lanes.  An early start never leaves the matrix (a block on an odd half
// word is never the first of the matrix), nor does a late end (the last block of a matrix of an even number of rows sits on
// an odd half word, and its scales' load ends with the block).
//
// The rest is the Q4_K product's: NW waves share a tile and split its super-blocks, each turning into digits exactly the
// activations it multiplies (or copying them, HANDED: the 64-byte pieces a SwiGLU epilogue left, whose chunk order is this
// kernel's too); loads run two units ahead across tile boundaries, every wave walks whole rounds of two steps; the finishing
// wave changes from tile to tile; epilogues: plain (+ residual, in place by one fire-and-forget add), SwiGLU over a gate tile
// and the up tile behind it (as floats, or as the digit planes the product behind takes), the cast of a value projection's
// rows into the value state, or the rotation of a q|k|v product with its cache append (ROPE).
//
// Q3_K (ELEMENT = NH_Q3_K; crates/neura-precision/src/ggml.rs:291-306) has the same sixteen scale groups of 16 in a super-block
// of 110 bytes: 32 bytes of third bits, 64 of bit pairs, twelve bytes of 6-bit scales and d.  Lane (r, q) takes the 16 bytes of
// bit pairs 32 h + 16 j .. and the 16 third-bit bytes 16 j .., and its four B operands are the codes 0..7
//     ((pairs >> 2 g) & 3) | (((third >> (4 h + g)) & 1) << 2)     of elements 128 h + 32 g + 16 j .. + 15, g = 0..3
// whose offset of 4 comes off against the activations' sums; the scales (stored 32 too large) and d come as one 16-byte load
// every lane issues.  Blocks of 110 bytes sit on odd half words as often as Q6_K's: the loads start at the 4-byte boundary
// below and two exchanges a step bring the pieces' last half words.
constexpr uint32_t Q6K_BLOCK_BYTES = 210;
constexpr uint32_t Q3K_BLOCK_BYTES = 110;
constexpr uint32_t Q6K_ZERO_BYTES = 304;  // what an idle A lane reads: four chunk offsets (0, 96, 192, 288) + 16 bytes

typedef uint32_t q6_u32x3 __attribute__((ext_vector_type(3)));
typedef q6_u32x3 q6_u32x3_a4 __attribute__((aligned(4)));
typedef u32x4 q6_u32x4_a4 __attribute__((aligned(4)));
template <int ELEMENT>
struct KqUnit;
template <>
struct KqUnit<NH_Q6_K> {
    u32x4 la, lb, qh;
    q6_u32x3 sc;
    uint32_t shift;  // 16 where the block sits on an odd half word (the loads then start two bytes early), else 0
};
template <>
struct KqUnit<NH_Q3_K> {
    u32x4 qs, hm, sc;  // bit pairs, third bits, the twelve scale bytes and d
    uint32_t shift;
};
typedef KqUnit<NH_Q6_K> Q6Unit;

static inline size_t q6k_tile16_lds(uint32_t nblk, uint32_t NW) {
    return (size_t)nblk * (TILE16_BLOCK_DIGITS + TILE16_BLOCK_PAIRS) + (size_t)NW * Q6K_ZERO_BYTES + (size_t)2 * NW * 16u * 4u + (size_t)NW * 4u + 64u;
}

// The leading arguments are what a wave needs before its first loads: plain words, handed over in scalar registers as the wave
// starts (-amdgpu-kernarg-preload-count).  `input` is x, or the digit planes with HANDED.
// SWIGLU: the matrix is a gate matrix with the up matrix `lead_to_w1` * 16 bytes further; a workgroup's unit of work is a pair of
// tiles (gate rows, then the same rows of up) and the pair's finishing wave writes silu(gate) * up.
// ROPE: a q|k|v product (up to three matrices stacked, the second `lead_to_w1` * 16 bytes and the third `lead_to_w2` * 16 bytes
// behind the first, ending at rows `lead_end0`, `lead_end1` and N) whose epilogue rotates the q and k rows and writes k and v
// into the states (rope_store): `lead_tile_rows` is then the rotation's width, and a tile holds channels c .. c + 7 of a head
// and their partners half a head further.
// The product itself, `block` of `lead_grid` workgroups, its LDS at `q6k_lds_bytes` (q6k_tile16_lds() of it).
template <int NW, bool HANDED, bool SWIGLU = false, int ELEMENT = NH_Q6_K, bool ROPE = false>
__device__ __forceinline__ void q6k_tile16_product(uint8_t *q6k_lds_bytes, const uint32_t block, const uint8_t *lead_w0, const void *lead_input, const float *lead_norm_w,
                                                   uint32_t lead_row_bytes, uint32_t lead_grid, uint32_t lead_tiles, uint32_t lead_tile_rows, int32_t lead_to_w1,
                                                   int32_t lead_to_w2, uint32_t lead_end0, uint32_t lead_end1, const GemvParams &p) {
    static_assert(!(HANDED && SWIGLU), "handed-over digit planes feed a plain product");
    static_assert(!ROPE || (!HANDED && !SWIGLU), "the rotation is folded into a product of floats with no other epilogue");
    static_assert(ELEMENT == NH_Q6_K || ELEMENT == NH_Q3_K, "super-blocks of sixteen scale groups of 16");
    constexpr bool Q3 = ELEMENT == NH_Q3_K;
    constexpr uint32_t BLOCK_BYTES = Q3 ? Q3K_BLOCK_BYTES : Q6K_BLOCK_BYTES;
    typedef KqUnit<ELEMENT> Unit;
    constexpr uint32_t NT = NW * 64;
    constexpr int D = 2;
    typedef int i32x4 __attribute__((ext_vector_type(4)));
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef const __attribute__((address_space(1))) q6_u32x4_a4 *global_uint4;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t nblk = lead_row_bytes / BLOCK_BYTES;
    const float *const x = static_cast<const float *>(lead_input);
    uint8_t *const digits = q6k_lds_bytes;
    uint8_t *const zeros = q6k_lds_bytes + (size_t)nblk * TILE16_BLOCK_DIGITS + wave * Q6K_ZERO_BYTES;
    f32x2 *const pairs = reinterpret_cast<f32x2 *>(q6k_lds_bytes + (size_t)nblk * TILE16_BLOCK_DIGITS + NW * Q6K_ZERO_BYTES);  // [block][chunk]: (sum, scale)
    float *const part = reinterpret_cast<float *>(pairs + (size_t)nblk * 16u);                                                  // [parity][wave][16]
    float *const red = part + 2u * NW * 16u;                                                                                    // [wave]

    auto fetch_the_rest = [&]() {
        __builtin_amdgcn_sched_barrier(0);
        NH_FETCH(p.y, p.residual, p.N, p.K, p.eps, p.append_value, p.rope_cursor, p.rope_v, p.rope_width, p.rope_capacity, p.rope_ring, p.rope_element, p.bias[0], p.refusal);
        if (SWIGLU) NH_FETCH(p.digits_out, p.tag_out);
        if (ROPE) NH_FETCH(p.rope_cosines, p.rope_sines, p.rope_k, p.rope_q_rows, p.rope_k_rows, p.rope_positions, p.bias[1], p.bias[2], p.end[0], p.end[1]);
        __builtin_amdgcn_sched_barrier(0);
    };
    const uint32_t r = lane & 15u, q = lane >> 4, h = q >> 1, j = q & 1u;
    const uint32_t tiles = lead_tiles;
    if (block >= tiles || block >= lead_grid) return;  // the whole workgroup: no barrier has been reached
    const uint32_t ntiles = (tiles - block + lead_grid - 1u) / lead_grid;
    const uint32_t count = wave < nblk ? (nblk - wave + NW - 1u) / NW : 0u;  // super-blocks of one tile this wave walks
    const uint32_t tile_rows = ROPE ? 16u : lead_tile_rows, row_bytes = lead_row_bytes;
    const uint8_t *const w0 = lead_w0;
    // a tile may hold fewer than 16 rows: the columns past them walk the tile's last row again and are never written
    const int64_t to_w1 = (int64_t)lead_to_w1 * 16, to_w2 = (int64_t)lead_to_w2 * 16;
    const uint32_t end0 = lead_end0, end1 = lead_end1;
    const uint32_t half_width = (ROPE ? lead_tile_rows : 16u) >> 1, tiles_per_head = max(half_width >> 3, 1u);
    auto lane_row = [w0, row_bytes, tile_rows, r, to_w1, to_w2, end0, end1, half_width, tiles_per_head](uint32_t tile) -> const uint8_t * {
        if (SWIGLU) return w0 + ((tile & 1u) ? to_w1 : (int64_t)0) + (int64_t)((size_t)((tile >> 1) * 16u + r) * row_bytes);
        if (ROPE) {
            const uint32_t n = (tile / tiles_per_head) * (2u * half_width) + (tile % tiles_per_head) * 8u + (r & 7u) + (r >> 3) * half_width;
            const bool in0 = n < end0, in1 = n < end1;
            return w0 + (in0 ? (int64_t)0 : (in1 ? to_w1 : to_w2)) + (int64_t)((size_t)(n - (in0 ? 0u : (in1 ? end0 : end1))) * row_bytes);
        }
        return w0 + (size_t)(tile * tile_rows + min(r, tile_rows - 1u)) * row_bytes;
    };
    // what the rotation's epilogue reads (the cursor, then cos, sin and bias of a tile's sixteen outputs) is fetched ahead
    uint32_t rope_position = 0;
    RopeOperands rope_held{0.0f, 1.0f, 0.0f};
    auto rope_row = [half_width, tiles_per_head, lane](uint32_t tile, uint32_t &c) -> uint32_t {
        c = (tile % tiles_per_head) * 8u + (lane & 7u);
        return (tile / tiles_per_head) * (2u * half_width) + c + ((lane >> 3) & 1u) * half_width;
    };
    const uint32_t first_tile = block, hop = lead_grid;
    // with SwiGLU the workgroup's unit of work is a pair: tiles 2 t (gate) and 2 t + 1 (up)
    auto tile_at = [first_tile, hop](uint32_t i) -> uint32_t {
        if (SWIGLU) return 2u * (first_tile + (i >> 1) * hop) + (i & 1u);
        return first_tile + i * hop;
    };
    const uint32_t walked = SWIGLU ? 2u * ntiles : ntiles;  // tiles this workgroup walks
    typedef const __attribute__((address_space(1))) q6_u32x3_a4 *global_uint3;
    const uint32_t at_low = 64u * h + 16u * j, at_high = 128u + 32u * h + 16u * j, at_scales = 192u + 8u * h;

    // Loads run D steps ahead of the arithmetic, across tile boundaries.  Every fetch issues its four loads: past the last step
    // the last unit is fetched again and dropped, so that the waits count exactly how many loads are newer than the one needed.
    Unit ring[D];
    uint32_t ahead_tile = 0, ahead_b = wave;
    const uint8_t *ahead_row = lane_row(tile_at(0));
    auto fetch = [&](Unit &u) {
        const uint8_t *at = ahead_row + (size_t)min(ahead_b, nblk - 1u) * BLOCK_BYTES;
        const uint8_t *down = reinterpret_cast<const uint8_t *>(reinterpret_cast<uintptr_t>(at) & ~(uintptr_t)3);
        if constexpr (Q3) {
            u.qs = *(global_uint4)(uintptr_t)(down + 32u + 32u * h + 16u * j);
            u.hm = *(global_uint4)(uintptr_t)(down + 16u * j);
            u.sc = *(global_uint4)(uintptr_t)(down + 96u);
        } else {
            u.la = *(global_uint4)(uintptr_t)(down + at_low);
            u.lb = *(global_uint4)(uintptr_t)(down + at_low + 32u);
            u.qh = *(global_uint4)(uintptr_t)(down + at_high);
            u.sc = *(global_uint3)(uintptr_t)(down + at_scales);
        }
        u.shift = ((uint32_t)reinterpret_cast<uintptr_t>(at) & 2u) * 8u;
        if (ahead_b + NW < nblk) {
            ahead_b += NW;
        } else if (ahead_tile + 1u < walked) {
            ahead_b = wave;
            ahead_tile++;
            ahead_row = lane_row(tile_at(ahead_tile));
        }
    };
    auto first_fetches = [&]() {
#pragma unroll
        for (int i = 0; i < D; i++) fetch(ring[i]);
    };

    // ---- activations -> three signed base-256 digit planes and a (sum, scale) pair per chunk of 16; the power-of-two scale is
    // that of the chunk's 64-element group (its largest magnitude lands in [2^21, 2^22)).  Unit e4 = tid + NT * j (four
    // consecutive activations) lies in super-block wave + NW * j: a wave turns into digits exactly the super-blocks it multiplies.
    {
        const uint32_t units = nblk * 64u;
        if (lane < Q6K_ZERO_BYTES / 4u) reinterpret_cast<uint32_t *>(zeros)[lane] = 0u;
        if (lane + 64u < Q6K_ZERO_BYTES / 4u) reinterpret_cast<uint32_t *>(zeros)[lane + 64u] = 0u;
        auto stage = [&](uint32_t e4, f32x4 v, f32x4 w, float rms) {
            if (lead_norm_w) {
#pragma unroll
                for (int i = 0; i < 4; i++) v[i] = __fmul_rn(__fmul_rn(v[i], rms), w[i]);
            }
            uint32_t top = 0;  // largest magnitude of the group as bits: infinities and NaNs sort above every finite value
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float element = v[i];  // a copy first: the bits of a vector element taken in place read element 0 every time
                top = max(top, __builtin_bit_cast(uint32_t, element) & 0x7fffffffu);
            }
            top = max(top, (uint32_t)dpp_int<DPP_QUAD_XOR1>((int)top));
            top = max(top, (uint32_t)dpp_int<DPP_QUAD_XOR2>((int)top));
            top = max(top, (uint32_t)dpp_int<DPP_ROW_ROR4>((int)top));
            top = max(top, (uint32_t)dpp_int<DPP_ROW_ROR8>((int)top));
            const uint32_t raw = top >> 23;
            const uint32_t exponent = min(max(raw, 22u), 254u);
            const float scale = __builtin_bit_cast(float, (275u - exponent) << 23);
            const float unscale = raw == 255u ? __builtin_bit_cast(float, 0x7fc00000u) : __builtin_bit_cast(float, (exponent - 21u) << 23);
            float total = 0.0f;
            uint32_t dg[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float rounded = rintf(v[i] * scale);
                total += rounded;
                dg[i] = signed_digits((int)rounded);  // bytes 0..2: signed digits, least significant first
            }
            const uint32_t lo01 = __builtin_amdgcn_perm(dg[1], dg[0], 0x05010400u), hi01 = __builtin_amdgcn_perm(dg[1], dg[0], 0x07030602u);
            const uint32_t lo23 = __builtin_amdgcn_perm(dg[3], dg[2], 0x05010400u), hi23 = __builtin_amdgcn_perm(dg[3], dg[2], 0x07030602u);
            const uint32_t plane2 = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);  // least significant digits of the four elements
            const uint32_t plane1 = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
            const uint32_t plane0 = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);  // most significant
            total += dpp<DPP_QUAD_XOR1>(total);
            total += dpp<DPP_QUAD_XOR2>(total);  // the four lanes of a chunk
            // unit e4: 64 units a super-block, 4 a chunk of 16 elements
            uint32_t *slot = reinterpret_cast<uint32_t *>(digits + (size_t)(e4 >> 2) * 48u) + (e4 & 3u);
            slot[0] = plane0, slot[4] = plane1, slot[8] = plane2;
            if ((e4 & 3u) == 0) pairs[e4 >> 2] = f32x2{total * unscale, unscale};
        };
        if constexpr (HANDED) {
            // a wave copies the super-blocks it walks, one 16-byte load a lane and block.  A chunk of 16 activations is 64 bytes in
            // memory: words 0..3 plane 0 | 4..6 plane 1, first twelve | 7 a tag || 8 plane 1, last four | 9..11 plane 2, first
            // twelve | 12 plane 2, last four | 13, 14 the (sum, scale) pair | 15 a tag; lane 4 c + piece holds words 4 piece .. + 3 of chunk c
            constexpr int MAXB = NW <= 8 ? 10 : 5;
            const uint32_t chunk = lane >> 2, piece = lane & 3u;
            for (uint32_t j0 = 0; j0 < count || j0 == 0; j0 += MAXB) {
                u32x4 held[MAXB];
#pragma unroll
                for (int i = 0; i < MAXB; i++) {
                    const uint32_t b = min(wave + NW * min(j0 + i, count ? count - 1u : 0u), nblk - 1u);
                    held[i] = *reinterpret_cast<const u32x4 *>(static_cast<const uint8_t *>(lead_input) + (size_t)b * TILE16_BLOCK_HANDED + lane * 16u);
                }
                if (j0 == 0) {
                    first_fetches();
                    fetch_the_rest();
                }
#pragma unroll
                for (int i = 0; i < MAXB; i++) {
                    if (j0 + i >= count) continue;
                    const uint32_t b = wave + NW * (j0 + i);
                    uint8_t *planes = digits + (size_t)b * TILE16_BLOCK_DIGITS + chunk * 48u;
                    if (piece == 0u) {
                        *reinterpret_cast<u32x4 *>(planes) = held[i];
                    } else if (piece == 1u) {
                        *reinterpret_cast<uint2 *>(planes + 16u) = uint2{held[i].x, held[i].y};
                        *reinterpret_cast<uint32_t *>(planes + 24u) = held[i].z;
                    } else if (piece == 2u) {
                        *reinterpret_cast<uint32_t *>(planes + 28u) = held[i].x;
                        *reinterpret_cast<uint2 *>(planes + 32u) = uint2{held[i].y, held[i].z};
                        *reinterpret_cast<uint32_t *>(planes + 40u) = held[i].w;
                    } else {
                        *reinterpret_cast<uint32_t *>(planes + 44u) = held[i].x;
                        const uint32_t sum_bits = held[i].y, scale_bits = held[i].z;
                        pairs[b * 16u + chunk] = f32x2{__builtin_bit_cast(float, sum_bits), __builtin_bit_cast(float, scale_bits)};
                    }
                }
            }
        } else {
            constexpr int MAXJ = 5;
            f32x4 held[MAXJ], weight[MAXJ];
            const bool resident = units <= MAXJ * NT;
            float rms = 1.0f;
            if (resident) {
#pragma unroll
                for (int i = 0; i < MAXJ; i++) {
                    const uint32_t e4 = tid + NT * i;
                    held[i] = e4 < units ? *reinterpret_cast<const f32x4 *>(x + 4u * e4) : f32x4{0.f, 0.f, 0.f, 0.f};
                }
                if (lead_norm_w) {
#pragma unroll
                    for (int i = 0; i < MAXJ; i++) {
                        const uint32_t e4 = tid + NT * i;
                        weight[i] = e4 < units ? *reinterpret_cast<const f32x4 *>(lead_norm_w + 4u * e4) : f32x4{0.f, 0.f, 0.f, 0.f};
                    }
                }
            }
            // the weights' loads go out behind the activations', which everything waits for first
            first_fetches();
            fetch_the_rest();
            if (ROPE && wave == 0 && lane < 16u) rope_position = p.rope_cursor[0];
            if (lead_norm_w) {
                // sum of squares of the whole row (crates/neura-kernel/src/task/norm.rs:69-83; the same fp32 adds in another order)
                float square = 0.0f;
                if (resident) {
#pragma unroll
                    for (int i = 0; i < MAXJ; i++)
#pragma unroll
                        for (int k = 0; k < 4; k++) square = __fadd_rn(square, __fmul_rn(held[i][k], held[i][k]));
                } else {
                    for (uint32_t e4 = tid; e4 < units; e4 += NT) {
                        const f32x4 v = *reinterpret_cast<const f32x4 *>(x + 4u * e4);
#pragma unroll
                        for (int k = 0; k < 4; k++) square = __fadd_rn(square, __fmul_rn(v[k], v[k]));
                    }
                }
                square = wave_sum(square);
                if (lane == 0) red[wave] = square;
                __syncthreads();
                float total = 0.0f;
#pragma unroll
                for (int w = 0; w < NW; w++) total += red[w];
                rms = rms_scale_of(total, p.K, p.eps);
            }
            if (resident) {
#pragma unroll
                for (int i = 0; i < MAXJ; i++) {
                    if (NT * i >= units) break;  // uniform over the workgroup
                    const uint32_t e4 = tid + NT * i;
                    if (e4 < units) stage(e4, held[i], weight[i], rms);  // whole groups of 16 lanes are in or out together
                }
            } else {
                for (uint32_t e4 = tid; e4 < units; e4 += NT)
                    stage(e4, *reinterpret_cast<const f32x4 *>(x + 4u * e4), lead_norm_w ? *reinterpret_cast<const f32x4 *>(lead_norm_w + 4u * e4) : f32x4{0.f, 0.f, 0.f, 0.f},
                          rms);
            }
        }
    }
    __builtin_amdgcn_wave_barrier();  // LDS serves a wave's accesses in order: the reads below see this wave's writes
    if (ROPE && wave == 0 && lane < 16u) {
        uint32_t c;
        const uint32_t n = rope_row(tile_at(0), c);
        rope_held = rope_operands(p, n, c, rope_position);
    }

    // ---- the walk
    const uint32_t m = lane & 15u;
    const bool feeds = (m >> 2) == q && (m & 3u) < 3u;  // A row m = 4 * slice + plane meets K slice `slice` only
    const uint8_t *const abase = feeds ? digits + (8u * h + j) * 48u + (m & 3u) * 16u : zeros;
    const uint32_t astride = feeds ? TILE16_BLOCK_DIGITS : 0u;
    const f32x2 *const pbase = pairs + 8u * h + j;
    const uint32_t pick = j ? 0x07050301u : 0x06040200u;  // the scales of chunks 8 h + 2 g + j out of the eight of half h
    const int beside = (int)((lane ^ 16u) * 4u), above = (int)(((lane + 16u) & 63u) * 4u), across = (int)((lane ^ 32u) * 4u);  // lanes of the same row
    float acc = 0.0f, gate = 0.0f;
    uint32_t parity = 0;
    struct Step {
        i32x4 c[4];
        f32x2 pr[4];
        uint32_t scales, d;
    };
    auto multiply = [&](const Unit &u, uint32_t b, Step &st) {
        const uint8_t *at = abase + (size_t)b * astride;
        const i32x4 a0 = *reinterpret_cast<const i32x4 *>(at), a1 = *reinterpret_cast<const i32x4 *>(at + 96);
        const i32x4 a2 = *reinterpret_cast<const i32x4 *>(at + 192), a3 = *reinterpret_cast<const i32x4 *>(at + 288);
#pragma unroll
        for (int g = 0; g < 4; g++) st.pr[g] = pbase[b * 16u + 2u * g];
        const uint32_t shift = u.shift;
        auto placed = [shift](const u32x4 &piece, uint32_t after) -> u32x4 {
            return u32x4{__builtin_amdgcn_alignbit(piece.y, piece.x, shift), __builtin_amdgcn_alignbit(piece.z, piece.y, shift),
                         __builtin_amdgcn_alignbit(piece.w, piece.z, shift), __builtin_amdgcn_alignbit(after, piece.w, shift)};
        };
        i32x4 b0, b1, b2, b3;
        if constexpr (Q3) {
            // The word that follows a piece in memory:
            //   bit pairs:  lane (h, j) <- the bit pairs of the lane 16 further;  (1, 1) <- its own scales' first word
            //   third bits: (h, 0) <- the third bits of (h, 1);  (h, 1) <- the bit pairs of (0, 0)
            const uint32_t qs0 = u.qs.x, hm0 = u.hm.x;
            const uint32_t got_qs = (uint32_t)__builtin_amdgcn_ds_bpermute(above, (int)qs0);
            const uint32_t after_hm = (uint32_t)__builtin_amdgcn_ds_bpermute(q == 1u ? beside : above, (int)(j ? hm0 : qs0));
            const uint32_t after_qs = q == 3u ? u.sc.x : got_qs;
            const u32x4 qs = placed(u.qs, after_qs), hm = placed(u.hm, after_hm) >> (4u * h);
            const u32x4 two = {0x03030303u, 0x03030303u, 0x03030303u, 0x03030303u}, third = {0x04040404u, 0x04040404u, 0x04040404u, 0x04040404u};
            b0 = (i32x4)((qs & two) | ((hm << 2) & third)), b1 = (i32x4)(((qs >> 2) & two) | ((hm << 1) & third));
            b2 = (i32x4)(((qs >> 4) & two) | (hm & third)), b3 = (i32x4)(((qs >> 6) & two) | ((hm >> 1) & third));
            // sixteen 6-bit scales: low nibbles in the first eight bytes (scales 0..7, then 8..15 in the high nibbles), bit pairs in
            // the last four; this lane's are 8 h + 2 g + j
            const uint32_t s0 = __builtin_amdgcn_alignbit(u.sc.y, u.sc.x, shift), s1 = __builtin_amdgcn_alignbit(u.sc.z, u.sc.y, shift);
            const uint32_t s2 = __builtin_amdgcn_alignbit(u.sc.w, u.sc.z, shift);
            const uint32_t first = ((s0 >> (4u * h)) & 0x0f0f0f0fu) | (((s2 >> (4u * h)) & 0x03030303u) << 4);
            const uint32_t second = ((s1 >> (4u * h)) & 0x0f0f0f0fu) | (((s2 >> (4u * h + 2u)) & 0x03030303u) << 4);
            st.scales = __builtin_amdgcn_perm(second, first, pick);
            st.d = (u.sc.w >> shift) & 0xffffu;
        } else {
            // The word that follows each of the lane's three pieces in memory is the first word of another piece of the row:
            //   first nibble piece:  lane (h, 0) <- first piece of (h, 1);  lane (h, 1) <- second piece of (h, 0)
            //   second nibble piece: (0, 0) <- second of (0, 1);  (0, 1) <- first of (1, 0);  (1, 0) <- second of (1, 1);  (1, 1) <- bit pairs of (0, 0)
            //   bit pairs:           (h, j) <- bit pairs of the lane 16 further;  (1, 1) <- the scales of (0, 0)
            // every lane offers what its reader wants and takes part in every exchange
            const uint32_t la0 = u.la.x, lb0 = u.lb.x, qh0 = u.qh.x, sc0 = u.sc.x, sc2 = u.sc.z;
            const uint32_t after_la = (uint32_t)__builtin_amdgcn_ds_bpermute(beside, (int)(j ? la0 : lb0));
            const uint32_t after_lb = (uint32_t)__builtin_amdgcn_ds_bpermute(above, (int)(q == 0u ? qh0 : (q == 2u ? la0 : lb0)));
            const uint32_t after_qh = (uint32_t)__builtin_amdgcn_ds_bpermute(above, (int)(q == 0u ? sc0 : qh0));
            const uint32_t from_upper = (uint32_t)__builtin_amdgcn_ds_bpermute(across, (int)sc2);
            const u32x4 la = placed(u.la, after_la), lb = placed(u.lb, after_lb), qh = placed(u.qh, after_qh);
            const u32x4 low = {0x0f0f0f0fu, 0x0f0f0f0fu, 0x0f0f0f0fu, 0x0f0f0f0fu}, high = {0x30303030u, 0x30303030u, 0x30303030u, 0x30303030u};
            b0 = (i32x4)((la & low) | ((qh << 4) & high)), b1 = (i32x4)((lb & low) | ((qh << 2) & high));
            b2 = (i32x4)(((la >> 4) & low) | (qh & high)), b3 = (i32x4)(((lb >> 4) & low) | ((qh >> 2) & high));
            st.scales = __builtin_amdgcn_perm(__builtin_amdgcn_alignbit(u.sc.z, u.sc.y, shift), __builtin_amdgcn_alignbit(u.sc.y, u.sc.x, shift), pick);
            st.d = ((h ? sc2 : from_upper) >> shift) & 0xffffu;  // d follows the sixteen scales: the third word of the upper lanes' twelve bytes
        }
        const i32x4 none = {0, 0, 0, 0};
        st.c[0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, b0, none, 0, 0, 0);
        st.c[1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1, b1, none, 0, 0, 0);
        st.c[2] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a2, b2, none, 0, 0, 0);
        st.c[3] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a3, b3, none, 0, 0, 0);
        asm volatile("" : "+v"(st.scales), "+v"(st.d));  // the unit is read by here
    };
    auto weigh = [&](const Step &st) {
        float whole = 0.0f;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const float planes = fmaf(fmaf((float)st.c[g][0], 256.0f, (float)st.c[g][1]), 256.0f, (float)st.c[g][2]);
            const float scale = Q3 ? (float)((st.scales >> (8 * g)) & 0xffu) - 32.0f : (float)(int8_t)(st.scales >> (8 * g));
            whole = fmaf(scale, fmaf(st.pr[g].y, planes, (Q3 ? -4.0f : -32.0f) * st.pr[g].x), whole);
        }
        acc = fmaf(half_to_float((uint16_t)st.d), whole, acc);
    };
    // The wave that finishes a tile (sums the waves' parts, runs the epilogue) changes from tile to tile (with SwiGLU from pair to
    // pair: the gate sum waits in its registers)
    auto tile_end = [&](uint32_t tile, uint32_t index) {
        const uint32_t finisher = ROPE ? 0u : (SWIGLU ? index >> 1 : index) % NW;
        float v = acc;
        v += __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));  // lane ^ 16
        v += __shfl_xor(v, 32, 64);
        if (q == 0) part[(parity * NW + wave) * 16u + r] = v;
        acc = 0.0f;
        __syncthreads();
        if (wave == finisher && q == 0 && r < tile_rows) {
            float total = 0.0f;
#pragma unroll
            for (int w = 0; w < NW; w++) total += part[(parity * NW + w) * 16u + r];
            const size_t n = (size_t)tile * tile_rows + r;
            if (ROPE) {
                uint32_t c;
                const uint32_t row = rope_row(tile, c);
                rope_store(p, total, row, lane >= 8u, rope_position, rope_held);
                if (tile + hop < tiles) {  // the next tile of this workgroup
                    const uint32_t next = rope_row(tile + hop, c);
                    rope_held = rope_operands(p, next, c, rope_position);
                }
            } else if (SWIGLU) {
                // (the pair's sixteen outputs either as floats or as chunk tile / 2 of the digit planes the product behind takes)
                if (!(tile & 1u)) gate = total;
                else if (p.digits_out) reinterpret_cast<uint32_t *>(p.digits_out + (size_t)(tile >> 1) * 64u)[r] = handed_piece_word(silu(gate) * total, r, p.tag_out);
                else p.y[(size_t)(tile >> 1) * 16u + r] = silu(gate) * total;
            } else if (p.residual == p.y) unsafeAtomicAdd(p.y + n, total);  // in place: one add per element, nothing to wait for
            else p.y[n] = p.residual ? p.residual[n] + total : total;
            if (!SWIGLU && !ROPE && p.append_value) {
                // a value projection of one token: its rows (+ bias) go into the value state at the cursor as halves, as
                // value_append_kernel would cast them
                const uint32_t cursor = p.rope_cursor[0];
                const float value = p.bias[0] ? total + p.bias[0][n] : total;
                const uint32_t slot = p.rope_ring ? cursor % p.rope_ring : cursor;
                if (slot >= p.rope_capacity) atomicMax(p.refusal, (uint32_t)REFUSAL_ORIGIN);
                else state_store(p.rope_v, p.rope_element, ((uint64_t)((uint32_t)n / p.rope_width) * p.rope_capacity + slot) * p.rope_width + (uint32_t)n % p.rope_width, value);
            }
        }
        parity ^= 1u;
    };
    if (count == 0) {  // more waves than super-blocks: this one only keeps the barriers
        for (uint32_t t = 0; t < walked; t++) tile_end(tile_at(t), t);
        return;
    }
    // Every wave walks whole rounds of D steps: the steps past its last tile multiply what was fetched again and publish nothing.
    uint32_t at_tile = 0, at_b = wave;
    const uint32_t steps = walked * count;
    for (uint32_t s0 = 0; s0 < steps; s0 += D) {
#pragma unroll
        for (int slot = 0; slot < D; slot++) {
            Step st;
            multiply(ring[slot], at_b, st);
            __builtin_amdgcn_sched_barrier(0);  // the fetch reuses this unit's registers: keep its loads behind their last use
            fetch(ring[slot]);
            __builtin_amdgcn_sched_barrier(0);
            weigh(st);
            at_b += NW;
            if (at_b >= nblk) {
                if (at_tile < walked) tile_end(tile_at(at_tile), at_tile);
                at_b = wave;
                at_tile++;
            }
        }
    }
}

}  // namespace nh
