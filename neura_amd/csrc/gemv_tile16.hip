// The Q4_K product of one activation row on 16-row tiles of the 16x16x64 integer MFMA: kernel and launcher.
// Built with the matrix-core results in vector registers (-amdgpu-mfma-vgpr-form): the sums are weighed right where they land.
#include "gemv_q6k_tile16.hpp"
#include "gemv_shared.hpp"

namespace nh {

// ---------------------------------------------------------------------------------------------------------------------
// One activation row against a Q4_K matrix on 16-row tiles of v_mfma_i32_16x16x64_i8: the decode step's product.
//
// A wave step covers one super-block of 16 rows.  Lane (r, q) = (lane % 16, lane / 16) fetches the 32 nibble bytes of
// group q of row r (two 128-bit loads) and the block header, and unpacks them with two masks and a shift a word into the B
// operands of four MFMAs: the sixteen low nibbles of each load are K slice q of one instruction, the high nibbles of
// another.  The activations are the A operand: row m = 4 * slice + plane holds one of three signed base-256 digit planes of
// the sixteen activations slice `slice` meets and zeros everywhere else, so C comes back with lane (r, q) holding the three
// plane sums of ITS OWN weights -- no sum crosses lanes and the lane that holds a sum holds the header that weighs it.  The
// digits carry 22 bits below a power-of-two scale per 64-element group (exact for the group's largest magnitudes, finer
// than fp32 rounding of the products for the rest), so the integer arithmetic is exact and what is left to fp32 is
// d * (sc . sums) - dmin * (m . activation sums) per group, as the reference weighs it (crates/neura-kernel/src/dot.rs:583-619).
//
// NW waves share a tile, wave w taking super-blocks w, w + NW, ... (and turning exactly those activations into digits,
// in its own corner of LDS, so no barrier stands between staging and walking); their sixteen partial sums meet in LDS once
// a tile.  Loads run D steps ahead across tile boundaries; workgroups take tiles blockIdx.x, blockIdx.x + gridDim.x, ...
// so that the device as a whole walks one window of the matrix from end to end.
// 0.9 vector instructions a weight (the vector kernel above: 2.4) with the multiply-adds on the matrix cores.
// Epilogues: y (+ in-place residual by one fire-and-forget add), SwiGLU over a gate tile and the up tile behind it, or the
// rotation with the cache append (tile rows = 8 channels c.. and their partners c + width/2.. of one head).
constexpr uint32_t TILE16_ZERO_BYTES = 208;    // what an idle A lane reads: four chunk offsets (0, 48, 96, 144) + 16 bytes
// (TILE16_APPEND: a plain product of one row that also casts its outputs into the value state -- a form of its own, so that the
// plain products of a step fetch and test nothing for it)
enum Tile16Mode { TILE16_PLAIN = 0, TILE16_SWIGLU = 1, TILE16_ROPE = 2, TILE16_APPEND = 3 };

static size_t tile16_lds(uint32_t nblk, uint32_t NW, uint32_t R, bool handed = false) {
    const size_t sums = handed ? (size_t)nblk * TILE16_BLOCK_PAIRS : (size_t)R * nblk * 64u;
    return (size_t)R * nblk * TILE16_BLOCK_DIGITS + (size_t)NW * TILE16_ZERO_BYTES + sums + (size_t)2 * NW * R * 16u * 4u + (size_t)NW * R * 4u + 64u;
}

struct Tile16Unit {
    u32x4 hdr, qa, qb;
};
// Q5_K: a super-block is Q4_K's with the codes' fifth bits between the header and the nibbles (176 bytes: 16 of header, 32 of
// fifth bits, 128 of nibbles; crates/neura-precision/src/ggml.rs:321-335).  Byte l of the 32 carries, in bits 2 g and 2 g + 1,
// the fifth bits of codes l and 32 + l of group g: lane (r, q) fetches all 32 bytes beside its group's nibbles (the four lanes
// of a row ask for the same bytes in one instruction) and sets bit 4 of its sixteen-code operands from them.  Scales,
// minimums, digit planes and the weighing are Q4_K's.
struct Tile16UnitFifth {
    u32x4 hdr, qa, qb, fa, fb;  // fa, fb: the fifth bits of codes l = 0..15 and 16..31 of every group
};
template <bool FIFTH>
struct Tile16UnitOf {
    typedef Tile16Unit type;
};
template <>
struct Tile16UnitOf<true> {
    typedef Tile16UnitFifth type;
};
// the B operands of a step: low and high nibbles of the unit's two nibble loads, with the fifth bit where the element has one
template <bool FIFTH, class UNIT>
__device__ __forceinline__ void tile16_codes(const UNIT &u, uint32_t q, u32x4 &la, u32x4 &ha, u32x4 &lb, u32x4 &hb) {
    const u32x4 mask = {0x0f0f0f0fu, 0x0f0f0f0fu, 0x0f0f0f0fu, 0x0f0f0f0fu};
    la = u.qa & mask, ha = (u.qa >> 4) & mask, lb = u.qb & mask, hb = (u.qb >> 4) & mask;
    if constexpr (FIFTH) {
        const u32x4 bit = {0x10101010u, 0x10101010u, 0x10101010u, 0x10101010u};
        const u32x4 fa = u.fa >> (2u * q), fb = u.fb >> (2u * q);  // bit 0: the low nibble's fifth bit, bit 1: the high nibble's
        la |= (fa << 4) & bit, ha |= (fa << 3) & bit, lb |= (fb << 4) & bit, hb |= (fb << 3) & bit;
    }
}

//
// R > 1: up to R activation rows (p.rows of them) meet the weights in one pass.  Every row has its own digit planes and sums in
// LDS; a step unpacks its weights once and runs the four MFMAs and the weighing once a row, so the weights are read once for
// all rows where one launch a row read them `rows` times.
//
// HANDED: the activations arrive as digit planes already (p.digits_in: per chunk of 16 one 64-byte piece -- three planes of
// 16 bytes, then the chunk's (sum, scale) pair), left there by the SwiGLU epilogue of the product before (p.digits_out),
// which holds a chunk's sixteen outputs in sixteen lanes of one wave when it is done and writes the piece as one whole,
// aligned 64 bytes (pieces smaller than the 32 bytes the memory checks as one cost a read-modify-write each).  The scale
// is then a chunk's own, not a group's, so the four MFMAs of a step keep their sums apart and each is weighed by its
// chunk's scale; the staging pass shrinks to a copy.
//
// A seam stands between two products of one launch (gemv_q4k_chain_kernel below).  The product behind it asks for its first
// weights at once -- they depend on nothing -- and then for its activations, which the product before may still be writing.
// What crosses a seam crosses it between compute units of different dies, whose L2 caches do not see each other's writes
// inside a launch, so it is stored and loaded at device scope (sc1: written through to memory, read past the L2) -- and it
// carries its own proof of arrival: every piece the memory writes as one (a 32-byte sector of a chunk of digit planes, an
// 8-byte (value, tag) pair of a float) ends in a tag word that names the launch's step and the seam, and a reader that
// finds another tag reads the piece again, `spin` times at most.  No flag, no barrier between workgroups and no wait for a
// store's acknowledgement: a workgroup that is done with one product walks into the next, and waits only where the very
// numbers it needs are not there yet.  A reader that runs out of turns writes REFUSAL_SEAM and goes on with what it has
// (every wave still reaches every barrier and the kernel ends); the host then runs the step again, one launch a product.
// NoSeam is a product that is a launch of its own.
struct NoSeam {
    static constexpr bool WAITS = false;         // the first weights are asked for before the activations
    static constexpr bool SHARED_IN = false;     // activations (and the residual) were written by this launch
    static constexpr bool SHARED_OUT = false;    // outputs are read by a later product of this launch
    static constexpr bool HANDS_RING = false;    // past its last unit the ring fetches the first units of the product behind the seam
    static constexpr bool TAKES_RING = false;    // the ring arrives with this product's first units in flight
    uint32_t spin = 0;
};

typedef float tile16_f32x4 __attribute__((ext_vector_type(4)));
// 16 bytes at `base + offset` (base uniform over the wave); SHARED: at device scope
template <bool SHARED>
__device__ __forceinline__ u32x4 tile16_load16(const void *base, uint32_t offset) {
    if constexpr (SHARED) {
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, 0xffffffff, 0x00020000);
        return __builtin_amdgcn_raw_buffer_load_b128(rsrc, offset, 0, 16);  // aux 16: sc1
    } else {
        typedef const __attribute__((address_space(1))) u32x4 *global_uint4;
        return *(global_uint4)(uintptr_t)(static_cast<const uint8_t *>(base) + offset);
    }
}
// the same, past the L2 (device scope) only where `past` says so: a reader's first look may be served by the L2 of its die --
// whatever it finds there carries its tag -- and only a piece found stale is read again from memory
__device__ __forceinline__ u32x4 tile16_load16_either(const void *base, uint32_t offset, bool past) {
    return past ? tile16_load16<true>(base, offset) : tile16_load16<false>(base, offset);
}
template <bool SHARED>
__device__ __forceinline__ tile16_f32x4 tile16_load4(const float *base, uint32_t element) {
    if constexpr (SHARED) return __builtin_bit_cast(tile16_f32x4, tile16_load16<true>(base, element * 4u));
    else return *reinterpret_cast<const tile16_f32x4 *>(base + element);
}
template <bool SHARED>
__device__ __forceinline__ void tile16_store_word(uint32_t *at, uint32_t word) {
    if constexpr (SHARED) __hip_atomic_store(at, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else *at = word;
}

// The product itself; `block` of `lead_grid` workgroups.
// `ring`: the units in flight, the caller's (a chained launch hands them from one product to the next: with HANDS_RING the
// fetches past this product's last unit ask for super-blocks wave, wave + NW, ... of `next_row`, this lane's weight row in
// the first tile the workgroup walks of the product behind the seam (nullptr: it walks none), which then TAKES_RING).
template <int NW, int D, int MODE, int R, bool HANDED, class SEAM, bool FIFTH = false>
__device__ __forceinline__ void tile16_product(uint8_t *tile16_lds_bytes, const uint32_t block, const SEAM seam, typename Tile16UnitOf<FIFTH>::type (&ring)[D], const uint8_t *next_row,
                                               uint32_t next_nblk, const uint8_t *lead_w0, const void *lead_input,
                                               const float *lead_norm_w, int32_t lead_to_w1, int32_t lead_to_w2, uint32_t lead_row_bytes, uint32_t lead_grid,
                                               uint32_t lead_tiles, uint32_t lead_tile_rows, uint32_t lead_end0, uint32_t lead_end1, const GemvParams &p) {
    static_assert(R == 1 || MODE != TILE16_ROPE, "the rotation is folded into the product of one row only");
    static_assert(!HANDED || (R == 1 && MODE == TILE16_PLAIN), "handed-over digit planes feed a plain product of one row");
    static_assert(MODE != TILE16_APPEND || (R == 1 && !SEAM::SHARED_IN && !SEAM::SHARED_OUT), "a value projection's append rides a product of one row with a launch of its own");
    static_assert(!(SEAM::WAITS || SEAM::SHARED_IN || SEAM::SHARED_OUT) || R == 1, "products of one row are chained");
    static_assert(!FIFTH || (R == 1 && !SEAM::HANDS_RING && !SEAM::TAKES_RING), "Q5_K: one row, a launch of its own");
    typedef typename Tile16UnitOf<FIFTH>::type Unit;
    constexpr uint32_t BLOCK_BYTES = FIFTH ? 176u : 144u, TO_NIBBLES = FIFTH ? 48u : 16u;  // a super-block, and from its start to its nibbles
    constexpr uint32_t NT = NW * 64;
    typedef int i32x4 __attribute__((ext_vector_type(4)));
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    typedef const __attribute__((address_space(1))) u32x4 *global_uint4;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t nblk = lead_row_bytes / BLOCK_BYTES;  // super-blocks a row
    const float *const x = static_cast<const float *>(lead_input);
    uint8_t *const digits = tile16_lds_bytes;
    const uint32_t row_digits = nblk * TILE16_BLOCK_DIGITS;  // digit planes of one activation row
    uint8_t *const zeros = tile16_lds_bytes + (size_t)R * row_digits + wave * TILE16_ZERO_BYTES;  // a wave's own zeros
    f32x4 *const sums = reinterpret_cast<f32x4 *>(tile16_lds_bytes + (size_t)R * row_digits + NW * TILE16_ZERO_BYTES);  // [row][block][group]
    float *const part = reinterpret_cast<float *>(sums + (HANDED ? (size_t)nblk * (TILE16_BLOCK_PAIRS / 16u) : (size_t)R * nblk * 4u));  // [parity][wave][row][16]
    float *const red = part + 2u * NW * R * 16u;                                  // [wave][row]

    // everything else a wave reads from `p` is asked for in one go once its first loads are out
    auto fetch_the_rest = [&]() {
        __builtin_amdgcn_sched_barrier(0);
        NH_FETCH(p.y, p.residual, p.N, p.K, p.rows, p.eps, p.digits_out);
        if (MODE == TILE16_APPEND) NH_FETCH(p.rope_cursor, p.rope_v, p.rope_width, p.rope_capacity, p.rope_ring, p.rope_element, p.bias[0], p.refusal);
        if (MODE == TILE16_ROPE)
            NH_FETCH(p.rope_cosines, p.rope_sines, p.rope_cursor, p.rope_k, p.rope_v, p.rope_width, p.rope_q_rows, p.rope_k_rows, p.rope_capacity, p.rope_positions,
                     p.rope_ring, p.rope_element, p.bias[0], p.bias[1], p.bias[2], p.refusal, p.end[0], p.end[1]);
        __builtin_amdgcn_sched_barrier(0);
    };
    const uint32_t r = lane & 15u, q = lane >> 4;
    // tiles of this workgroup: blockIdx.x, blockIdx.x + lead_grid, ... (with SwiGLU a pair of tiles: gate rows, then the up rows)
    const uint32_t tiles = lead_tiles;
    // what a wave with nothing (more) to fetch here asks for on behalf of the product behind the seam
    auto hand_on = [&]() {
        if constexpr (SEAM::HANDS_RING) {
#pragma unroll
            for (int i = 0; i < D; i++) {
                const uint8_t *at = (next_row ? next_row : lead_w0 + q * 32u) + (size_t)(next_row ? min(wave + NW * (uint32_t)i, next_nblk - 1u) : 0u) * 144u;
                ring[i].hdr = *(global_uint4)(uintptr_t)(at - q * 32u);
                ring[i].qa = *(global_uint4)(uintptr_t)(at + 16u);
                ring[i].qb = *(global_uint4)(uintptr_t)(at + 32u);
            }
        }
    };
    if (block >= tiles || block >= lead_grid) {  // the whole workgroup: no barrier has been reached
        hand_on();
        return;
    }
    const uint32_t ntiles = (tiles - block + lead_grid - 1u) / lead_grid;
    const uint32_t count = wave < nblk ? (nblk - wave + NW - 1u) / NW : 0u;  // super-blocks of one tile this wave walks

    // the weight row lane r reads in tile `tile`; with the rotation folded in a tile holds channels c0 .. c0 + 7 of a head and
    // their partners half a head further (written with selects over scalars captured by value: nothing here may end up indexed)
    const uint8_t *const w0 = lead_w0;
    const int64_t to_w1 = (int64_t)lead_to_w1 * 16, to_w2 = (int64_t)lead_to_w2 * 16;  // handed over in units of 16 bytes
    const uint32_t end0 = lead_end0, end1 = lead_end1;
    const uint32_t row_bytes = lead_row_bytes;
    // (with the rotation folded in the tile rows' word carries the rotation's width: such tiles are always whole)
    const uint32_t half_width = (MODE == TILE16_ROPE ? lead_tile_rows : 16u) >> 1, tiles_per_head = max(half_width >> 3, 1u);
    const uint32_t first_tile = block, hop = lead_grid;
    // a plain tile may hold fewer than 16 rows (a matrix of 3584 rows is 256 tiles of 14, one a compute unit, where it is 224
    // of 16): the columns past them walk the tile's last row again and are never written
    const uint32_t tile_rows = MODE == TILE16_PLAIN || MODE == TILE16_APPEND ? lead_tile_rows : 16u;
    auto lane_row = [w0, to_w1, to_w2, end0, end1, row_bytes, half_width, tiles_per_head, tile_rows, r, q](uint32_t tile) -> const uint8_t * {
        (void)tile_rows;  // the SwiGLU form's tiles are whole
        int64_t offset;
        if (MODE == TILE16_SWIGLU) {
            offset = ((tile & 1u) ? to_w1 : (int64_t)0) + (int64_t)((tile >> 1) * 16u + r) * row_bytes;
        } else {
            uint32_t n = tile * tile_rows + min(r, tile_rows - 1u);
            if (MODE == TILE16_ROPE) n = (tile / tiles_per_head) * (2u * half_width) + (tile % tiles_per_head) * 8u + (r & 7u) + (r >> 3) * half_width;
            const bool in0 = n < end0, in1 = n < end1;
            const int64_t matrix = in0 ? (int64_t)0 : (in1 ? to_w1 : to_w2);
            const uint32_t before = in0 ? 0u : (in1 ? end0 : end1);
            offset = matrix + (int64_t)(n - before) * row_bytes;
        }
        return w0 + offset + q * 32u;
    };
    // with SwiGLU the workgroup's unit of work is a pair: tiles 2j (gate) and 2j + 1 (up)
    auto tile_at = [first_tile, hop](uint32_t i) -> uint32_t {
        if (MODE == TILE16_SWIGLU) return 2u * (first_tile + (i >> 1) * hop) + (i & 1u);
        return first_tile + i * hop;
    };
    const uint32_t walked = MODE == TILE16_SWIGLU ? 2u * ntiles : ntiles;  // tiles this workgroup walks

    // Loads run D steps ahead of the arithmetic, across tile boundaries.  Every fetch issues its three loads: past the last
    // step the last unit is fetched again and dropped, so that every path issues the same loads in the same order and the
    // waits count exactly how many loads are newer than the one needed.
    uint32_t ahead_tile = 0, ahead_b = wave;
    const uint8_t *ahead_row = lane_row(tile_at(0));
    // HANDS_RING: once this wave's last unit is asked for, the fetches that would ask for it again ask for units 0, 1, ... of the
    // product behind the seam instead (the first `pad` of them still are fillers: the walk below runs whole rounds of D steps,
    // and the last D fetches are the ones whose units stay in the ring)
    bool exhausted = count == 0;
    int32_t beyond = -(int32_t)((D - (walked * count) % D) % D);
    auto advance = [&]() {
        if (ahead_b + NW < nblk) {
            ahead_b += NW;
        } else if (ahead_tile + 1u < walked) {
            ahead_b = wave;
            ahead_tile++;
            ahead_row = lane_row(tile_at(ahead_tile));
        } else {
            exhausted = true;
        }
    };
    auto fetch = [&](Unit &u) {
        const uint8_t *at = ahead_row + (size_t)min(ahead_b, nblk - 1u) * BLOCK_BYTES;
        if constexpr (SEAM::HANDS_RING) {
            if (exhausted && next_row) at = next_row + (size_t)min(wave + NW * (uint32_t)max(beyond, 0), next_nblk - 1u) * 144u;
            if (exhausted) beyond++;
        }
        u.hdr = *(global_uint4)(uintptr_t)(at - q * 32u);
        u.qa = *(global_uint4)(uintptr_t)(at + TO_NIBBLES);
        u.qb = *(global_uint4)(uintptr_t)(at + TO_NIBBLES + 16u);
        if constexpr (FIFTH) {
            u.fa = *(global_uint4)(uintptr_t)(at - q * 32u + 16u);
            u.fb = *(global_uint4)(uintptr_t)(at - q * 32u + 32u);
        }
        advance();
    };
    // TAKES_RING: the product before asked for this wave's first D units; the fetches here go on behind them
    auto first_fetches = [&]() {
#pragma unroll
        for (int i = 0; i < D; i++) {
            if constexpr (SEAM::TAKES_RING) advance();
            else fetch(ring[i]);
        }
    };

    // what the rotation's epilogue reads (the cursor, then cos, sin and bias of a tile's sixteen outputs) is fetched ahead:
    // the cursor with the activations, a tile's operands a tile early
    uint32_t rope_position = 0;
    RopeOperands rope_held{0.0f, 1.0f, 0.0f};
    constexpr bool CHAINED = SEAM::SHARED_IN || SEAM::SHARED_OUT;  // one of several products of a launch
    // the tag words of what this product reads and writes across a seam: the seam's number below the step's (a device word
    // that the step's first kernel moves on, so that what the step before left in the same place never passes for fresh)
    uint32_t tag_in = 0, tag_out = 0;
    float residual_held = 0.0f;  // chained: the residual of this workgroup's first tile (lanes 0..15), asked for ahead
    auto rope_row = [half_width, tiles_per_head, lane](uint32_t tile, uint32_t &c) -> uint32_t {
        c = (tile % tiles_per_head) * 8u + (lane & 7u);
        return (tile / tiles_per_head) * (2u * half_width) + c + ((lane >> 3) & 1u) * half_width;
    };

    // ---- handed-over planes (HANDED): one 16-byte piece a lane and super-block, into the LDS layout the walk reads
    constexpr int LATE = HANDED && SEAM::SHARED_IN ? 3 : 0;  // super-blocks a wave may look at only when its walk reaches them
    u32x4 late_held[LATE > 0 ? LATE : 1];
    uint32_t late_count = 0, early_count = 0;
    const uint32_t chunk = lane >> 2, piece = lane & 3u;
    auto handed_load = [&](uint32_t b, bool past) -> u32x4 {
        if constexpr (SEAM::SHARED_IN) return tile16_load16_either(lead_input, b * TILE16_BLOCK_HANDED + lane * 16u, past);
        else return tile16_load16<false>(lead_input, b * TILE16_BLOCK_HANDED + lane * 16u);
    };
    auto handed_put = [&](uint32_t b, const u32x4 &held) {
        uint8_t *planes = digits + (size_t)b * TILE16_BLOCK_DIGITS + chunk * 48u;
        uint8_t *const pairs = reinterpret_cast<uint8_t *>(sums);
        if (piece == 0u) {
            *reinterpret_cast<u32x4 *>(planes) = held;
        } else if (piece == 1u) {
            *reinterpret_cast<uint2 *>(planes + 16u) = uint2{held.x, held.y};
            *reinterpret_cast<uint32_t *>(planes + 24u) = held.z;
        } else if (piece == 2u) {
            *reinterpret_cast<uint32_t *>(planes + 28u) = held.x;
            *reinterpret_cast<uint2 *>(planes + 32u) = uint2{held.y, held.z};
            *reinterpret_cast<uint32_t *>(planes + 40u) = held.w;
        } else {
            *reinterpret_cast<uint32_t *>(planes + 44u) = held.x;
            *reinterpret_cast<uint2 *>(pairs + (size_t)b * TILE16_BLOCK_PAIRS + chunk * 8u) = uint2{held.y, held.z};
        }
    };
    // the late super-blocks' planes: read again past the L2 while any is stale, then put where the walk reads them
    auto late_stage = [&]() {
        if constexpr (LATE > 0) {
            for (uint32_t turn = 0;; turn++) {
                bool stale = false;
#pragma unroll
                for (int l = 0; l < LATE; l++) stale = stale || ((uint32_t)l < late_count && (piece & 1u) && late_held[l].w != tag_in);
                if (__builtin_amdgcn_ballot_w64(stale) == 0 && seam.spin) break;
                if (turn >= seam.spin) {
                    if (lane == 0) atomicMax(p.refusal, (uint32_t)REFUSAL_SEAM);
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
#pragma unroll
                for (int l = 0; l < LATE; l++) late_held[l] = handed_load(min(wave + NW * (early_count + l), nblk - 1u), true);
            }
#pragma unroll
            for (int l = 0; l < LATE; l++)
                if ((uint32_t)l < late_count) handed_put(wave + NW * (early_count + l), late_held[l]);
        }
    };

    // ---- activations -> three signed base-256 digit planes per 16 elements, a power-of-two scale per 64-element group.
    // Unit e4 = tid + NT * j (four consecutive activations) lies in super-block wave + NW * j: a wave turns into digits
    // exactly the super-blocks it multiplies.
    {
        const uint32_t units = nblk * 64u;
        if (lane < TILE16_ZERO_BYTES / 4u) reinterpret_cast<uint32_t *>(zeros)[lane] = 0u;
        auto stage = [&](uint32_t e4, f32x4 v, f32x4 w, float rms, uint8_t *row_planes, f32x4 *row_sums) {
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
            const float scale = __builtin_bit_cast(float, (275u - exponent) << 23);  // the group's largest magnitude lands in [2^21, 2^22)
            const float unscale = raw == 255u ? __builtin_bit_cast(float, 0x7fc00000u) : __builtin_bit_cast(float, (exponent - 21u) << 23);
            float total = 0.0f;
            uint32_t dg[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float rounded = rintf(v[i] * scale);
                total += rounded;
                dg[i] = signed_digits((int)rounded);  // bytes 0..2: signed digits, least significant first; byte 3 is zero below 2^23
            }
            const uint32_t lo01 = __builtin_amdgcn_perm(dg[1], dg[0], 0x05010400u), hi01 = __builtin_amdgcn_perm(dg[1], dg[0], 0x07030602u);
            const uint32_t lo23 = __builtin_amdgcn_perm(dg[3], dg[2], 0x05010400u), hi23 = __builtin_amdgcn_perm(dg[3], dg[2], 0x07030602u);
            const uint32_t plane2 = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);  // digit 0 (least significant) of the four elements
            const uint32_t plane1 = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
            const uint32_t plane0 = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);  // digit 2 (most significant)
            total += dpp<DPP_QUAD_XOR1>(total);
            total += dpp<DPP_QUAD_XOR2>(total);
            total += dpp<0x141>(total);  // half mirror: the other quad of the eight lanes of a sub-block
            // unit e4: 64 units a super-block, 16 a group, 8 a sub-block, 4 a chunk of 16 elements
            uint32_t *slot = reinterpret_cast<uint32_t *>(row_planes + (size_t)(e4 >> 2) * 48u) + (e4 & 3u);
            slot[0] = plane0, slot[4] = plane1, slot[8] = plane2;
            float *s = reinterpret_cast<float *>(row_sums + (e4 >> 4));  // (low sub-block sum, high sub-block sum, unscale, -)
            if ((e4 & 7u) == 0) s[(e4 >> 3) & 1u] = total * unscale;
            if ((e4 & 15u) == 0) s[2] = unscale;
        };
        if constexpr (HANDED) {
            // a wave copies the super-blocks it walks, one 16-byte load a lane and block.
            // A chunk of 16 activations is 64 bytes in memory, two sectors that each end in a tag word:
            //   words 0..3 plane 0 | 4..6 plane 1, first twelve | 7 tag || 8 plane 1, last four | 9..11 plane 2, first twelve |
            //   12 plane 2, last four | 13, 14 the (sum, scale) pair | 15 tag
            // lane 4 c + piece holds words 4 piece .. 4 piece + 3 of chunk c
            constexpr int MAXB = NW <= 8 ? 10 : 5;  // super-blocks a wave copies at once: ffn_down at eight waves has ten, all asked for together
            if constexpr (SEAM::WAITS) {
                // behind a seam: the first weights are asked for before the planes, which may not be there yet
                first_fetches();
                fetch_the_rest();
            }
            if constexpr (SEAM::SHARED_IN) tag_in = p.tag_in + 128u * *p.tick;
            // Behind a seam the planes of a wave's last super-blocks may be the ones the product before writes last (p.late_from:
            // the first such super-block): they are asked for with the others and looked at only when the walk reaches them,
            // by which time they have long arrived -- the walk does not wait at its start for what it needs at its end.
            if constexpr (LATE > 0) {
                uint32_t late = 0;
                for (uint32_t j = 0; j < count; j++) late += wave + NW * j >= p.late_from ? 1u : 0u;
                late_count = min(late, (uint32_t)LATE);
            }
            const uint32_t early = count - late_count;
            early_count = early;
            for (uint32_t j0 = 0; j0 < early || (j0 == 0 && LATE > 0); j0 += MAXB) {
                u32x4 held[MAXB];
                for (uint32_t turn = 0;; turn++) {
#pragma unroll
                    for (int j = 0; j < MAXB; j++) {
                        const uint32_t b = min(wave + NW * min(j0 + j, early ? early - 1u : 0u), nblk - 1u);
                        held[j] = handed_load(b, turn > 0);
                    }
                    if (j0 == 0 && turn == 0) {
                        if constexpr (LATE > 0) {
#pragma unroll
                            for (int l = 0; l < LATE; l++) late_held[l] = handed_load(min(wave + NW * (early + l), nblk - 1u), false);
                        }
                        if constexpr (!SEAM::WAITS) {
                            first_fetches();
                            fetch_the_rest();
                        }
                    }
                    if constexpr (!SEAM::SHARED_IN) break;
                    bool stale = false;
#pragma unroll
                    for (int j = 0; j < MAXB; j++) stale = stale || ((piece & 1u) && held[j].w != tag_in);
                    if ((__builtin_amdgcn_ballot_w64(stale) == 0 || early == 0) && seam.spin) break;  // (no turns at all: the tests' way to the refusal)
                    if (turn >= seam.spin) {
                        if (lane == 0) atomicMax(p.refusal, (uint32_t)REFUSAL_SEAM);
                        break;
                    }
                    __builtin_amdgcn_s_sleep(1);
                }
#pragma unroll
                for (int j = 0; j < MAXB; j++)
                    if (j0 + j < early) handed_put(wave + NW * (j0 + j), held[j]);
            }
            if (!SEAM::WAITS && LATE == 0 && count == 0) {
                first_fetches();
                fetch_the_rest();
            }
            if (CHAINED && p.residual && q == 0 && r < tile_rows)
                residual_held = __hip_atomic_load(p.residual + first_tile * tile_rows + r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else if constexpr (R > 1) {
            // the weights' loads go out first; every row's activations follow (twice where the norm is folded in: once for
            // the row's sum of squares, once for the digits -- the second pass finds them in the cache)
            first_fetches();
            fetch_the_rest();
            const uint32_t rows = min(p.rows, (uint32_t)R);
            if (lead_norm_w) {
                for (uint32_t row = 0; row < rows; row++) {
                    float square = 0.0f;
                    for (uint32_t e4 = tid; e4 < units; e4 += NT) {
                        const f32x4 v = *reinterpret_cast<const f32x4 *>(x + (size_t)row * p.K + 4u * e4);
#pragma unroll
                        for (int i = 0; i < 4; i++) square = __fadd_rn(square, __fmul_rn(v[i], v[i]));
                    }
                    square = wave_sum(square);
                    if (lane == 0) red[wave * R + row] = square;
                }
                __syncthreads();
            }
            for (uint32_t row = 0; row < rows; row++) {
                float rms = 1.0f;
                if (lead_norm_w) {
                    float total = 0.0f;
#pragma unroll
                    for (int w = 0; w < NW; w++) total += red[w * R + row];
                    rms = rms_scale_of(total, p.K, p.eps);
                }
                for (uint32_t e4 = tid; e4 < units; e4 += NT)
                    stage(e4, *reinterpret_cast<const f32x4 *>(x + (size_t)row * p.K + 4u * e4),
                          lead_norm_w ? *reinterpret_cast<const f32x4 *>(lead_norm_w + 4u * e4) : f32x4{0.f, 0.f, 0.f, 0.f}, rms, digits + (size_t)row * row_digits,
                          sums + (size_t)row * nblk * 4u);
            }
        } else {
        constexpr int MAXJ = 5;
        f32x4 held[MAXJ], weight[MAXJ];
        const bool resident = units <= MAXJ * NT;
        float rms = 1.0f;
        if constexpr (SEAM::WAITS) {
            // behind a seam: the first weights are asked for before the activations, which may not be there yet
            first_fetches();
            fetch_the_rest();
        }
        if constexpr (SEAM::SHARED_IN) {
            tag_in = p.tag_in + 128u * *p.tick;
            // the row arrives as (value, tag) pairs of eight bytes, written as one by the product before: four activations
            // are two 16-byte loads, read again until every pair of the wave carries this seam's tag (launch_chain takes no
            // row that does not fit the registers)
            if (lead_norm_w) {
#pragma unroll
                for (int j = 0; j < MAXJ; j++) {
                    const uint32_t e4 = tid + NT * j;
                    weight[j] = e4 < units ? *reinterpret_cast<const f32x4 *>(lead_norm_w + 4u * e4) : f32x4{0.f, 0.f, 0.f, 0.f};
                }
            }
            for (uint32_t turn = 0;; turn++) {
                bool stale = false;
#pragma unroll
                for (int j = 0; j < MAXJ; j++) {
                    const uint32_t e4 = tid + NT * j;
                    held[j] = f32x4{0.f, 0.f, 0.f, 0.f};
                    if (e4 < units) {
                        const u32x4 low = tile16_load16_either(lead_input, 32u * e4, turn > 0), high = tile16_load16_either(lead_input, 32u * e4 + 16u, turn > 0);
                        // (each word is copied to a scalar first: the bits of a vector element taken in place read element 0 every time)
                        const uint32_t v0 = low.x, v1 = low.z, v2 = high.x, v3 = high.z;
                        held[j] = f32x4{__builtin_bit_cast(float, v0), __builtin_bit_cast(float, v1), __builtin_bit_cast(float, v2), __builtin_bit_cast(float, v3)};
                        stale = stale || low.y != tag_in || low.w != tag_in || high.y != tag_in || high.w != tag_in;
                    }
                }
                if (__builtin_amdgcn_ballot_w64(stale) == 0 && seam.spin) break;  // (no turns at all: the tests' way to the refusal)
                if (turn >= seam.spin) {
                    if (lane == 0) atomicMax(p.refusal, (uint32_t)REFUSAL_SEAM);
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
        } else if (resident) {
#pragma unroll
            for (int j = 0; j < MAXJ; j++) {
                const uint32_t e4 = tid + NT * j;
                held[j] = e4 < units ? *reinterpret_cast<const f32x4 *>(x + 4u * e4) : f32x4{0.f, 0.f, 0.f, 0.f};
            }
            if (lead_norm_w) {
#pragma unroll
                for (int j = 0; j < MAXJ; j++) {
                    const uint32_t e4 = tid + NT * j;
                    weight[j] = e4 < units ? *reinterpret_cast<const f32x4 *>(lead_norm_w + 4u * e4) : f32x4{0.f, 0.f, 0.f, 0.f};
                }
            }
        }
        // the weights' loads go out behind the activations', which everything waits for first
        if constexpr (!SEAM::WAITS) {
            first_fetches();
            fetch_the_rest();
        }
        if (MODE == TILE16_ROPE && wave == 0 && lane < 16u) rope_position = p.rope_cursor[0];
        // the first tile's residual, where this launch wrote it or reads what is written here: asked for now, added at the tile's end
        if (CHAINED && MODE == TILE16_PLAIN && p.residual && q == 0 && r < tile_rows)
            residual_held = __hip_atomic_load(p.residual + first_tile * tile_rows + r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (lead_norm_w) {
            // sum of squares of the whole row (crates/neura-kernel/src/task/norm.rs:69-83; the same fp32 adds in another order)
            float square = 0.0f;
            if (resident) {
#pragma unroll
                for (int j = 0; j < MAXJ; j++)
#pragma unroll
                    for (int i = 0; i < 4; i++) square = __fadd_rn(square, __fmul_rn(held[j][i], held[j][i]));
            } else {
                for (uint32_t e4 = tid; e4 < units; e4 += NT) {
                    const f32x4 v = *reinterpret_cast<const f32x4 *>(x + 4u * e4);
#pragma unroll
                    for (int i = 0; i < 4; i++) square = __fadd_rn(square, __fmul_rn(v[i], v[i]));
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
            for (int j = 0; j < MAXJ; j++) {
                if (NT * j >= units) break;  // uniform over the workgroup
                const uint32_t e4 = tid + NT * j;
                if (e4 < units) stage(e4, held[j], weight[j], rms, digits, sums);  // whole groups of 16 lanes are in or out together
            }
        } else {
            for (uint32_t e4 = tid; e4 < units; e4 += NT)
                stage(e4, *reinterpret_cast<const f32x4 *>(x + 4u * e4), lead_norm_w ? *reinterpret_cast<const f32x4 *>(lead_norm_w + 4u * e4) : f32x4{0.f, 0.f, 0.f, 0.f}, rms,
                      digits, sums);
        }
        }
    }
    __builtin_amdgcn_wave_barrier();  // LDS serves a wave's accesses in order: the reads below see this wave's writes
    if (MODE == TILE16_ROPE && wave == 0 && lane < 16u) {
        uint32_t c;
        const uint32_t n = rope_row(tile_at(0), c);
        rope_held = rope_operands(p, n, c, rope_position);
    }
    // (planes that leave through a kernel boundary carry the seam's number alone: their reader does not look at tags, and the
    // step's word would be a load from memory that the walk's start waits for)
    if constexpr (SEAM::SHARED_OUT) tag_out = p.tag_out + (p.tick ? 128u * *p.tick : 0u);
    else if (MODE == TILE16_SWIGLU && R == 1) tag_out = p.tag_out;

    // ---- the walk
    const ScaleLane lane_scales = scale_lane(q);
    const uint32_t m = lane & 15u;
    const bool feeds = (m >> 2) == q && (m & 3u) < 3u;  // A row m = 4 * slice + plane meets K slice `slice` only
    const uint8_t *const abase = feeds ? digits + q * 192u + (m & 3u) * 16u : zeros;
    const uint32_t astride = feeds ? TILE16_BLOCK_DIGITS : 0u;
    const uint32_t arow = feeds ? row_digits : 0u;  // from one activation row's planes to the next one's
    constexpr int RQ = (R + 3) / 4;                 // rows an epilogue lane finishes: q, q + 4, ...
    float acc[R], gate[RQ];
#pragma unroll
    for (int row = 0; row < R; row++) acc[row] = 0.0f;
#pragma unroll
    for (int i = 0; i < RQ; i++) gate[i] = 0.0f;
    uint32_t parity = 0;
    // One step in two halves with the next fetch between them: everything that reads the fetched registers (nibbles, header)
    // comes first, so the fetch can reuse them, and the weighing of the sums follows while the loads are under way.
    struct Step {
        i32x4 cl, ch;
        f32x4 s;
        uint32_t sc, mn, dd;
    };
    auto multiply = [&](const Unit &u, uint32_t b, Step &st) {
        const uint8_t *at = abase + (size_t)b * astride;
        const i32x4 a00 = *reinterpret_cast<const i32x4 *>(at), a01 = *reinterpret_cast<const i32x4 *>(at + 48);
        const i32x4 a10 = *reinterpret_cast<const i32x4 *>(at + 96), a11 = *reinterpret_cast<const i32x4 *>(at + 144);
        st.s = sums[b * 4u + q];
        u32x4 la_, ha_, lb_, hb_;
        tile16_codes<FIFTH>(u, q, la_, ha_, lb_, hb_);
        const i32x4 la = (i32x4)la_, ha = (i32x4)ha_, lb = (i32x4)lb_, hb = (i32x4)hb_;
        half2_t sc, mn;
        scale_pairs(u.hdr, lane_scales, sc, mn);
        st.sc = __builtin_bit_cast(uint32_t, sc), st.mn = __builtin_bit_cast(uint32_t, mn), st.dd = u.hdr.x;
        i32x4 cl = {0, 0, 0, 0}, ch = {0, 0, 0, 0};
        cl = __builtin_amdgcn_mfma_i32_16x16x64_i8(a00, la, cl, 0, 0, 0);
        ch = __builtin_amdgcn_mfma_i32_16x16x64_i8(a10, ha, ch, 0, 0, 0);
        cl = __builtin_amdgcn_mfma_i32_16x16x64_i8(a01, lb, cl, 0, 0, 0);
        ch = __builtin_amdgcn_mfma_i32_16x16x64_i8(a11, hb, ch, 0, 0, 0);
        st.cl = cl, st.ch = ch;
        asm volatile("" : "+v"(st.sc), "+v"(st.mn), "+v"(st.dd));  // the header is read by here
    };
    auto weigh = [&](const Step &st) {
        const half2_t sc = __builtin_bit_cast(half2_t, st.sc), mn = __builtin_bit_cast(half2_t, st.mn), dd = __builtin_bit_cast(half2_t, st.dd);
        // (c0 * 256 + c1) fits 24 bits: one conversion for two planes
        const float fl = fmaf((float)((st.cl[0] << 8) + st.cl[1]), 256.0f, (float)st.cl[2]);
        const float fh = fmaf((float)((st.ch[0] << 8) + st.ch[1]), 256.0f, (float)st.ch[2]);
        const float weighed = fmaf((float)sc.x, fl, (float)sc.y * fh);    // scales and minimums arrive * 2^-24 (half subnormals)
        const float floor_ = fmaf((float)mn.x, st.s.x, (float)mn.y * st.s.y);
        const float d24 = (float)dd.x * (16777216.0f * st.s.z), m24 = (float)dd.y * -16777216.0f;
        acc[0] = fmaf(d24, weighed, fmaf(m24, floor_, acc[0]));
    };
    // handed-over planes: a chunk of 16 has its own scale, so the four MFMAs keep their sums apart
    struct HandedStep {
        i32x4 c[4];
        f32x4 low, high;  // (sum, scale) of chunks 0, 1 and of chunks 2, 3 of the lane's group
        uint32_t sc, mn, dd;
    };
    auto multiply_handed = [&](const Unit &u, uint32_t b, HandedStep &st) {
        const uint8_t *at = abase + (size_t)b * astride;
        const i32x4 a00 = *reinterpret_cast<const i32x4 *>(at), a01 = *reinterpret_cast<const i32x4 *>(at + 48);
        const i32x4 a10 = *reinterpret_cast<const i32x4 *>(at + 96), a11 = *reinterpret_cast<const i32x4 *>(at + 144);
        st.low = sums[b * 8u + 2u * q], st.high = sums[b * 8u + 2u * q + 1u];
        u32x4 la_, ha_, lb_, hb_;
        tile16_codes<FIFTH>(u, q, la_, ha_, lb_, hb_);
        const i32x4 la = (i32x4)la_, ha = (i32x4)ha_, lb = (i32x4)lb_, hb = (i32x4)hb_;
        half2_t sc, mn;
        scale_pairs(u.hdr, lane_scales, sc, mn);
        st.sc = __builtin_bit_cast(uint32_t, sc), st.mn = __builtin_bit_cast(uint32_t, mn), st.dd = u.hdr.x;
        const i32x4 none = {0, 0, 0, 0};
        st.c[0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a00, la, none, 0, 0, 0);
        st.c[2] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a10, ha, none, 0, 0, 0);
        st.c[1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a01, lb, none, 0, 0, 0);
        st.c[3] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a11, hb, none, 0, 0, 0);
        asm volatile("" : "+v"(st.sc), "+v"(st.mn), "+v"(st.dd));  // the header is read by here
    };
    auto weigh_handed = [&](const HandedStep &st) {
        const half2_t sc = __builtin_bit_cast(half2_t, st.sc), mn = __builtin_bit_cast(half2_t, st.mn), dd = __builtin_bit_cast(half2_t, st.dd);
        float f[4];
#pragma unroll
        for (int i = 0; i < 4; i++) f[i] = fmaf((float)((st.c[i][0] << 8) + st.c[i][1]), 256.0f, (float)st.c[i][2]);
        const float fl = fmaf(st.low.y, f[0], st.low.w * f[1]), fh = fmaf(st.high.y, f[2], st.high.w * f[3]);  // scales are powers of two
        const float weighed = fmaf((float)sc.x, fl, (float)sc.y * fh);
        const float floor_ = fmaf((float)mn.x, st.low.x + st.low.z, (float)mn.y * (st.high.x + st.high.z));
        const float d24 = (float)dd.x * 16777216.0f, m24 = (float)dd.y * -16777216.0f;
        acc[0] = fmaf(d24, weighed, fmaf(m24, floor_, acc[0]));
    };
    // R > 1: the weights are unpacked once, the next fetch goes out, and every row then runs its four MFMAs and its weighing.
    // Only the twelve lanes that feed the matrix cores read their operands from LDS; the other lanes' operand registers are
    // cleared once and never written again (a read by all 64 lanes costs LDS eight clocks a time, most of them for zeros).
    constexpr int G = R < 4 ? R : (NW > 8 ? 2 : 4);  // rows a phase; sixteen waves a workgroup leave a wave 128 registers
    i32x4 a[G][4];
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
        for (int k = 0; k < 4; k++) a[g][k] = i32x4{0, 0, 0, 0};
    auto step_rows = [&](Unit &u, uint32_t b) {
        const u32x4 mask = {0x0f0f0f0fu, 0x0f0f0f0fu, 0x0f0f0f0fu, 0x0f0f0f0fu};
        const i32x4 la = (i32x4)(u.qa & mask), ha = (i32x4)((u.qa >> 4) & mask);
        const i32x4 lb = (i32x4)(u.qb & mask), hb = (i32x4)((u.qb >> 4) & mask);
        half2_t sc, mn;
        scale_pairs(u.hdr, lane_scales, sc, mn);
        const half2_t dd = __builtin_bit_cast(half2_t, u.hdr.x);
        float scx = (float)sc.x, scy = (float)sc.y, mnx = (float)mn.x, mny = (float)mn.y;
        float d24 = (float)dd.x * 16777216.0f, m24 = (float)dd.y * -16777216.0f;
        asm volatile("" : "+v"(scx), "+v"(scy), "+v"(mnx), "+v"(mny), "+v"(d24), "+v"(m24));  // the header is read by here
        __builtin_amdgcn_sched_barrier(0);
        fetch(u);
        __builtin_amdgcn_sched_barrier(0);
        // Rows go four at a time through three phases -- every operand read from LDS, every MFMA, every weighing -- so that
        // a row's reads and matrix-core results are waited for behind the other rows' work, not one row after another.
#pragma unroll
        for (int first = 0; first < R; first += G) {
            const uint8_t *at = abase + (size_t)b * astride + (size_t)first * arow;
            const f32x4 *s = sums + b * 4u + q + (size_t)first * nblk * 4u;
            i32x4 cl[G], ch[G];
            f32x4 rs[G];
            if (feeds) {
#pragma unroll
                for (int g = 0; g < G; g++) {
                    const uint8_t *from = at + (size_t)g * arow;
                    a[g][0] = *reinterpret_cast<const i32x4 *>(from), a[g][1] = *reinterpret_cast<const i32x4 *>(from + 48);
                    a[g][2] = *reinterpret_cast<const i32x4 *>(from + 96), a[g][3] = *reinterpret_cast<const i32x4 *>(from + 144);
                }
            }
#pragma unroll
            for (int g = 0; g < G; g++) {
                rs[g] = *s;
                s += nblk * 4u;
            }
            __builtin_amdgcn_sched_barrier(0);
            const i32x4 none = {0, 0, 0, 0};
#pragma unroll
            for (int g = 0; g < G; g++) {
                cl[g] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[g][0], la, none, 0, 0, 0);
                ch[g] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[g][2], ha, none, 0, 0, 0);
            }
#pragma unroll
            for (int g = 0; g < G; g++) {
                cl[g] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[g][1], lb, cl[g], 0, 0, 0);
                ch[g] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[g][3], hb, ch[g], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int g = 0; g < G; g++) {
                const float fl = fmaf((float)((cl[g][0] << 8) + cl[g][1]), 256.0f, (float)cl[g][2]);
                const float fh = fmaf((float)((ch[g][0] << 8) + ch[g][1]), 256.0f, (float)ch[g][2]);
                const float weighed = fmaf(scx, fl, scy * fh);
                const float floor_ = fmaf(mnx, rs[g].x, mny * rs[g].y);
                acc[first + g] = fmaf(d24 * rs[g].z, weighed, fmaf(m24, floor_, acc[first + g]));
            }
        }
    };
    // The wave that finishes a tile (sums the waves' parts, runs the epilogue) changes from tile to tile (with SwiGLU from pair
    // to pair: the gate sum waits in its registers), so that no wave falls behind the others by an epilogue a tile.
    auto tile_end = [&](uint32_t tile, uint32_t index) {
        const uint32_t finisher = MODE == TILE16_ROPE ? 0u : (MODE == TILE16_SWIGLU ? index >> 1 : index) % NW;
#pragma unroll
        for (int row = 0; row < R; row++) {
            float v = acc[row];
            v += __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));  // lane ^ 16
            v += __shfl_xor(v, 32, 64);
            if (q == 0) part[((parity * NW + wave) * R + row) * 16u + r] = v;
            acc[row] = 0.0f;
        }
        __syncthreads();
        if (wave == finisher) {
#pragma unroll
          for (int i = 0; i < RQ; i++) {
            // lane (r, q) finishes output r of activation rows q, q + 4, ...
            const uint32_t row = q + 4u * i;
            if (row >= min(p.rows, (uint32_t)R)) break;
            float total = 0.0f;
#pragma unroll
            for (int w = 0; w < NW; w++) total += part[((parity * NW + w) * R + row) * 16u + r];
            if (MODE == TILE16_SWIGLU) {
                if (!(tile & 1u)) {
                    gate[i] = total;
                } else if (R == 1 && p.digits_out) {
                    // the sixteen outputs of this pair are chunk tile / 2 of the next product's activations
                    const uint32_t word = handed_piece_word(silu(gate[i]) * total, r, tag_out);
                    tile16_store_word<SEAM::SHARED_OUT>(reinterpret_cast<uint32_t *>(p.digits_out + (size_t)(tile >> 1) * 64u) + r, word);
                } else {
                    tile16_store_word<SEAM::SHARED_OUT>(reinterpret_cast<uint32_t *>(p.y + (size_t)row * (p.N / 2u) + (tile >> 1) * 16u + r),
                                                        __builtin_bit_cast(uint32_t, silu(gate[i]) * total));
                }
            } else if (MODE == TILE16_ROPE) {
                uint32_t c;
                const uint32_t n = rope_row(tile, c);
                rope_store(p, total, n, lane >= 8u, rope_position, rope_held);
                if (tile + hop < tiles) {  // the next tile of this workgroup
                    const uint32_t next = rope_row(tile + hop, c);
                    rope_held = rope_operands(p, next, c, rope_position);
                }
            } else if (r < tile_rows) {
                const size_t n = (size_t)row * p.N + tile * tile_rows + r;
                if constexpr (CHAINED) {
                    // what another die wrote or will read inside this launch goes past the L2: no add in the cache, the
                    // residual read at device scope (the first tile's was asked for ahead) and the sum stored at device scope
                    float old = 0.0f;
                    if (p.residual) old = index == 0 ? residual_held : __hip_atomic_load(p.residual + n, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    const float value = old + total;
                    tile16_store_word<true>(reinterpret_cast<uint32_t *>(p.y + n), __builtin_bit_cast(uint32_t, value));
                    // for the product behind the seam: the number with the seam's tag beside it, eight bytes stored as one
                    if (SEAM::SHARED_OUT && p.pairs_out)
                        __hip_atomic_store(reinterpret_cast<unsigned long long *>(p.pairs_out) + n,
                                           (unsigned long long)__builtin_bit_cast(uint32_t, value) | ((unsigned long long)tag_out << 32), __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
                } else if (p.residual == p.y) {
                    // in place (the decoder's residual stream): one add per element, nothing to wait for
                    unsafeAtomicAdd(p.y + n, total);
                } else {
                    p.y[n] = p.residual ? p.residual[n] + total : total;
                }
                if constexpr (MODE == TILE16_APPEND) {
                    // a value projection of one token: its rows (+ bias) go into the value state at the cursor, as
                    // value_append_kernel would cast them
                    const uint32_t cursor = p.rope_cursor[0];
                    const float value = p.bias[0] ? total + p.bias[0][n] : total;
                    const uint32_t slot = p.rope_ring ? cursor % p.rope_ring : cursor;
                    if (slot >= p.rope_capacity) atomicMax(p.refusal, (uint32_t)REFUSAL_ORIGIN);
                    else state_store(p.rope_v, p.rope_element, ((uint64_t)((uint32_t)n / p.rope_width) * p.rope_capacity + slot) * p.rope_width + (uint32_t)n % p.rope_width, value);
                }
            }
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
            if constexpr (R > 1) {
                step_rows(ring[slot], at_b);
            } else if constexpr (HANDED) {
                if (LATE > 0 && late_count && s0 + slot == early_count) late_stage();
                HandedStep st;
                multiply_handed(ring[slot], at_b, st);
                __builtin_amdgcn_sched_barrier(0);
                fetch(ring[slot]);
                __builtin_amdgcn_sched_barrier(0);
                weigh_handed(st);
            } else {
                Step st;
                multiply(ring[slot], at_b, st);
                __builtin_amdgcn_sched_barrier(0);  // the fetch reuses this unit's registers: keep its loads behind their last use
                fetch(ring[slot]);
                __builtin_amdgcn_sched_barrier(0);
                weigh(st);
            }
            at_b += NW;
            if (at_b >= nblk) {
                if (at_tile < walked) tile_end(tile_at(at_tile), at_tile);
                at_b = wave;
                at_tile++;
            }
        }
    }
}

// The leading arguments are what a wave needs before it can ask for its first activations and weights.  They are plain words
// so that the hardware can hand them over in scalar registers when it starts the wave (the file is built with
// -amdgpu-kernarg-preload-count): the wave's first loads then go out without waiting for a load of its parameters
// (about 0.5 us); everything else sits in `p` and is fetched meanwhile.  `input` is x, or the digit planes with HANDED.
template <int NW, int D, int MODE, int R, bool HANDED = false, bool FIFTH = false>
__global__ __launch_bounds__(NW * 64) void gemv_q4k_tile16_kernel(const uint8_t *lead_w0, const void *lead_input, const float *lead_norm_w, int32_t lead_to_w1,
                                                                  int32_t lead_to_w2, uint32_t lead_row_bytes, uint32_t lead_grid, uint32_t lead_tiles,
                                                                  uint32_t lead_tile_rows, uint32_t lead_end0, uint32_t lead_end1, GemvParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t tile16_lds_bytes[];
    typename Tile16UnitOf<FIFTH>::type ring[D];
    tile16_product<NW, D, MODE, R, HANDED, NoSeam, FIFTH>(tile16_lds_bytes, blockIdx.x, NoSeam{}, ring, nullptr, 0u, lead_w0, lead_input, lead_norm_w, lead_to_w1, lead_to_w2,
                                                          lead_row_bytes, lead_grid, lead_tiles, lead_tile_rows, lead_end0, lead_end1, p);
}

// ---------------------------------------------------------------------------------------------------------------------
// Two to eight activation rows against a Q4_K matrix, four rows to an MFMA, the sub-block scales inside the operand.
//
// The block-diagonal operand above spends a whole MFMA on one activation row (its A rows are slices of that row), so every
// further row costs four more of them: measured, 4.7 us a row on gate|up, all of it matrix-core time.  Here the sixteen A rows
// are (activation row, digit plane) pairs -- row m = 4 i + plane, four activation rows an instruction -- and an MFMA's K runs
// over a whole 64-element group, which it may because the weights enter already multiplied by their sub-block's scale: a six-
// bit scale is sc = 8 hi + lo with hi, lo < 8, and nibble * hi and nibble * lo (at most 105) are both bytes, so two MFMAs a
// group, accumulated over the four groups of a super-block, leave 8 * C_hi + C_lo = sum of digit * nibble * sc in integers, exact.
// One multiplication makes four such bytes (a word of nibbles times hi or lo: no byte carries into the next).  What is left to
// fp32 per super-block and activation row is one conversion of the three plane sums, the activation scale and d; the minimums
// come off against sub-block sums as in the one-row kernel.  The activations' power-of-two scale is a super-block's here, not
// a 64-element group's (the digits of a super-block meet in one integer sum): 22 bits below the largest magnitude of 256.
// Lane (r, s) = (lane % 16, lane / 16) supplies, for every group, the eight bytes 8 s .. 8 s + 7 of weight row r -- low nibbles
// elements 8 s .., high nibbles elements 32 + 8 s .. -- and the digit planes are staged in that order (slot 16 s + 8 half + t of
// a group's 64), so an operand is one aligned 16-byte read; it receives C column r, rows 4 s .. 4 s + 3: the three plane sums
// of activation row s against ITS weight row, so again no sum crosses lanes.  A wave turns into digits exactly the
// super-blocks it walks, all rows' activations asked for at once.  Launched for three and four rows (P = 1): there it beats
// the block-diagonal form by 13 % a layer (gate|up 25.9 against 30.7 us); at two rows that form is ahead (21.8 against 23.7),
// and two passes over the unpacked weights (P = 2, rows 0..3 then 4..7) tie with the 32-row and half-precision tiles at five
// to eight rows (gate|up 34 against 36 us, the plain products 16 against 14) -- turning eight rows into digits in every
// workgroup (6.6 us) is what bounds them -- so those keep their kernels.
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
struct Rows4Unit {
    u32x4 hdr;
    u32x2 w[4];
};

static size_t rows4_row_stride(uint32_t nblk) {
    const size_t bytes = (size_t)nblk * TILE16_BLOCK_DIGITS + 64u;  // the idle A rows (plane 3) read 64 bytes past a group
    return (bytes + 255u) / 256u * 256u + 64u;  // rows 64 bytes apart modulo the banks' 256: the four rows of an operand read spread over them
}
static size_t rows4_lds(uint32_t nblk, uint32_t NW, uint32_t rows) {
    return rows * rows4_row_stride(nblk) + (size_t)rows * nblk * 48u + (size_t)2 * NW * 64u * (rows / 4u) * 4u + (size_t)NW * rows * 4u + 64u;
}

template <int NW, int D, int MODE, int P>
__global__ __launch_bounds__(NW * 64) void gemv_q4k_rows4_kernel(GEMV_LEAD_PARAMETERS) {
    GEMV_TAKE_LEAD;
    static_assert(MODE == TILE16_PLAIN || MODE == TILE16_SWIGLU, "no rotation is folded into a product of several rows");
    extern __shared__ __attribute__((aligned(16))) uint8_t rows4_lds_bytes[];
    constexpr uint32_t NT = NW * 64, ROWS = 4 * P;
    typedef int i32x4 __attribute__((ext_vector_type(4)));
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    typedef const __attribute__((address_space(1))) u32x4 *global_uint4;
    typedef const __attribute__((address_space(1))) u32x2 *global_uint2;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t nblk = p.nblk;
    const uint32_t row_stride = (uint32_t)(((size_t)nblk * TILE16_BLOCK_DIGITS + 64u + 255u) / 256u * 256u + 64u);
    uint8_t *const digits = rows4_lds_bytes;
    float *const sums = reinterpret_cast<float *>(rows4_lds_bytes + (size_t)ROWS * row_stride);  // [row][block][8 sums, 4 scales]
    float *const part = sums + (size_t)ROWS * nblk * 12u;                                          // [parity][wave][pass][lane]
    float *const red = part + 2u * NW * P * 64u;                                                   // [wave][row]
    const uint32_t r = lane & 15u, s = lane >> 4;
    const uint32_t tiles = p.row_groups;
    if (blockIdx.x >= tiles) return;
    const uint32_t ntiles = (tiles - blockIdx.x + gridDim.x - 1u) / gridDim.x;
    const uint32_t count = wave < nblk ? (nblk - wave + NW - 1u) / NW : 0u;
    const uint32_t rows = min(p.rows, ROWS);

    const uint8_t *const w0 = p.W[0];
    const int64_t to_w1 = p.W[1] - p.W[0], to_w2 = p.W[2] - p.W[0];
    const uint32_t end0 = p.end[0], end1 = p.end[1], row_bytes = p.row_bytes;
    const uint32_t first_tile = blockIdx.x, hop = gridDim.x;
    const uint32_t tile_rows = MODE == TILE16_PLAIN ? p.tile_rows : 16u;
    auto lane_row = [w0, to_w1, to_w2, end0, end1, row_bytes, tile_rows, r, s](uint32_t tile) -> const uint8_t * {
        (void)tile_rows;
        int64_t offset;
        if (MODE == TILE16_SWIGLU) {
            offset = ((tile & 1u) ? to_w1 : (int64_t)0) + (int64_t)((tile >> 1) * 16u + r) * row_bytes;
        } else {
            const uint32_t n = tile * tile_rows + min(r, tile_rows - 1u);
            const bool in0 = n < end0, in1 = n < end1;
            const int64_t matrix = in0 ? (int64_t)0 : (in1 ? to_w1 : to_w2);
            const uint32_t before = in0 ? 0u : (in1 ? end0 : end1);
            offset = matrix + (int64_t)(n - before) * row_bytes;
        }
        return w0 + offset + s * 8u;
    };
    auto tile_at = [first_tile, hop](uint32_t i) -> uint32_t {
        if (MODE == TILE16_SWIGLU) return 2u * (first_tile + (i >> 1) * hop) + (i & 1u);
        return first_tile + i * hop;
    };
    const uint32_t walked = MODE == TILE16_SWIGLU ? 2u * ntiles : ntiles;

    Rows4Unit ring[D];
    uint32_t ahead_tile = 0, ahead_b = wave;
    const uint8_t *ahead_row = lane_row(tile_at(0));
    auto fetch = [&](Rows4Unit &u) {
        const uint8_t *at = ahead_row + (size_t)min(ahead_b, nblk - 1u) * 144u;
        u.hdr = *(global_uint4)(uintptr_t)(at - s * 8u);
#pragma unroll
        for (int g = 0; g < 4; g++) u.w[g] = *(global_uint2)(uintptr_t)(at + 16u + 32u * g);
        if (ahead_b + NW < nblk) {
            ahead_b += NW;
        } else if (ahead_tile + 1u < walked) {
            ahead_b = wave;
            ahead_tile++;
            ahead_row = lane_row(tile_at(ahead_tile));
        }
    };
#pragma unroll
    for (int i = 0; i < D; i++) fetch(ring[i]);

    // ---- activations -> digit planes: unit e4 = tid + NT * j (four consecutive activations) lies in super-block wave + NW * j
    {
        const uint32_t units = p.K / 4u;
        auto stage = [&](uint32_t row, uint32_t e4, f32x4 v, f32x4 w, float rms) {
            if (p.norm_w) {
#pragma unroll
                for (int i = 0; i < 4; i++) v[i] = __fmul_rn(__fmul_rn(v[i], rms), w[i]);
            }
            uint32_t top = 0;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float element = v[i];
                top = max(top, __builtin_bit_cast(uint32_t, element) & 0x7fffffffu);
            }
            // the largest magnitude of the super-block: its 64 units are the 64 lanes of this wave
            top = max(top, (uint32_t)dpp_int<DPP_QUAD_XOR1>((int)top));
            top = max(top, (uint32_t)dpp_int<DPP_QUAD_XOR2>((int)top));
            top = max(top, (uint32_t)dpp_int<DPP_ROW_ROR4>((int)top));
            top = max(top, (uint32_t)dpp_int<DPP_ROW_ROR8>((int)top));
            top = max(top, (uint32_t)__builtin_amdgcn_ds_swizzle((int)top, 0x401F));  // lane ^ 16
            top = max(top, (uint32_t)__shfl_xor((int)top, 32, 64));
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
                dg[i] = signed_digits((int)rounded);
            }
            const uint32_t lo01 = __builtin_amdgcn_perm(dg[1], dg[0], 0x05010400u), hi01 = __builtin_amdgcn_perm(dg[1], dg[0], 0x07030602u);
            const uint32_t lo23 = __builtin_amdgcn_perm(dg[3], dg[2], 0x05010400u), hi23 = __builtin_amdgcn_perm(dg[3], dg[2], 0x07030602u);
            const uint32_t plane2 = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);  // least significant digits
            const uint32_t plane1 = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
            const uint32_t plane0 = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);  // most significant
            total += dpp<DPP_QUAD_XOR1>(total);
            total += dpp<DPP_QUAD_XOR2>(total);
            total += dpp<0x141>(total);  // the other quad of the eight lanes of a sub-block
            // unit e4: 64 a super-block, 16 a group, 8 a sub-block.  Elements e = 4 (e4 % 16) .. + 3 of their group sit in slot
            // 16 ((e % 32) / 8) + 8 (e / 32) + e % 8 of the group's 64: the order the weights' bytes unpack in
            const uint32_t e = 4u * (e4 & 15u);
            const uint32_t seat = 16u * ((e & 31u) >> 3) + 8u * (e >> 5) + (e & 7u);
            uint8_t *group = digits + (size_t)row * row_stride + (size_t)(e4 >> 6) * TILE16_BLOCK_DIGITS + ((e4 >> 4) & 3u) * 192u + seat;
            *reinterpret_cast<uint32_t *>(group) = plane0, *reinterpret_cast<uint32_t *>(group + 64) = plane1, *reinterpret_cast<uint32_t *>(group + 128) = plane2;
            float *held = sums + (size_t)row * nblk * 12u + (size_t)(e4 >> 6) * 12u;
            if ((e4 & 7u) == 0) held[(e4 >> 3) & 7u] = total * unscale;
            if ((e4 & 63u) == 0) held[8] = unscale;
        };
        constexpr int MAXJ = 2;
        if (units <= MAXJ * NT) {
            // every row's activations are asked for at once and wait in registers: a row at a time pays a round trip to the
            // cache a row
            f32x4 held[ROWS][MAXJ], weight[MAXJ];
#pragma unroll
            for (int row = 0; row < (int)ROWS; row++)
#pragma unroll
                for (int j = 0; j < MAXJ; j++) {
                    const uint32_t e4 = tid + NT * j;
                    held[row][j] = (uint32_t)row < rows && e4 < units ? *reinterpret_cast<const f32x4 *>(p.x + (size_t)row * p.K + 4u * e4) : f32x4{0.f, 0.f, 0.f, 0.f};
                }
            float rms[ROWS];
#pragma unroll
            for (int row = 0; row < (int)ROWS; row++) rms[row] = 1.0f;
            if (p.norm_w) {
#pragma unroll
                for (int j = 0; j < MAXJ; j++) {
                    const uint32_t e4 = tid + NT * j;
                    weight[j] = e4 < units ? *reinterpret_cast<const f32x4 *>(p.norm_w + 4u * e4) : f32x4{0.f, 0.f, 0.f, 0.f};
                }
#pragma unroll
                for (int row = 0; row < (int)ROWS; row++) {
                    float square = 0.0f;  // the row's sum of squares, thread by thread in the order the row-at-a-time loop adds them
#pragma unroll
                    for (int j = 0; j < MAXJ; j++)
#pragma unroll
                        for (int i = 0; i < 4; i++) square = __fadd_rn(square, __fmul_rn(held[row][j][i], held[row][j][i]));
                    square = wave_sum(square);
                    if (lane == 0) red[wave * ROWS + row] = square;
                }
                __syncthreads();
#pragma unroll
                for (int row = 0; row < (int)ROWS; row++) {
                    float total = 0.0f;
#pragma unroll
                    for (int w = 0; w < NW; w++) total += red[w * ROWS + row];
                    rms[row] = rms_scale_of(total, p.K, p.eps);
                }
            }
#pragma unroll
            for (int row = 0; row < (int)ROWS; row++) {
                if ((uint32_t)row >= rows) break;
#pragma unroll
                for (int j = 0; j < MAXJ; j++) {
                    const uint32_t e4 = tid + NT * j;
                    if (e4 < units) stage(row, e4, held[row][j], weight[j], rms[row]);  // whole groups of 16 lanes are in or out together
                }
            }
        } else {
            if (p.norm_w) {
                for (uint32_t row = 0; row < rows; row++) {
                    float square = 0.0f;
                    for (uint32_t e4 = tid; e4 < units; e4 += NT) {
                        const f32x4 v = *reinterpret_cast<const f32x4 *>(p.x + (size_t)row * p.K + 4u * e4);
#pragma unroll
                        for (int i = 0; i < 4; i++) square = __fadd_rn(square, __fmul_rn(v[i], v[i]));
                    }
                    square = wave_sum(square);
                    if (lane == 0) red[wave * ROWS + row] = square;
                }
                __syncthreads();
            }
            for (uint32_t row = 0; row < rows; row++) {
                float rms = 1.0f;
                if (p.norm_w) {
                    float total = 0.0f;
#pragma unroll
                    for (int w = 0; w < NW; w++) total += red[w * ROWS + row];
                    rms = rms_scale_of(total, p.K, p.eps);
                }
                for (uint32_t e4 = tid; e4 < units; e4 += NT)
                    stage(row, e4, *reinterpret_cast<const f32x4 *>(p.x + (size_t)row * p.K + 4u * e4),
                          p.norm_w ? *reinterpret_cast<const f32x4 *>(p.norm_w + 4u * e4) : f32x4{0.f, 0.f, 0.f, 0.f}, rms);
            }
        }
    }
    __builtin_amdgcn_wave_barrier();  // LDS serves a wave's accesses in order: the reads below see this wave's writes

    // ---- the walk.  A row m = 4 i + plane of pass `pass` is activation row 4 pass + i; lane (m, s) reads digits 16 s .. of a group
    const uint32_t m = lane & 15u;
    const uint8_t *const abase = digits + (size_t)(m >> 2) * row_stride + (m & 3u) * 64u + s * 16u;
    const float *const sbase = sums + (size_t)s * nblk * 12u;  // this lane's activation row of pass 0 is row s
    float acc[P], gate[P];
#pragma unroll
    for (int i = 0; i < P; i++) acc[i] = 0.0f, gate[i] = 0.0f;
    uint32_t parity = 0;
    auto step = [&](Rows4Unit &u, uint32_t b) {
        // the eight scales and minimums of the row (crates/neura-precision/src/ggml.rs:127-136), four to a word
        const uint32_t sc_words[2] = {u.hdr.y & 0x3f3f3f3fu, (u.hdr.w & 0x0f0f0f0fu) | ((u.hdr.y >> 2) & 0x30303030u)};
        const uint32_t mn_words[2] = {u.hdr.z & 0x3f3f3f3fu, ((u.hdr.w >> 4) & 0x0f0f0f0fu) | ((u.hdr.z >> 2) & 0x30303030u)};
        // the lane's weights times their scale's two digits, a group an operand: bytes 0..7 the low nibbles (sub-block 2 g),
        // bytes 8..15 the high ones (sub-block 2 g + 1)
        i32x4 high_part[4], low_part[4];
        float mn[8];
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const uint32_t word = sc_words[g >> 1], shift = 16u * (g & 1u);
            const uint32_t hi_a = (word >> (shift + 3u)) & 7u, lo_a = (word >> shift) & 7u;            // sub-block 2 g
            const uint32_t hi_b = (word >> (shift + 11u)) & 7u, lo_b = (word >> (shift + 8u)) & 7u;    // sub-block 2 g + 1
            const uint32_t n0 = u.w[g].x & 0x0f0f0f0fu, n1 = u.w[g].y & 0x0f0f0f0fu;
            const uint32_t n2 = (u.w[g].x >> 4) & 0x0f0f0f0fu, n3 = (u.w[g].y >> 4) & 0x0f0f0f0fu;
            // a word of four nibbles times a digit below 8, as two packed 16-bit products: no byte carries into the next
            // (a full 32-bit multiplication runs at a quarter of the rate)
            typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));
            auto times = [](uint32_t nibbles, uint32_t digit) -> int {
                const u16x2 both = {(uint16_t)digit, (uint16_t)digit};
                return __builtin_bit_cast(int, __builtin_bit_cast(u16x2, nibbles) * both);
            };
            high_part[g] = i32x4{times(n0, hi_a), times(n1, hi_a), times(n2, hi_b), times(n3, hi_b)};
            low_part[g] = i32x4{times(n0, lo_a), times(n1, lo_a), times(n2, lo_b), times(n3, lo_b)};
            mn[2 * g] = (float)((mn_words[g >> 1] >> shift) & 0xffu), mn[2 * g + 1] = (float)((mn_words[g >> 1] >> (shift + 8u)) & 0xffu);
        }
        const half2_t dd = __builtin_bit_cast(half2_t, u.hdr.x);
        float scale_d = (float)dd.x, scale_m = -(float)dd.y;
        asm volatile("" : "+v"(scale_d), "+v"(scale_m));  // the header is read by here
        __builtin_amdgcn_sched_barrier(0);
        fetch(u);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int pass = 0; pass < P; pass++) {
            const uint8_t *at = abase + (size_t)pass * 4u * row_stride + (size_t)b * TILE16_BLOCK_DIGITS;
            const float *held = sbase + (size_t)pass * 4u * nblk * 12u + (size_t)b * 12u;
            i32x4 a[4];
#pragma unroll
            for (int g = 0; g < 4; g++) a[g] = *reinterpret_cast<const i32x4 *>(at + 192 * g);
            const f32x4 s0 = *reinterpret_cast<const f32x4 *>(held), s1 = *reinterpret_cast<const f32x4 *>(held + 4);
            const float unscale = held[8];
            i32x4 ch = {0, 0, 0, 0}, cl = {0, 0, 0, 0};
#pragma unroll
            for (int g = 0; g < 4; g++) {
                ch = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[g], high_part[g], ch, 0, 0, 0);
                cl = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[g], low_part[g], cl, 0, 0, 0);
            }
            // plane sums of digit * nibble * scale, below 2^25 each; the three planes meet in fp32
            const float t0 = (float)(8 * ch[0] + cl[0]), t1 = (float)(8 * ch[1] + cl[1]), t2 = (float)(8 * ch[2] + cl[2]);
            const float weighed = fmaf(fmaf(t0, 256.0f, t1), 256.0f, t2) * unscale;
            float floor_ = mn[0] * s0[0];
            floor_ = fmaf(mn[1], s0[1], floor_), floor_ = fmaf(mn[2], s0[2], floor_), floor_ = fmaf(mn[3], s0[3], floor_);
            floor_ = fmaf(mn[4], s1[0], floor_), floor_ = fmaf(mn[5], s1[1], floor_), floor_ = fmaf(mn[6], s1[2], floor_), floor_ = fmaf(mn[7], s1[3], floor_);
            acc[pass] = fmaf(scale_d, weighed, fmaf(scale_m, floor_, acc[pass]));
        }
    };
    // lane (r, s) holds output r of activation rows s (pass 0) and 4 + s (pass 1): the waves' parts meet in LDS, and the wave
    // whose turn it is sums them and runs the epilogue
    auto tile_end = [&](uint32_t tile, uint32_t index) {
        const uint32_t finisher = (MODE == TILE16_SWIGLU ? index >> 1 : index) % NW;
#pragma unroll
        for (int pass = 0; pass < P; pass++) {
            part[((parity * NW + wave) * P + pass) * 64u + lane] = acc[pass];
            acc[pass] = 0.0f;
        }
        __syncthreads();
        if (wave == finisher) {
#pragma unroll
            for (int pass = 0; pass < P; pass++) {
                const uint32_t row = 4u * pass + s;
                float total = 0.0f;
#pragma unroll
                for (int w = 0; w < NW; w++) total += part[((parity * NW + w) * P + pass) * 64u + lane];
                if (row >= rows) continue;
                if (MODE == TILE16_SWIGLU) {
                    if (tile & 1u) p.y[(size_t)row * (p.N / 2u) + (tile >> 1) * 16u + r] = silu(gate[pass]) * total;
                    else gate[pass] = total;
                } else if (r < tile_rows) {
                    const size_t n = (size_t)row * p.N + tile * tile_rows + r;
                    if (p.residual == p.y) unsafeAtomicAdd(p.y + n, total);
                    else p.y[n] = p.residual ? p.residual[n] + total : total;
                }
            }
        }
        parity ^= 1u;
    };
    if (count == 0) {
        for (uint32_t t = 0; t < walked; t++) tile_end(tile_at(t), t);
        return;
    }
    uint32_t at_tile = 0, at_b = wave;
    const uint32_t steps = walked * count;
    for (uint32_t s0 = 0; s0 < steps; s0 += D) {
#pragma unroll
        for (int slot = 0; slot < D; slot++) {
            step(ring[slot], at_b);
            at_b += NW;
            if (at_b >= nblk) {
                if (at_tile < walked) tile_end(tile_at(at_tile), at_tile);
                at_b = wave;
                at_tile++;
            }
        }
    }
}

// ---- the 16-row tile kernel (one activation row, Q4_K)
// NEURA_HIP_TILE16=0 keeps it out (the vector and the other matrix-core forms then take one row as before), as does a forced
// NEURA_HIP_MFMA form.  Otherwise it takes every Q4_K product of one row whose matrices end on tile boundaries, and of two
// to four rows (NEURA_HIP_TILE16_ROWS lowers that) where all their digit planes fit the workgroup's LDS.  From five rows on
// the MFMAs and the weighing, both paid once a row, cost more than the weights' bytes: the 32-row tiles take those.
constexpr uint32_t TILE16_MOST_ROWS = 4;
static uint32_t tile16_row_form(uint32_t rows) { return rows <= 1u ? 1u : (rows <= 2u ? 2u : 4u); }

bool tile16_takes(const GemvArgs &a) {
    if ((a.element != NH_Q4_K && a.element != NH_Q5_K) || a.rows < 1 || a.rows > TILE16_MOST_ROWS || a.K % 256u != 0 || a.K == 0) return false;
    if (env_int("NEURA_HIP_TILE16", 1) == 0 || env_int("NEURA_HIP_MFMA", 1) != 1) return false;
    // Q5_K (one row): the same tiles with the fifth bit beside the nibble; NEURA_HIP_Q5K_TILE16=0 leaves it to the staged kernel
    if (a.element == NH_Q5_K && (a.rows != 1 || a.merge || env_int("NEURA_HIP_Q5K_TILE16", 1) == 0)) return false;
    // a value projection that casts its rows into the value state: one row, whole heads, no other epilogue
    if (a.append_value && (a.rows != 1 || a.swiglu || a.rope || a.residual || a.digits_in || a.digits_out || a.W[1] || a.W[2] || !a.append_value->width ||
                           a.N % a.append_value->width))
        return false;
    for (int m = 0; m < 3; m++)
        if (a.W[m] && ((uintptr_t)a.W[m] & 15u)) return false;
    if (a.rows > 1 && (a.rope || a.rows > (uint32_t)env_int("NEURA_HIP_TILE16_ROWS", (int)TILE16_MOST_ROWS))) return false;
    if (a.rows > 1 && (env_int("NEURA_HIP_MFMA32", 1) == 2 || env_int("NEURA_HIP_F16_TILES", 1) == 2)) return false;  // another form is forced
    if (((uintptr_t)a.x & 15u) || (a.norm_w && ((uintptr_t)a.norm_w & 15u))) return false;
    if (a.N < 16u || a.N % 16u != 0) return false;
    if (a.swiglu) {
        if (a.residual || a.rope || a.end[0] != a.N / 2 || (a.N / 2) % 16u != 0) return false;
    } else if (a.rope) {
        const uint32_t width = a.rope->width;
        if (a.residual || width < 16u || width % 16u != 0) return false;
        if (a.rope->q_rows % width || a.rope->k_rows % width || a.N % width || a.rope->q_rows > a.rope->k_rows || a.rope->k_rows > a.N) return false;
        if (a.end[0] % width || a.end[1] % width || a.end[2] != a.N) return false;
    } else if (a.end[0] % 16u != 0 || a.end[1] % 16u != 0) {
        return false;
    }
    for (int m = 1; m < 3; m++) {  // the matrices stacked behind the first are named by their distance from it in 16-byte units
        if (!a.W[m]) continue;
        const int64_t apart = static_cast<const uint8_t *>(a.W[m]) - static_cast<const uint8_t *>(a.W[0]);
        if (apart % 16 != 0 || apart / 16 > INT32_MAX || apart / 16 < INT32_MIN) return false;
    }
    if (a.digits_out && (!a.swiglu || a.rows != 1 || a.N % 512u != 0 || ((uintptr_t)a.digits_out & 63u))) return false;
    if (a.digits_in && (a.swiglu || a.rope || a.norm_w || a.rows != 1 || ((uintptr_t)a.digits_in & 15u))) return false;
    const uint32_t nblk = a.K / 256u;
    return tile16_lds(nblk, nblk > 32u ? 16u : 8u, tile16_row_form(a.rows), a.digits_in != nullptr) <= 160u * 1024u;
}

// A SwiGLU product of one row ends with a chunk's sixteen outputs in sixteen lanes of one wave: it can leave them as the digit
// planes the product behind it would otherwise make of them again (NEURA_HIP_TILE16_HANDED=0 keeps the floats).
size_t gemv_digit_bytes(uint32_t K) { return (size_t)(K / 256u) * TILE16_BLOCK_HANDED; }

bool gemv_hands_digits(const GemvArgs &producer, const GemvArgs &consumer) {
    if (env_int("NEURA_HIP_TILE16_HANDED", 1) == 0) return false;
    if (!producer.swiglu || producer.rows != 1 || consumer.rows != 1 || consumer.K != producer.N / 2u || consumer.K % 256u != 0) return false;
    if (consumer.swiglu || consumer.rope || consumer.norm_w) return false;
    GemvArgs from = producer, to = consumer;
    from.digits_out = nullptr, to.digits_in = nullptr;
    if (!tile16_takes(from) && !q6k_tile16_takes(from)) return false;  // (both leave the same pieces)
    if (consumer.element == NH_Q6_K || consumer.element == NH_Q3_K) {
        // the Q6_K and Q3_K tiles read the same pieces in the same chunk order
        alignas(16) static const uint8_t somewhere[16] = {};
        to.digits_in = somewhere;
        return q6k_tile16_takes(to);
    }
    if (!tile16_takes(to)) return false;
    const uint32_t nblk = to.K / 256u;
    return tile16_lds(nblk, nblk > 32u ? 16u : 8u, 1u, true) <= 160u * 1024u;
}

// ---- three and four rows, four to an MFMA.  NEURA_HIP_ROWS4=0 keeps the kernel out, as does any other form forced by its switch.
bool rows4_takes(const GemvArgs &a) {
    if (a.element != NH_Q4_K || a.rows < 3 || a.rows > 4 || a.K % 256u != 0 || a.K == 0 || a.rope || a.digits_in || a.digits_out) return false;
    if (env_int("NEURA_HIP_ROWS4", 1) == 0 || env_int("NEURA_HIP_TILE16", 1) == 0 || env_int("NEURA_HIP_MFMA", 1) != 1) return false;
    if (env_int("NEURA_HIP_MFMA32", 1) == 2 || env_int("NEURA_HIP_F16_TILES", 1) == 2 || env_int("NEURA_HIP_TILE16_ROWS", 8) < (int)a.rows) return false;
    if (((uintptr_t)a.x & 15u) || (a.norm_w && ((uintptr_t)a.norm_w & 15u))) return false;
    if (a.N < 16u || a.N % 16u != 0) return false;
    if (a.swiglu) {
        if (a.residual || a.end[0] != a.N / 2 || (a.N / 2) % 16u != 0) return false;
    } else if (a.end[0] % 16u != 0 || a.end[1] % 16u != 0) {
        return false;
    }
    return rows4_lds(a.K / 256u, 8u, 4u) <= 160u * 1024u;
}

template <int NW, int MODE, int P>
static hipError_t launch_rows4_instance(nh_device *d, const GemvParams &p, uint32_t grid, size_t lds) {
    static bool raised = false;
    if (!raised && lds > 64u * 1024u) {
        hipError_t error = hipFuncSetAttribute((const void *)gemv_q4k_rows4_kernel<NW, 2, MODE, P>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (error != hipSuccess) return error;
        raised = true;
    }
    hipLaunchKernelGGL((gemv_q4k_rows4_kernel<NW, 2, MODE, P>), dim3(grid), dim3(NW * 64), lds, d->stream, GEMV_LEAD(p));
    return hipGetLastError();
}

template <int MODE, int P>
static hipError_t launch_rows4_waves(nh_device *d, const GemvParams &p, uint32_t waves, uint32_t grid, size_t lds) {
    switch (waves) {
    case 4: return launch_rows4_instance<4, MODE, P>(d, p, grid, lds);
    case 7: return launch_rows4_instance<7, MODE, P>(d, p, grid, lds);
    default: return launch_rows4_instance<8, MODE, P>(d, p, grid, lds);
    }
}

int32_t launch_rows4(nh_device *d, const GemvArgs &a) {
    GemvParams p{};
    for (int s = 0; s < 3; s++) {
        p.W[s] = static_cast<const uint8_t *>(a.W[s] ? a.W[s] : a.W[0]);
        p.end[s] = a.end[s];
    }
    p.x = a.x, p.y = a.y, p.residual = a.residual, p.norm_w = a.norm_w;
    p.N = a.N, p.K = a.K, p.swiglu = a.swiglu, p.eps = a.eps, p.rows = a.rows;
    p.row_bytes = (uint32_t)payload_bytes(a.element, a.K);
    p.nblk = a.K / 256u;
    const uint32_t waves = p.nblk <= 8u ? 4u : (p.nblk <= 14u ? 7u : 8u);
    // tiles and rounds as the one-row kernel deals them: a plain tile holds the number of rows, 16 down to 12, that leaves the
    // fewest compute units idle in the last round
    p.tile_rows = 16;
    if (!a.swiglu) {
        auto idle = [&](uint32_t rows) {
            const uint32_t tiles = a.N / rows, rounds = (tiles + (uint32_t)d->compute_units - 1u) / (uint32_t)d->compute_units;
            return 65536u - (uint32_t)((uint64_t)tiles * 65536u / ((uint64_t)rounds * (uint32_t)d->compute_units));
        };
        for (uint32_t rows = 15; rows >= 12; rows--) {
            if (a.N % rows || a.end[0] % rows || a.end[1] % rows) continue;
            if (idle(rows) + 3277u < idle(p.tile_rows)) p.tile_rows = rows;
        }
    }
    const uint32_t units = a.swiglu ? a.N / 32u : a.N / p.tile_rows;
    p.row_groups = units;
    const uint32_t rounds = (units + (uint32_t)d->compute_units - 1u) / (uint32_t)d->compute_units;
    const uint32_t grid = (units + rounds - 1u) / rounds;
    const size_t lds = rows4_lds(p.nblk, waves, 4u);
    profile_mark(d);
    hipError_t launched = a.swiglu ? launch_rows4_waves<TILE16_SWIGLU, 1>(d, p, waves, grid, lds) : launch_rows4_waves<TILE16_PLAIN, 1>(d, p, waves, grid, lds);
    NH_HIP(launched);
    profile_mark(d);
    if (d->profile) d->profile_bytes += (uint64_t)a.N * p.row_bytes;
    return NH_OK;
}

template <int NW, int D, int MODE, int R, bool HANDED = false, bool FIFTH = false>
static hipError_t launch_tile16_instance(nh_device *d, const GemvParams &p, uint32_t grid, size_t lds) {
    static bool raised = false;  // a workgroup may hold more than the default 64 KiB of LDS once the kernel says so
    if (!raised && lds > 64u * 1024u) {
        hipError_t error = hipFuncSetAttribute((const void *)gemv_q4k_tile16_kernel<NW, D, MODE, R, HANDED, FIFTH>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (error != hipSuccess) return error;
        raised = true;
    }
    hipLaunchKernelGGL((gemv_q4k_tile16_kernel<NW, D, MODE, R, HANDED, FIFTH>), dim3(grid), dim3(NW * 64), lds, d->stream, p.W[0],
                       HANDED ? static_cast<const void *>(p.digits_in) : static_cast<const void *>(p.x), p.norm_w, (int32_t)((p.W[1] - p.W[0]) / 16),
                       (int32_t)((p.W[2] - p.W[0]) / 16), p.row_bytes, grid, p.row_groups, MODE == TILE16_ROPE ? p.rope_width : p.tile_rows, p.end[0], p.end[1], p);
    return hipGetLastError();
}

// a plain product of one row whose activations arrive as digit planes
static hipError_t launch_tile16_handed(nh_device *d, const GemvParams &p, uint32_t waves, uint32_t grid, size_t lds) {
    switch (waves) {
    case 4: return launch_tile16_instance<4, 2, TILE16_PLAIN, 1, true>(d, p, grid, lds);
    case 7: return launch_tile16_instance<7, 2, TILE16_PLAIN, 1, true>(d, p, grid, lds);
    default: return launch_tile16_instance<8, 2, TILE16_PLAIN, 1, true>(d, p, grid, lds);
    }
}

template <int MODE, int R>
static hipError_t launch_tile16_rows(nh_device *d, const GemvParams &p, uint32_t waves, uint32_t grid, size_t lds) {
    switch (waves) {
    case 4: return launch_tile16_instance<4, 2, MODE, R>(d, p, grid, lds);
    case 6: return launch_tile16_instance<6, 2, MODE, R>(d, p, grid, lds);
    case 7: return launch_tile16_instance<7, 2, MODE, R>(d, p, grid, lds);
    case 8: return launch_tile16_instance<8, 2, MODE, R>(d, p, grid, lds);
    default: return launch_tile16_instance<16, 2, MODE, R>(d, p, grid, lds);
    }
}

template <int MODE>
static hipError_t launch_tile16_mode(nh_device *d, const GemvParams &p, uint32_t waves, uint32_t grid, size_t lds) {
    if constexpr (MODE != TILE16_ROPE) {
        switch (tile16_row_form(p.rows)) {
        case 1: break;
        case 2: return launch_tile16_rows<MODE, 2>(d, p, waves, grid, lds);
        default: return launch_tile16_rows<MODE, 4>(d, p, waves, grid, lds);
        }
    }
    return launch_tile16_rows<MODE, 1>(d, p, waves, grid, lds);
}

// Q5_K: one row, every mode
template <int MODE, bool HANDED>
static hipError_t launch_tile16_fifth(nh_device *d, const GemvParams &p, uint32_t waves, uint32_t grid, size_t lds) {
    switch (waves) {
    case 4: return launch_tile16_instance<4, 2, MODE, 1, HANDED, true>(d, p, grid, lds);
    case 6: return launch_tile16_instance<6, 2, MODE, 1, HANDED, true>(d, p, grid, lds);
    case 7: return launch_tile16_instance<7, 2, MODE, 1, HANDED, true>(d, p, grid, lds);
    case 8: return launch_tile16_instance<8, 2, MODE, 1, HANDED, true>(d, p, grid, lds);
    default: return launch_tile16_instance<16, 2, MODE, 1, HANDED, true>(d, p, grid, lds);
    }
}

// what a launch of the 16-row tile product is made of: the parameter block, waves a workgroup, workgroups, LDS
struct Tile16Launch {
    GemvParams p;
    uint32_t waves, grid;
    size_t lds;
};

static Tile16Launch tile16_plan(nh_device *d, const GemvArgs &a, uint32_t fixed_waves = 0) {
    Tile16Launch plan{};
    GemvParams &p = plan.p;
    for (int s = 0; s < 3; s++) {
        p.W[s] = static_cast<const uint8_t *>(a.W[s] ? a.W[s] : a.W[0]);
        p.end[s] = a.end[s];
    }
    p.x = a.x, p.y = a.y, p.residual = a.residual, p.norm_w = a.norm_w;
    p.N = a.N, p.K = a.K, p.swiglu = a.swiglu, p.eps = a.eps, p.rows = a.rows;
    p.digits_out = a.digits_out, p.digits_in = a.digits_in;
    p.tick = d->tick, p.tag_in = a.tag_in, p.tag_out = a.tag_out, p.pairs_out = static_cast<uint2 *>(a.pairs_out);
    p.late_from = 0xffffffffu;
    p.refusal = d->refusal;

    p.row_bytes = (uint32_t)payload_bytes(a.element, a.K);
    p.nblk = a.K / 256u;
    p.rope_width = 16;  // the kernel derives a tile's rows from it only where the rotation is folded in
    if (a.rope) {
        p.rope_cosines = a.rope->cosines, p.rope_sines = a.rope->sines, p.rope_cursor = a.rope->cursor, p.rope_k = a.rope->cache_k, p.rope_v = a.rope->cache_v;
        p.rope_width = a.rope->width, p.rope_q_rows = a.rope->q_rows, p.rope_k_rows = a.rope->k_rows, p.rope_capacity = a.rope->capacity;
        p.rope_positions = a.rope->positions, p.rope_ring = a.rope->ring, p.rope_element = a.rope->element;
        p.refusal = d->refusal;
        for (int s = 0; s < 3; s++) p.bias[s] = a.bias[s];
    }
    if (a.append_value) {  // (a plain product: the width here is the value heads', not a tile's)
        p.append_value = 1u, p.rope_v = a.append_value->cache_v, p.rope_cursor = a.append_value->cursor, p.rope_width = a.append_value->width;
        p.rope_capacity = a.append_value->capacity, p.rope_ring = a.append_value->ring, p.rope_element = a.append_value->element, p.bias[0] = a.bias[0];
    }
    // waves of a workgroup share a tile and split its super-blocks: about two steps a wave
    // (sixteen on deep rows, where turning the activations into digits is the larger part of a wave's work; eight where the
    // digits arrive ready: fewer loads in flight a compute unit stream faster, as the shallow products show)
    plan.waves = fixed_waves ? fixed_waves : (p.nblk <= 8u ? 4u : (p.nblk <= 14u ? 7u : (p.nblk <= 32u || a.digits_in ? 8u : 16u)));
    // one row against short rows (the 1.5B shape's 1536 columns are six super-blocks): a wave a super-block keeps more bytes in
    // flight a compute unit than four waves of two steps -- measured on that shape, a decode step 0.963 -> 0.898 ms
    // (two to four rows take the same waves: a row of theirs is then, bit for bit, what the one-row product gives)
    if (!fixed_waves && !a.digits_in && p.nblk > 4u && p.nblk <= 8u) plan.waves = p.nblk <= 6u ? 6u : 8u;
    // units of work: tiles, or with SwiGLU pairs (a gate tile and the up tile behind it); every workgroup takes the same
    // number of them, one workgroup a compute unit when there are that many
    // A plain tile holds the number of rows, 16 down to 12, that leaves the fewest compute units idle in the last round.
    p.tile_rows = 16;
    if (!a.swiglu && !a.rope) {
        auto idle = [&](uint32_t rows) {  // share of the rounds' slots left empty, in 1/65536
            const uint32_t tiles = a.N / rows, rounds = (tiles + (uint32_t)d->compute_units - 1u) / (uint32_t)d->compute_units;
            return 65536u - (uint32_t)((uint64_t)tiles * 65536u / ((uint64_t)rounds * (uint32_t)d->compute_units));
        };
        for (uint32_t rows = 15; rows >= 12; rows--) {
            if (a.N % rows || a.end[0] % rows || a.end[1] % rows) continue;
            // fewer rows a tile stage the activations more often: taken only where they fill at least a twentieth more of the device
            if (idle(rows) + 3277u < idle(p.tile_rows)) p.tile_rows = rows;
        }
    }
    const uint32_t units = a.swiglu ? a.N / 32u : a.N / p.tile_rows;
    p.row_groups = units;
    const uint32_t rounds = (units + (uint32_t)d->compute_units - 1u) / (uint32_t)d->compute_units;
    plan.grid = (units + rounds - 1u) / rounds;
    plan.lds = tile16_lds(p.nblk, plan.waves, tile16_row_form(a.rows), a.digits_in != nullptr);
    return plan;
}

int32_t launch_tile16(nh_device *d, const GemvArgs &a) {
    const Tile16Launch plan = tile16_plan(d, a);
    const GemvParams &p = plan.p;
    const uint32_t waves = plan.waves, grid = plan.grid;
    const size_t lds = plan.lds;
    profile_mark(d);
    hipError_t launched;
    if (a.append_value)
        launched = a.element == NH_Q5_K ? launch_tile16_fifth<TILE16_APPEND, false>(d, p, waves, grid, lds) : launch_tile16_rows<TILE16_APPEND, 1>(d, p, waves, grid, lds);
    else if (a.element == NH_Q5_K)
        launched = a.digits_in ? launch_tile16_fifth<TILE16_PLAIN, true>(d, p, waves, grid, lds)
                   : a.swiglu  ? launch_tile16_fifth<TILE16_SWIGLU, false>(d, p, waves, grid, lds)
                   : a.rope    ? launch_tile16_fifth<TILE16_ROPE, false>(d, p, waves, grid, lds)
                               : launch_tile16_fifth<TILE16_PLAIN, false>(d, p, waves, grid, lds);
    else
        launched = a.digits_in ? launch_tile16_handed(d, p, waves, grid, lds)
                   : a.swiglu  ? launch_tile16_mode<TILE16_SWIGLU>(d, p, waves, grid, lds)
                   : a.rope    ? launch_tile16_mode<TILE16_ROPE>(d, p, waves, grid, lds)
                               : launch_tile16_mode<TILE16_PLAIN>(d, p, waves, grid, lds);
    NH_HIP(launched);
    profile_mark(d);
    if (d->profile) d->profile_bytes += (uint64_t)a.N * p.row_bytes;
    return NH_OK;
}

// ---------------------------------------------------------------------------------------------------------------------
// Two independent one-row products over the same activation row in one launch: a Q4_K (FIFTH: Q5_K) q|k product with the rotation
// folded in and the Q6_K value projection that casts its rows into the value state -- what a layer of a Q4_K_M or Q5_K_M file asks
// for where the value projection is stored in Q6_K.  The first `lead_grid` workgroups run the Q4_K product, the others the Q6_K one; neither
// waits for the other.  As two launches the pair takes 6.1 + 6.5 us, and nearly all of either is the launch and the first
// round trips.
struct Q6kBeside {
    const uint8_t *w0;
    const float *norm_w;
    uint32_t row_bytes, grid, tiles, tile_rows;
    GemvParams p;
};
template <int NW, bool FIFTH = false>
__global__ __launch_bounds__(NW * 64) void gemv_q4k_rope_beside_q6k_kernel(const uint8_t *lead_w0, const void *lead_input, const float *lead_norm_w, int32_t lead_to_w1,
                                                                           int32_t lead_to_w2, uint32_t lead_row_bytes, uint32_t lead_grid, uint32_t lead_tiles,
                                                                           uint32_t lead_tile_rows, uint32_t lead_end0, uint32_t lead_end1, GemvParams p, Q6kBeside beside) {
    extern __shared__ __attribute__((aligned(16))) uint8_t pair_lds_bytes[];
    if (blockIdx.x < lead_grid) {
        typename Tile16UnitOf<FIFTH>::type ring[2];
        tile16_product<NW, 2, TILE16_ROPE, 1, false, NoSeam, FIFTH>(pair_lds_bytes, blockIdx.x, NoSeam{}, ring, nullptr, 0u, lead_w0, lead_input, lead_norm_w, lead_to_w1, lead_to_w2, lead_row_bytes,
                                                     lead_grid, lead_tiles, lead_tile_rows, lead_end0, lead_end1, p);
    } else {
        q6k_tile16_product<NW, false, false>(pair_lds_bytes, blockIdx.x - lead_grid, beside.w0, lead_input, beside.norm_w, beside.row_bytes, beside.grid, beside.tiles,
                                             beside.tile_rows, 0, 0, 0u, 0u, beside.p);
    }
}

template <int NW, bool FIFTH>
static hipError_t launch_pair_instance(nh_device *d, const Tile16Launch &first, const Q6kLaunch &second) {
    const size_t lds = first.lds > second.lds ? first.lds : second.lds;
    static bool raised = false;
    if (!raised && lds > 64u * 1024u) {
        hipError_t error = hipFuncSetAttribute((const void *)gemv_q4k_rope_beside_q6k_kernel<NW, FIFTH>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (error != hipSuccess) return error;
        raised = true;
    }
    const GemvParams &p = first.p;
    Q6kBeside beside{second.p.W[0], second.p.norm_w, second.p.row_bytes, second.grid, second.p.row_groups, second.p.tile_rows, second.p};
    hipLaunchKernelGGL((gemv_q4k_rope_beside_q6k_kernel<NW, FIFTH>), dim3(first.grid + second.grid), dim3(NW * 64), lds, d->stream, p.W[0], static_cast<const void *>(p.x), p.norm_w,
                       (int32_t)((p.W[1] - p.W[0]) / 16), (int32_t)((p.W[2] - p.W[0]) / 16), p.row_bytes, first.grid, p.row_groups, p.rope_width, p.end[0], p.end[1], p, beside);
    return hipGetLastError();
}

// NEURA_HIP_PAIR=0 keeps the two launches
bool gemv_pairs(nh_device *d, const GemvArgs &rotated, const GemvArgs &value) {
    if (env_int("NEURA_HIP_PAIR", 1) == 0) return false;
    if ((rotated.element != NH_Q4_K && rotated.element != NH_Q5_K) || !rotated.rope || rotated.rows != 1 || !tile16_takes(rotated)) return false;
    if (value.element != NH_Q6_K || !value.append_value || value.rows != 1 || value.digits_in || !q6k_tile16_takes(value)) return false;
    if (rotated.x != value.x || rotated.norm_w != value.norm_w || rotated.K != value.K || rotated.eps != value.eps) return false;
    const uint32_t waves = tile16_plan(d, rotated).waves;
    return waves == q6k_tile16_plan(d, value).waves && (waves == 4u || waves == 7u || waves == 8u);
}

int32_t launch_gemv_pair(nh_device *d, const GemvArgs &rotated, const GemvArgs &value) {
    if (!gemv_pairs(d, rotated, value)) return fail(NH_E_ARGUMENT, "these two products do not share a launch (ask gemv_pairs first)");
    const Tile16Launch first = tile16_plan(d, rotated);
    const Q6kLaunch second = q6k_tile16_plan(d, value);
    profile_mark(d);
    hipError_t launched;
    if (rotated.element == NH_Q5_K)
        launched = first.waves == 4u ? launch_pair_instance<4, true>(d, first, second) : first.waves == 7u ? launch_pair_instance<7, true>(d, first, second) : launch_pair_instance<8, true>(d, first, second);
    else
        launched = first.waves == 4u ? launch_pair_instance<4, false>(d, first, second) : first.waves == 7u ? launch_pair_instance<7, false>(d, first, second) : launch_pair_instance<8, false>(d, first, second);
    NH_HIP(launched);
    profile_mark(d);
    if (d->profile) d->profile_bytes += (uint64_t)rotated.N * first.p.row_bytes + (uint64_t)value.N * second.p.row_bytes;
    return NH_OK;
}

// ---------------------------------------------------------------------------------------------------------------------
// Several dependent one-row products in one launch (crates/neura-kernel/src/scheduler.rs:110-166 runs a whole program as one
// persistent kernel; here it is the products between two attentions of a decode step: attn_output, gate|up, ffn_down and the
// q|k|v product of the layer behind, or the head).  One workgroup of eight waves a compute unit, all resident at once; every
// stage is the 16-row tile product above, with the seams its comment describes: a workgroup walks from one product into the
// next with nothing between them but a barrier of its own waves (they share LDS), asks for the next product's first
// weights, and reads its activations as tagged pieces until they are this step's.
struct ChainStage {
    const uint8_t *w0;
    const void *input;
    const float *norm_w;
    int32_t to_w1, to_w2;
    uint32_t row_bytes, grid, tiles, tile_rows, end0, end1;
    GemvParams p;
};
constexpr int CHAIN_STAGES_MOST = 4;
struct ChainParams {
    ChainStage stage[CHAIN_STAGES_MOST];
    uint32_t spin;  // times a reader may read a stale piece again
    uint32_t stages;  // bit s: stage s runs (all of them, unless a test splits a chain over several launches)
    uint32_t second_lds;  // where ffn_down's part of LDS begins, behind the other products'
};

template <bool WAITS_, bool IN_, bool OUT_, bool HANDS_ = false, bool TAKES_ = false>
struct ChainSeam {
    static constexpr bool WAITS = WAITS_, SHARED_IN = IN_, SHARED_OUT = OUT_, HANDS_RING = HANDS_, TAKES_RING = TAKES_;
    uint32_t spin;
};

enum ChainProgram { CHAIN_FFN = 0, CHAIN_O_FFN = 1, CHAIN_O_FFN_QKV = 2, CHAIN_O_FFN_HEAD = 3 };

#define CHAIN_STAGE_ARGUMENTS(s) (s).w0, (s).input, (s).norm_w, (s).to_w1, (s).to_w2, (s).row_bytes, (s).grid, (s).tiles, (s).tile_rows, (s).end0, (s).end1, (s).p

// this lane's weight row in the first tile workgroup `block` walks of a plain one-matrix stage (nullptr: it walks none)
__device__ __forceinline__ const uint8_t *chain_first_row(const ChainStage &stage, uint32_t block) {
    if (block >= stage.tiles || block >= stage.grid) return nullptr;
    const uint32_t lane = threadIdx.x & 63u, r = lane & 15u, q = lane >> 4;
    const uint32_t n = block * stage.tile_rows + min(r, stage.tile_rows - 1u);
    return stage.w0 + (size_t)n * stage.row_bytes + q * 32u;
}

template <int PROGRAM>
__global__ __launch_bounds__(512) void gemv_q4k_chain_kernel(ChainParams c) {
    extern __shared__ __attribute__((aligned(16))) uint8_t chain_lds_bytes[];
    constexpr bool LEADS = PROGRAM != CHAIN_FFN;                                        // attn_output in front
    constexpr bool TRAILS = PROGRAM == CHAIN_O_FFN_QKV || PROGRAM == CHAIN_O_FFN_HEAD;  // a product behind ffn_down
    const uint32_t block = blockIdx.x;
    Tile16Unit ring[2];
    int at = 0;
    if constexpr (LEADS) {
        // attn_output: x is the attention's output (the launch before); y = h + ..., which gate|up reads as tagged pairs
        if (c.stages & 1u)
            tile16_product<8, 2, TILE16_PLAIN, 1, false>(chain_lds_bytes, block, ChainSeam<false, false, true>{c.spin}, ring, nullptr, 0u,
                                                         CHAIN_STAGE_ARGUMENTS(c.stage[at]));
        __syncthreads();  // these two products stage their activations in the same part of LDS
        at++;
    }
    // gate|up with SwiGLU: leaves tagged digit planes; past its last unit its ring asks for ffn_down's first weights
    const ChainStage &down = c.stage[at + 1];
    if (c.stages & (1u << at))
        tile16_product<8, 2, TILE16_SWIGLU, 1, false>(chain_lds_bytes, block, ChainSeam<LEADS, LEADS, true, true, false>{c.spin}, ring,
                                                      chain_first_row(down, block), down.row_bytes / 144u, CHAIN_STAGE_ARGUMENTS(c.stage[at]));
    at++;
    // ffn_down over the digit planes, h += ...: in a part of LDS of its own (no wave waits for another between the two
    // products), its first weights in flight, the planes of its last super-blocks looked at when the walk reaches them
    if (c.stages & (1u << at)) {
        if (c.stages & (1u << (at - 1)))
            tile16_product<8, 2, TILE16_PLAIN, 1, true>(chain_lds_bytes + c.second_lds, block, ChainSeam<false, true, TRAILS, false, true>{c.spin}, ring, nullptr, 0u,
                                                        CHAIN_STAGE_ARGUMENTS(c.stage[at]));
        else  // (a launch of this stage alone: nothing handed it a ring)
            tile16_product<8, 2, TILE16_PLAIN, 1, true>(chain_lds_bytes + c.second_lds, block, ChainSeam<false, true, TRAILS, false, false>{c.spin}, ring, nullptr, 0u,
                                                        CHAIN_STAGE_ARGUMENTS(c.stage[at]));
    }
    at++;
    if constexpr (TRAILS) {
        // (every wave that gets here has passed ffn_down's barrier, which none reaches before it is done with gate|up's LDS)
        if constexpr (PROGRAM == CHAIN_O_FFN_QKV)
            tile16_product<8, 2, TILE16_ROPE, 1, false>(chain_lds_bytes, block, ChainSeam<true, true, false>{c.spin}, ring, nullptr, 0u, CHAIN_STAGE_ARGUMENTS(c.stage[at]));
        else
            tile16_product<8, 2, TILE16_PLAIN, 1, false>(chain_lds_bytes, block, ChainSeam<true, true, false>{c.spin}, ring, nullptr, 0u, CHAIN_STAGE_ARGUMENTS(c.stage[at]));
    }
}

static bool chain_stage_takes(const GemvArgs &a) {
    if (a.element != NH_Q4_K || !tile16_takes(a) || a.rows != 1) return false;
    return tile16_lds(a.K / 256u, 8u, 1u, a.digits_in != nullptr) <= 160u * 1024u;
}

// Whether launch_chain takes these products as one launch: attn_output (or none), gate|up handing its digits to ffn_down, and
// behind them the next q|k|v with the rotation folded in, or the head (or none).  NEURA_HIP_CHAIN: 0 (the default: measured, the
// chained launch takes as long as its products one by one and a little more) keeps one launch a product, 1 chains gate|up and
// ffn_down, 2 attn_output in front of them, 3 the product behind them as well.
int gemv_chain_level() { return env_int("NEURA_HIP_CHAIN", 0); }

bool gemv_chains(nh_device *d, const GemvArgs *lead, const GemvArgs &gate_up, const GemvArgs &down, const GemvArgs *trail) {
    const int wanted = gemv_chain_level();
    if (wanted <= 0 || !d->tick || d->compute_units < 1) return false;
    if (lead && wanted < 2) return false;
    if (trail && wanted < 3) return false;
    if (!gate_up.digits_out || !down.digits_in || gate_up.digits_out != down.digits_in || !gate_up.tag_out || gate_up.tag_out != down.tag_in) return false;
    if (!chain_stage_takes(gate_up) || !chain_stage_takes(down)) return false;
    // the ring handed across the seam holds the first two units of every wave of ffn_down's first tile
    if (down.K / 256u < 16u) return false;
    if (tile16_lds(gate_up.K / 256u, 8u, 1u, false) + 256u + tile16_lds(down.K / 256u, 8u, 1u, true) > 160u * 1024u) return false;
    if (lead && tile16_lds(lead->K / 256u, 8u, 1u, false) + 256u + tile16_lds(down.K / 256u, 8u, 1u, true) > 160u * 1024u) return false;
    if (trail && tile16_lds(trail->K / 256u, 8u, 1u, false) + 256u + tile16_lds(down.K / 256u, 8u, 1u, true) > 160u * 1024u) return false;
    // a row handed on as (value, tag) pairs is held in registers while its reader looks at the tags: five units of four a thread
    constexpr uint32_t HELD_MOST = 5u * 512u * 4u;
    if (lead) {
        if (!chain_stage_takes(*lead) || lead->swiglu || lead->rope || lead->digits_in || lead->digits_out) return false;
        if (!lead->pairs_out || lead->pairs_out != (const void *)gate_up.x || !lead->tag_out || lead->tag_out != gate_up.tag_in || gate_up.K > HELD_MOST) return false;
    }
    if (trail) {
        if (!chain_stage_takes(*trail) || trail->swiglu || trail->digits_in || trail->digits_out || trail->residual) return false;
        if (!down.pairs_out || down.pairs_out != (const void *)trail->x || !down.tag_out || down.tag_out != trail->tag_in || trail->K > HELD_MOST) return false;
    }
    return true;
}

template <int PROGRAM>
static hipError_t launch_chain_program(nh_device *d, const ChainParams &c, uint32_t grid, size_t lds) {
    static bool raised = false;
    if (!raised) {
        hipError_t error = hipFuncSetAttribute((const void *)gemv_q4k_chain_kernel<PROGRAM>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (error != hipSuccess) return error;
        raised = true;
    }
    hipLaunchKernelGGL((gemv_q4k_chain_kernel<PROGRAM>), dim3(grid), dim3(512), lds, d->stream, c);
    return hipGetLastError();
}

int32_t launch_chain(nh_device *d, const GemvArgs *lead, const GemvArgs &gate_up, const GemvArgs &down, const GemvArgs *trail, uint32_t spin) {
    ChainParams c{};
    const GemvArgs *stages[CHAIN_STAGES_MOST] = {nullptr, nullptr, nullptr, nullptr};
    int count = 0;
    if (lead) stages[count++] = lead;
    stages[count++] = &gate_up;
    stages[count++] = &down;
    if (trail) stages[count++] = trail;
    size_t lds = 0, lds_down = 0;
    uint64_t bytes = 0;
    uint32_t late_from = 0xffffffffu;
    for (int s = 0; s < count; s++) {
        Tile16Launch plan = tile16_plan(d, *stages[s], 8u);
        if (stages[s] == &gate_up) {
            // the first of ffn_down's super-blocks that holds an output of gate|up's last round of pairs
            const uint32_t pairs = plan.p.row_groups, last_round = (pairs - 1u) / plan.grid;
            late_from = last_round * plan.grid / 16u;
        }
        if (stages[s] == &down) plan.p.late_from = late_from;
        const GemvParams &p = plan.p;
        ChainStage &stage = c.stage[s];
        stage.w0 = p.W[0];
        stage.input = p.digits_in ? static_cast<const void *>(p.digits_in) : static_cast<const void *>(p.x);
        stage.norm_w = p.norm_w;
        stage.to_w1 = (int32_t)((p.W[1] - p.W[0]) / 16), stage.to_w2 = (int32_t)((p.W[2] - p.W[0]) / 16);
        stage.row_bytes = p.row_bytes, stage.grid = plan.grid, stage.tiles = p.row_groups;
        stage.tile_rows = stages[s]->rope ? p.rope_width : p.tile_rows;
        stage.end0 = p.end[0], stage.end1 = p.end[1];
        stage.p = p;
        if (stages[s] == &down) lds_down = plan.lds;
        else if (plan.lds > lds) lds = plan.lds;
        bytes += (uint64_t)stages[s]->N * p.row_bytes;
    }
    // ffn_down stages its planes behind the other products' part of LDS; one workgroup a compute unit: more LDS than two of
    // them could share
    c.second_lds = (uint32_t)((lds + 255u) / 256u * 256u);
    lds = c.second_lds + lds_down;
    if (lds < 84u * 1024u) lds = 84u * 1024u;
    c.spin = spin;
    const uint32_t grid = (uint32_t)d->compute_units;
    profile_mark(d);
    hipError_t launched = hipSuccess;
    // NEURA_HIP_CHAIN_SPLIT=1 (a test's switch): every stage a launch of its own of the same kernel, the seams' tags unchanged
    const bool split = env_int("NEURA_HIP_CHAIN_SPLIT", 0) == 1;
    for (int part = 0; part < (split ? count : 1) && launched == hipSuccess; part++) {
        c.stages = split ? 1u << part : 0xffu;
        if (!lead) launched = launch_chain_program<CHAIN_FFN>(d, c, grid, lds);
        else if (!trail) launched = launch_chain_program<CHAIN_O_FFN>(d, c, grid, lds);
        else if (trail->rope) launched = launch_chain_program<CHAIN_O_FFN_QKV>(d, c, grid, lds);
        else launched = launch_chain_program<CHAIN_O_FFN_HEAD>(d, c, grid, lds);
    }
    NH_HIP(launched);
    profile_mark(d);
    if (d->profile) d->profile_bytes += bytes;
    return NH_OK;
}

__global__ __launch_bounds__(64) void tick_kernel(uint32_t *tick) {
    if (threadIdx.x == 0) *tick = *tick + 1u;
}

int32_t launch_tick(nh_device *d) {
    if (!d->tick) return NH_OK;
    hipLaunchKernelGGL(tick_kernel, dim3(1), dim3(64), 0, d->stream, d->tick);
    NH_HIP(hipGetLastError());
    return NH_OK;
}

}  // namespace nh
