// Causal grouped-query attention over an fp16 K/V cache (flash-decoding form).
//
// One workgroup serves one (kv head, plane, query row, key section): the `groups` query
// heads that share the kv head ride along, so every K/V row is fetched once for all of them.
// A section is walked in tiles of 64 keys, three passes per tile:
//   scores  a key row of `WIDTH` halves is read by WIDTH/8 lanes with one 128-bit load each and
//           dotted with the query heads in registers (DPP sums across the lanes of a key); the
//           value rows of the tile go to LDS as they arrive;
//   weights one wave per query head, one lane per key: tile maximum, exp, running (top, mass);
//   values  every thread owns a few channels and a slice of the tile's keys and adds
//           weight * value from LDS, so no accumulator ever crosses lanes.
// Rescaling happens once per tile, not per key.  The slices meet in LDS at the end; sections
// are merged by a second kernel (crates/neura-kernel/src/task/attention.rs:619-671 does the
// same fold).  The next tile's K/V rows are in flight during the weight and value passes.
#include "blocks.hpp"
#include "common.hpp"

#include <cstdlib>

namespace nh {

constexpr int MAX_GROUPS = 8;

struct AttentionParams {
    const float *q;
    float *out;
    float *partial;      // [unit][section][group][width + 2] when sections > 1
    uint64_t q_sh, q_sb, q_sr, o_sh, o_sb, o_sr;
    const uint16_t *cache_k, *cache_v;  // as bytes of another element for attention_any_kernel
    uint32_t heads, kv_heads, groups, batch, rows, capacity, keys, sections;
    const uint32_t *cursor;
    float scale;
    uint32_t *refusal;
    uint32_t reach;  // 0, or the span of a ring of `keys` slots
};

__device__ __forceinline__ void fetch_parameters(const AttentionParams &p) {
    NH_FETCH(p.q, p.out, p.partial, p.q_sh, p.q_sb, p.q_sr, p.o_sh, p.o_sb, p.o_sr, p.cache_k, p.cache_v, p.heads, p.kv_heads, p.groups, p.batch, p.rows,
             p.capacity, p.keys, p.sections, p.cursor, p.scale, p.refusal, p.reach);
}

// A ring cache (Cache::windowed, crates/neura-decoder/src/cache.rs:311-317, :391-394): once `written` positions have gone
// in, slot `at` holds the latest position below `written` that lands on it (key_position,
// crates/neura-kernel/src/task/attention.rs:103-108), and a query weighs the `reach` positions up to its own
// (weighed, :136-144).  The one division is done once: the slots up to `last` hold base + at, the others base - keys + at.
struct Ring {
    uint32_t base, last, keys, reach;
    __device__ Ring(uint32_t keys, uint32_t written, uint32_t reach) : keys(keys), reach(reach) {
        if (written <= keys) {
            base = 0u, last = keys - 1u;
        } else {
            last = (written - 1u) % keys;
            base = written - 1u - last;
        }
    }
    __device__ __forceinline__ bool seen(uint32_t at, uint32_t position) const {
        const uint32_t held = at <= last ? base + at : base - keys + at;
        return held <= position && position - held < reach;
    }
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void unpack8(const u32x4 &raw, float (&out)[8]) {
    const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
        out[2 * j] = half_to_float((uint16_t)(words[j] & 0xffffu));
        out[2 * j + 1] = half_to_float((uint16_t)(words[j] >> 16));
    }
}

// sum over the LPK lanes that share a key: DPP adds inside a row of 16 lanes
template <int LPK>
__device__ __forceinline__ float key_sum(float v) {
    static_assert(LPK == 4 || LPK == 8 || LPK == 16 || LPK == 32, "lanes per key");
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, false));  // lane ^ 1
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, false));  // lane ^ 2
    if (LPK >= 8) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false));  // half mirror: the other quad of 8
    if (LPK >= 16) v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, false));  // mirror: the other half of 16
    if (LPK >= 32) v += __shfl_xor(v, 16, 64);
    return v;
}

// the K and V rows (8 halves per lane) of the T steps of one tile; `first` is this lane's key in step 0
template <int T, int STEP, int WIDTH>
__device__ __forceinline__ void fetch_tile(u32x4 (&kraw)[T], u32x4 (&vraw)[T], const uint16_t *__restrict__ cache_k,
                                           const uint16_t *__restrict__ cache_v, uint64_t plane, uint32_t first, uint32_t capacity, uint32_t dl) {
#pragma unroll
    for (int s = 0; s < T; s++) {
        const uint32_t at_key = min(first + s * STEP, capacity - 1u);
        const uint64_t at = (plane + at_key) * WIDTH + dl * 8u;
        kraw[s] = *reinterpret_cast<const u32x4 *>(cache_k + at);
        vraw[s] = *reinterpret_cast<const u32x4 *>(cache_v + at);
    }
}

template <int WIDTH>
__global__ __launch_bounds__(256) void attention_kernel(AttentionParams p) {
    constexpr int LPK = WIDTH / 8;                       // lanes per key in the score pass
    constexpr int KPW = 64 / LPK, STEP = 4 * KPW;        // keys per wave and per workgroup step
    constexpr int TK = 64, T = TK / STEP;                // keys and steps per tile
    constexpr int DPT = WIDTH >= 64 ? WIDTH / 64 : 1;    // channels per thread in the value pass
    constexpr int TPS = WIDTH / DPT;                     // threads per key slice in the value pass
    constexpr int SLICES = 256 / TPS, KPS = TK / SLICES; // key slices of a tile and keys per slice
    // the tile's value rows, and once the last tile is done the slices' sums, share one buffer
    constexpr size_t VT_BYTES = sizeof(uint16_t) * TK * WIDTH, MERGED_BYTES = sizeof(float) * SLICES * MAX_GROUPS * WIDTH;
    __shared__ __attribute__((aligned(16))) uint8_t shared_rows[VT_BYTES > MERGED_BYTES ? VT_BYTES : MERGED_BYTES];
    uint16_t(*vt)[WIDTH] = reinterpret_cast<uint16_t(*)[WIDTH]>(shared_rows);
    float(*merged)[MAX_GROUPS][WIDTH] = reinterpret_cast<float(*)[MAX_GROUPS][WIDTH]>(shared_rows);
    __shared__ __attribute__((aligned(16))) float scores[TK][MAX_GROUPS];  // scores, then weights, of the tile's keys
    __shared__ float tile_scale[MAX_GROUPS];                               // exp(old top - new top) per query head
    __shared__ float stat_top[MAX_GROUPS], stat_mass[MAX_GROUPS];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t sub = lane / LPK, dl = lane % LPK;
    const uint32_t unit = blockIdx.x;  // (kv head, plane, row)
    const uint32_t row = unit % p.rows;
    const uint32_t b = (unit / p.rows) % p.batch, kvh = unit / p.rows / p.batch;
    const uint32_t section = blockIdx.y;
    const uint32_t G = p.groups;

    // A section is a fixed span of the window, whatever the cursor says: the K and V rows of its first tile
    // go out before the cursor has even arrived (rows past the visible keys are fetched and dropped).
    const uint32_t chunk = (p.keys + p.sections - 1u) / p.sections;
    const uint32_t begin = min(p.keys, section * chunk);
    const uint64_t plane = ((uint64_t)kvh * p.batch + b) * p.capacity;
    const uint32_t mine = wave * KPW + sub;  // this lane's key inside a step
    u32x4 kraw[T], vraw[T];
    fetch_tile<T, STEP, WIDTH>(kraw, vraw, p.cache_k, p.cache_v, plane, begin + mine, p.capacity, dl);

    uint32_t origin = p.cursor ? p.cursor[b] : 0u;
    if (!p.reach && origin + p.rows > p.keys) {  // refusal::ORIGIN (attention.rs:250-252)
        if (tid == 0) atomicMax(p.refusal, (uint32_t)REFUSAL_ORIGIN);
        origin = p.keys - p.rows;
    }
    // key `at` counts iff at <= origin + row; in a ring every written slot is walked and asked what it holds
    const uint32_t position = origin + row;
    const uint32_t visible = min(p.keys, p.reach ? origin + p.rows : position + 1u);
    const uint32_t last = min(visible, begin + chunk);
    const Ring ring(p.keys, origin + p.rows, p.reach);

    float qr[MAX_GROUPS][8];
#pragma unroll
    for (int g = 0; g < MAX_GROUPS; g++) {
#pragma unroll
        for (int j = 0; j < 8; j++) qr[g][j] = 0.0f;
        if (g < (int)G) {
            const float *src = p.q + (uint64_t)(kvh * G + g) * p.q_sh + (uint64_t)b * p.q_sb + (uint64_t)row * p.q_sr + dl * 8u;
#pragma unroll
            for (int j = 0; j < 8; j++) qr[g][j] = src[j];
        }
    }
    // value pass: this thread sums DPT channels over the keys of one slice of every tile
    const uint32_t slice = tid / TPS, channel = (tid % TPS) * DPT;
    float acc[MAX_GROUPS][DPT];
#pragma unroll
    for (int g = 0; g < MAX_GROUPS; g++)
#pragma unroll
        for (int d = 0; d < DPT; d++) acc[g][d] = 0.0f;
    // softmax statistics: wave w keeps the running top and mass of query heads w and w + 4 (the same in all its lanes)
    float top[2] = {-INFINITY, -INFINITY}, mass[2] = {0.0f, 0.0f};

    for (uint32_t tile = begin; tile < last; tile += TK) {
        // ---- scores of the tile's 64 keys; its value rows go to LDS as they are
#pragma unroll
        for (int s = 0; s < T; s++) {
            const uint32_t local = s * STEP + mine, key = tile + local;
            *reinterpret_cast<u32x4 *>(&vt[local][dl * 8u]) = vraw[s];
            float kf[8];
            unpack8(kraw[s], kf);
#pragma unroll
            for (int g = 0; g < MAX_GROUPS; g++) {
                if (g < (int)G) {
                    float score = 0.0f;
#pragma unroll
                    for (int j = 0; j < 8; j++) score = fmaf(qr[g][j], kf[j], score);
                    score = key_sum<LPK>(score) * p.scale;
                    if (dl == 0) scores[local][g] = key < last && (!p.reach || ring.seen(key, position)) ? score : -INFINITY;
                }
            }
        }
        if (tile + TK < last) fetch_tile<T, STEP, WIDTH>(kraw, vraw, p.cache_k, p.cache_v, plane, tile + TK + mine, p.capacity, dl);  // in flight during the rest of this tile
        __syncthreads();
        // ---- weights: one lane per key, one wave per query head
#pragma unroll
        for (int gi = 0; gi < 2; gi++) {
            const uint32_t g = wave + 4u * gi;
            if (g < G) {
                const float score = scores[lane][g];
                const float next = fmaxf(top[gi], wave_max(score));
                const float weight = score == -INFINITY ? 0.0f : softmax_exp(score - next);
                const float rescale = top[gi] == -INFINITY ? 0.0f : softmax_exp(top[gi] - next);
                mass[gi] = fmaf(mass[gi], rescale, wave_sum(weight));
                top[gi] = next;
                scores[lane][g] = weight;
                if (lane == 0) tile_scale[g] = rescale;
            }
        }
        __syncthreads();
        // ---- values: acc = acc * rescale + sum over this slice's keys of weight * value
#pragma unroll
        for (int g = 0; g < MAX_GROUPS; g++) {
            const float rescale = g < (int)G ? tile_scale[g] : 0.0f;
#pragma unroll
            for (int d = 0; d < DPT; d++) acc[g][d] *= rescale;
        }
#pragma unroll
        for (int kk = 0; kk < KPS; kk++) {
            const uint32_t local = slice * KPS + kk;
            float v[DPT];
            if (DPT == 1) {
                v[0] = half_to_float(vt[local][channel]);
            } else if (DPT == 2) {
                const uint32_t pair = *reinterpret_cast<const uint32_t *>(&vt[local][channel]);
                v[0] = half_to_float((uint16_t)(pair & 0xffffu)), v[1 % DPT] = half_to_float((uint16_t)(pair >> 16));
            } else {
                const uint2 quad = *reinterpret_cast<const uint2 *>(&vt[local][channel]);
                v[0] = half_to_float((uint16_t)(quad.x & 0xffffu)), v[1 % DPT] = half_to_float((uint16_t)(quad.x >> 16));
                v[2 % DPT] = half_to_float((uint16_t)(quad.y & 0xffffu)), v[3 % DPT] = half_to_float((uint16_t)(quad.y >> 16));
            }
            const float4 w0 = *reinterpret_cast<const float4 *>(&scores[local][0]), w1 = *reinterpret_cast<const float4 *>(&scores[local][4]);
            // heads past G hold stale weights: their sums are never read
#pragma unroll
            for (int d = 0; d < DPT; d++) {
                acc[0][d] = fmaf(w0.x, v[d], acc[0][d]), acc[1][d] = fmaf(w0.y, v[d], acc[1][d]);
                acc[2][d] = fmaf(w0.z, v[d], acc[2][d]), acc[3][d] = fmaf(w0.w, v[d], acc[3][d]);
                acc[4][d] = fmaf(w1.x, v[d], acc[4][d]), acc[5][d] = fmaf(w1.y, v[d], acc[5][d]);
                acc[6][d] = fmaf(w1.z, v[d], acc[6][d]), acc[7][d] = fmaf(w1.w, v[d], acc[7][d]);
            }
        }
        __syncthreads();  // the next tile overwrites vt and scores
    }
    // ---- the slices meet in LDS
#pragma unroll
    for (int g = 0; g < MAX_GROUPS; g++) {
        if (g < (int)G) {
#pragma unroll
            for (int d = 0; d < DPT; d++) merged[slice][g][channel + d] = acc[g][d];
        }
    }
#pragma unroll
    for (int gi = 0; gi < 2; gi++) {
        const uint32_t g = wave + 4u * gi;
        if (g < G && lane == 0) stat_top[g] = top[gi], stat_mass[g] = mass[gi];
    }
    __syncthreads();
    for (uint32_t index = tid; index < G * WIDTH; index += 256) {
        const uint32_t g = index / WIDTH, c = index % WIDTH;
        float value = 0.0f;
#pragma unroll
        for (int s = 0; s < SLICES; s++) value += merged[s][g][c];
        const float largest = stat_top[g], total = stat_mass[g];
        const uint32_t head = kvh * G + g;
        if (p.sections > 1) {
            float *dst = p.partial + (((uint64_t)unit * p.sections + section) * G + g) * (WIDTH + 2);
            dst[c] = value;
            if (c == 0) {
                dst[WIDTH] = largest;
                dst[WIDTH + 1] = total;
            }
        } else {
            float normalized = total > 0.0f ? 1.0f / total : 0.0f;
            p.out[(uint64_t)head * p.o_sh + (uint64_t)b * p.o_sb + (uint64_t)row * p.o_sr + c] = value * normalized;
        }
    }
}

// Fold of the sections of one (unit, query head): crates/neura-kernel/src/task/attention.rs:619-671.
// One workgroup per (unit, group, block of 32 channels).  Thread s first turns the statistics of
// section s into its weight; then thread (channel, stripe) sums its channel over every eighth
// section -- all of its loads in flight at once -- and the eight stripes meet in LDS.
// (The leading arguments are what the first loads need: the hardware hands them to a wave in scalar registers as it starts.)
// J: sections a stripe sums at most (8 J >= sections): no more loads than the sections ask for, to the next power of two.
template <int J>
__global__ __launch_bounds__(256) void attention_fold_kernel(const float *lead_partial, uint32_t lead_sections, uint32_t lead_groups, uint32_t width,
                                                             AttentionParams p) {
    __shared__ float weights[256], masses[256], held[256], stripes[8][32];
    const uint32_t G = lead_groups, tid = threadIdx.x, sections = lead_sections;
    const uint32_t blocks = (width + 31u) / 32u;
    const uint32_t cblock = blockIdx.x % blocks, ug = blockIdx.x / blocks;
    const uint32_t unit = ug / G, g = ug % G;
    const float *src = lead_partial + ((uint64_t)unit * sections * G + g) * (width + 2);
    const uint32_t hop = G * (width + 2u);  // one section further (a unit's partials are far fewer than 2^32 numbers)
    float top = -INFINITY, mass = 0.0f;
    {
        const float *stats = src + min(tid, sections - 1u) * hop + width;
        const float read_top = stats[0], read_mass = stats[1];
        if (tid < sections) top = read_top, mass = read_mass;
    }
    // the channel sums do not wait for the weights: fetch first.  Every load is issued whatever its section (past the last
    // one it reads the last again and is dropped): loads under a condition each got a branch of their own, and the address
    // arithmetic between them waited for the loads before -- eight round trips one after another where one is enough.
    const uint32_t c = cblock * 32u + (tid & 31u), stripe = tid >> 5;
    const float *column = src + min(c, width - 1u);
    float values[J];
#pragma unroll
    for (int j = 0; j < J; j++) values[j] = column[min(stripe + 8u * j, sections - 1u) * hop];
#pragma unroll
    for (int j = 0; j < J; j++)
        if (stripe + 8u * j >= sections || c >= width) values[j] = 0.0f;
    // the largest top and the weighed mass: a wave each, then the four waves' words
    const float wave_top = wave_max(top);
    if ((tid & 63u) == 0) held[tid >> 6] = wave_top;
    __syncthreads();
    const float largest = fmaxf(fmaxf(held[0], held[1]), fmaxf(held[2], held[3]));
    const float weight = top == -INFINITY ? 0.0f : softmax_exp(top - largest);
    weights[tid] = weight;
    const float wave_mass = wave_sum(mass * weight);
    if ((tid & 63u) == 0) masses[tid >> 6] = wave_mass;
    __syncthreads();
    const float total = (masses[0] + masses[1]) + (masses[2] + masses[3]);
    const float normalized = total > 0.0f ? 1.0f / total : 0.0f;
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < J; j++) {
        const uint32_t s = stripe + 8u * j;
        if (s < sections) sum = fmaf(values[j], weights[s], sum);
    }
    stripes[stripe][tid & 31u] = sum;
    __syncthreads();
    if (tid < 32 && c < width) {
        // where the row goes is worked out here, behind the loads: it needs parameters the first loads do not wait for
        const uint32_t row = unit % p.rows;
        const uint32_t b = (unit / p.rows) % p.batch, kvh = unit / p.rows / p.batch;
        float value = ((stripes[0][tid] + stripes[1][tid]) + (stripes[2][tid] + stripes[3][tid])) +
                      ((stripes[4][tid] + stripes[5][tid]) + (stripes[6][tid] + stripes[7][tid]));
        p.out[(uint64_t)(kvh * G + g) * p.o_sh + (uint64_t)b * p.o_sb + (uint64_t)row * p.o_sr + c] = value * normalized;
    }
}


// Eight numbers of a key or value state as eight halves (four words) for the matrix cores, and for single states the eight
// residues * 2^11 beside them.  Halves go as they lie.  bfloat16 numbers become the halves they equal (every bfloat16 between
// 2^-17 and 65504 in magnitude is a half; smaller ones land within 2^-25).  Single numbers enter as two half planes, the value
// rounded to half and its residue * 2^11 -- 22 bits of each, as the queries and the weights do.  States past the halves' range
// (65504) overflow here as they would in half states.
template <int CE, int WORDS>
__device__ __forceinline__ void states_as_halves(const u32x4 (&raw)[WORDS], u32x4 &value, u32x4 &residue) {
    if constexpr (CE == NH_F16) {
        value = raw[0];
    } else if constexpr (CE == NH_BF16) {
        const uint32_t words[4] = {raw[0].x, raw[0].y, raw[0].z, raw[0].w};
        uint32_t out[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t word = words[i];
            const _Float16 low = (_Float16)__builtin_bit_cast(float, word << 16), high = (_Float16)__builtin_bit_cast(float, word & 0xffff0000u);
            out[i] = (uint32_t)__builtin_bit_cast(uint16_t, low) | ((uint32_t)__builtin_bit_cast(uint16_t, high) << 16);
        }
        value = u32x4{out[0], out[1], out[2], out[3]};
    } else {
        const uint32_t words[8] = {raw[0].x, raw[0].y, raw[0].z, raw[0].w, raw[WORDS - 1].x, raw[WORDS - 1].y, raw[WORDS - 1].z, raw[WORDS - 1].w};
        uint32_t out[4], fine_out[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t first = words[2 * i], second = words[2 * i + 1];
            const float a = __builtin_bit_cast(float, first), b = __builtin_bit_cast(float, second);
            const _Float16 a_high = (_Float16)a, b_high = (_Float16)b;
            const _Float16 a_low = (_Float16)((a - (float)a_high) * 2048.0f), b_low = (_Float16)((b - (float)b_high) * 2048.0f);
            out[i] = (uint32_t)__builtin_bit_cast(uint16_t, a_high) | ((uint32_t)__builtin_bit_cast(uint16_t, b_high) << 16);
            fine_out[i] = (uint32_t)__builtin_bit_cast(uint16_t, a_low) | ((uint32_t)__builtin_bit_cast(uint16_t, b_low) << 16);
        }
        value = u32x4{out[0], out[1], out[2], out[3]};
        residue = u32x4{fine_out[0], fine_out[1], fine_out[2], fine_out[3]};
    }
}

// ---------------------------------------------------------------- several query rows: the matrix cores --------
//
// A chunk of query rows (a fill) against the same cache, on v_mfma_f32_32x32x16_f16.  One workgroup serves one
// (kv head, plane) and a block of query rows; each of its four waves owns 32 "columns" -- RPW = 32 / groups query
// rows times the query heads of the group -- and all four share the key and value tiles of 32 keys the workgroup
// stages in LDS.  Per tile and wave:
//   scores  S^T[key][column] = K[key][:] . q[column][:]: the key rows are the A operand as they lie (a lane reads 8
//           halves of its key), the queries the B operand, held in registers as two half planes (value and residue, so
//           fp32 queries lose nothing).  C hands lane (column, half) sixteen of the tile's 32 keys: a column's maximum
//           and sum never leave its two lanes.
//   values  O^T[channel][column] += V^T[channel][key] . P^T[key][column]: the weights go back in as the B operand
//           straight from the registers C left them in (again as value and residue planes), and the value tile, which
//           the workgroup wrote to LDS transposed, is the A operand in that same key order.
// The running maximum, sum and the 32 x 64 accumulators of a column live in its two lanes; nothing is folded afterwards.
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// CE: what the states hold (states_as_halves above); single states stage a second plane of key and value residues and cost
// one more MFMA a product.
// SPLIT: two sets of four waves share the block of query rows and take every other key tile each (the walk of a long row
// block is a chain of tiles, each a chain of MFMAs and a softmax with one wave a SIMD: two sets halve it); the two meet in
// LDS at the end, lane by lane, as two partial softmaxes do.  Single states stage twice the planes and keep one set.
template <int WIDTH, int CE = NH_F16, bool SPLIT = false>
__global__ __launch_bounds__(SPLIT ? 512 : 256) void attention_tile_kernel(AttentionParams p, uint32_t rows_per_wave) {
    fetch_parameters(p);
    static_assert(!SPLIT || CE != NH_F32, "two sets of staged tiles of single states do not fit the static LDS");
    constexpr int SETS = SPLIT ? 2 : 1;
    constexpr int TK = 32;                       // keys per tile
    constexpr int STEPS = WIDTH / 16;            // MFMA steps over the channels of a score
    constexpr int BLOCKS = WIDTH / 32;           // 32-channel blocks of the output
    constexpr int KPITCH = WIDTH + 8;            // halves per staged key row (the pad spreads the banks)
    constexpr int VPITCH = TK + 4;               // halves per staged value channel
    constexpr int PLANES = CE == NH_F32 ? 2 : 1;  // values, and for single states their residues * 2^11
    constexpr int WORDS = CE == NH_F32 ? 2 : 1;   // 16-byte loads that hold eight stored numbers
    constexpr uint32_t STORED = CE == NH_F32 ? 4u : 2u;
    constexpr size_t KT_BYTES = sizeof(uint16_t) * SETS * PLANES * TK * KPITCH, VT_BYTES = sizeof(uint16_t) * SETS * PLANES * WIDTH * VPITCH;
    __shared__ __attribute__((aligned(16))) uint8_t tile_lds[KT_BYTES + VT_BYTES];  // the staged key tiles, then the value tiles
    uint16_t(*const kt_planes)[PLANES][TK][KPITCH] = reinterpret_cast<uint16_t(*)[PLANES][TK][KPITCH]>(tile_lds);
    uint16_t(*const vt_planes)[PLANES][WIDTH][VPITCH] = reinterpret_cast<uint16_t(*)[PLANES][WIDTH][VPITCH]>(tile_lds + KT_BYTES);
    const uint32_t set = SPLIT ? threadIdx.x >> 8 : 0u;  // which of the two sets of waves; tid, wave: within the set
    uint16_t(*const kt)[KPITCH] = kt_planes[set][0];
    uint16_t(*const vt)[VPITCH] = vt_planes[set][0];
    uint16_t(*const kt_fine)[KPITCH] = kt_planes[set][PLANES - 1];
    uint16_t(*const vt_fine)[VPITCH] = vt_planes[set][PLANES - 1];
    const uint32_t tid = threadIdx.x & 255u, lane = tid & 63u, wave = tid >> 6;
    const uint32_t n = lane & 31u, h = lane >> 5;
    const uint32_t G = p.groups;
    const uint32_t b = blockIdx.x % p.batch, kvh = blockIdx.x / p.batch;
    const uint64_t plane = ((uint64_t)kvh * p.batch + b) * p.capacity;

    uint32_t origin = p.cursor ? p.cursor[b] : 0u;
    if (!p.reach && origin + p.rows > p.keys) {  // refusal::ORIGIN (attention.rs:250-252)
        if (tid == 0) atomicMax(p.refusal, (uint32_t)REFUSAL_ORIGIN);
        origin = p.keys - p.rows;
    }
    const Ring ring(p.keys, origin + p.rows, p.reach);
    // this lane's column: a query row and a query head of the group
    const uint32_t block_row = blockIdx.y * 4u * rows_per_wave;
    const uint32_t row = block_row + wave * rows_per_wave + n / G, g = n % G;
    const bool held = n < rows_per_wave * G && row < p.rows;
    const uint32_t limit = origin + min(row, p.rows - 1u);  // the last key this column sees (its own position)
    // the workgroup walks up to the last key its last row sees; a ring is walked whole, every slot asked what it holds
    const uint32_t last_row = min(p.rows, block_row + 4u * rows_per_wave) - 1u;
    const uint32_t span = min(p.keys, p.reach ? origin + p.rows : origin + last_row + 1u);
    const uint32_t wave_first = block_row + wave * rows_per_wave;
    const uint32_t wave_span = wave_first >= p.rows ? 0u : (p.reach ? span : min(p.keys, origin + min(p.rows, wave_first + rows_per_wave)));

    // queries as two half planes: q = value + residue, both halves
    half8_t q_value[STEPS], q_residue[STEPS];
    {
        const float *src = p.q + (uint64_t)(kvh * G + g) * p.q_sh + (uint64_t)b * p.q_sb + (uint64_t)min(row, p.rows - 1u) * p.q_sr;
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const float value = held ? src[16 * s + 8 * h + i] : 0.0f;
                const _Float16 high = (_Float16)value;
                q_value[s][i] = high;
                q_residue[s][i] = (_Float16)((value - (float)high) * 2048.0f);  // scaled up, clear of the subnormal halves
            }
        }
    }
    f32x16 acc[BLOCKS];
#pragma unroll
    for (int d = 0; d < BLOCKS; d++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[d][r] = 0.0f;
    float top = -INFINITY, mass = 0.0f;

    // the pieces of a tile this thread stages: 16 bytes of a key row and of a value row each
    constexpr int PIECES = TK * WIDTH / 8 / 256;  // per thread and tile
    u32x4 kraw[PIECES][WORDS], vraw[PIECES][WORDS];
    const uint8_t *const k_bytes = reinterpret_cast<const uint8_t *>(p.cache_k), *const v_bytes = reinterpret_cast<const uint8_t *>(p.cache_v);
    auto fetch = [&](uint32_t tile) {
#pragma unroll
        for (int k = 0; k < PIECES; k++) {
            const uint32_t piece = tid + 256u * k, key = piece / (WIDTH / 8), chunk = piece % (WIDTH / 8);
            const uint64_t at = (plane + min(tile + key, p.capacity - 1u)) * WIDTH + chunk * 8u;
#pragma unroll
            for (int w = 0; w < WORDS; w++) {
                kraw[k][w] = *reinterpret_cast<const u32x4 *>(k_bytes + at * STORED + 16u * w);
                vraw[k][w] = *reinterpret_cast<const u32x4 *>(v_bytes + at * STORED + 16u * w);
            }
        }
    };
    // set s walks tiles s, s + SETS, ...; both sets meet every barrier of every round
    if (set * TK < span) fetch(set * TK);
    for (uint32_t first = 0; first < span; first += SETS * TK) {
        const uint32_t tile = first + set * TK;
        const bool have = tile < span;
        __syncthreads();  // the last tile's readers are done
#pragma unroll
        for (int k = 0; k < PIECES; k++) {
            if (!have) break;
            const uint32_t piece = tid + 256u * k, key = piece / (WIDTH / 8), chunk = piece % (WIDTH / 8);
            u32x4 k_words, k_fine = {0u, 0u, 0u, 0u}, v_words, v_fine = {0u, 0u, 0u, 0u};
            states_as_halves<CE, WORDS>(kraw[k], k_words, k_fine);
            states_as_halves<CE, WORDS>(vraw[k], v_words, v_fine);
            *reinterpret_cast<u32x4 *>(&kt[key][chunk * 8u]) = k_words;
            if constexpr (CE == NH_F32) *reinterpret_cast<u32x4 *>(&kt_fine[key][chunk * 8u]) = k_fine;
            // rows past the written keys may hold anything, and a weight of zero does not silence a NaN
            const uint32_t keep = tile + key < span ? 0xffffffffu : 0u;
            // groups of four keys change places by the channel block (chunk / 4), or the chunks a store instruction touches share four banks
            const uint32_t column = (((key >> 2) ^ (chunk >> 2)) << 2) | (key & 3u);
            {
                const uint32_t words[4] = {v_words.x & keep, v_words.y & keep, v_words.z & keep, v_words.w & keep};
#pragma unroll
                for (int i = 0; i < 8; i++) vt[chunk * 8u + i][column] = (uint16_t)(words[i >> 1] >> (16 * (i & 1)));
            }
            if constexpr (CE == NH_F32) {
                const uint32_t words[4] = {v_fine.x & keep, v_fine.y & keep, v_fine.z & keep, v_fine.w & keep};
#pragma unroll
                for (int i = 0; i < 8; i++) vt_fine[chunk * 8u + i][column] = (uint16_t)(words[i >> 1] >> (16 * (i & 1)));
            }
        }
        if (tile + SETS * TK < span) fetch(tile + SETS * TK);  // in flight while this tile is multiplied
        __syncthreads();
        if (!have || tile >= wave_span) continue;  // keys none of this wave's rows see (every wave still meets the barriers)

        // ---- scores
        f32x16 scores, fine;
#pragma unroll
        for (int r = 0; r < 16; r++) scores[r] = 0.0f, fine[r] = 0.0f;
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            const half8_t keys = *reinterpret_cast<const half8_t *>(&kt[n][16 * s + 8 * h]);
            scores = __builtin_amdgcn_mfma_f32_32x32x16_f16(keys, q_value[s], scores, 0, 0, 0);
            fine = __builtin_amdgcn_mfma_f32_32x32x16_f16(keys, q_residue[s], fine, 0, 0, 0);
            if constexpr (CE == NH_F32)
                fine = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const half8_t *>(&kt_fine[n][16 * s + 8 * h]), q_value[s], fine, 0, 0, 0);
        }
        // ---- weights: register 4j + e of lane (column, h) is key 8j + 4h + e of the tile
        float tile_top = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const uint32_t key = tile + 8u * (r >> 2) + 4u * h + (r & 3);
            const bool seen = held && key < p.keys && (p.reach ? ring.seen(key, limit) : key <= limit);
            scores[r] = seen ? fmaf(fine[r], 1.0f / 2048.0f, scores[r]) * p.scale : -INFINITY;
            tile_top = fmaxf(tile_top, scores[r]);
        }
        tile_top = fmaxf(tile_top, __shfl_xor(tile_top, 32, 64));
        const float next = fmaxf(top, tile_top);
        const float rescale = top == -INFINITY ? 0.0f : softmax_exp(top - next);
        float tile_mass = 0.0f;
        half8_t w_value[2], w_residue[2], w_small[2];  // w_small: the weights * 2^-11, for the values' residues (single states)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const float weight = scores[r] == -INFINITY ? 0.0f : softmax_exp(scores[r] - next);
            tile_mass += weight;
            // the weights ride 2^10 up (undone with the mass at the end): their residues stay normal halves
            const float raised = weight * 1024.0f;
            const _Float16 high = (_Float16)raised;
            // key slots of the second product: step t takes registers 8t .. 8t + 7 in order
            w_value[r >> 3][r & 7] = high;
            w_residue[r >> 3][r & 7] = (_Float16)(raised - (float)high);
            w_small[r >> 3][r & 7] = (_Float16)(CE == NH_F32 ? raised * (1.0f / 2048.0f) : 0.0f);
        }
        tile_mass += __shfl_xor(tile_mass, 32, 64);
        mass = fmaf(mass, rescale, tile_mass);
        top = next;
        // ---- values
#pragma unroll
        for (int d = 0; d < BLOCKS; d++) {
#pragma unroll
            for (int r = 0; r < 16; r++) acc[d][r] *= rescale;
#pragma unroll
            for (int t = 0; t < 2; t++) {
                // slots 8h + i of step t: keys 16t + 4h + i (i < 4) and 16t + 8 + 4h + (i - 4), as the weights lie
                half8_t values;
                // channels 32 d + n lie in chunks 4 d .. 4 d + 3: their key groups sit d places off
                const uint2 low = *reinterpret_cast<const uint2 *>(&vt[32 * d + n][4 * ((4 * t + h) ^ d)]);
                const uint2 high = *reinterpret_cast<const uint2 *>(&vt[32 * d + n][4 * ((4 * t + 2 + h) ^ d)]);
                const u32x4 joined = {low.x, low.y, high.x, high.y};
                values = __builtin_bit_cast(half8_t, joined);
                acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_f16(values, w_value[t], acc[d], 0, 0, 0);
                acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_f16(values, w_residue[t], acc[d], 0, 0, 0);
                if constexpr (CE == NH_F32) {
                    const uint2 low_fine = *reinterpret_cast<const uint2 *>(&vt_fine[32 * d + n][4 * ((4 * t + h) ^ d)]);
                    const uint2 high_fine = *reinterpret_cast<const uint2 *>(&vt_fine[32 * d + n][4 * ((4 * t + 2 + h) ^ d)]);
                    const half8_t residues = __builtin_bit_cast(half8_t, u32x4{low_fine.x, low_fine.y, high_fine.x, high_fine.y});
                    acc[d] = __builtin_amdgcn_mfma_f32_32x32x16_f16(residues, w_small[t], acc[d], 0, 0, 0);
                }
            }
        }
    }
    if constexpr (SPLIT) {
        // ---- the two sets meet lane by lane: the second leaves its maximum, its mass and its sums (a 32-channel block a
        // round) where the tiles were staged, the first joins them as two partial softmaxes join
        static_assert(KT_BYTES + VT_BYTES >= sizeof(float) * 256 * 18, "the staged tiles' LDS holds a round of the meeting");
        float *const meet = reinterpret_cast<float *>(tile_lds);
        float mine = 1.0f, theirs = 0.0f;
#pragma unroll
        for (int d = 0; d < BLOCKS; d++) {
            __syncthreads();  // the walk (or the round before) is done with this LDS
            if (set == 1u) {
                if (d == 0) meet[16 * 256 + tid] = top, meet[17 * 256 + tid] = mass;
#pragma unroll
                for (int r = 0; r < 16; r++) meet[r * 256 + tid] = acc[d][r];
            }
            __syncthreads();
            if (set == 0u) {
                if (d == 0) {
                    const float other_top = meet[16 * 256 + tid], other_mass = meet[17 * 256 + tid];
                    const float next = fmaxf(top, other_top);
                    mine = top == -INFINITY ? 0.0f : softmax_exp(top - next);
                    theirs = other_top == -INFINITY ? 0.0f : softmax_exp(other_top - next);
                    mass = fmaf(mass, mine, other_mass * theirs);
                    top = next;
                }
#pragma unroll
                for (int r = 0; r < 16; r++) acc[d][r] = fmaf(acc[d][r], mine, meet[r * 256 + tid] * theirs);
            }
        }
        if (set == 1u) return;
    }
    if (!held) return;
    // register 4j + e of block d is channel 32d + 8j + 4h + e of this lane's column
    const float normalized = mass > 0.0f ? 1.0f / (mass * 1024.0f) : 0.0f;
    float *dst = p.out + (uint64_t)(kvh * G + g) * p.o_sh + (uint64_t)b * p.o_sb + (uint64_t)row * p.o_sr;
#pragma unroll
    for (int d = 0; d < BLOCKS; d++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float4 out4 = {acc[d][4 * j] * normalized, acc[d][4 * j + 1] * normalized, acc[d][4 * j + 2] * normalized, acc[d][4 * j + 3] * normalized};
            *reinterpret_cast<float4 *>(dst + 32 * d + 8 * j + 4 * h) = out4;
        }
}


// ---------------------------------------------------------------- one query row, many planes: the matrix cores ------
//
// A decode step of several planes walks as many key tiles as a long fill, one query row each; the row-at-a-time kernel
// spends its time in the multiply-adds of the scores and the value sums.  Here the ≤16 query heads of a group are the 16
// columns of v_mfma_f32_16x16x32_f16.  A workgroup serves one (kv head, plane, section of the window); each of its four
// waves walks every fourth tile of 32 keys on its own -- no barrier inside the walk -- and the four meet once in LDS.
// Per tile and wave:
//   scores  S[key][column]: the key rows are the A operand straight from the cache (lane (key % 16, kq) loads the 8 halves
//           32 s + 8 kq .. of its key), the queries the B operand as value and residue * 2^11 half planes in registers.
//           C hands lane (column, kq) the keys 4 kq + e and 16 + 4 kq + e of the tile: a column's statistics live in four lanes.
//   values  O^T[channel][column] += V^T[channel][key] . P^T[key][column]: the weights (* 2^10, value and residue planes) go
//           back in as the B operand from the registers C left them in -- slots 0..3 the keys 4 kq + e, slots 4..7 the keys
//           16 + 4 kq + e -- and the value rows, which the wave wrote to its own corner of LDS as they lie, are the A operand in
//           that same key order, transposed by the read (ds_read_b64_tr_b16, two a lane).
typedef float f32x4_t __attribute__((ext_vector_type(4)));

// The leading arguments are what the first loads (cursor, queries, the first key and value tile) need: plain words that the
// hardware hands to a wave in scalar registers as it starts (batch and query heads a group share a word); the rest is in `p`.
// TK = 16 (one plane a kv head: a decode step of few planes): tiles of sixteen keys, so that sections of 64 keys give every
// compute unit a workgroup and a wave half the work; the value product then runs on v_mfma_f32_16x16x16_f16 (K = the tile's keys).
// CE: what the states hold (states_as_halves above): single states cost one more MFMA a product -- the key residues against the
// query values, the value residues against the weights * 2^-11.
template <int WIDTH, int TK = 32, int CE = NH_F16>
__global__ __launch_bounds__(256) void attention_decode_tile_kernel(const uint32_t *lead_cursor, const float *lead_q, const uint16_t *lead_k, const uint16_t *lead_v,
                                                                    uint32_t lead_q_sh, uint32_t lead_q_sb, uint32_t lead_keys, uint32_t lead_sections,
                                                                    uint32_t lead_capacity, uint32_t lead_batch_groups, AttentionParams p) {
    constexpr int KB = TK / 16;             // 16-key blocks of a tile
    constexpr int STEPS = WIDTH / 32;       // MFMA steps over the channels of a score
    constexpr int BLOCKS = WIDTH / 16;      // 16-channel blocks of the output
    constexpr int VROW = WIDTH + 16;        // halves per staged value row: the four rows a read's sixteen lanes touch fall into different banks
    constexpr int PIECES = TK * WIDTH / 8 / 64;  // 16-byte pieces of a value tile per lane
    // the waves' value corners and, once every wave has left the walk, their sums share one buffer
    constexpr size_t VT_BYTES = sizeof(uint16_t) * 4 * TK * VROW, MERGED_BYTES = sizeof(float) * 4 * 16 * (WIDTH + 4), STATS_BYTES = sizeof(float) * 8 * 16;
    constexpr size_t ROWS_BYTES = VT_BYTES > MERGED_BYTES ? VT_BYTES : MERGED_BYTES;
    __shared__ __attribute__((aligned(16))) uint8_t shared_rows[ROWS_BYTES + STATS_BYTES];
    uint16_t(*vt)[TK][VROW] = reinterpret_cast<uint16_t(*)[TK][VROW]>(shared_rows);
    float(*merged)[16][WIDTH + 4] = reinterpret_cast<float(*)[16][WIDTH + 4]>(shared_rows);  // per wave and column: the weighed channel sums (rows 16 bytes apart in phase)
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t n = lane & 15u, kq = lane >> 4;
    const uint32_t G = lead_batch_groups & 0xffffu, batch = lead_batch_groups >> 16;
    const uint32_t keys_held = lead_keys, sections = lead_sections, capacity = lead_capacity;
    const uint32_t unit = blockIdx.x, section = blockIdx.y;
    const uint32_t b = unit % batch, kvh = unit / batch;
    const uint64_t plane = ((uint64_t)kvh * batch + b) * capacity;

    // what does not need the cursor comes first: the cursor's load, the queries' and the first tile's are then all in flight
    // together instead of one round trip to memory behind the other
    const uint32_t origin_read = lead_cursor ? lead_cursor[b] : 0u;
    const uint32_t chunk = (keys_held + sections - 1u) / sections;
    const uint32_t begin = min(keys_held, section * chunk);
    const bool held = n < G;

    // the queries of this lane's column, as they lie; they become two half planes once the first tile has been asked for
    float q_raw[STEPS][8];
    {
        const float *src = lead_q + (uint64_t)(kvh * G + min(n, G - 1u)) * lead_q_sh + (uint64_t)b * lead_q_sb;
        // a column past the group reads the group's last head: its scores are masked, and no column reaches another's sums
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            const float4 low = *reinterpret_cast<const float4 *>(src + 32 * s + 8 * kq), high = *reinterpret_cast<const float4 *>(src + 32 * s + 8 * kq + 4);
            q_raw[s][0] = low.x, q_raw[s][1] = low.y, q_raw[s][2] = low.z, q_raw[s][3] = low.w;
            q_raw[s][4] = high.x, q_raw[s][5] = high.y, q_raw[s][6] = high.z, q_raw[s][7] = high.w;
        }
    }
    f32x4_t acc[BLOCKS];
#pragma unroll
    for (int d = 0; d < BLOCKS; d++) acc[d] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    float top = -INFINITY, mass = 0.0f;

    constexpr int WORDS = CE == NH_F32 ? 2 : 1;              // 16-byte loads that hold eight stored numbers
    constexpr uint32_t STORED = CE == NH_F32 ? 4u : 2u;      // bytes a stored number
    const uint8_t *const k_bytes = reinterpret_cast<const uint8_t *>(lead_k), *const v_bytes = reinterpret_cast<const uint8_t *>(lead_v);
    u32x4 kraw[KB][STEPS][WORDS], vraw[PIECES][WORDS];
    auto fetch_keys = [&](uint32_t tile) {
#pragma unroll
        for (int kb = 0; kb < KB; kb++)
#pragma unroll
            for (int s = 0; s < STEPS; s++) {
                const uint64_t at = (plane + min(tile + 16u * kb + n, capacity - 1u)) * WIDTH + 32u * s + 8u * kq;
#pragma unroll
                for (int w = 0; w < WORDS; w++) kraw[kb][s][w] = *reinterpret_cast<const u32x4 *>(k_bytes + at * STORED + 16u * w);
            }
    };
    auto fetch_values = [&](uint32_t tile) {
#pragma unroll
        for (int i = 0; i < PIECES; i++) {
            const uint32_t piece = lane + 64u * i, key = piece / (WIDTH / 8), part = piece % (WIDTH / 8);
            const uint64_t at = (plane + min(tile + key, capacity - 1u)) * WIDTH + part * 8u;
#pragma unroll
            for (int w = 0; w < WORDS; w++) vraw[i][w] = *reinterpret_cast<const u32x4 *>(v_bytes + at * STORED + 16u * w);
        }
    };
    // the first tile's rows are asked for whether or not the cursor has reached them (the addresses are clamped to the cache)
    uint32_t tile = begin + wave * TK;
    __builtin_amdgcn_sched_barrier(0);  // the queries' loads stay ahead of the tile's, their first use behind them
    if (tile < min(keys_held, begin + chunk)) fetch_keys(tile), fetch_values(tile);
    __builtin_amdgcn_sched_barrier(0);
    half8_t q_value[STEPS], q_residue[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; s++)
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const _Float16 high = (_Float16)q_raw[s][i];
            q_value[s][i] = high;
            q_residue[s][i] = (_Float16)((q_raw[s][i] - (float)high) * 2048.0f);
        }
    uint32_t origin = origin_read;
    if (!p.reach && origin + 1u > keys_held) {  // refusal::ORIGIN (attention.rs:250-252)
        if (tid == 0) atomicMax(p.refusal, (uint32_t)REFUSAL_ORIGIN);
        origin = keys_held - 1u;
    }
    const Ring ring(keys_held, origin + 1u, p.reach);
    const uint32_t visible = min(keys_held, origin + 1u);  // a ring too: the slots written so far
    const uint32_t last = min(visible, begin + chunk);
    for (; tile < last; tile += 4 * TK) {
        // ---- scores
        f32x4_t scores[KB], fine[KB];
#pragma unroll
        for (int kb = 0; kb < KB; kb++) {
            scores[kb] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f}, fine[kb] = scores[kb];
#pragma unroll
            for (int s = 0; s < STEPS; s++) {
                u32x4 key_words, key_residues = {0u, 0u, 0u, 0u};
                states_as_halves<CE, WORDS>(kraw[kb][s], key_words, key_residues);
                const half8_t keys = __builtin_bit_cast(half8_t, key_words);
                scores[kb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(keys, q_value[s], scores[kb], 0, 0, 0);
                fine[kb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(keys, q_residue[s], fine[kb], 0, 0, 0);
                if constexpr (CE == NH_F32) fine[kb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, key_residues), q_value[s], fine[kb], 0, 0, 0);
            }
        }
        const uint32_t next = tile + 4 * TK;
        if (next < last) fetch_keys(next);  // in flight during the rest of this tile
        // ---- weights: register e of block kb is key 16 kb + 4 kq + e of the tile, for this lane's column
        float tile_top = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < KB; kb++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const uint32_t key = tile + 16u * kb + 4u * kq + e;
                const bool seen = held && key < last && (!p.reach || ring.seen(key, origin));
                scores[kb][e] = seen ? fmaf(fine[kb][e], 1.0f / 2048.0f, scores[kb][e]) * p.scale : -INFINITY;
                tile_top = fmaxf(tile_top, scores[kb][e]);
            }
        tile_top = fmaxf(tile_top, __shfl_xor(tile_top, 16, 64));
        tile_top = fmaxf(tile_top, __shfl_xor(tile_top, 32, 64));
        const float newer = fmaxf(top, tile_top);
        const float rescale = top == -INFINITY ? 0.0f : softmax_exp(top - newer);
        float tile_mass = 0.0f;
        half8_t w_value, w_residue, w_small;  // with sixteen keys a tile the low four slots only; w_small: the weights * 2^-11, for the values' residues
#pragma unroll
        for (int i = 0; i < 8; i++) w_value[i] = (_Float16)0.0f, w_residue[i] = (_Float16)0.0f, w_small[i] = (_Float16)0.0f;
#pragma unroll
        for (int kb = 0; kb < KB; kb++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float weight = scores[kb][e] == -INFINITY ? 0.0f : softmax_exp(scores[kb][e] - newer);
                tile_mass += weight;
                // the weights ride 2^10 up (undone with the mass at the end): their residues stay normal halves
                const float raised = weight * 1024.0f;
                const _Float16 high = (_Float16)raised;
                w_value[4 * kb + e] = high;
                w_residue[4 * kb + e] = (_Float16)(raised - (float)high);
                if constexpr (CE == NH_F32) w_small[4 * kb + e] = (_Float16)(raised * (1.0f / 2048.0f));
            }
        tile_mass += __shfl_xor(tile_mass, 16, 64);
        tile_mass += __shfl_xor(tile_mass, 32, 64);
        mass = fmaf(mass, rescale, tile_mass);
        top = newer;
        // ---- the tile's value rows, transposed, into this wave's corner of LDS (single states: the values' plane, then their
        // residues' plane through the same corner)
        u32x4 v_words[PIECES], v_fine[PIECES];
#pragma unroll
        for (int i = 0; i < PIECES; i++) {
            v_fine[i] = u32x4{0u, 0u, 0u, 0u};
            states_as_halves<CE, WORDS>(vraw[i], v_words[i], v_fine[i]);
        }
        auto stage_plane = [&](const u32x4 (&plane_words)[PIECES]) {
#pragma unroll
            for (int i = 0; i < PIECES; i++) {
                const uint32_t piece = lane + 64u * i, key = piece / (WIDTH / 8), part = piece % (WIDTH / 8);
                // rows past the walked keys may hold anything, and a weight of zero does not silence a NaN
                const uint32_t keep = tile + key < last ? 0xffffffffu : 0u;
                *reinterpret_cast<u32x4 *>(&vt[wave][key][part * 8u]) = u32x4{plane_words[i].x & keep, plane_words[i].y & keep, plane_words[i].z & keep, plane_words[i].w & keep};
            }
        };
        // ds_read_b64_tr_b16 hands lane 4 k + a of a group of sixteen, which points at four halves, element (lane % 4) of the pieces
        // its lanes a, a + 4, a + 8, a + 12 point at: with lane (k, a) of group kq at key 4 kq + k, channels 16 d + 4 a .., lane n
        // receives channel 16 d + n of keys 4 kq .. 4 kq + 3 -- the A operand, transposed on the way out of LDS
        typedef short short4_t __attribute__((ext_vector_type(4)));
        typedef __attribute__((address_space(3))) short4_t *lds_short4;
        auto transposed = [&](uint32_t first_key, int d) -> uint2 {
            return __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4)&vt[wave][first_key + 4u * kq + (n >> 2)][16 * d + 4 * (n & 3u)]));
        };
        stage_plane(v_words);
        if (next < last) fetch_values(next);
        __builtin_amdgcn_wave_barrier();  // LDS serves a wave's accesses in order: the reads below see these writes
        // ---- values
#pragma unroll
        for (int d = 0; d < BLOCKS; d++) {
#pragma unroll
            for (int e = 0; e < 4; e++) acc[d][e] *= rescale;
            const uint2 low = transposed(0u, d);
            if constexpr (TK == 32) {
                const uint2 high = transposed(16u, d);
                const half8_t values = __builtin_bit_cast(half8_t, u32x4{low.x, low.y, high.x, high.y});
                acc[d] = __builtin_amdgcn_mfma_f32_16x16x32_f16(values, w_value, acc[d], 0, 0, 0);
                acc[d] = __builtin_amdgcn_mfma_f32_16x16x32_f16(values, w_residue, acc[d], 0, 0, 0);
            } else {
                typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
                const half4_t values = __builtin_bit_cast(half4_t, low);
                const half4_t first = {w_value[0], w_value[1], w_value[2], w_value[3]}, second = {w_residue[0], w_residue[1], w_residue[2], w_residue[3]};
                acc[d] = __builtin_amdgcn_mfma_f32_16x16x16f16(values, first, acc[d], 0, 0, 0);
                acc[d] = __builtin_amdgcn_mfma_f32_16x16x16f16(values, second, acc[d], 0, 0, 0);
            }
        }
        __builtin_amdgcn_wave_barrier();  // the next plane, or the next tile, overwrites the corner
        if constexpr (CE == NH_F32) {
            stage_plane(v_fine);
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int d = 0; d < BLOCKS; d++) {
                const uint2 low = transposed(0u, d);
                if constexpr (TK == 32) {
                    const uint2 high = transposed(16u, d);
                    const half8_t values = __builtin_bit_cast(half8_t, u32x4{low.x, low.y, high.x, high.y});
                    acc[d] = __builtin_amdgcn_mfma_f32_16x16x32_f16(values, w_small, acc[d], 0, 0, 0);
                } else {
                    typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
                    const half4_t third = {w_small[0], w_small[1], w_small[2], w_small[3]};
                    acc[d] = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(half4_t, low), third, acc[d], 0, 0, 0);
                }
            }
            __builtin_amdgcn_wave_barrier();
        }
    }
    // ---- the four waves meet: register e of block d is channel 16 d + 4 kq + e of this lane's column
    // a wave's sums are weighed by e^(its top - the largest of the four) before they leave its registers: the four tops and
    // masses of a column cross in LDS first (lanes kq = 0 hold a column's statistics; every lane of the column reads them back)
    float(*tops)[16] = reinterpret_cast<float(*)[16]>(shared_rows + ROWS_BYTES);  // [4 waves][16 columns], then the masses
    float(*masses)[16] = tops + 4;
    if (kq == 0) tops[wave][n] = top, masses[wave][n] = mass;
    __syncthreads();  // the statistics are out, and every wave is done with its corner
    float largest = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; w++) largest = fmaxf(largest, tops[w][n]);
    const float mine = top == -INFINITY ? 0.0f : softmax_exp(top - largest) * (1.0f / 1024.0f);
#pragma unroll
    for (int d = 0; d < BLOCKS; d++)
        *reinterpret_cast<f32x4_t *>(&merged[wave][n][16 * d + 4 * kq]) = acc[d] * mine;
    __syncthreads();
    for (uint32_t index = tid; index < G * WIDTH; index += 256) {
        const uint32_t g = index / WIDTH, c = index % WIDTH;
        const float value = (merged[0][g][c] + merged[1][g][c]) + (merged[2][g][c] + merged[3][g][c]);
        float total = 0.0f, highest = -INFINITY;
        if (c == 0 || sections == 1) {
#pragma unroll
            for (int w = 0; w < 4; w++) highest = fmaxf(highest, tops[w][g]);
#pragma unroll
            for (int w = 0; w < 4; w++) total = fmaf(masses[w][g], tops[w][g] == -INFINITY ? 0.0f : softmax_exp(tops[w][g] - highest), total);
        }
        if (sections > 1) {
            float *dst = p.partial + (((uint64_t)unit * sections + section) * G + g) * (WIDTH + 2);
            dst[c] = value;
            if (c == 0) dst[WIDTH] = highest, dst[WIDTH + 1] = total;
        } else {
            const float normalized = total > 0.0f ? 1.0f / total : 0.0f;
            p.out[(uint64_t)(kvh * G + g) * p.o_sh + (uint64_t)b * p.o_sb + c] = value * normalized;
        }
    }
}

// ---------------------------------------------------------------- states of any element ------------------------------
//
// Keys and values held as single, bfloat16 (or half) numbers (Cache::new(.., element), crates/neura-decoder/src/cache.rs:130-134).
// One workgroup per (kv head, plane, row, section of the window), three plain passes over the section's keys: the scores of
// every (query head of the group, key) pair into LDS (a thread a pair, neighbouring threads the heads of one key, so a key
// row is fetched once and shared); a wave per query head for the largest score, the weights e^(score - largest) and their
// mass; a thread per (query head, channel) for the weighed sum of the value rows.  The section's sums leave in the layout
// attention_fold_kernel merges (or normalised, when one section covers the window).  fp32 throughout, no matrix cores: this
// is the form for elements the tile kernels do not read, built to be right rather than fast.
constexpr uint32_t ANY_KEYS = 256;  // keys a section holds at most: 16 query heads x 256 scores of LDS

template <int CE>
__global__ __launch_bounds__(256) void attention_any_kernel(AttentionParams p, uint32_t width) {
    fetch_parameters(p);
    __shared__ float scores[16 * ANY_KEYS];
    __shared__ float tops[16], masses[16];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t unit = blockIdx.x, section = blockIdx.y;
    const uint32_t row = unit % p.rows;
    const uint32_t b = (unit / p.rows) % p.batch, kvh = unit / p.rows / p.batch;
    const uint32_t G = p.groups;
    const uint32_t chunk = (p.keys + p.sections - 1u) / p.sections;
    const uint32_t begin = min(p.keys, section * chunk);
    const uint64_t plane = ((uint64_t)kvh * p.batch + b) * p.capacity;
    uint32_t origin = p.cursor ? p.cursor[b] : 0u;
    if (!p.reach && origin + p.rows > p.keys) {  // refusal::ORIGIN (attention.rs:250-252)
        if (tid == 0) atomicMax(p.refusal, (uint32_t)REFUSAL_ORIGIN);
        origin = p.keys - p.rows;
    }
    const uint32_t position = origin + row;
    const uint32_t visible = min(p.keys, p.reach ? origin + p.rows : position + 1u);
    const uint32_t last = min(visible, begin + chunk);
    const uint32_t n = last > begin ? last - begin : 0u;
    const Ring ring(p.keys, origin + p.rows, p.reach);
    // ---- scores
    for (uint32_t pair = tid; pair < n * G; pair += 256) {
        const uint32_t g = pair % G, key = begin + pair / G;
        float score = -INFINITY;
        if (!p.reach || ring.seen(key, position)) {
            const float *q = p.q + (uint64_t)(kvh * G + g) * p.q_sh + (uint64_t)b * p.q_sb + (uint64_t)row * p.q_sr;
            float total = 0.0f;
            for (uint32_t c = 0; c < width; c++) total = fmaf(q[c], cache_load<CE>(p.cache_k, (plane + key) * width + c), total);
            score = total * p.scale;
        }
        scores[g * ANY_KEYS + pair / G] = score;
    }
    __syncthreads();
    // ---- weights: wave w takes query heads w, w + 4, ...
    for (uint32_t g = wave; g < G; g += 4) {
        float top = -INFINITY;
        for (uint32_t k = lane; k < n; k += 64) top = fmaxf(top, scores[g * ANY_KEYS + k]);
        top = wave_max(top);
        float mass = 0.0f;
        for (uint32_t k = lane; k < n; k += 64) {
            const float score = scores[g * ANY_KEYS + k];
            const float weight = score == -INFINITY ? 0.0f : softmax_exp(score - top);
            scores[g * ANY_KEYS + k] = weight;
            mass += weight;
        }
        mass = wave_sum(mass);
        if (lane == 0) tops[g] = top, masses[g] = mass;
    }
    __syncthreads();
    // ---- values
    for (uint32_t index = tid; index < G * width; index += 256) {
        const uint32_t g = index / width, c = index % width;
        float value = 0.0f;
        for (uint32_t k = 0; k < n; k++) {
            const float weight = scores[g * ANY_KEYS + k];
            // a slot no query weighs may hold anything, and a weight of zero does not silence a NaN
            if (weight != 0.0f) value = fmaf(weight, cache_load<CE>(p.cache_v, (plane + begin + k) * width + c), value);
        }
        if (p.sections > 1) {
            float *dst = p.partial + (((uint64_t)unit * p.sections + section) * G + g) * (width + 2);
            dst[c] = value;
            if (c == 0) dst[width] = tops[g], dst[width + 1] = masses[g];
        } else {
            const float normalized = masses[g] > 0.0f ? 1.0f / masses[g] : 0.0f;
            p.out[(uint64_t)(kvh * G + g) * p.o_sh + (uint64_t)b * p.o_sb + (uint64_t)row * p.o_sr + c] = value * normalized;
        }
    }
}

// the fold with as many loads a thread as the sections ask for
template <typename... Args>
static void launch_fold(uint32_t sections, dim3 grid, dim3 block, size_t lds, hipStream_t stream, Args... args) {
    if (sections <= 32u) hipLaunchKernelGGL(attention_fold_kernel<4>, grid, block, lds, stream, args...);
    else if (sections <= 64u) hipLaunchKernelGGL(attention_fold_kernel<8>, grid, block, lds, stream, args...);
    else if (sections <= 128u) hipLaunchKernelGGL(attention_fold_kernel<16>, grid, block, lds, stream, args...);
    else hipLaunchKernelGGL(attention_fold_kernel<32>, grid, block, lds, stream, args...);
}

int32_t launch_attention(nh_device *d, const AttentionArgs &a) {
    AttentionParams p{};
    p.q = a.q, p.out = a.out;
    p.q_sh = a.q_sh, p.q_sb = a.q_sb, p.q_sr = a.q_sr, p.o_sh = a.o_sh, p.o_sb = a.o_sb, p.o_sr = a.o_sr;
    p.cache_k = a.cache_k, p.cache_v = a.cache_v;
    p.heads = a.heads, p.kv_heads = a.kv_heads, p.groups = a.heads / a.kv_heads;
    p.batch = a.batch, p.rows = a.rows, p.capacity = a.capacity, p.keys = a.keys;
    p.cursor = a.cursor, p.scale = a.scale, p.refusal = d->refusal, p.reach = a.reach;
    if (a.unmerged) *a.unmerged = SectionSums{nullptr, 0u, 0u, 0u};
    if (p.groups > (uint32_t)MAX_GROUPS) return fail(NH_E_ARGUMENT, "%u query heads share a key head where this kernel rides %d", p.groups, MAX_GROUPS);
    uint32_t units = a.kv_heads * a.batch * a.rows;
    if (!units) return NH_OK;
    if (a.cache_element != NH_F16 && a.cache_element != NH_F32 && a.cache_element != NH_BF16)
        return fail(NH_E_ARGUMENT, "a cache holds keys and values in single, half or bfloat16 storage, and element %d carries another grid", a.cache_element);
    // one query row a plane over single or bfloat16 states rides the matrix cores too (NEURA_HIP_ATTENTION_ANY=1: the plain fp32 kernel)
    const char *const asked = a.cache_element != NH_F16 ? getenv("NEURA_HIP_ATTENTION_ANY") : nullptr;  // read at every launch: the tests switch it
    const bool plain_states = asked && asked[0] == '1';
    const bool decode_tiles = a.rows == 1 && (a.width == 64 || a.width == 128) && p.groups <= 16 && ((uintptr_t)a.cache_k & 15u) == 0 &&
                              ((uintptr_t)a.cache_v & 15u) == 0 && ((uintptr_t)a.q & 15u) == 0 && a.q_sh % 4 == 0 && a.q_sb % 4 == 0;
    const bool fill_tiles = a.rows >= 4 && (a.width == 64 || a.width == 128) && p.groups >= 1 && ((uintptr_t)a.out & 15u) == 0 && a.o_sh % 4 == 0 &&
                            a.o_sb % 4 == 0 && a.o_sr % 4 == 0 && ((uintptr_t)a.cache_k & 15u) == 0 && ((uintptr_t)a.cache_v & 15u) == 0;
    if (a.cache_element != NH_F16 && (plain_states || !(decode_tiles || fill_tiles))) {
        if (p.groups > 16u) return fail(NH_E_ARGUMENT, "%u query heads share a key head where this kernel rides 16", p.groups);
        // sections of at most ANY_KEYS keys, enough of them to fill the device where the units alone do not
        uint32_t sections = (a.keys + ANY_KEYS - 1u) / ANY_KEYS;
        const uint32_t wanted = ((uint32_t)d->compute_units * 2u + units - 1u) / units, most = (a.keys + 31u) / 32u;
        if (sections < wanted) sections = wanted < most ? wanted : most;
        if (sections < 1u) sections = 1u;
        if (sections > 256u) return fail(NH_E_ARGUMENT, "a window of %u keys is more than 256 sections of %u", a.keys, ANY_KEYS);
        p.sections = sections;
        if (p.sections > 1) {
            p.partial = static_cast<float *>(scratch(d, (size_t)p.sections * a.heads * a.batch * a.rows * (a.width + 2) * sizeof(float)));
            if (!p.partial) return NH_E_MEMORY;
        }
        dim3 grid(units, p.sections);
        if (a.cache_element == NH_F32) hipLaunchKernelGGL(attention_any_kernel<NH_F32>, grid, dim3(256), 0, d->stream, p, a.width);
        else hipLaunchKernelGGL(attention_any_kernel<NH_BF16>, grid, dim3(256), 0, d->stream, p, a.width);
        NH_HIP(hipGetLastError());
        if (p.sections > 1) {
            launch_fold(p.sections, dim3(units * p.groups * ((a.width + 31) / 32)), dim3(256), 0, d->stream, p.partial, p.sections, p.groups, a.width, p);
            NH_HIP(hipGetLastError());
        }
        return NH_OK;
    }
    // a chunk of query rows goes to the matrix cores
    if (fill_tiles) {
        const uint32_t rows_per_wave = 32u / p.groups;
        dim3 grid(a.kv_heads * a.batch, (a.rows + 4u * rows_per_wave - 1u) / (4u * rows_per_wave));
        p.sections = 1;
        // two sets of waves a workgroup where the block's walk is long enough to be worth their meeting (four tiles and more);
        // NEURA_HIP_FILL_SPLIT=0 keeps one set
        static const bool split_wanted = [] { const char *v = getenv("NEURA_HIP_FILL_SPLIT"); return !(v && v[0] == '0'); }();
        const bool split = split_wanted && a.cache_element != NH_F32 && a.keys >= 128u;
#define FILL_TILE(WIDTH)                                                                                                                           \
    do {                                                                                                                                           \
        if (a.cache_element == NH_F16 && split) hipLaunchKernelGGL((attention_tile_kernel<WIDTH, NH_F16, true>), grid, dim3(512), 0, d->stream, p, rows_per_wave);   \
        else if (a.cache_element == NH_BF16 && split) hipLaunchKernelGGL((attention_tile_kernel<WIDTH, NH_BF16, true>), grid, dim3(512), 0, d->stream, p, rows_per_wave); \
        else if (a.cache_element == NH_F16) hipLaunchKernelGGL((attention_tile_kernel<WIDTH, NH_F16>), grid, dim3(256), 0, d->stream, p, rows_per_wave);   \
        else if (a.cache_element == NH_BF16) hipLaunchKernelGGL((attention_tile_kernel<WIDTH, NH_BF16>), grid, dim3(256), 0, d->stream, p, rows_per_wave); \
        else hipLaunchKernelGGL((attention_tile_kernel<WIDTH, NH_F32>), grid, dim3(256), 0, d->stream, p, rows_per_wave);                             \
    } while (0)
        if (a.width == 64) FILL_TILE(64);
        else FILL_TILE(128);
#undef FILL_TILE
        NH_HIP(hipGetLastError());
        return NH_OK;
    }
    // one query row a plane: the group's query heads are the columns of the matrix cores
    {
        const bool aligned = ((uintptr_t)a.cache_k & 15u) == 0 && ((uintptr_t)a.cache_v & 15u) == 0 && ((uintptr_t)a.q & 15u) == 0 && a.q_sh % 4 == 0 &&
                             a.q_sb % 4 == 0;
        const uint32_t planes = a.kv_heads * a.batch;
        if (aligned && a.rows == 1 && (a.width == 64 || a.width == 128) && p.groups <= 16) {
            // sections of at least 256 keys (two tiles a wave) where the planes alone fill the chip; where they do not (eight
            // planes and fewer: measured even at twelve, slower from sixteen on), of 64 (one tile of sixteen keys a wave);
            // enough workgroups to fill the chip twice over.  NEURA_HIP_ATTENTION_TK16=<planes> moves the line (0: never).
            static const uint32_t thin_below = [] { const char *v = getenv("NEURA_HIP_ATTENTION_TK16"); return v ? (uint32_t)atoi(v) : 12u; }();
            const bool thin = planes < thin_below;
            const uint32_t thinnest = thin ? 64u : planes >= 8 ? 256u : 128u;
            uint32_t wanted_sections = ((uint32_t)d->compute_units * 2 + planes - 1) / planes;
            const uint32_t most = (a.keys + thinnest - 1) / thinnest;
            p.sections = wanted_sections < 1 ? 1 : (wanted_sections > most ? most : wanted_sections);
            if (p.sections > 256) p.sections = 256;
            // the caller's next product merges the sections itself: no more of them than it takes, and only where sections that
            // few stay under 128 keys (two tiles a wave)
            const bool leave = a.unmerged && a.batch == 1 && thin && most <= 2u * MERGED_SECTIONS_MOST;
            if (leave && p.sections > MERGED_SECTIONS_MOST) p.sections = MERGED_SECTIONS_MOST;
            if (p.sections > 1) {
                p.partial = static_cast<float *>(scratch(d, (size_t)p.sections * a.heads * a.batch * (a.width + 2) * sizeof(float)));
                if (!p.partial) return NH_E_MEMORY;
            }
            dim3 grid(planes, p.sections);
            if (p.q_sh > UINT32_MAX || p.q_sb > UINT32_MAX || p.batch > 0xffffu) return fail(NH_E_ARGUMENT, "query strides and planes past what the decode attention takes");
            const uint32_t batch_groups = (p.batch << 16) | p.groups;
#define DECODE_TILE_OF(WIDTH, TK, CE)                                                                                                                            \
    hipLaunchKernelGGL((attention_decode_tile_kernel<WIDTH, TK, CE>), grid, dim3(256), 0, d->stream, p.cursor, p.q, p.cache_k, p.cache_v, (uint32_t)p.q_sh, \
                       (uint32_t)p.q_sb, p.keys, p.sections, p.capacity, batch_groups, p)
#define DECODE_TILE(WIDTH, TK)                                                                                                                                   \
    do {                                                                                                                                                         \
        if (a.cache_element == NH_F16) DECODE_TILE_OF(WIDTH, TK, NH_F16);                                                                                        \
        else if (a.cache_element == NH_BF16) DECODE_TILE_OF(WIDTH, TK, NH_BF16);                                                                                 \
        else DECODE_TILE_OF(WIDTH, TK, NH_F32);                                                                                                                  \
    } while (0)
            if (a.width == 64) {
                if (thin) DECODE_TILE(64, 16);
                else DECODE_TILE(64, 32);
            } else {
                if (thin) DECODE_TILE(128, 16);
                else DECODE_TILE(128, 32);
            }
#undef DECODE_TILE
#undef DECODE_TILE_OF
            NH_HIP(hipGetLastError());
            if (p.sections > 1 && leave) {
                *a.unmerged = SectionSums{p.partial, p.sections, p.groups, a.width};
            } else if (p.sections > 1) {
                launch_fold(p.sections, dim3(planes * p.groups * ((a.width + 31) / 32)), dim3(256), 0, d->stream, p.partial, p.sections, p.groups, a.width, p);
                NH_HIP(hipGetLastError());
            }
            return NH_OK;
        }
    }
    // sections of the context: enough workgroups to fill the chip four times over, none thinner
    // than 64 keys (thinner sections cost more in the fold than they gain in the walk)
    const uint32_t thinnest = 64u;
    uint32_t wanted = ((uint32_t)d->compute_units * 4 + units - 1) / units;
    uint32_t most = (a.keys + thinnest - 1) / thinnest;
    p.sections = wanted < 1 ? 1 : (wanted > most ? most : wanted);
    if (p.sections > 256) p.sections = 256;
    if (p.sections > 1) {
        p.partial = static_cast<float *>(scratch(d, (size_t)p.sections * a.heads * a.batch * a.rows * (a.width + 2) * sizeof(float)));
        if (!p.partial) return NH_E_MEMORY;
    }
    dim3 grid(units, p.sections), block(256);
    switch (a.width) {
    case 32: hipLaunchKernelGGL(attention_kernel<32>, grid, block, 0, d->stream, p); break;
    case 64: hipLaunchKernelGGL(attention_kernel<64>, grid, block, 0, d->stream, p); break;
    case 128: hipLaunchKernelGGL(attention_kernel<128>, grid, block, 0, d->stream, p); break;
    case 256: hipLaunchKernelGGL(attention_kernel<256>, grid, block, 0, d->stream, p); break;
    default: return fail(NH_E_ARGUMENT, "a head of %u numbers fits none of the widths 32, 64, 128, 256 this kernel walks", a.width);
    }
    NH_HIP(hipGetLastError());
    if (p.sections > 1) {
        launch_fold(p.sections, dim3(units * p.groups * ((a.width + 31) / 32)), dim3(256), 0, d->stream, p.partial, p.sections, p.groups, a.width, p);
        NH_HIP(hipGetLastError());
    }
    return NH_OK;
}

}  // namespace nh
