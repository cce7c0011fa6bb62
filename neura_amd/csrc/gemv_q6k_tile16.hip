// The Q6_K and Q3_K products of one activation row on 16-row tiles of the 16x16x64 integer MFMA: kernel and launcher.
// Built with the matrix-core results in vector registers (-amdgpu-mfma-vgpr-form).
#include "gemv_q6k_tile16.hpp"

namespace nh {

template <int NW, bool HANDED, bool SWIGLU = false, int ELEMENT = NH_Q6_K, bool ROPE = false>
__global__ __launch_bounds__(NW * 64) void gemv_q6k_tile16_kernel(const uint8_t *lead_w0, const void *lead_input, const float *lead_norm_w, uint32_t lead_row_bytes,
                                                                  uint32_t lead_grid, uint32_t lead_tiles, uint32_t lead_tile_rows, int32_t lead_to_w1, int32_t lead_to_w2,
                                                                  uint32_t lead_end0, uint32_t lead_end1, GemvParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t q6k_lds_bytes[];
    q6k_tile16_product<NW, HANDED, SWIGLU, ELEMENT, ROPE>(q6k_lds_bytes, blockIdx.x, lead_w0, lead_input, lead_norm_w, lead_row_bytes, lead_grid, lead_tiles, lead_tile_rows,
                                                          lead_to_w1, lead_to_w2, lead_end0, lead_end1, p);
}

// NEURA_HIP_Q6K_TILE16=0 keeps the kernel out (the staged kernel then takes Q6_K and Q3_K as before).  Otherwise it takes every such product
// of one row and one matrix that ends on a tile boundary (or a gate and an up matrix with SwiGLU), with no other epilogue than the
// residual or the cast of a value projection's rows into the value state: the head, ffn_down, attn_v and attn_output of a k-quant
// mix, gate|up of a file stored in Q6_K or Q3_K; or up to three matrices stacked with the rotation folded in (the q|k or q|k|v
// product of such a file).
bool q6k_tile16_takes(const GemvArgs &a) {
    if ((a.element != NH_Q6_K && a.element != NH_Q3_K) || a.rows != 1 || a.K % 256u != 0 || a.K == 0 || a.merge) return false;
    if (a.digits_out && (!a.swiglu || a.N % 512u != 0 || ((uintptr_t)a.digits_out & 63u))) return false;  // whole super-blocks of planes
    if (env_int("NEURA_HIP_Q6K_TILE16", 1) == 0) return false;
    auto stacked = [&a](int m) {  // a matrix behind the first is named by its distance from it in 16-byte units
        const int64_t apart = static_cast<const uint8_t *>(a.W[m]) - static_cast<const uint8_t *>(a.W[0]);
        return apart % 16 == 0 && apart / 16 <= INT32_MAX && apart / 16 >= INT32_MIN;
    };
    if (a.swiglu) {  // gate and up stacked: pairs of whole tiles, no other epilogue
        if (!a.W[1] || a.W[2] || a.residual || a.append_value || a.digits_in || a.rope || a.end[0] != a.N / 2u || a.N % 32u != 0 || !stacked(1)) return false;
    } else if (a.rope) {  // whole heads, every matrix ending on one; biases ride along
        const uint32_t width = a.rope->width;
        if (a.residual || a.append_value || a.digits_in || width < 16u || width % 16u != 0) return false;
        if (a.rope->q_rows % width || a.rope->k_rows % width || a.N % width || a.rope->q_rows > a.rope->k_rows || a.rope->k_rows > a.N) return false;
        if (a.end[0] % width || a.end[1] % width || a.end[2] != a.N) return false;
        if ((a.W[1] && !stacked(1)) || (a.W[2] && !stacked(2))) return false;
    } else if (a.W[1] || a.W[2] || a.end[0] != a.N) {
        return false;
    }
    if (a.append_value) {  // a value projection that casts its rows into the value state: whole heads, no other epilogue
        if (a.residual || a.digits_in || !a.append_value->width || a.N % a.append_value->width) return false;
    } else if (a.bias[0] && !a.rope) {
        return false;
    }
    if ((a.bias[1] || a.bias[2]) && !a.rope) return false;
    if (a.N < 16u || a.N % 16u != 0) return false;
    if (a.digits_in) {
        if (a.norm_w || ((uintptr_t)a.digits_in & 15u)) return false;
    } else if (((uintptr_t)a.x & 15u) || (a.norm_w && ((uintptr_t)a.norm_w & 15u))) {
        return false;
    }
    if ((uintptr_t)a.W[0] & 3u) return false;  // the first block on a 4-byte boundary: no load starts before the matrix
    const uint32_t nblk = a.K / 256u;
    return q6k_tile16_lds(nblk, nblk > 32u && !a.digits_in ? 16u : 8u) <= 160u * 1024u;
}

template <int NW, bool HANDED, bool SWIGLU = false, int ELEMENT = NH_Q6_K, bool ROPE = false>
static hipError_t launch_q6k_tile16_instance(nh_device *d, const GemvParams &p, uint32_t grid, size_t lds) {
    static bool raised = false;  // a workgroup may hold more than the default 64 KiB of LDS once the kernel says so
    if (!raised && lds > 64u * 1024u) {
        hipError_t error = hipFuncSetAttribute((const void *)gemv_q6k_tile16_kernel<NW, HANDED, SWIGLU, ELEMENT, ROPE>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (error != hipSuccess) return error;
        raised = true;
    }
    hipLaunchKernelGGL((gemv_q6k_tile16_kernel<NW, HANDED, SWIGLU, ELEMENT, ROPE>), dim3(grid), dim3(NW * 64), lds, d->stream, p.W[0],
                       HANDED ? static_cast<const void *>(p.digits_in) : static_cast<const void *>(p.x), p.norm_w, p.row_bytes, grid, p.row_groups,
                       ROPE ? p.rope_width : p.tile_rows, (int32_t)((p.W[1] - p.W[0]) / 16), (int32_t)((p.W[2] - p.W[0]) / 16), p.end[0], p.end[1], p);
    return hipGetLastError();
}

Q6kLaunch q6k_tile16_plan(nh_device *d, const GemvArgs &a) {
    Q6kLaunch plan{};
    GemvParams &p = plan.p;
    for (int s = 0; s < 3; s++) {
        p.W[s] = static_cast<const uint8_t *>(a.W[0]);
        p.end[s] = a.N;
    }
    if (a.swiglu) p.W[1] = static_cast<const uint8_t *>(a.W[1]), p.end[0] = a.N / 2u;
    if (a.rope) {
        for (int s = 0; s < 3; s++) {
            if (a.W[s]) p.W[s] = static_cast<const uint8_t *>(a.W[s]);
            p.end[s] = a.end[s], p.bias[s] = a.bias[s];
        }
        p.rope_cosines = a.rope->cosines, p.rope_sines = a.rope->sines, p.rope_cursor = a.rope->cursor, p.rope_k = a.rope->cache_k, p.rope_v = a.rope->cache_v;
        p.rope_width = a.rope->width, p.rope_q_rows = a.rope->q_rows, p.rope_k_rows = a.rope->k_rows, p.rope_capacity = a.rope->capacity;
        p.rope_positions = a.rope->positions, p.rope_ring = a.rope->ring, p.rope_element = a.rope->element, p.refusal = d->refusal;
    }
    p.x = a.x, p.y = a.y, p.residual = a.residual, p.norm_w = a.norm_w;
    p.N = a.N, p.K = a.K, p.eps = a.eps, p.rows = 1, p.swiglu = a.swiglu;
    p.digits_in = a.digits_in, p.digits_out = a.digits_out, p.tag_out = a.tag_out;
    if (a.append_value) {
        p.append_value = 1u, p.rope_v = a.append_value->cache_v, p.rope_cursor = a.append_value->cursor, p.rope_width = a.append_value->width;
        p.rope_capacity = a.append_value->capacity, p.rope_ring = a.append_value->ring, p.rope_element = a.append_value->element, p.bias[0] = a.bias[0], p.refusal = d->refusal;
    }
    p.row_bytes = (uint32_t)payload_bytes(a.element, a.K);
    p.nblk = a.K / 256u;
    // waves of a workgroup share a tile and split its super-blocks: about two steps a wave; sixteen on deep rows whose
    // activations the waves turn into digits themselves, eight where the digits arrive ready
    plan.waves = p.nblk <= 8u ? 4u : (p.nblk <= 14u ? 7u : (p.nblk <= 32u || a.digits_in ? 8u : 16u));
    // a tile holds the number of rows, 16 down to 12, that leaves the fewest compute units idle in the last round
    p.tile_rows = 16;
    auto idle = [&](uint32_t rows) {  // share of the rounds' slots left empty, in 1/65536
        const uint32_t tiles = a.N / rows, rounds = (tiles + (uint32_t)d->compute_units - 1u) / (uint32_t)d->compute_units;
        return 65536u - (uint32_t)((uint64_t)tiles * 65536u / ((uint64_t)rounds * (uint32_t)d->compute_units));
    };
    for (uint32_t rows = 15; rows >= 12 && !a.swiglu && !a.rope; rows--) {
        if (a.N % rows) continue;
        if (idle(rows) + 3277u < idle(p.tile_rows)) p.tile_rows = rows;
    }
    const uint32_t units = a.swiglu ? a.N / 32u : a.N / p.tile_rows;
    p.row_groups = units;
    const uint32_t rounds = (units + (uint32_t)d->compute_units - 1u) / (uint32_t)d->compute_units;
    plan.grid = (units + rounds - 1u) / rounds;
    plan.lds = q6k_tile16_lds(p.nblk, plan.waves);
    return plan;
}

template <int ELEMENT>
static hipError_t launch_q6k_tile16_of(nh_device *d, const GemvArgs &a, const Q6kLaunch &plan) {
    const GemvParams &p = plan.p;
    const uint32_t waves = plan.waves, grid = plan.grid;
    const size_t lds = plan.lds;
    if (a.rope) {
        return waves == 4u   ? launch_q6k_tile16_instance<4, false, false, ELEMENT, true>(d, p, grid, lds)
               : waves == 7u ? launch_q6k_tile16_instance<7, false, false, ELEMENT, true>(d, p, grid, lds)
               : waves == 8u ? launch_q6k_tile16_instance<8, false, false, ELEMENT, true>(d, p, grid, lds)
                             : launch_q6k_tile16_instance<16, false, false, ELEMENT, true>(d, p, grid, lds);
    }
    if (a.swiglu) {
        return waves == 4u   ? launch_q6k_tile16_instance<4, false, true, ELEMENT>(d, p, grid, lds)
               : waves == 7u ? launch_q6k_tile16_instance<7, false, true, ELEMENT>(d, p, grid, lds)
               : waves == 8u ? launch_q6k_tile16_instance<8, false, true, ELEMENT>(d, p, grid, lds)
                             : launch_q6k_tile16_instance<16, false, true, ELEMENT>(d, p, grid, lds);
    }
    if (a.digits_in) {
        return waves == 4u   ? launch_q6k_tile16_instance<4, true, false, ELEMENT>(d, p, grid, lds)
               : waves == 7u ? launch_q6k_tile16_instance<7, true, false, ELEMENT>(d, p, grid, lds)
                             : launch_q6k_tile16_instance<8, true, false, ELEMENT>(d, p, grid, lds);
    }
    return waves == 4u   ? launch_q6k_tile16_instance<4, false, false, ELEMENT>(d, p, grid, lds)
           : waves == 7u ? launch_q6k_tile16_instance<7, false, false, ELEMENT>(d, p, grid, lds)
           : waves == 8u ? launch_q6k_tile16_instance<8, false, false, ELEMENT>(d, p, grid, lds)
                         : launch_q6k_tile16_instance<16, false, false, ELEMENT>(d, p, grid, lds);
}

int32_t launch_q6k_tile16(nh_device *d, const GemvArgs &a) {
    const Q6kLaunch plan = q6k_tile16_plan(d, a);
    profile_mark(d);
    NH_HIP(a.element == NH_Q3_K ? launch_q6k_tile16_of<NH_Q3_K>(d, a, plan) : launch_q6k_tile16_of<NH_Q6_K>(d, a, plan));
    profile_mark(d);
    if (d->profile) d->profile_bytes += (uint64_t)a.N * plan.p.row_bytes;
    return NH_OK;
}

}  // namespace nh
