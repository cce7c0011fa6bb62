// The decoder: the hand-scheduled kernel sequence that stands where the reference compiles
// its answer / fill / reset programs, and the C ABI operator entry points.
#include "common.hpp"

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <vector>

using namespace nh;

struct nh_model {
    nh_device *d = nullptr;
    nh_weights *weights = nullptr;
    nh_model_config c{};
    int32_t element = 0;
    uint32_t capacity = 0, window = 0;
    uint32_t positions = 0;  // rows of the rotation's tables: every position a cursor can name
    bool ring = false;       // the window is a ring (a bounded batch, crates/neura-generate/src/batch.rs:313-325)
    const uint8_t *token_embd = nullptr, *output = nullptr;
    const float *output_norm = nullptr;
    std::vector<const float *> attn_norm, ffn_norm;
    std::vector<const uint8_t *> attn_q, attn_k, attn_v, attn_o, ffn_gate, ffn_up, ffn_down;
    // the element of every matrix: [token_embd, output, then per layer q, k, v, o, gate, up, down]
    std::vector<int32_t> elements;
    std::vector<const float *> bias_q, bias_k, bias_v;  // per layer, nullptr where a projection has none
    std::vector<uint8_t *> cache_k, cache_v;  // numbers of c.cache_element, `eb` bytes each
    size_t cache_elements = 0;  // per layer and per K or V
    size_t eb = 2;
    // the shared prefix (Cache::with_shared, crates/neura-decoder/src/cache.rs:138-161): one plane per layer,
    // [kv_heads][1][capacity][head_dim], allocated when a prefix is first kept
    std::vector<uint8_t *> shared_k, shared_v;
    // activations; T = rows * batch flattened token rows, t = row * batch + plane
    float *h = nullptr, *xn = nullptr, *qkv = nullptr, *att = nullptr, *act = nullptr, *up = nullptr, *logits = nullptr;
    float *rope_cos = nullptr, *rope_sin = nullptr;  // [capacity][head_dim / 2], for the rotation folded into the q|k|v product
    uint32_t *inputs_dev = nullptr;  // [tokens T_max | cursors B | draws B x 4 words | mask bytes B]
    uint32_t *chosen_dev = nullptr;
    uint8_t *inputs_host = nullptr;  // pinned mirror of inputs_dev
    uint32_t *chosen_host = nullptr; // pinned [B + 1]: chosen tokens, then the refusal word
    uint32_t *chosen_mapped = nullptr;  // the same words as the device addresses them: a step's last kernel writes them there
    uint32_t max_tokens = 0;
    // the decode step captured as a HIP graph: [0] all planes active, [1] some plane masked, [2], [3] the same with a sampled choice
    hipGraphExec_t decode_graph[4] = {nullptr, nullptr, nullptr, nullptr};
    uint64_t graph_moved[4] = {0, 0, 0, 0};  // nh_device::moved when each graph was recorded
    bool graph_warmed[4] = {false, false, false, false};  // the variant has run once outside a capture
    bool use_graph = true;
    // Dependent products of a decode step as one launch with seams between them (launch_chain) until a seam's wait runs out
    // once: the step is then run again one launch a product, and so is every later one.
    bool chain = true;
    uint32_t chain_spin = 1u << 18;  // times a reader at a seam may read a stale piece again (NEURA_HIP_CHAIN_SPIN)
    uint2 *pairs = nullptr;          // [hidden] (value, tag): the residual stream as a chained launch hands it from product to product
    uint32_t seam_fallbacks = 0;     // steps run again because a seam gave up
};

namespace {

// whether rocprofv3 launched this process: it names its tool library in the environment of what it runs
bool traced_by_rocprofiler() {
    const char *tools = getenv("ROCP_TOOL_LIBRARIES");
    if (tools && tools[0]) return true;
    const char *preloaded = getenv("LD_PRELOAD");
    return preloaded && strstr(preloaded, "rocprofiler-sdk") != nullptr;
}

uint32_t qkv_width(const nh_model *m) { return (m->c.heads + 2 * m->c.kv_heads) * m->c.head_dim; }

void release(nh_model *m) {
    if (!m) return;
    (void)hipStreamSynchronize(m->d->stream);
    for (hipGraphExec_t graph : m->decode_graph)
        if (graph) (void)hipGraphExecDestroy(graph);
    for (auto p : m->cache_k) (void)hipFree(p);
    for (auto p : m->cache_v) (void)hipFree(p);
    for (auto p : m->shared_k) (void)hipFree(p);
    for (auto p : m->shared_v) (void)hipFree(p);
    float *buffers[] = {m->h, m->xn, m->qkv, m->att, m->act, m->up, m->logits, m->rope_cos, m->rope_sin};
    for (float *p : buffers)
        if (p) (void)hipFree(p);
    if (m->pairs) (void)hipFree(m->pairs);
    if (m->inputs_dev) (void)hipFree(m->inputs_dev);
    if (m->chosen_dev) (void)hipFree(m->chosen_dev);
    if (m->inputs_host) (void)hipHostFree(m->inputs_host);
    if (m->chosen_host) (void)hipHostFree(m->chosen_host);
    delete m;
}

template <typename T>
bool device_array(T *&out, size_t count) {
    void *held = nullptr;
    if (hipMalloc(&held, (count ? count : 1) * sizeof(T)) != hipSuccess) return false;
    out = static_cast<T *>(held);
    return true;
}

// writes tokens / cursors / draws / mask through the pinned staging buffer in one copy
int32_t stage_inputs(nh_model *m, const uint32_t *tokens, uint32_t count, const uint32_t *cursors, const uint8_t *mask, uint32_t batch,
                     const nh_draw *draws = nullptr) {
    static_assert(sizeof(nh_draw) == 16, "a draw is four words");
    uint32_t *words = reinterpret_cast<uint32_t *>(m->inputs_host);
    memcpy(words, tokens, (size_t)count * 4);
    memcpy(words + m->max_tokens, cursors, (size_t)batch * 4);
    if (draws) memcpy(words + m->max_tokens + batch, draws, (size_t)batch * sizeof(nh_draw));
    uint8_t *mask_bytes = reinterpret_cast<uint8_t *>(words + m->max_tokens + 5 * (size_t)batch);
    for (uint32_t b = 0; b < batch; b++) mask_bytes[b] = mask ? (mask[b] ? 1 : 0) : 1;
    size_t bytes = ((size_t)m->max_tokens + 5 * (size_t)batch) * 4 + batch;
    NH_HIP(hipMemcpyAsync(m->inputs_dev, m->inputs_host, bytes, hipMemcpyHostToDevice, m->d->stream));
    return NH_OK;
}

const uint32_t *dev_tokens(const nh_model *m) { return m->inputs_dev; }
const uint32_t *dev_cursor(const nh_model *m) { return m->inputs_dev + m->max_tokens; }
const nh_draw *dev_draws(const nh_model *m) { return reinterpret_cast<const nh_draw *>(m->inputs_dev + m->max_tokens + m->c.batch); }
const uint8_t *dev_mask(const nh_model *m) { return reinterpret_cast<const uint8_t *>(m->inputs_dev + m->max_tokens + 5 * (size_t)m->c.batch); }

enum { EMBD = 0, HEAD = 1, Q = 0, K_ = 1, V = 2, O = 3, GATE = 4, UP = 5, DOWN = 6 };
int32_t element_at(const nh_model *m, uint32_t layer, int which) { return m->elements[2 + 7 * layer + which]; }

GemvArgs narrow(const nh_model *m, int32_t element, const uint8_t *W, uint32_t N, uint32_t K, const float *x, uint32_t rows, float *y) {
    GemvArgs a{};
    a.element = element;
    a.W[0] = W, a.W[1] = nullptr, a.W[2] = nullptr;
    a.end[0] = a.end[1] = a.end[2] = N;
    a.N = N, a.K = K, a.x = x, a.rows = rows, a.y = y;
    return a;
}

// all layers over T = rows * batch token rows whose inputs are already staged on the device
int32_t forward(nh_model *m, uint32_t rows, bool any_inactive, bool products_only = false) {
    nh_device *d = m->d;
    const nh_model_config &c = m->c;
    const uint32_t B = c.batch, T = rows * B, H = c.hidden, hd = c.head_dim;
    const uint32_t QW = c.heads * hd, KW = c.kv_heads * hd, QKV = QW + 2 * KW, F = c.ffn;
    const uint8_t *mask = any_inactive ? dev_mask(m) : nullptr;
    const bool wide = T > 8;  // more rows than the narrow product takes
    int32_t status;
    const bool chains = m->chain && T == 1 && !mask && gemv_chain_level() > 0;
    // what one product of a chained launch hands another carries tag words that name the pass: the device's tick moves on
    // before any is written
    if (chains && (status = launch_tick(d)) != NH_OK) return status;
    if (!products_only && (status = launch_gather(d, m->elements[EMBD], m->token_embd, c.vocab, H, dev_tokens(m), T, B, mask, m->h)) != NH_OK)
        return status;
    const float scale = 1.0f / sqrtf((float)hd);
    for (uint32_t L = 0; L < c.layers; L++) {
        bool roped = false;
        if (wide) {
            const uint8_t *mats[3] = {m->attn_q[L], m->attn_k[L], m->attn_v[L]};
            const float *biases[3] = {m->bias_q[L], m->bias_k[L], m->bias_v[L]};
            const uint32_t widths[3] = {QW, KW, KW};
            const bool alike = element_at(m, L, Q) == element_at(m, L, K_) && element_at(m, L, Q) == element_at(m, L, V);
            const bool stacked = alike && gemm_stacks(element_at(m, L, Q), H, m->h, mats[0], mats[1], mats[2], QW, QW + KW);
            uint32_t column = 0;
            if (!stacked && (status = launch_rmsnorm(d, m->h, nullptr, m->attn_norm[L], c.eps, T, H, m->xn, nullptr)) != NH_OK) return status;
            if (stacked) {
                // q|k|v as one product (the key and value projections alone are a few dozen workgroups each), the norm
                // done by the pass that packs the rows
                GemmArgs g{element_at(m, L, Q), mats[0], QKV, H, m->h, NH_F32, T, m->qkv, nullptr, QKV};
                g.W_more[0] = mats[1], g.W_more[1] = mats[2], g.end[0] = QW, g.end[1] = QW + KW;
                g.norm_w = m->attn_norm[L], g.eps = c.eps;
                if ((status = launch_gemm(d, g)) != NH_OK) return status;
                for (int s = 0; s < 3; s++) {
                    if (biases[s] && (status = launch_columns(d, m->qkv + column, QKV, biases[s], m->qkv + column, QKV, T, widths[s])) != NH_OK) return status;
                    column += widths[s];
                }
            } else {
                for (int s = 0; s < 3; s++) {
                    GemmArgs g{element_at(m, L, Q + s), mats[s], widths[s], H, m->xn, NH_F32, T, m->qkv + column, nullptr, QKV};
                    if ((status = launch_gemm(d, g)) != NH_OK) return status;
                    if (biases[s] && (status = launch_columns(d, m->qkv + column, QKV, biases[s], m->qkv + column, QKV, T, widths[s])) != NH_OK) return status;
                    column += widths[s];
                }
            }
        } else {
            const bool biased = m->bias_q[L] || m->bias_k[L] || m->bias_v[L];
            const bool alike = element_at(m, L, Q) == element_at(m, L, K_) && element_at(m, L, Q) == element_at(m, L, V);
            GemvArgs a = narrow(m, element_at(m, L, Q), m->attn_q[L], QKV, H, m->h, T, m->qkv);
            a.W[1] = m->attn_k[L], a.W[2] = m->attn_v[L];
            a.end[0] = QW, a.end[1] = QW + KW, a.end[2] = QKV;
            a.norm_w = m->attn_norm[L], a.eps = c.eps;
            // one token of one active plane: the rotation, the biases and the cache append ride in the product's epilogue
            // (the epilogue casts what it appends into the states' element)
            const bool halves = true;
            RopeFusion rope{m->rope_cos, m->rope_sin, dev_cursor(m), reinterpret_cast<uint16_t *>(m->cache_k[L]), reinterpret_cast<uint16_t *>(m->cache_v[L]),
                            hd, QW, QW + KW, m->capacity, m->positions, m->ring ? m->window : 0u, c.cache_element};
            // (five to eight planes of one token each: the same from the product of the 32-row tiles, every plane at its own cursor)
            if (halves && alike && !products_only && rows == 1 && !mask && gemv_fuses_rope(a, rope)) {
                a.rope = &rope;
                a.bias[0] = m->bias_q[L], a.bias[1] = m->bias_k[L], a.bias[2] = m->bias_v[L];
                roped = true;
            }
            // the same with a value projection stored otherwise (a Q4_K_M file keeps some in Q6_K): q|k go out rotated from
            // one product, the value row follows from its own product through a small append
            GemvArgs qk = narrow(m, element_at(m, L, Q), m->attn_q[L], QW + KW, H, m->h, T, m->qkv);
            qk.W[1] = m->attn_k[L];
            qk.end[0] = QW, qk.end[1] = QW + KW, qk.end[2] = QW + KW;
            qk.norm_w = m->attn_norm[L], qk.eps = c.eps;
            RopeFusion rope_qk = rope;
            const bool split_value = halves && !alike && element_at(m, L, Q) == element_at(m, L, K_) && !products_only && T == 1 && !mask &&
                                     gemv_fuses_rope(qk, rope_qk);
            if (roped || (alike && (!biased || products_only))) {
                if ((status = launch_gemv(d, a)) != NH_OK) return status;
            } else if (split_value) {
                qk.rope = &rope_qk;
                qk.bias[0] = m->bias_q[L], qk.bias[1] = m->bias_k[L];
                GemvArgs value = narrow(m, element_at(m, L, V), m->attn_v[L], KW, H, m->h, T, m->xn);
                value.norm_w = m->attn_norm[L], value.eps = c.eps;
                // a K-quant product on the tiles (or on the staged kernel, of one K slice) casts its rows into the value state itself;
                // others leave that to a small kernel
                value.append_value = &rope_qk, value.bias[0] = m->bias_v[L];
                const bool appends = gemv_appends_value(value) && !(getenv("NEURA_HIP_APPEND_VALUE") && getenv("NEURA_HIP_APPEND_VALUE")[0] == '0');
                if (!appends) value.append_value = nullptr, value.bias[0] = nullptr;
                if (gemv_pairs(d, qk, value)) {  // both in one launch: neither waits for the other
                    if ((status = launch_gemv_pair(d, qk, value)) != NH_OK) return status;
                } else {
                    if ((status = launch_gemv(d, qk)) != NH_OK) return status;
                    if ((status = launch_gemv(d, value)) != NH_OK) return status;
                }
                if (!appends && (status = launch_value_append(d, m->xn, m->bias_v[L], m->cache_v[L], c.kv_heads, hd, m->capacity, dev_cursor(m),
                                                              m->ring ? m->window : 0u, c.cache_element)) != NH_OK)
                    return status;
                roped = true;
            } else {
                // matrices of different elements, or biases outside the folded rotation: one product each, placed side by side
                const uint8_t *mats[3] = {m->attn_q[L], m->attn_k[L], m->attn_v[L]};
                const float *biases[3] = {m->bias_q[L], m->bias_k[L], m->bias_v[L]};
                const uint32_t widths[3] = {QW, KW, KW};
                uint32_t column = 0;
                for (int s = 0; s < 3; s++) {
                    GemvArgs one = narrow(m, element_at(m, L, Q + s), mats[s], widths[s], H, m->h, T, m->xn);
                    one.norm_w = m->attn_norm[L], one.eps = c.eps;
                    if ((status = launch_gemv(d, one)) != NH_OK) return status;
                    if ((status = launch_columns(d, m->xn, widths[s], products_only ? nullptr : biases[s], m->qkv + column, QKV, T, widths[s])) != NH_OK) return status;
                    column += widths[s];
                }
            }
        }
        if (!products_only && !roped && (status = launch_rope_append(d, m->qkv, c.heads, c.kv_heads, hd, B, rows, m->cache_k[L], m->cache_v[L],
                                                           m->capacity, m->window, dev_cursor(m), mask, c.rope_base, m->ring, c.cache_element, m->rope_cos, m->rope_sin,
                                                           m->positions)) != NH_OK)
            return status;
        AttentionArgs at{};
        at.q = m->qkv, at.out = m->att;
        at.q_sh = hd, at.q_sb = QKV, at.q_sr = (uint64_t)B * QKV;
        at.o_sh = hd, at.o_sb = QW, at.o_sr = (uint64_t)B * QW;
        at.cache_k = reinterpret_cast<const uint16_t *>(m->cache_k[L]), at.cache_v = reinterpret_cast<const uint16_t *>(m->cache_v[L]);
        at.cache_element = c.cache_element;
        at.heads = c.heads, at.kv_heads = c.kv_heads, at.batch = B, at.rows = rows, at.width = hd;
        at.capacity = m->capacity, at.keys = m->window, at.cursor = dev_cursor(m), at.scale = scale;
        at.reach = m->ring ? m->window : 0u;
        // one row through a product that merges the attention's sections as it stages its row: the attention leaves them unmerged
        SectionSums sums{};
        GemvArgs o{};
        if (!wide) {
            o = narrow(m, element_at(m, L, O), m->attn_o[L], H, QW, m->att, T, m->h);
            o.residual = m->h;
            if (gemv_merges_sections(o, hd)) at.unmerged = &sums;
        }
        if (!products_only && (status = launch_attention(d, at)) != NH_OK) return status;
        if (wide) {
            GemmArgs o{element_at(m, L, O), m->attn_o[L], H, QW, m->att, NH_F32, T, m->h, m->h, H};
            if ((status = launch_gemm(d, o)) != NH_OK) return status;
            // where the matrix cores take both projections the norm rides in the pass that packs the rows for the gate
            // projection, and the up projection multiplies those same packed rows
            const bool paired = element_at(m, L, GATE) == element_at(m, L, UP) &&
                                gemm_stacks(element_at(m, L, GATE), H, m->h, m->ffn_gate[L], nullptr, nullptr, 0, 0) &&
                                gemm_stacks(element_at(m, L, UP), H, m->h, m->ffn_up[L], nullptr, nullptr, 0, 0);
            if (!paired && (status = launch_rmsnorm(d, m->h, nullptr, m->ffn_norm[L], c.eps, T, H, m->xn, nullptr)) != NH_OK) return status;
            GemmArgs g{element_at(m, L, GATE), m->ffn_gate[L], F, H, paired ? m->h : m->xn, NH_F32, T, m->act, nullptr, F};
            GemmArgs u{element_at(m, L, UP), m->ffn_up[L], F, H, paired ? m->h : m->xn, NH_F32, T, m->up, nullptr, F};
            if (paired) g.norm_w = m->ffn_norm[L], g.eps = c.eps, u.packed = true;
            if ((status = launch_gemm(d, g)) != NH_OK) return status;
            if ((status = launch_gemm(d, u)) != NH_OK) return status;
            // silu(gate) * up is formed as the down projection packs its rows, or by a kernel of its own
            const bool gated = gemm_stacks(element_at(m, L, DOWN), F, m->up, m->ffn_down[L], nullptr, nullptr, 0, 0);
            if (!gated && (status = launch_silu_mul(d, m->act, m->up, (uint64_t)T * F, m->act)) != NH_OK) return status;
            GemmArgs dn{element_at(m, L, DOWN), m->ffn_down[L], H, F, gated ? m->up : m->act, NH_F32, T, m->h, m->h, H};
            if (gated) dn.gate = m->act;
            if ((status = launch_gemm(d, dn)) != NH_OK) return status;
        } else {
            if (sums.sections) o.merge = &sums;
            GemvArgs dn = narrow(m, element_at(m, L, DOWN), m->ffn_down[L], H, F, m->act, T, m->h);
            dn.residual = m->h;
            bool chained = false;
            const uint32_t seam = 1u + 4u * (L % 31u);  // the numbers of this layer's seams: seam (h), seam + 1 (digit planes), ...
            if (chains && !o.merge && element_at(m, L, GATE) == element_at(m, L, UP)) {
                GemvArgs gu = narrow(m, element_at(m, L, GATE), m->ffn_gate[L], 2 * F, H, m->h, T, m->act);
                gu.W[1] = m->ffn_up[L];
                gu.end[0] = F, gu.end[1] = gu.end[2] = 2 * F;
                gu.swiglu = 1, gu.norm_w = m->ffn_norm[L], gu.eps = c.eps;
                if (gemv_hands_digits(gu, dn) && gemv_digit_bytes(F) <= (size_t)F * sizeof(float)) {
                    gu.digits_out = reinterpret_cast<uint8_t *>(m->up), dn.digits_in = reinterpret_cast<const uint8_t *>(m->up);
                    gu.tag_out = dn.tag_in = seam + 1u;
                    // with attn_output in front, gate|up reads the residual stream as the pairs attn_output leaves beside it
                    GemvArgs lead = o, behind = gu;
                    lead.pairs_out = m->pairs, lead.tag_out = seam;
                    behind.x = reinterpret_cast<const float *>(m->pairs), behind.tag_in = seam;
                    if (gemv_chains(d, &lead, behind, dn, nullptr)) {
                        if ((status = launch_chain(d, &lead, behind, dn, nullptr, m->chain_spin)) != NH_OK) return status;
                        chained = true;
                    } else if (gemv_chains(d, nullptr, gu, dn, nullptr)) {
                        if ((status = launch_gemv(d, o)) != NH_OK) return status;
                        if ((status = launch_chain(d, nullptr, gu, dn, nullptr, m->chain_spin)) != NH_OK) return status;
                        chained = true;
                    }
                    dn.digits_in = nullptr, dn.tag_in = 0;
                }
            }
            if (chained) continue;
            if ((status = launch_gemv(d, o)) != NH_OK) return status;
            if (element_at(m, L, GATE) == element_at(m, L, UP)) {
                GemvArgs gu = narrow(m, element_at(m, L, GATE), m->ffn_gate[L], 2 * F, H, m->h, T, m->act);
                gu.W[1] = m->ffn_up[L];
                gu.end[0] = F, gu.end[1] = gu.end[2] = 2 * F;
                gu.swiglu = 1, gu.norm_w = m->ffn_norm[L], gu.eps = c.eps;
                // one row: silu(gate) * up goes to the down projection as the digit planes it multiplies (they fit the up
                // projection's idle buffer), not as floats it would turn into digits again
                if (gemv_hands_digits(gu, dn) && gemv_digit_bytes(F) <= (size_t)F * sizeof(float))
                    gu.digits_out = reinterpret_cast<uint8_t *>(m->up), dn.digits_in = reinterpret_cast<const uint8_t *>(m->up), gu.tag_out = dn.tag_in = seam + 1u;
                if ((status = launch_gemv(d, gu)) != NH_OK) return status;
            } else {
                GemvArgs g = narrow(m, element_at(m, L, GATE), m->ffn_gate[L], F, H, m->h, T, m->act);
                GemvArgs u = narrow(m, element_at(m, L, UP), m->ffn_up[L], F, H, m->h, T, m->up);
                g.norm_w = u.norm_w = m->ffn_norm[L], g.eps = u.eps = c.eps;
                if ((status = launch_gemv(d, g)) != NH_OK) return status;
                if ((status = launch_gemv(d, u)) != NH_OK) return status;
                if ((status = launch_silu_mul(d, m->act, m->up, (uint64_t)T * F, m->act)) != NH_OK) return status;
            }
            if ((status = launch_gemv(d, dn)) != NH_OK) return status;
        }
        if (!products_only && mask && (status = launch_mask_rows(d, m->h, rows, B, H, mask)) != NH_OK) return status;
    }
    return NH_OK;
}

__global__ __launch_bounds__(64) void publish_kernel(const uint32_t *chosen, const uint32_t *refusal, uint32_t batch, uint32_t *host) {
    for (uint32_t i = threadIdx.x; i <= batch; i += 64u) host[i] = i < batch ? chosen[i] : *refusal;
}

// every kernel of one decode step: the layers, then logits = rms(hidden) . head^T and the greedy
// choice (examples/qwen/model.rs:81-84, crates/neura-generate/src/sampling.rs:69-71)
int32_t decode_kernels(nh_model *m, bool any_inactive, bool sampled) {
    int32_t status;
    if ((status = forward(m, 1, any_inactive)) != NH_OK) return status;
    GemvArgs head = narrow(m, m->output == m->token_embd ? m->elements[EMBD] : m->elements[HEAD], m->output, m->c.vocab, m->c.hidden, m->h, m->c.batch, m->logits);
    head.norm_w = m->output_norm, head.eps = m->c.eps;
    if ((status = launch_gemv(m->d, head)) != NH_OK) return status;
    // the choices and the refusal word go to the host's pinned words from a kernel of the step (part of the recorded graph): the
    // two device-to-host copies they would otherwise take are two more operations behind every step.  The greedy choice's
    // last kernel writes them itself; a sampled step has a kernel for it.
    if (!sampled) return launch_argmax(m->d, m->logits, m->c.batch, m->c.vocab, m->chosen_dev, m->chosen_mapped, m->d->refusal);
    status = launch_sample(m->d, m->logits, m->c.batch, m->c.vocab, dev_draws(m), m->chosen_dev);
    if (status != NH_OK || !m->chosen_mapped) return status;
    hipLaunchKernelGGL(publish_kernel, dim3(1), dim3(64), 0, m->d->stream, m->chosen_dev, m->d->refusal, m->c.batch, m->chosen_mapped);
    NH_HIP(hipGetLastError());
    return NH_OK;
}

}  // namespace

extern "C" {

nh_model *nh_model_create(nh_device *device, const nh_model_config *config, nh_weights *weights, const nh_tensor_table *table) {
    if (!device || !config || !weights || !table) {
        fail(NH_E_ARGUMENT, "a model names no device, config, arena or tensor table");
        return nullptr;
    }
    const nh_model_config &c = *config;
    if (c.cache_element != NH_F16 && c.cache_element != NH_BF16 && c.cache_element != NH_F32) {  // crates/neura-decoder/src/cache.rs:130-134
        fail(NH_E_ARGUMENT, "a cache holds keys and values in single, half or bfloat16 storage, and element %d carries another grid", c.cache_element);
        return nullptr;
    }
    if (!c.layers || !c.hidden || !c.heads || !c.kv_heads || !c.head_dim || !c.ffn || !c.vocab || !c.context || !c.batch ||
        c.heads % c.kv_heads || c.head_dim % 8) {
        fail(NH_E_ARGUMENT, "a decoder of %u layers, %u hidden, %u/%u heads of %u, %u ffn, %u vocab, %u context, %u planes holds no model",
             c.layers, c.hidden, c.heads, c.kv_heads, c.head_dim, c.ffn, c.vocab, c.context, c.batch);
        return nullptr;
    }
    std::vector<int32_t> elements(2 + 7 * (size_t)c.layers, table->matrix_element);
    if (table->matrix_elements) elements.assign(table->matrix_elements, table->matrix_elements + elements.size());
    for (int32_t element : elements) {
        if (element != NH_Q8_0 && element != NH_Q4_K && !staged_super_block(element)) {
            fail(NH_E_ARGUMENT, "a decoder multiplies Q8_0, Q3_K, Q4_K, Q5_K or Q6_K matrices, and this table names element %d", element);
            return nullptr;
        }
        uint32_t block = block_elements(element);
        if (c.hidden % block || c.ffn % block || (c.heads * c.head_dim) % block) {
            fail(NH_E_ARGUMENT, "rows of %u, %u and %u numbers are not whole blocks of %u", c.hidden, c.ffn, c.heads * c.head_dim, block);
            return nullptr;
        }
    }
    if (!(c.rope_base > 1.0f) || !std::isfinite(c.rope_base)) {  // refusal::KNOB, crates/neura-kernel/src/task/rope.rs:33-36
        fail(NH_E_ARGUMENT, "a rope base of %f turns nothing", (double)c.rope_base);
        return nullptr;
    }
    // crates/neura-generate/src/batch.rs:315-322
    if (c.window > c.context) {
        fail(NH_E_ARGUMENT, "a batch keeps a window of %u tokens over a context of %u", c.window, c.context);
        return nullptr;
    }
    // states of another element than half are read by the plain attention kernel, in at most 256 sections of 256 keys, and
    // by more than 16 query heads a key head not at all: refused here, not at the first step
    if (c.cache_element != NH_F16 && ((c.window ? c.window : c.context) > 256u * 256u || c.heads / c.kv_heads > 16u)) {
        fail(NH_E_ARGUMENT, "single and bfloat16 states are attended over at most %u keys by at most 16 query heads a key head, not %u keys by %u",
             256u * 256u, c.window ? c.window : c.context, c.heads / c.kv_heads);
        return nullptr;
    }
    if (c.window && (c.max_rows ? c.max_rows : 1u) > c.window) {
        fail(NH_E_ARGUMENT, "a batch fills chunks of %u rows into a window of %u tokens", c.max_rows, c.window);
        return nullptr;
    }
    nh_model *m = new nh_model();
    m->d = device, m->weights = weights, m->c = c, m->element = table->matrix_element;
    m->elements = elements;
    uint32_t widest = c.max_rows ? c.max_rows : 1;
    m->ring = c.window != 0;                          // BatchSpec::window names one: the caches are rings of it
    m->window = c.window ? c.window : c.context;      // crates/neura-generate/src/batch.rs:313-314
    m->capacity = m->window + widest;                 // crates/neura-generate/src/batch.rs:323-325
    m->positions = c.context + widest;
    m->max_tokens = widest * c.batch;
    size_t arena = nh_weights_bytes(weights);
    auto at = [&](uint64_t offset, uint64_t bytes, const char *name) -> const uint8_t * {
        if (offset % 16 || offset > arena || bytes > arena - offset) {
            fail(NH_E_ARGUMENT, "the tensor %s of %llu bytes at %llu does not sit 16-byte aligned inside an arena of %zu bytes", name,
                 (unsigned long long)bytes, (unsigned long long)offset, arena);
            return nullptr;
        }
        return static_cast<const uint8_t *>(nh_weights_at(weights, offset));
    };
    const uint32_t H = c.hidden, QW = c.heads * c.head_dim, KW = c.kv_heads * c.head_dim, F = c.ffn;
    auto matrix_bytes = [&](int32_t element, uint64_t n, uint64_t k) { return n * payload_bytes(element, k); };
    bool ok = true;
    ok = ok && (m->token_embd = at(table->token_embd, matrix_bytes(elements[EMBD], c.vocab, H), "token_embd.weight"));
    m->output = m->token_embd;  // tied head unless the table names one (examples/qwen/model.rs:81-84)
    if (ok && table->output != UINT64_MAX) ok = (m->output = at(table->output, matrix_bytes(elements[HEAD], c.vocab, H), "output.weight")) != nullptr;
    ok = ok && (m->output_norm = reinterpret_cast<const float *>(at(table->output_norm, (uint64_t)H * 4, "output_norm.weight")));
    for (uint32_t L = 0; ok && L < c.layers; L++) {
        const uint8_t *p;
        ok = ok && (p = at(table->attn_norm[L], (uint64_t)H * 4, "attn_norm.weight"));
        if (ok) m->attn_norm.push_back(reinterpret_cast<const float *>(p));
        ok = ok && (p = at(table->ffn_norm[L], (uint64_t)H * 4, "ffn_norm.weight"));
        if (ok) m->ffn_norm.push_back(reinterpret_cast<const float *>(p));
        ok = ok && (p = at(table->attn_q[L], matrix_bytes(element_at(m, L, Q), QW, H), "attn_q.weight"));
        if (ok) m->attn_q.push_back(p);
        ok = ok && (p = at(table->attn_k[L], matrix_bytes(element_at(m, L, K_), KW, H), "attn_k.weight"));
        if (ok) m->attn_k.push_back(p);
        ok = ok && (p = at(table->attn_v[L], matrix_bytes(element_at(m, L, V), KW, H), "attn_v.weight"));
        if (ok) m->attn_v.push_back(p);
        ok = ok && (p = at(table->attn_output[L], matrix_bytes(element_at(m, L, O), H, QW), "attn_output.weight"));
        if (ok) m->attn_o.push_back(p);
        ok = ok && (p = at(table->ffn_gate[L], matrix_bytes(element_at(m, L, GATE), F, H), "ffn_gate.weight"));
        if (ok) m->ffn_gate.push_back(p);
        ok = ok && (p = at(table->ffn_up[L], matrix_bytes(element_at(m, L, UP), F, H), "ffn_up.weight"));
        if (ok) m->ffn_up.push_back(p);
        ok = ok && (p = at(table->ffn_down[L], matrix_bytes(element_at(m, L, DOWN), H, F), "ffn_down.weight"));
        if (ok) m->ffn_down.push_back(p);
        const uint64_t *bias_tables[3] = {table->attn_q_bias, table->attn_k_bias, table->attn_v_bias};
        std::vector<const float *> *held[3] = {&m->bias_q, &m->bias_k, &m->bias_v};
        const uint32_t bias_rows[3] = {QW, KW, KW};
        const char *bias_names[3] = {"attn_q.bias", "attn_k.bias", "attn_v.bias"};
        for (int s = 0; ok && s < 3; s++) {
            const float *bias = nullptr;
            if (bias_tables[s] && bias_tables[s][L] != UINT64_MAX) {
                ok = (p = at(bias_tables[s][L], (uint64_t)bias_rows[s] * 4, bias_names[s])) != nullptr;
                bias = reinterpret_cast<const float *>(p);
            }
            held[s]->push_back(bias);
        }
    }
    if (!ok) {
        release(m);
        return nullptr;
    }
    if (hipSetDevice(device->index) != hipSuccess) {
        fail(NH_E_DEVICE, "device %d cannot be made current", device->index);
        release(m);
        return nullptr;
    }
    const size_t T = m->max_tokens;
    m->cache_elements = (size_t)c.kv_heads * c.batch * m->capacity * c.head_dim;
    m->eb = c.cache_element == NH_F32 ? 4 : 2;
    ok = device_array(m->h, T * H) && device_array(m->xn, T * (H > QW ? H : QW)) && device_array(m->qkv, T * (QW + 2 * KW)) &&
         device_array(m->att, T * QW) && device_array(m->act, T * F) && device_array(m->up, T * F) &&
         device_array(m->logits, (size_t)c.batch * c.vocab) && device_array(m->inputs_dev, T + 6 * c.batch + 4) &&
         device_array(m->chosen_dev, c.batch) && device_array(m->rope_cos, (size_t)m->positions * (c.head_dim / 2)) &&
         device_array(m->rope_sin, (size_t)m->positions * (c.head_dim / 2)) && device_array(m->pairs, (size_t)H) &&
         hipMemsetAsync(m->pairs, 0, (size_t)H * sizeof(uint2), device->stream) == hipSuccess &&
         hipMemsetAsync(m->up, 0, T * F * sizeof(float), device->stream) == hipSuccess;
    for (uint32_t L = 0; ok && L < c.layers; L++) {
        uint8_t *k = nullptr, *v = nullptr;
        ok = device_array(k, m->cache_elements * m->eb);
        if (ok) m->cache_k.push_back(k);
        ok = ok && device_array(v, m->cache_elements * m->eb);
        if (ok && v) m->cache_v.push_back(v);
        if (ok) ok = hipMemsetAsync(k, 0, m->cache_elements * m->eb, device->stream) == hipSuccess &&
                     hipMemsetAsync(v, 0, m->cache_elements * m->eb, device->stream) == hipSuccess;
    }
    ok = ok && hipHostMalloc((void **)&m->inputs_host, (T + 6 * c.batch + 4) * 4, hipHostMallocDefault) == hipSuccess &&
         hipHostMalloc((void **)&m->chosen_host, ((size_t)c.batch + 1) * 4, hipHostMallocDefault) == hipSuccess;
    if (const char *held = getenv("NEURA_HIP_PUBLISH"); ok && !(held && held[0] == '0')) ok = hipHostGetDevicePointer((void **)&m->chosen_mapped, m->chosen_host, 0) == hipSuccess;
    // everything a captured step touches exists before the capture: the split partials of the
    // products (at most 5 slices x 4 rows), of the attention (at most 256 sections) and of the
    // greedy choice, and the rope table
    {
        size_t widest = (size_t)(2 * F > c.vocab ? 2 * F : c.vocab);
        size_t products = 8 * 4 * widest * sizeof(float);
        size_t sections = (size_t)256 * c.heads * T * (c.head_dim + 2) * sizeof(float);
        size_t choice = (size_t)c.batch * 1024 * 8;
        // the wide product packs its fp32 activations as two half rows each, with their sub-block sums and a scale per row
        size_t deepest = (size_t)(F > QW ? F : QW);
        if (H > deepest) deepest = H;
        size_t split_rows = T > 8 ? gemm_q4k_scratch_bytes(T, (uint32_t)deepest, false) : 0;
        size_t wanted = products > sections ? products : sections;
        if (choice > wanted) wanted = choice;
        if (split_rows > wanted) wanted = split_rows;
        ok = ok && scratch(device, wanted) != nullptr && rope_frequencies(device, c.rope_base, c.head_dim) != nullptr &&
             launch_rope_angles(device, c.rope_base, c.head_dim, m->positions, m->rope_cos, m->rope_sin) == NH_OK;
    }
    {
        // Decode steps replay a recorded HIP graph unless NEURA_HIP_GRAPH=0 -- or the process runs under rocprofv3: with the
        // profiler's queue interception in place, hipGraphLaunch has died in a host copy past a page-aligned address (the
        // same address in every such run) once a few thousand packets had gone through the queue, where eager launches of
        // the same kernels trace cleanly.  Kernel durations are the same either way, so traced runs step eagerly.
        const char *held = getenv("NEURA_HIP_GRAPH");
        const bool traced = traced_by_rocprofiler();
        if (held && held[0] == '1' && traced) {
            fail(NH_E_ARGUMENT, "NEURA_HIP_GRAPH=1 asks for recorded decode steps in a process traced by rocprofv3: that combination has crashed "
                                "inside hipGraphLaunch; traced processes step eagerly");
            release(m);
            return nullptr;
        }
        m->use_graph = !(held && held[0] == '0') && !traced;
        // NEURA_HIP_CHAIN_SPIN: the reads of the flag words a seam's wait may take (0: every wait gives up at once, which is how
        // the tests reach the step that is run again)
        if (const char *spin = getenv("NEURA_HIP_CHAIN_SPIN"); spin && spin[0]) m->chain_spin = (uint32_t)strtoul(spin, nullptr, 10);
    }
    ok = ok && hipStreamSynchronize(device->stream) == hipSuccess;
    if (!ok) {
        fail(NH_E_MEMORY, "device %d holds no caches and activations of this decoder", device->index);
        release(m);
        return nullptr;
    }
    return m;
}

void nh_model_destroy(nh_model *model) { release(model); }

uint32_t nh_model_capacity(const nh_model *model) { return model ? model->capacity : 0; }

uint32_t nh_model_seam_fallbacks(const nh_model *model) { return model ? model->seam_fallbacks : 0; }

static int32_t decode_step(nh_model *m, const uint32_t *tokens, const uint32_t *cursors, const uint8_t *mask, uint32_t batch,
                           const nh_draw *draws, uint32_t *chosen_out) {
    NH_REQUIRE(m && tokens && cursors && chosen_out, "a decode step names no model, tokens, cursors or result");
    NH_REQUIRE(batch == m->c.batch, "a decode step of %u planes feeds a model of %u planes", batch, m->c.batch);
    bool any_inactive = false;
    for (uint32_t b = 0; b < batch; b++) {
        bool active = !mask || mask[b];
        any_inactive |= !active;
        // crates/neura-generate/src/batch.rs:1627-1632: a plane answers only below its context
        NH_REQUIRE(!active || cursors[b] < m->c.context, "plane %u at cursor %u of a context of %u no longer answers", b, cursors[b],
                   m->c.context);
    }
    nh_device *d = m->d;
    int32_t status;
    if (draws && (status = check_draws(draws, batch)) != NH_OK) return status;
    if ((status = stage_inputs(m, tokens, batch, cursors, mask, batch, draws)) != NH_OK) return status;
    // Every kernel of the step reads its token, cursor and mask from device memory and no launch
    // shape depends on them, so the step is captured once per mask variant and replayed.
    // Profiled steps run eagerly (event records do not belong in a graph).
    const int variant = (any_inactive ? 1 : 0) + (draws ? 2 : 0);
    for (int attempt = 0;; attempt++) {
        hipGraphExec_t &graph = m->decode_graph[variant];
        // The first step of a variant runs eagerly: its launchers grow the device scratch to what the variant needs (an
        // allocation, which does not belong inside a stream capture; the outgrown block is kept until nh_close).
        if (m->use_graph && traced_by_rocprofiler()) return fail(NH_E_DEVICE, "a recorded decode step is never launched in a process traced by rocprofv3");
        if (m->use_graph && !d->profile && m->graph_warmed[variant]) {
            if (graph && m->graph_moved[variant] != d->moved) {
                // the device scratch or rope table moved since the capture (another model or operator call grew it)
                (void)hipGraphExecDestroy(graph);
                graph = nullptr;
            }
            if (!graph) {
                m->graph_moved[variant] = d->moved;
                NH_HIP(hipStreamBeginCapture(d->stream, hipStreamCaptureModeThreadLocal));
                status = decode_kernels(m, any_inactive, draws != nullptr);
                hipGraph_t recorded = nullptr;
                hipError_t ended = hipStreamEndCapture(d->stream, &recorded);
                if (status != NH_OK) {
                    if (recorded) (void)hipGraphDestroy(recorded);
                    return status;
                }
                if (ended != hipSuccess) return hip_fail(ended, "hipStreamEndCapture");
                hipError_t built = hipGraphInstantiate(&graph, recorded, nullptr, nullptr, 0);
                (void)hipGraphDestroy(recorded);
                if (built != hipSuccess) {
                    graph = nullptr;
                    return hip_fail(built, "hipGraphInstantiate");
                }
            }
            NH_HIP(hipGraphLaunch(graph, d->stream));
        } else {
            if ((status = decode_kernels(m, any_inactive, draws != nullptr)) != NH_OK) return status;
            m->graph_warmed[variant] = true;
        }
        if (!m->chosen_mapped) {
            NH_HIP(hipMemcpyAsync(m->chosen_host, m->chosen_dev, (size_t)batch * 4, hipMemcpyDeviceToHost, d->stream));
            NH_HIP(hipMemcpyAsync(m->chosen_host + batch, d->refusal, 4, hipMemcpyDeviceToHost, d->stream));
        }
        NH_HIP(hipStreamSynchronize(d->stream));
        if (m->chosen_host[batch] != REFUSAL_SEAM || attempt > 0) break;
        // A seam of a chained launch gave up (not every workgroup was resident, or one was held up past the wait's bound):
        // what the step wrote behind it is not to be trusted.  Every kernel of a step reads its inputs from where the host
        // staged them and writes the same cache rows again, so the step is simply run once more, one launch a product, and
        // the model stays that way; recorded steps hold chained launches and are dropped.
        NH_HIP(hipMemsetAsync(d->refusal, 0, sizeof(uint32_t), d->stream));
        NH_HIP(hipStreamSynchronize(d->stream));
        m->chain = false;
        m->seam_fallbacks++;
        for (hipGraphExec_t &held : m->decode_graph) {
            if (held) (void)hipGraphExecDestroy(held);
            held = nullptr;
        }
    }
    if (m->chosen_host[batch] != REFUSAL_NONE) return check_refusal(d, "a decode step");
    memcpy(chosen_out, m->chosen_host, (size_t)batch * 4);
    return NH_OK;
}

int32_t nh_decode_step(nh_model *m, const uint32_t *tokens, const uint32_t *cursors, const uint8_t *mask, uint32_t batch,
                       uint32_t *chosen_out) {
    return decode_step(m, tokens, cursors, mask, batch, nullptr, chosen_out);
}

int32_t nh_decode_step_sampled(nh_model *m, const uint32_t *tokens, const uint32_t *cursors, const uint8_t *mask, uint32_t batch,
                               const nh_draw *host_draws, uint32_t *chosen_out) {
    NH_REQUIRE(host_draws, "a sampled decode step names no draws");
    return decode_step(m, tokens, cursors, mask, batch, host_draws, chosen_out);
}

int32_t nh_prefill(nh_model *m, const uint32_t *tokens, uint32_t rows, const uint32_t *cursors, const uint8_t *mask, uint32_t batch) {
    NH_REQUIRE(m && tokens && cursors, "a fill names no model, tokens or cursors");
    NH_REQUIRE(batch == m->c.batch, "a fill of %u planes feeds a model of %u planes", batch, m->c.batch);
    NH_REQUIRE(rows >= 1 && rows * batch <= m->max_tokens, "a fill of %u rows feeds a model built for chunks of %u rows", rows,
               m->max_tokens / m->c.batch);
    bool any_inactive = false;
    for (uint32_t b = 0; b < batch; b++) {
        bool active = !mask || mask[b];
        any_inactive |= !active;
        NH_REQUIRE(!active || (uint64_t)cursors[b] + rows <= m->c.context, "plane %u at cursor %u fills %u rows past a context of %u", b,
                   cursors[b], rows, m->c.context);
    }
    int32_t status;
    if ((status = stage_inputs(m, tokens, rows * batch, cursors, mask, batch)) != NH_OK) return status;
    if ((status = forward(m, rows, any_inactive)) != NH_OK) return status;
    return check_refusal(m->d, "a fill");
}

int32_t nh_model_time_products(nh_model *m, uint32_t steps, double *seconds_out, uint64_t *launches_out, uint64_t *bytes_out) {
    NH_REQUIRE(m && steps && seconds_out && launches_out && bytes_out, "a product timing names no model, no step or no result");
    nh_device *d = m->d;
    // count launches and bytes with the per-launch profile of one untimed pass, then time
    // `steps` passes of the same launches between one pair of events
    int32_t status;
    if ((status = nh_profile_begin(d)) != NH_OK) return status;
    status = forward(m, 1, false, true);
    if (status == NH_OK) {
        GemvArgs head = narrow(m, m->output == m->token_embd ? m->elements[EMBD] : m->elements[HEAD], m->output, m->c.vocab, m->c.hidden, m->h, m->c.batch, m->logits);
        head.norm_w = m->output_norm, head.eps = m->c.eps;
        status = launch_gemv(d, head);
    }
    double ignored = 0.0;
    int32_t ended = nh_profile_end(d, &ignored, launches_out, bytes_out);
    if (status != NH_OK) return status;
    if (ended != NH_OK) return ended;
    if ((status = nh_timer_start(d)) != NH_OK) return status;
    for (uint32_t step = 0; step < steps; step++) {
        if ((status = forward(m, 1, false, true)) != NH_OK) return status;
        GemvArgs head = narrow(m, m->output == m->token_embd ? m->elements[EMBD] : m->elements[HEAD], m->output, m->c.vocab, m->c.hidden, m->h, m->c.batch, m->logits);
        head.norm_w = m->output_norm, head.eps = m->c.eps;
        if ((status = launch_gemv(d, head)) != NH_OK) return status;
    }
    if ((status = nh_timer_stop(d, seconds_out)) != NH_OK) return status;
    *launches_out *= steps;
    *bytes_out *= steps;
    return NH_OK;
}

int32_t nh_model_reset(nh_model *m, const uint8_t *reset, uint32_t batch) {
    NH_REQUIRE(m && reset && batch == m->c.batch, "a reset names no model, no flags or another plane count");
    const size_t plane = (size_t)m->capacity * m->c.head_dim;
    for (uint32_t L = 0; L < m->c.layers; L++)
        for (uint32_t head = 0; head < m->c.kv_heads; head++)
            for (uint32_t b = 0; b < batch; b++) {
                if (!reset[b]) continue;
                size_t at = ((size_t)head * batch + b) * plane;
                NH_HIP(hipMemsetAsync(m->cache_k[L] + at * m->eb, 0, plane * m->eb, m->d->stream));
                NH_HIP(hipMemsetAsync(m->cache_v[L] + at * m->eb, 0, plane * m->eb, m->d->stream));
            }
    return NH_OK;
}

// the shared planes, zeroed, on first use
static int32_t shared_planes(nh_model *m) {
    if (!m->shared_k.empty()) return NH_OK;
    const size_t bytes = (size_t)m->c.kv_heads * m->capacity * m->c.head_dim * m->eb;
    for (uint32_t L = 0; L < m->c.layers; L++) {
        uint8_t *k = nullptr, *v = nullptr;
        if (hipMalloc((void **)&k, bytes) != hipSuccess || hipMalloc((void **)&v, bytes) != hipSuccess) {
            if (k) (void)hipFree(k);
            return fail(NH_E_MEMORY, "no room for the %zu bytes a shared prefix of layer %u holds", 2 * bytes, L);
        }
        m->shared_k.push_back(k), m->shared_v.push_back(v);
        NH_HIP(hipMemsetAsync(k, 0, bytes, m->d->stream));
        NH_HIP(hipMemsetAsync(v, 0, bytes, m->d->stream));
    }
    return NH_OK;
}

int32_t nh_model_keep_prefix(nh_model *m, uint32_t plane_index) {
    NH_REQUIRE(m && plane_index < m->c.batch, "a prefix is kept from a plane of the model");
    int32_t status = shared_planes(m);
    if (status != NH_OK) return status;
    const size_t plane = (size_t)m->capacity * m->c.head_dim;
    for (uint32_t L = 0; L < m->c.layers; L++)
        for (uint32_t head = 0; head < m->c.kv_heads; head++) {
            const size_t from = ((size_t)head * m->c.batch + plane_index) * plane, to = (size_t)head * plane;
            NH_HIP(hipMemcpyAsync(m->shared_k[L] + to * m->eb, m->cache_k[L] + from * m->eb, plane * m->eb, hipMemcpyDeviceToDevice, m->d->stream));
            NH_HIP(hipMemcpyAsync(m->shared_v[L] + to * m->eb, m->cache_v[L] + from * m->eb, plane * m->eb, hipMemcpyDeviceToDevice, m->d->stream));
        }
    return NH_OK;
}

int32_t nh_model_reset_shared(nh_model *m, const uint8_t *reset, const uint8_t *share, uint32_t batch) {
    NH_REQUIRE(m && reset && share && batch == m->c.batch, "a reset names no model, no flags or another plane count");
    bool any = false;
    for (uint32_t b = 0; b < batch; b++) any |= share[b] != 0;
    int32_t status = any ? shared_planes(m) : NH_OK;
    if (status != NH_OK) return status;
    const size_t plane = (size_t)m->capacity * m->c.head_dim;
    for (uint32_t L = 0; L < m->c.layers; L++)
        for (uint32_t head = 0; head < m->c.kv_heads; head++)
            for (uint32_t b = 0; b < batch; b++) {
                const size_t at = ((size_t)head * batch + b) * plane;
                if (share[b]) {  // select(share, prefix, blank): the prefix wins over the reset (cache.rs:231-238)
                    NH_HIP(hipMemcpyAsync(m->cache_k[L] + at * m->eb, m->shared_k[L] + (size_t)head * plane * m->eb, plane * m->eb, hipMemcpyDeviceToDevice, m->d->stream));
                    NH_HIP(hipMemcpyAsync(m->cache_v[L] + at * m->eb, m->shared_v[L] + (size_t)head * plane * m->eb, plane * m->eb, hipMemcpyDeviceToDevice, m->d->stream));
                } else if (reset[b]) {
                    NH_HIP(hipMemsetAsync(m->cache_k[L] + at * m->eb, 0, plane * m->eb, m->d->stream));
                    NH_HIP(hipMemsetAsync(m->cache_v[L] + at * m->eb, 0, plane * m->eb, m->d->stream));
                }
            }
    return NH_OK;
}

int32_t nh_model_shared_write(nh_model *m, uint32_t layer, int32_t value_not_key, const void *host_src) {
    NH_REQUIRE(m && host_src && layer < m->c.layers, "a shared prefix write names no model, no bytes or no layer %u", layer);
    int32_t status = shared_planes(m);
    if (status != NH_OK) return status;
    return nh_upload(m->d, value_not_key ? m->shared_v[layer] : m->shared_k[layer], host_src, (size_t)m->c.kv_heads * m->capacity * m->c.head_dim * m->eb);
}

int32_t nh_model_shared_read(nh_model *m, uint32_t layer, int32_t value_not_key, void *host_dst) {
    NH_REQUIRE(m && host_dst && layer < m->c.layers, "a shared prefix read names no model, no bytes or no layer %u", layer);
    int32_t status = shared_planes(m);
    if (status != NH_OK) return status;
    return nh_download(m->d, host_dst, value_not_key ? m->shared_v[layer] : m->shared_k[layer], (size_t)m->c.kv_heads * m->capacity * m->c.head_dim * m->eb);
}

int32_t nh_model_logits(nh_model *m, float *host_out) {
    NH_REQUIRE(m && host_out, "a logits read names no model or no result");
    return nh_download(m->d, host_out, m->logits, (size_t)m->c.batch * m->c.vocab * 4);
}

int32_t nh_model_cache_write(nh_model *m, uint32_t layer, int32_t value_not_key, const void *host_src) {
    NH_REQUIRE(m && host_src && layer < m->c.layers, "a cache write names no model, no bytes or no layer %u", layer);
    return nh_upload(m->d, value_not_key ? m->cache_v[layer] : m->cache_k[layer], host_src, m->cache_elements * m->eb);
}

int32_t nh_model_cache_read(nh_model *m, uint32_t layer, int32_t value_not_key, void *host_dst) {
    NH_REQUIRE(m && host_dst && layer < m->c.layers, "a cache read names no model, no bytes or no layer %u", layer);
    return nh_download(m->d, host_dst, value_not_key ? m->cache_v[layer] : m->cache_k[layer], m->cache_elements * m->eb);
}

// ---- operator entry points ---------------------------------------------------------------

static bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

int32_t nh_dequant(nh_device *device, int32_t element, const void *dev_src, uint64_t elements, float *dev_dst) {
    NH_REQUIRE(device && dev_src && dev_dst, "a dequantisation names no device or no buffer");
    uint32_t block = block_elements(element);
    NH_REQUIRE(block, "element %d carries no reader", element);
    NH_REQUIRE(elements % block == 0, "%llu numbers are not whole blocks of %u", (unsigned long long)elements, block);
    return launch_dequant(device, element, dev_src, elements, dev_dst);
}

int32_t nh_convert_half(nh_device *device, const float *dev_src, uint64_t elements, uint16_t *dev_dst) {
    NH_REQUIRE(device && dev_src && dev_dst, "a conversion names no device or no buffer");
    return launch_convert_half(device, dev_src, elements, dev_dst);
}

int32_t nh_pack_q8_0(nh_device *device, const float *dev_src, uint64_t elements, void *dev_dst) {
    NH_REQUIRE(device && dev_src && dev_dst, "a packing names no device or no buffer");
    NH_REQUIRE(aligned16(dev_src) && ((uintptr_t)dev_dst & 3u) == 0, "a packing reads from a 16-byte boundary and writes from a 4-byte one");
    return launch_pack_q8_0(device, dev_src, elements, static_cast<uint8_t *>(dev_dst));
}

int32_t nh_gemv(nh_device *device, int32_t element, const void *dev_W, uint32_t N, uint32_t K, const float *dev_x, uint32_t rows,
                float *dev_y, const nh_epilogue *epilogue) {
    NH_REQUIRE(device && dev_W && dev_x && dev_y, "a product names no device or no buffer");
    NH_REQUIRE(element == NH_Q8_0 || element == NH_Q4_K || staged_super_block(element),
               "a narrow product walks Q8_0, Q3_K, Q4_K, Q5_K or Q6_K weights, not element %d", element);
    NH_REQUIRE(N > 0 && K > 0 && K % block_elements(element) == 0, "a row of %u numbers is not whole blocks of %u", K, block_elements(element));
    NH_REQUIRE(rows >= 1 && rows <= 8, "a narrow product takes one to eight rows, not %u", rows);
    NH_REQUIRE(aligned16(dev_W) && aligned16(dev_x), "a product reads its weights and activations from 16-byte aligned addresses");
    GemvArgs a{};
    a.element = element;
    a.W[0] = dev_W, a.W[1] = nullptr, a.W[2] = nullptr;
    a.end[0] = a.end[1] = a.end[2] = N;
    a.N = N, a.K = K, a.x = dev_x, a.rows = rows, a.y = dev_y;
    if (epilogue) {
        a.residual = epilogue->residual;
        a.swiglu = epilogue->swiglu;
        NH_REQUIRE(!(a.swiglu && a.residual), "a product fuses swiglu or a residual, not both");
        if (a.swiglu) {
            NH_REQUIRE(N % 2 == 0, "a swiglu product halves %u rows", N);
            a.W[1] = static_cast<const uint8_t *>(dev_W) + (size_t)(N / 2) * payload_bytes(element, K);
            a.end[0] = N / 2;
            // Q6_K, Q5_K and Q3_K rows are read through aligned copies whatever their own alignment
            NH_REQUIRE(staged_super_block(element) || aligned16(a.W[1]), "the up half of a swiglu product starts off a 16-byte boundary");
        }
    }
    return launch_gemv(device, a);
}

int32_t nh_gemm(nh_device *device, int32_t element, const void *dev_W, uint32_t N, uint32_t K, const void *dev_X, int32_t x_element,
                uint32_t M, float *dev_Y, const nh_epilogue *epilogue) {
    NH_REQUIRE(device && dev_W && dev_X && dev_Y, "a product names no device or no buffer");
    NH_REQUIRE(element == NH_Q8_0 || element == NH_Q4_K || staged_super_block(element),
               "a wide product walks Q8_0, Q3_K, Q4_K, Q5_K or Q6_K weights, not element %d", element);
    NH_REQUIRE(x_element == NH_F32 || x_element == NH_F16, "a wide product takes fp32 or fp16 activations, not element %d", x_element);
    NH_REQUIRE(N > 0 && K > 0 && M > 0 && K % block_elements(element) == 0, "a row of %u numbers is not whole blocks of %u", K,
               block_elements(element));
    NH_REQUIRE(aligned16(dev_W) && aligned16(dev_X), "a product reads its weights and activations from 16-byte aligned addresses");
    NH_REQUIRE(!(epilogue && epilogue->swiglu), "a wide product fuses no swiglu");
    GemmArgs a{element, dev_W, N, K, dev_X, x_element, M, dev_Y, epilogue ? epilogue->residual : nullptr, N};
    return launch_gemm(device, a);
}

int32_t nh_rmsnorm(nh_device *device, const float *dev_x, const float *dev_residual, const float *dev_w, float eps, uint32_t rows,
                   uint32_t C, float *dev_out, float *dev_sum_out) {
    NH_REQUIRE(device && dev_x && dev_out && C > 0, "a norm names no device, no buffer or no column");
    return launch_rmsnorm(device, dev_x, dev_residual, dev_w, eps, rows, C, dev_out, dev_sum_out);
}

int32_t nh_rope(nh_device *device, const float *dev_x, uint32_t planes, uint32_t batch, uint32_t rows, uint32_t width,
                const uint32_t *dev_cursor, float base, float *dev_out) {
    NH_REQUIRE(device && dev_x && dev_out, "a rope names no device or no buffer");
    NH_REQUIRE(width >= 2 && width % 2 == 0, "a rope turns pairs, and %u numbers leave one over", width);
    NH_REQUIRE(std::isfinite(base) && base > 1.0f, "a rope base of %f turns nothing", (double)base);
    return launch_rope(device, dev_x, planes, batch, rows, width, dev_cursor, base, dev_out);
}

static bool cache_holds(int32_t element) { return element == NH_F16 || element == NH_BF16 || element == NH_F32; }

int32_t nh_cache_write(nh_device *device, const float *dev_k, const float *dev_v, uint16_t *dev_cache_k, uint16_t *dev_cache_v,
                       uint32_t kv_heads, uint32_t batch, uint32_t rows, uint32_t width, uint32_t capacity, uint32_t window,
                       const uint32_t *dev_cursor, const uint8_t *dev_mask, int32_t ring) {
    return nh_cache_write_element(device, dev_k, dev_v, dev_cache_k, dev_cache_v, kv_heads, batch, rows, width, capacity, window, dev_cursor, dev_mask,
                                  ring, NH_F16);
}

int32_t nh_cache_write_element(nh_device *device, const float *dev_k, const float *dev_v, void *dev_cache_k, void *dev_cache_v,
                               uint32_t kv_heads, uint32_t batch, uint32_t rows, uint32_t width, uint32_t capacity, uint32_t window,
                               const uint32_t *dev_cursor, const uint8_t *dev_mask, int32_t ring, int32_t cache_element) {
    NH_REQUIRE(device && dev_k && dev_v && dev_cache_k && dev_cache_v && dev_cursor, "a cache write names no device or no buffer");
    // crates/neura-decoder/src/cache.rs:130-134
    NH_REQUIRE(cache_holds(cache_element), "a cache holds keys and values in single, half or bfloat16 storage, and element %d carries another grid",
               cache_element);
    // crates/neura-decoder/src/cache.rs:113-125, :328-335
    NH_REQUIRE(kv_heads > 0 && width > 0 && batch > 0, "a cache of %u planes of %u heads of %u numbers holds no key", batch, kv_heads, width);
    NH_REQUIRE(window > 0 && window <= capacity, "a cache of %u positions keeps a window of %u positions", capacity, window);
    NH_REQUIRE(rows > 0 && rows <= window, "a cache of a %u position window takes %u rows at a time", window, rows);
    NH_REQUIRE(!dev_mask || rows <= capacity - window, "a masked chunk of %u rows holds only %u scratch rows", rows, capacity - window);
    int32_t status = launch_cache_write(device, dev_k, dev_v, dev_cache_k, dev_cache_v, kv_heads, batch, rows, width, capacity, window,
                                        dev_cursor, dev_mask, ring != 0, cache_element);
    return status != NH_OK ? status : check_refusal(device, "a cache write");
}

int32_t nh_attention(nh_device *device, const float *dev_q, const uint16_t *dev_cache_k, const uint16_t *dev_cache_v, uint32_t heads,
                     uint32_t kv_heads, uint32_t batch, uint32_t rows, uint32_t width, uint32_t capacity, uint32_t keys, uint32_t reach,
                     const uint32_t *dev_cursor, float scale, float *dev_out) {
    return nh_attention_element(device, dev_q, dev_cache_k, dev_cache_v, heads, kv_heads, batch, rows, width, capacity, keys, reach, dev_cursor, scale,
                                dev_out, NH_F16);
}

int32_t nh_attention_element(nh_device *device, const float *dev_q, const void *dev_cache_k, const void *dev_cache_v, uint32_t heads,
                             uint32_t kv_heads, uint32_t batch, uint32_t rows, uint32_t width, uint32_t capacity, uint32_t keys,
                             uint32_t reach, const uint32_t *dev_cursor, float scale, float *dev_out, int32_t cache_element) {
    NH_REQUIRE(device && dev_q && dev_cache_k && dev_cache_v && dev_out, "an attention names no device or no buffer");
    NH_REQUIRE(cache_holds(cache_element), "a cache holds keys and values in single, half or bfloat16 storage, and element %d carries another grid",
               cache_element);
    // crates/neura-decoder/src/cache.rs:383-388
    NH_REQUIRE(kv_heads > 0 && heads % kv_heads == 0, "a query of %u heads reads a cache of %u key heads", heads, kv_heads);
    NH_REQUIRE(keys > 0 && keys <= capacity && rows > 0 && rows <= keys, "%u rows weigh %u keys of a cache of %u positions", rows, keys, capacity);
    NH_REQUIRE(std::isfinite(scale) && scale != 0.0f, "an attention scale of %f weighs nothing", (double)scale);  // attention.rs:128-132
    NH_REQUIRE(aligned16(dev_cache_k) && aligned16(dev_cache_v), "an attention reads its caches from 16-byte aligned addresses");
    AttentionArgs a{};
    a.q = dev_q, a.out = dev_out;
    a.q_sh = a.o_sh = (uint64_t)batch * rows * width;
    a.q_sb = a.o_sb = (uint64_t)rows * width;
    a.q_sr = a.o_sr = width;
    a.cache_k = static_cast<const uint16_t *>(dev_cache_k), a.cache_v = static_cast<const uint16_t *>(dev_cache_v);
    a.heads = heads, a.kv_heads = kv_heads, a.batch = batch, a.rows = rows, a.width = width, a.capacity = capacity, a.keys = keys;
    a.cursor = dev_cursor, a.scale = scale, a.reach = reach, a.cache_element = cache_element;
    int32_t status = launch_attention(device, a);
    return status != NH_OK ? status : check_refusal(device, "an attention");
}

int32_t nh_gather(nh_device *device, int32_t element, const void *dev_table, uint32_t vocab, uint32_t width, const uint32_t *dev_tokens,
                  uint32_t count, uint32_t batch, const uint8_t *dev_mask, float *dev_out) {
    NH_REQUIRE(device && dev_table && dev_tokens && dev_out, "a gather names no device or no buffer");
    uint32_t block = block_elements(element);
    NH_REQUIRE(block && width % block == 0, "a row of %u numbers is not whole blocks of element %d", width, element);
    NH_REQUIRE(batch > 0, "a gather spreads its mask over no plane");
    int32_t status = launch_gather(device, element, dev_table, vocab, width, dev_tokens, count, batch, dev_mask, dev_out);
    return status != NH_OK ? status : check_refusal(device, "a gather");
}

int32_t nh_sample(nh_device *device, const float *dev_logits, uint32_t rows, uint32_t n, const nh_draw *host_draws, uint32_t *dev_out) {
    NH_REQUIRE(device && dev_logits && host_draws && dev_out, "a sample names no device, logits, draws or result");
    NH_REQUIRE(rows <= 4096, "a sample draws at most 4096 rows a call, not %u", rows);
    int32_t status = check_draws(host_draws, rows);
    if (status != NH_OK) return status;
    if (!rows) return NH_OK;
    // the draws ride in a small buffer of their own: the scratch belongs to the kernels
    nh_draw *draws = nullptr;
    NH_HIP(hipMalloc((void **)&draws, (size_t)rows * sizeof(nh_draw)));
    hipError_t copied = hipMemcpyAsync(draws, host_draws, (size_t)rows * sizeof(nh_draw), hipMemcpyHostToDevice, device->stream);
    if (copied == hipSuccess) status = launch_sample(device, dev_logits, rows, n, draws, dev_out);
    (void)hipStreamSynchronize(device->stream);
    (void)hipFree(draws);
    if (copied != hipSuccess) return hip_fail(copied, "hipMemcpyAsync");
    return status;
}

int32_t nh_argmax(nh_device *device, const float *dev_values, uint32_t rows, uint32_t n, uint32_t *dev_out) {
    NH_REQUIRE(device && dev_values && dev_out && n > 0, "a choice names no device, no buffer or no value");
    return launch_argmax(device, dev_values, rows, n, dev_out);
}

int32_t nh_argmax_static(nh_device *device, const float *dev_values, uint32_t rows, uint32_t n, uint32_t *dev_out) {
    NH_REQUIRE(device && dev_values && dev_out && n > 0, "a choice names no device, no buffer or no value");
    return launch_argmax_static(device, dev_values, rows, n, dev_out);
}

}  // extern "C"
