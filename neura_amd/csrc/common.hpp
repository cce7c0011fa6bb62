// Shared declarations of libneura_hip.so: the device handle, error reporting and the
// launcher prototypes each kernel file exports to the C ABI layer.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <vector>

#include "../../include/neura_hip.h"

namespace nh {

constexpr uint32_t Q8_0_BLOCK = 32, Q8_0_BYTES = 34;
constexpr uint32_t Q4_K_BLOCK = 256, Q4_K_BYTES = 144;
constexpr uint32_t Q6_K_BLOCK = 256, Q6_K_BYTES = 210;
constexpr uint32_t Q5_K_BLOCK = 256, Q5_K_BYTES = 176;
constexpr uint32_t Q3_K_BLOCK = 256, Q3_K_BYTES = 110;
constexpr uint32_t WAVE = 64;

int32_t fail(int32_t code, const char *format, ...) __attribute__((format(printf, 2, 3)));
int32_t hip_fail(hipError_t error, const char *what);

#define NH_HIP(call)                                              \
    do {                                                          \
        hipError_t nh_hip_error_ = (call);                        \
        if (nh_hip_error_ != hipSuccess) return ::nh::hip_fail(nh_hip_error_, #call); \
    } while (0)

#define NH_REQUIRE(condition, ...)                                \
    do {                                                          \
        if (!(condition)) return ::nh::fail(NH_E_ARGUMENT, __VA_ARGS__); \
    } while (0)

inline uint64_t payload_bytes(int32_t element, uint64_t elements) {
    switch (element) {
    case NH_Q8_0: return (elements + Q8_0_BLOCK - 1) / Q8_0_BLOCK * Q8_0_BYTES;
    case NH_Q4_K: return (elements + Q4_K_BLOCK - 1) / Q4_K_BLOCK * Q4_K_BYTES;
    case NH_Q6_K: return (elements + Q6_K_BLOCK - 1) / Q6_K_BLOCK * Q6_K_BYTES;
    case NH_Q5_K: return (elements + Q5_K_BLOCK - 1) / Q5_K_BLOCK * Q5_K_BYTES;
    case NH_Q3_K: return (elements + Q3_K_BLOCK - 1) / Q3_K_BLOCK * Q3_K_BYTES;
    case NH_F16: return elements * 2;
    case NH_F32: return elements * 4;
    default: return 0;
    }
}

// the super-block formats whose rows the narrow product stages raw in LDS
inline bool staged_super_block(int32_t element) { return element == NH_Q6_K || element == NH_Q5_K || element == NH_Q3_K; }

inline uint32_t block_elements(int32_t element) {
    switch (element) {
    case NH_Q8_0: return Q8_0_BLOCK;
    case NH_Q4_K: return Q4_K_BLOCK;
    case NH_Q3_K:
    case NH_Q5_K:
    case NH_Q6_K: return Q6_K_BLOCK;
    case NH_F16:
    case NH_F32: return 1;
    default: return 0;
    }
}

}  // namespace nh

// One device = one HIP stream, a pair of timing events and a few scratch buffers that
// grow on demand (split-K / split-context partials, argmax partials, the refusal word).
struct nh_device {
    int32_t index = 0;
    hipStream_t stream = nullptr;
    hipEvent_t started = nullptr, stopped = nullptr;
    int32_t compute_units = 0;
    void *scratch = nullptr;  // device scratch, `scratch_bytes` long
    size_t scratch_bytes = 0;
    std::vector<void *> retired;  // scratch blocks that were outgrown: released by nh_close, never before
    // counts the times the scratch was replaced by a larger block: a captured graph holds its address and is
    // recorded again when this no longer matches the count at its capture
    uint64_t moved = 0;
    uint32_t *refusal = nullptr;  // device word: 0 = none, else a refusal code
    uint32_t *tick = nullptr;  // device word that launch_tick moves on at the start of every pass over a decoder's layers: part of every tag word
    uint8_t *static_scratch = nullptr;  // this device's copy of the file-scope array nh_argmax_static works in (argmax.hip)
    struct RopeTable {
        float base;
        uint32_t width;
        float *table;  // device inverse frequencies pow(base, -2c/width), c < width / 2
    };
    std::vector<RopeTable> rope_tables;  // one per (base, width) met so far; entries never move
    // per-launch timing of the narrow products (nh_profile_*): event pairs on the stream
    bool profile = false;
    std::vector<hipEvent_t> profile_events;  // start, stop, start, stop, ...
    size_t profile_used = 0;
    uint64_t profile_bytes = 0;              // weight bytes the timed launches walked
};

namespace nh {

// grows the device scratch to at least `bytes`; returns nullptr on failure (error recorded)
void *scratch(nh_device *device, size_t bytes);
// device table of pow(base, -2c/width), c < width/2, computed on the host in fp32
const float *rope_frequencies(nh_device *device, float base, uint32_t width);
// reads and clears the refusal word; returns NH_OK or NH_E_REFUSAL with a message
int32_t check_refusal(nh_device *device, const char *what);

// records the next profiling event on the stream (no-op unless profiling is on)
void profile_mark(nh_device *device);

// REFUSAL_SEAM: a workgroup of a chained launch gave up waiting for the others (launch_chain); it ranks below the refusals of an
// input, which atomicMax keeps
enum Refusal : uint32_t { REFUSAL_NONE = 0, REFUSAL_SEAM = 1, REFUSAL_INDEX = 2, REFUSAL_ORIGIN = 3 };

// ---- launchers (each validates nothing: the C ABI layer checks shapes first) ----
int32_t launch_dequant(nh_device *d, int32_t element, const void *src, uint64_t elements, float *dst);
int32_t launch_convert_half(nh_device *d, const float *src, uint64_t elements, uint16_t *dst);

// Rotation and cache append folded into the q|k|v product of one token (one activation row, one plane):
// output rows [0, q_rows) are rotated and written to y, rows [q_rows, k_rows) are rotated, rounded to fp16 and
// written to the key cache at the cursor, the rest are rounded to fp16 into the value cache.
struct RopeFusion {
    const float *cosines, *sines;  // [positions][width / 2]: cos and sin of f32(position) * pow(base, -2c/width)
    const uint32_t *cursor;        // device: a word a plane (a product of one row reads the first)
    uint16_t *cache_k, *cache_v;
    uint32_t width, q_rows, k_rows, capacity;
    uint32_t positions;  // rows of the two tables
    uint32_t ring;       // 0, or the span of a ring cache: position p is written to slot p % ring
    int32_t element = NH_F16;  // what the two states hold (NH_F16, NH_BF16 or NH_F32: cache_k and cache_v then point at numbers of that size)
};

// NH_FETCH(p.a, p.b, ...): every scalar load of the named kernel parameters goes out at once, before the kernel's first
// wait.  Left alone the compiler loads each parameter where it is first used: a parameter block that spans several cache
// lines then costs one round trip to memory after another (about 0.3 us each) before the kernel's first vector load is
// issued.  At most thirty names a statement; statements that follow one another still share one wait.
#define NH_FETCH_1(a) "s"(a)
#define NH_FETCH_2(a, ...) "s"(a), NH_FETCH_1(__VA_ARGS__)
#define NH_FETCH_3(a, ...) "s"(a), NH_FETCH_2(__VA_ARGS__)
#define NH_FETCH_4(a, ...) "s"(a), NH_FETCH_3(__VA_ARGS__)
#define NH_FETCH_5(a, ...) "s"(a), NH_FETCH_4(__VA_ARGS__)
#define NH_FETCH_6(a, ...) "s"(a), NH_FETCH_5(__VA_ARGS__)
#define NH_FETCH_7(a, ...) "s"(a), NH_FETCH_6(__VA_ARGS__)
#define NH_FETCH_8(a, ...) "s"(a), NH_FETCH_7(__VA_ARGS__)
#define NH_FETCH_9(a, ...) "s"(a), NH_FETCH_8(__VA_ARGS__)
#define NH_FETCH_10(a, ...) "s"(a), NH_FETCH_9(__VA_ARGS__)
#define NH_FETCH_11(a, ...) "s"(a), NH_FETCH_10(__VA_ARGS__)
#define NH_FETCH_12(a, ...) "s"(a), NH_FETCH_11(__VA_ARGS__)
#define NH_FETCH_13(a, ...) "s"(a), NH_FETCH_12(__VA_ARGS__)
#define NH_FETCH_14(a, ...) "s"(a), NH_FETCH_13(__VA_ARGS__)
#define NH_FETCH_15(a, ...) "s"(a), NH_FETCH_14(__VA_ARGS__)
#define NH_FETCH_16(a, ...) "s"(a), NH_FETCH_15(__VA_ARGS__)
#define NH_FETCH_17(a, ...) "s"(a), NH_FETCH_16(__VA_ARGS__)
#define NH_FETCH_18(a, ...) "s"(a), NH_FETCH_17(__VA_ARGS__)
#define NH_FETCH_19(a, ...) "s"(a), NH_FETCH_18(__VA_ARGS__)
#define NH_FETCH_20(a, ...) "s"(a), NH_FETCH_19(__VA_ARGS__)
#define NH_FETCH_21(a, ...) "s"(a), NH_FETCH_20(__VA_ARGS__)
#define NH_FETCH_22(a, ...) "s"(a), NH_FETCH_21(__VA_ARGS__)
#define NH_FETCH_23(a, ...) "s"(a), NH_FETCH_22(__VA_ARGS__)
#define NH_FETCH_24(a, ...) "s"(a), NH_FETCH_23(__VA_ARGS__)
#define NH_FETCH_25(a, ...) "s"(a), NH_FETCH_24(__VA_ARGS__)
#define NH_FETCH_26(a, ...) "s"(a), NH_FETCH_25(__VA_ARGS__)
#define NH_FETCH_27(a, ...) "s"(a), NH_FETCH_26(__VA_ARGS__)
#define NH_FETCH_28(a, ...) "s"(a), NH_FETCH_27(__VA_ARGS__)
#define NH_FETCH_29(a, ...) "s"(a), NH_FETCH_28(__VA_ARGS__)
#define NH_FETCH_30(a, ...) "s"(a), NH_FETCH_29(__VA_ARGS__)
#define NH_FETCH_COUNT(_1, _2, _3, _4, _5, _6, _7, _8, _9, _10, _11, _12, _13, _14, _15, _16, _17, _18, _19, _20, _21, _22, _23, _24, _25, _26, _27, _28, _29, _30, N, ...) N
#define NH_FETCH_PASTE(a, b) a##b
#define NH_FETCH_PICK(n) NH_FETCH_PASTE(NH_FETCH_, n)
#define NH_FETCH(...)                                                                                                                                    \
    asm volatile("" ::NH_FETCH_PICK(NH_FETCH_COUNT(__VA_ARGS__, 30, 29, 28, 27, 26, 25, 24, 23, 22, 21, 20, 19, 18, 17, 16, 15, 14, 13, 12, 11, 10, 9, 8, 7, 6, 5, 4, \
                                                   3, 2, 1))(__VA_ARGS__))

// The sums a decode attention left a section of the keys each, not merged yet: per (unit, section, query head of the group)
// `width` weighed channel sums, then the section's largest score and its mass (what attention_fold_kernel reads).
struct SectionSums {
    const float *partial;
    uint32_t sections, groups, width;
};

struct GemvArgs {
    int32_t element;
    const void *W[3];  // up to three matrices stacked along N; unused entries are nullptr
    uint32_t end[3];   // first output row past each matrix (end[2] == N); with swiglu W[0] = gate, W[1] = up
    uint32_t N, K;
    const float *x;    // [rows][K]
    uint32_t rows;
    float *y;          // [rows][N] (or [rows][N/2] with swiglu)
    const float *residual;
    int32_t swiglu;
    // optional fused RMSNorm of x: x' = x / sqrt(mean(x^2)+eps) * norm_w
    const float *norm_w;
    float eps;
    const RopeFusion *rope = nullptr;  // only where gemv_fuses_rope() says so
    const float *bias[3] = {nullptr, nullptr, nullptr};  // one per stacked matrix, added before the rotation: only together with `rope`
    // Only where gemv_hands_digits() says so: a SwiGLU product leaves its outputs as digit planes (digits_out, in place of y)
    // and the product that follows reads them (digits_in, in place of x) instead of turning floats into digits again.
    uint8_t *digits_out = nullptr;
    const uint8_t *digits_in = nullptr;
    // Only where gemv_merges_sections() says so: the activation row is the attention output these sections merge into
    // (x is not read); the product merges them as it stages its row, and the attention's own fold launch falls away.
    const SectionSums *merge = nullptr;
    // Only for a one-row product of a staged K-quant (Q6_K, Q5_K, Q3_K) over one K slice (K <= 4096): the value projection of a
    // token whose q|k went out rotated from their own product -- its rows (+ bias[0]) are also cast into the value state
    // (cache_v, cursor, width, capacity and ring of this RopeFusion; halves), what launch_value_append does from y.
    const RopeFusion *append_value = nullptr;
    // Products chained into one launch (launch_chain), and a SwiGLU product that hands digit planes on: the numbers (1..127) of
    // the seams this product reads and writes across -- what is handed over carries them as tag words -- and, for a plain
    // product whose outputs another product of the same launch reads, where it leaves them as (value, tag) pairs beside y;
    // then x of the product behind it is that same array.
    uint32_t tag_in = 0, tag_out = 0;
    void *pairs_out = nullptr;
};
int32_t launch_gemv(nh_device *d, const GemvArgs &args);
// whether launch_gemv can merge attention sections of `width` channels a head into the activation row of this product
bool gemv_merges_sections(const GemvArgs &args, uint32_t width);
constexpr uint32_t MERGED_SECTIONS_MOST = 16;  // sections such a product merges at most
// whether `producer` (a SwiGLU product of one row) can hand its outputs to `consumer` as digit planes, and the bytes they take
bool gemv_hands_digits(const GemvArgs &producer, const GemvArgs &consumer);
size_t gemv_digit_bytes(uint32_t K);
// A Q4_K q|k product that folds the rotation in and the Q6_K value projection that appends its own rows, both over the same
// activation row, as one launch (a layer of a Q4_K_M file whose value projection is stored in Q6_K): gemv_pairs() says whether.
bool gemv_pairs(nh_device *d, const GemvArgs &rotated, const GemvArgs &value);
int32_t launch_gemv_pair(nh_device *d, const GemvArgs &rotated, const GemvArgs &value);
// Several dependent one-row Q4_K products as one launch with seams between them: attn_output (`lead`, or nullptr), gate|up
// handing its digit planes to ffn_down, and behind them the next q|k|v with the rotation folded in or the head (`trail`, or
// nullptr).  gemv_chains() says whether launch_chain takes them.
// `spin`: how often a reader may read a piece again whose tag is not the seam's before it gives up with REFUSAL_SEAM.
int gemv_chain_level();  // NEURA_HIP_CHAIN: 0 (the default) one launch a product, 1 gate|up with ffn_down, 2 attn_output in front, 3 a product behind
bool gemv_chains(nh_device *d, const GemvArgs *lead, const GemvArgs &gate_up, const GemvArgs &down, const GemvArgs *trail);
int32_t launch_chain(nh_device *d, const GemvArgs *lead, const GemvArgs &gate_up, const GemvArgs &down, const GemvArgs *trail, uint32_t spin);
// whether a one-row product with `append_value` set casts its rows into the value state from its own epilogue
bool gemv_appends_value(const GemvArgs &a);
// moves the device's tick word on: once at the start of every pass over a decoder's layers, before anything that writes tags
int32_t launch_tick(nh_device *d);
// whether launch_gemv can fold `rope` into this product (else the caller runs the rotation as its own kernel)
bool gemv_fuses_rope(const GemvArgs &args, const RopeFusion &rope);

struct GemmArgs {
    int32_t element;
    const void *W;
    uint32_t N, K;
    const void *X;  // [M][K]
    int32_t x_element;
    uint32_t M;
    float *Y;                // [M][ldy], the first N of every row are written
    const float *residual;   // [M][ldy] or nullptr
    uint32_t ldy;
    // Optional, Q4_K on the matrix cores only (gemm_stacks() says when): two more matrices stacked along N behind W, as the
    // narrow product stacks q|k|v.  end[s] = first output column past matrix s (end[2] == N); unused entries: W_more nullptr.
    const void *W_more[2] = {nullptr, nullptr};
    uint32_t end[2] = {0, 0};
    // the activations were packed by the launch before this one (same X, M, K, nothing else launched on the device's
    // scratch in between): skip the packing pass
    bool packed = false;
    // what the packing pass works on, instead of X as it lies (fp32 X only; the results are the ones the separate kernels give):
    //   norm_w: the rows of X normalised as launch_rmsnorm(X, nullptr, norm_w, eps) writes them;
    //   gate:   silu(gate) * X, element by element, as launch_silu_mul(gate, X) writes it (gate: [M][K] like X).
    const float *norm_w = nullptr;
    float eps = 0.0f;
    const float *gate = nullptr;
};
int32_t launch_gemm(nh_device *d, const GemmArgs &args);
// whether launch_gemm takes a product of this element and depth with matrices stacked along N at these boundaries, or with
// activations the launch before packed
bool gemm_stacks(int32_t element, uint32_t K, const void *X, const void *W0, const void *W1, const void *W2, uint32_t end0, uint32_t end1);
// device scratch a Q4_K wide product over M rows of K activations packs them into
size_t gemm_q4k_scratch_bytes(uint32_t M, uint32_t K, bool half_rows);

int32_t launch_rmsnorm(nh_device *d, const float *x, const float *residual, const float *w, float eps, uint32_t rows, uint32_t C,
                       float *out, float *sum_out);
int32_t launch_rope(nh_device *d, const float *x, uint32_t planes, uint32_t batch, uint32_t rows, uint32_t width,
                    const uint32_t *cursor, float base, float *out);
int32_t launch_cache_write(nh_device *d, const float *k, const float *v, void *cache_k, void *cache_v, uint32_t kv_heads,
                           uint32_t batch, uint32_t rows, uint32_t width, uint32_t capacity, uint32_t window, const uint32_t *cursor,
                           const uint8_t *mask, bool ring, int32_t cache_element = NH_F16);

// q / out addressing: element (head, plane, row, c) at head*sh + plane*sb + row*sr + c
struct AttentionArgs {
    const float *q;
    float *out;
    uint64_t q_sh, q_sb, q_sr, o_sh, o_sb, o_sr;
    const uint16_t *cache_k, *cache_v;
    uint32_t heads, kv_heads, batch, rows, width, capacity, keys;
    const uint32_t *cursor;
    float scale;
    uint32_t reach = 0;  // 0, or the span of a ring cache of `keys` slots (Cache::windowed): the last `reach` positions are weighed
    int32_t cache_element = NH_F16;  // what the caches hold: NH_F16 (the matrix-core kernels), NH_BF16 or NH_F32 (the kernel for any element)
    // Where the caller's next product merges the sections itself (gemv_merges_sections): a decode step of one plane may leave
    // its sections unmerged (at most MERGED_SECTIONS_MOST of them) and say here where they are; sections == 0 on return
    // means `out` holds the merged rows as always.
    SectionSums *unmerged = nullptr;
};
int32_t launch_attention(nh_device *d, const AttentionArgs &args);

// fused decode-side step: rope(q,k) + fp16 cache append from a token-major qkv buffer
// qkv [T][(heads + 2 kv_heads) * width], t = row * batch + plane; q is roped in place.
// cos / sin of every (position, channel pair) the rotation can meet, computed as the rotation kernels compute them
int32_t launch_rope_angles(nh_device *d, float base, uint32_t width, uint32_t positions, float *cosines, float *sines);
int32_t launch_rope_append(nh_device *d, float *qkv, uint32_t heads, uint32_t kv_heads, uint32_t width, uint32_t batch, uint32_t rows,
                           void *cache_k, void *cache_v, uint32_t capacity, uint32_t window, const uint32_t *cursor,
                           const uint8_t *mask, float base, bool ring, int32_t cache_element = NH_F16, const float *cosines = nullptr,
                           const float *sines = nullptr, uint32_t positions = 0);  // (a model's table of cosines and sines, where it has one)

// one token of one plane: v (+ bias) as halves into the value state at cursor[0] (at cursor[0] % ring when the cache is a ring)
int32_t launch_value_append(nh_device *d, const float *v, const float *bias, void *cache_v, uint32_t kv_heads, uint32_t width, uint32_t capacity,
                            const uint32_t *cursor, uint32_t ring, int32_t cache_element = NH_F16);
int32_t launch_columns(nh_device *d, const float *src, uint32_t lds, const float *bias, float *dst, uint32_t ldd, uint32_t rows, uint32_t n);

int32_t launch_pack_q8_0(nh_device *d, const float *src, uint64_t elements, uint8_t *dst);
int32_t launch_gather(nh_device *d, int32_t element, const void *table, uint32_t vocab, uint32_t width, const uint32_t *tokens,
                      uint32_t count, uint32_t batch, const uint8_t *mask, float *out);
// `published`, where given: pinned host words [rows + 1] as the device addresses them; the last kernel writes every row's choice
// there too, and behind them the word at `refusal` (what a decode step's caller reads once the stream has drained)
int32_t launch_argmax(nh_device *d, const float *values, uint32_t rows, uint32_t n, uint32_t *out, uint32_t *published = nullptr,
                      const uint32_t *refusal = nullptr);
// the same choice with its partials in a file-scope device array: no allocation, at most 64 rows
int32_t argmax_static_setup(nh_device *d);
int32_t launch_argmax_static(nh_device *d, const float *values, uint32_t rows, uint32_t n, uint32_t *out);
// sampled choice: `draws` is device memory, one entry a row; check_draws refuses what the reference's host asserts refuse
int32_t launch_sample(nh_device *d, const float *logits, uint32_t rows, uint32_t n, const nh_draw *draws, uint32_t *out);
int32_t check_draws(const nh_draw *draws, uint32_t rows);
int32_t launch_silu_mul(nh_device *d, const float *gate, const float *up, uint64_t n, float *out);
int32_t launch_mask_rows(nh_device *d, float *x, uint32_t rows, uint32_t batch, uint32_t width, const uint8_t *mask);

}  // namespace nh
