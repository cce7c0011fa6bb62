/*
 * neura_hip.h -- C ABI of libneura_hip.so: the MI355X (gfx950) implementation of the
 * quantized-GGUF decoder path of formetaohy/Neura.
 *
 * The reference has no C ABI: the path sits behind its Rust crates neura-runtime /
 * neura-gpu (dispatch), neura-decoder (model helpers) and neura-generate (generation loop).
 * Each entry point below names the reference interface it stands in for, as path:line under
 * the reference root.  A Rust `neura-hip-sys` crate binds these symbols one to one.
 *
 * Conventions
 *   - every function that returns int32_t returns 0 on success and a negative NH_E_* code on
 *     failure; nh_last_error() then returns a thread-local message.  The reference panics
 *     with a prose message in the same situations (a binding turns the code into a panic).
 *   - handles are opaque; one nh_device owns one HIP stream and is used from one thread at a
 *     time (the reference's Runtime is used through `&mut Batch`, one thread).
 *   - "dev" pointers are device memory of that nh_device; "host" pointers are caller memory.
 *   - matrices are GGUF tensors in place: W is [N][K] row-major, K contiguous, stored as raw
 *     ggml blocks (crates/neura-decoder/src/parameter.rs:5-15, crates/neura-runtime/src/store.rs:77-141).
 *   - element ids are ggml type ids (crates/neura-gguf/src/header.rs:150-162).
 *   - all work is enqueued on the device's stream; host-visible results are complete when the
 *     call that returns them (nh_download, nh_decode_step, nh_timer_stop, nh_sync) returns.
 */
#ifndef NEURA_HIP_H
#define NEURA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct nh_device nh_device;
typedef struct nh_weights nh_weights;
typedef struct nh_model nh_model;

enum {
    NH_F32 = 0,   /* Element::Single   */
    NH_F16 = 1,   /* Element::Half     */
    NH_BF16 = 30, /* Element::Bfloat16: a key / value cache element only (crates/neura-decoder/src/cache.rs:130-134) */
    NH_Q8_0 = 8,  /* Element::Q8_0: 32 elements / 34 bytes  (crates/neura-abi/src/element.rs:155-158) */
    NH_Q3_K = 11, /* Element::Q3K: 256 elements / 110 bytes (crates/neura-abi/src/element.rs:171-174) */
    NH_Q4_K = 12, /* Element::Q4K: 256 elements / 144 bytes (crates/neura-abi/src/element.rs:159-162) */
    NH_Q5_K = 13, /* Element::Q5K: 256 elements / 176 bytes (crates/neura-abi/src/element.rs:163-166) */
    NH_Q6_K = 14  /* Element::Q6K: 256 elements / 210 bytes (crates/neura-abi/src/element.rs:167-170) */
};

enum {
    NH_OK = 0,
    NH_E_ARGUMENT = -1, /* a shape, pointer or element the call cannot take */
    NH_E_DEVICE = -2,   /* a HIP call failed (GpuUnavailable, crates/neura-runtime/src/runtime.rs:183) */
    NH_E_MEMORY = -3,   /* device allocation failed */
    NH_E_REFUSAL = -4   /* the device refused an index or origin (crates/neura-abi/src/refusal.rs:73-96) */
};

/* Epilogue of a product: the reference fuses these through `chained`
 * (crates/neura-kernel/src/pointwise.rs:90-104). */
typedef struct nh_epilogue {
    const float *residual; /* dev, [rows][N] or NULL: y = residual + W·x (residual add, examples/qwen/mlp.rs:35) */
    int32_t swiglu;        /* 1: W holds gate rows [0,N/2) then up rows [N/2,N); y[rows][N/2] = silu(gate)·up
                              (examples/qwen/mlp.rs:31-33, crates/neura-pointwise/src/op.rs:163) */
} nh_epilogue;

/* ---- device, memory, timing : replaces crates/neura-gpu/src/native.rs:231-425 -------------- */

/* Runtime::open (crates/neura-runtime/src/runtime.rs:183).  NULL when no usable gfx950 device. */
nh_device *nh_open(int32_t device_index);
void nh_close(nh_device *device);
/* thread-local message of the last failed call on this thread ("" if none) */
const char *nh_last_error(void);
/* NativeDevice::create_buffer (crates/neura-gpu/src/native.rs:231); contents are zeroed */
void *nh_alloc(nh_device *device, size_t bytes);
int32_t nh_free(nh_device *device, void *dev);
/* NativeDevice::write_host / read_host (crates/neura-gpu/src/native.rs:231-425); both are
 * complete on return */
int32_t nh_upload(nh_device *device, void *dev_dst, const void *host_src, size_t bytes);
int32_t nh_download(nh_device *device, void *host_dst, const void *dev_src, size_t bytes);
/* Command::Copy (crates/neura-gpu/src/submission.rs:17-35): device to device, enqueued */
int32_t nh_copy(nh_device *device, void *dev_dst, const void *dev_src, size_t bytes);
/* Command::Clear (crates/neura-gpu/src/submission.rs:17-35) */
int32_t nh_clear(nh_device *device, void *dev, size_t bytes);
/* NativeDevice::wait (crates/neura-gpu/src/native.rs:231-425) */
int32_t nh_sync(nh_device *device);
/* Run::seconds (crates/neura-runtime/src/runtime.rs:130-135): device time between the two
 * calls, taken with HIP events on the device's own stream */
int32_t nh_timer_start(nh_device *device);
int32_t nh_timer_stop(nh_device *device, double *seconds_out);

/* Per-kernel timing as the reference's benchmark takes it (GPU timestamps around each
 * submission, crates/neura-gpu/src/native/vulkan.rs:1234-1276; examples/benchmark/measure.rs:4-33):
 * between begin and end every narrow-product launch on this device is bracketed by a HIP event
 * pair on the device's stream.  end returns the summed device seconds of those launches, their
 * count and the weight bytes they walked (payload bytes, counted once per launch:
 * examples/benchmark/product.rs:103-105). */
int32_t nh_profile_begin(nh_device *device);
int32_t nh_profile_end(nh_device *device, double *seconds_out, uint64_t *launches_out, uint64_t *bytes_out);

/* ---- weight arena : replaces Runtime::load (crates/neura-runtime/src/runtime.rs:356-367) ---- */

/* one arena of `bytes`; tensors are poured verbatim at 256-byte aligned offsets the caller
 * picks (crates/neura-plan/src/layout.rs:29-36) */
nh_weights *nh_weights_create(nh_device *device, size_t bytes);
void nh_weights_destroy(nh_weights *weights);
/* pour_one (crates/neura-runtime/src/store.rs:77-141): raw ggml bytes, no repacking */
int32_t nh_weights_put(nh_weights *weights, size_t at, const void *host_bytes, size_t bytes);
/* device address of arena offset `at` */
void *nh_weights_at(nh_weights *weights, size_t at);
size_t nh_weights_bytes(const nh_weights *weights);

/* ---- operators : replace the run_<kind> bodies of crates/neura-kernel ---------------------- */

/* fetch_q8_0 / fetch_q3_k / fetch_q4_k / fetch_q5_k / fetch_q6_k / fetch_half (crates/neura-kernel/src/fetch.rs:236-303, :95-98) ==
 * unpack (crates/neura-precision/src/ggml.rs:211-216, :291-350, :394-407): bit-exact fp32 values of NH_Q8_0, NH_Q3_K, NH_Q4_K,
 * NH_Q5_K, NH_Q6_K, NH_F16 or NH_F32 storage */
int32_t nh_dequant(nh_device *device, int32_t element, const void *dev_src, uint64_t elements, float *dev_dst);
/* run_convert_half (crates/neura-kernel/src/task/convert.rs:229-249): fp32 -> fp16 RNE */
int32_t nh_convert_half(nh_device *device, const float *dev_src, uint64_t elements, uint16_t *dev_dst);
/* run_convert_q8_0 with q8_0_quantum and q8_0_code (crates/neura-kernel/src/task/convert.rs:355-430), the device twin of
 * the host's q8_0 encoder (crates/neura-precision/src/ggml.rs:209-216): `elements` fp32 numbers into ceil(elements / 32) blocks
 * of 34 bytes (a ragged last block counts zeros behind its numbers).  dev_dst holds the blocks rounded up to a four-byte word;
 * the two bytes behind an odd number of blocks are written as zero, as the host's pack writes them.  dev_src on a 16-byte
 * boundary. */
int32_t nh_pack_q8_0(nh_device *device, const float *dev_src, uint64_t elements, void *dev_dst);
/* narrow product, rows <= 8 (template_run_matmul_folded{,_fused,_quad},
 * crates/neura-kernel/src/task/matmul.rs:376-803): y[r][n] = sum_k x[r][k]·W[n][k], fp32; W in NH_Q8_0, NH_Q3_K, NH_Q4_K,
 * NH_Q5_K or NH_Q6_K blocks (the dots of crates/neura-kernel/src/dot.rs:471-797) */
int32_t nh_gemv(nh_device *device, int32_t element, const void *dev_W, uint32_t N, uint32_t K, const float *dev_x, uint32_t rows,
                float *dev_y, const nh_epilogue *epilogue);
/* wide product (template_run_matmul_codes / _run, crates/neura-kernel/src/task/matmul.rs:943-1221):
 * X [M][K] in x_element (NH_F32 or NH_F16), Y fp32 [M][N]; W in the same five block formats */
int32_t nh_gemm(nh_device *device, int32_t element, const void *dev_W, uint32_t N, uint32_t K, const void *dev_X, int32_t x_element,
                uint32_t M, float *dev_Y, const nh_epilogue *epilogue);
/* run_norm NORM_RMS (crates/neura-kernel/src/task/norm.rs:55-130, :350-369):
 * v = x (+ residual); out = v / sqrt(mean(v^2) + eps) * w.  sum_out (may be NULL) receives v. */
int32_t nh_rmsnorm(nh_device *device, const float *dev_x, const float *dev_residual, const float *dev_w, float eps, uint32_t rows,
                   uint32_t C, float *dev_out, float *dev_sum_out);
/* run_rope (crates/neura-kernel/src/task/rope.rs:52-123): rotate-half over all `width`
 * channels of x [planes][batch][rows][width]; position = cursor[plane of batch] + row */
int32_t nh_rope(nh_device *device, const float *dev_x, uint32_t planes, uint32_t batch, uint32_t rows, uint32_t width,
                const uint32_t *dev_cursor, float base, float *dev_out);
/* Cache::write / write_masked (crates/neura-decoder/src/cache.rs:267-352): cast to fp16 then
 * scatter rows.  k, v are fp32 [kv_heads][batch][rows][width]; the caches are fp16
 * [kv_heads][batch][capacity][width]; row index = cursor[b] + row, or window + row for a
 * plane whose dev_mask byte is 0 (dev_mask may be NULL = all active).  ring != 0 is Cache::windowed (cache.rs:67-69,
 * :311-317; crates/neura-decoder/src/layout.rs:32-36): the window is a ring, row index = (cursor[b] + row) mod window. */
int32_t nh_cache_write(nh_device *device, const float *dev_k, const float *dev_v, uint16_t *dev_cache_k, uint16_t *dev_cache_v,
                       uint32_t kv_heads, uint32_t batch, uint32_t rows, uint32_t width, uint32_t capacity, uint32_t window,
                       const uint32_t *dev_cursor, const uint8_t *dev_mask, int32_t ring);
/* Cache::attend -> run_attention (+ run_attention_fold) (crates/neura-decoder/src/cache.rs:366-406,
 * crates/neura-kernel/src/task/attention.rs:309-671): causal GQA attention of q
 * [heads][batch][rows][width] over fp16 caches [kv_heads][batch][capacity][width], the first
 * `keys` rows visible; key `at` is weighed iff at <= cursor[b] + row.  out like q.
 * reach (AttentionOptions::reach, cache.rs:391-394; key_position / weighed, attention.rs:103-108, :136-144): 0, or the
 * span of a ring of `keys` slots -- slot `at` then holds the latest position below cursor[b] + rows that lands on it, a query
 * weighs the `reach` positions up to its own, and a cursor past `keys` is no refusal. */
int32_t nh_attention(nh_device *device, const float *dev_q, const uint16_t *dev_cache_k, const uint16_t *dev_cache_v, uint32_t heads,
                     uint32_t kv_heads, uint32_t batch, uint32_t rows, uint32_t width, uint32_t capacity, uint32_t keys, uint32_t reach,
                     const uint32_t *dev_cursor, float scale, float *dev_out);
/* nh_cache_write and nh_attention over states of another element (Cache::new(.., Element::Single | Half | Bfloat16),
 * crates/neura-decoder/src/cache.rs:130-134; the reference's cache tests run Single and Half, tests/cache.rs:17): the caches
 * are arrays of `cache_element` (NH_F16, NH_BF16 or NH_F32), everything else as above.  Chunks of one row and of four and more rows at head widths 64 and 128 ride the
 * same matrix-core kernels whatever the element (bfloat16 as the halves they equal, single as two half planes). */
int32_t nh_cache_write_element(nh_device *device, const float *dev_k, const float *dev_v, void *dev_cache_k, void *dev_cache_v,
                               uint32_t kv_heads, uint32_t batch, uint32_t rows, uint32_t width, uint32_t capacity, uint32_t window,
                               const uint32_t *dev_cursor, const uint8_t *dev_mask, int32_t ring, int32_t cache_element);
int32_t nh_attention_element(nh_device *device, const float *dev_q, const void *dev_cache_k, const void *dev_cache_v, uint32_t heads,
                             uint32_t kv_heads, uint32_t batch, uint32_t rows, uint32_t width, uint32_t capacity, uint32_t keys,
                             uint32_t reach, const uint32_t *dev_cursor, float scale, float *dev_out, int32_t cache_element);
/* run_gather (crates/neura-kernel/src/task/select.rs:29-49): out[t][:] = dequant(table[token[t]]),
 * times mask[t % batch] when dev_mask != NULL.  A token id >= vocab is refused. */
int32_t nh_gather(nh_device *device, int32_t element, const void *dev_table, uint32_t vocab, uint32_t width, const uint32_t *dev_tokens,
                  uint32_t count, uint32_t batch, const uint8_t *dev_mask, float *dev_out);
/* run_argmax (crates/neura-kernel/src/task/choice.rs:355-368): per row, lowest index wins ties */
int32_t nh_argmax(nh_device *device, const float *dev_values, uint32_t rows, uint32_t n, uint32_t *dev_out);
/* No counterpart in the reference.  nh_argmax for callers that cannot allocate (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): the same two kernels and the same result, with the section partials in a
 * 512 KiB array that is part of the library's device image (one copy per GPU, held until the process ends) instead of the
 * device scratch that nh_argmax may grow.  It calls no hipMalloc, hipFree or allocating routine.  rows <= 64 (any n); more
 * is refused with NH_E_ARGUMENT.  Nothing in the array has to start at zero (every partial is written before it is read).
 * All calls on one GPU share that GPU's array: calls that overlap on one GPU (two streams, two handles) race. */
int32_t nh_argmax_static(nh_device *device, const float *dev_values, uint32_t rows, uint32_t n, uint32_t *dev_out);

/* What one row draws with (Sampling::Sampled and the per-plane states of a sampled batch,
 * crates/neura-generate/src/sampling.rs:3-36, crates/neura-generate/src/batch.rs:383-386): the seed's 32 bits as the
 * kernel hashes them, the temperature the logits are divided by, the number of largest logits kept (1..64) and the
 * cumulative softmax mass the kept ones are cut at (0 < cumulative <= 1). */
typedef struct nh_draw {
    uint32_t seed;
    float temperature;
    uint32_t keep;
    float cumulative;
} nh_draw;
/* graph.sample over logits * recip(temperature) (crates/neura-generate/src/sampling.rs:69-94; run_sample / run_sample_fold,
 * crates/neura-kernel/src/task/choice.rs:933-989, :1109-1123, :1270-1359): per row the `keep` largest values, cut where
 * their running softmax mass plus the mass outside them reaches cumulative * total, then the largest of
 * value + gumbel_noise(seed, column) (choice.rs:81-89), the lowest column among equals.  keep == 1 is the argmax.
 * `host_draws`: rows entries of caller memory.  A row holds at most 262144 columns. */
int32_t nh_sample(nh_device *device, const float *dev_logits, uint32_t rows, uint32_t n, const nh_draw *host_draws, uint32_t *dev_out);

/* ---- decoder model : replaces the compiled answer / fill programs of Batch ------------------ */

/* Qwen2-style decoder (composition of examples/qwen/model.rs:92-103, attention.rs:98-154,
 * mlp.rs:29-36 without the qwen35 q-gate and q/k norms). */
typedef struct nh_model_config {
    uint32_t layers, hidden, heads, kv_heads, head_dim, ffn, vocab;
    uint32_t context;    /* BatchSpec.context */
    uint32_t batch;      /* BatchSpec.batch (planes) */
    uint32_t max_rows;   /* widest fill chunk (BatchSpec.chunks[0]), 1 if none */
    uint32_t window;     /* BatchSpec.window (crates/neura-generate/src/batch.rs:148-152): 0 = none; else the caches are rings of
                            `window` positions (+ max_rows scratch rows) and a sequence attends to its last `window` tokens */
    float rope_base;     /* <arch>.rope.freq_base */
    float eps;           /* <arch>.attention.layer_norm_rms_epsilon */
    int32_t cache_element; /* what the key and value states hold (Cache::new(.., element), crates/neura-decoder/src/cache.rs:63,
                              :130-134): NH_F16, NH_BF16 or NH_F32 -- NH_F32 is 0, so a config that never names it keeps single
                              precision states as the reference's own example does (examples/qwen/main.rs:107); the headline
                              workload names NH_F16.  Every element takes the fused kernels (single and bfloat16 states are
                              read onto the matrix cores as halves: magnitudes past 65504 overflow as in half states).
                              Keys and values are cast on their way in (graph.cast, cache.rs:347-348;
                              bfloat16 rounds to nearest even, crates/neura-kernel/src/task/convert.rs:86-89) */
} nh_model_config;

/* where each tensor sits in the arena (byte offsets) and its element.  Per layer arrays have
 * `layers` entries.  output == UINT64_MAX ties the head to token_embd (examples/qwen/model.rs:81-84). */
typedef struct nh_tensor_table {
    int32_t matrix_element; /* element of every matrix: NH_Q8_0, NH_Q3_K, NH_Q4_K, NH_Q5_K or NH_Q6_K */
    uint64_t token_embd, output, output_norm;
    const uint64_t *attn_norm, *attn_q, *attn_k, *attn_v, *attn_output, *ffn_norm, *ffn_gate, *ffn_up, *ffn_down;
    /* Optional, NULL = absent.
     * matrix_elements: the element of each matrix where a file mixes them (a Q4_K_M file keeps some matrices in Q6_K;
     * neura-gguf hands every tensor over with its own element, crates/neura-gguf/src/header.rs:10-17):
     * [token_embd, output, then per layer attn_q, attn_k, attn_v, attn_output, ffn_gate, ffn_up, ffn_down], 2 + 7 * layers
     * entries of NH_Q8_0 / NH_Q3_K / NH_Q4_K / NH_Q5_K / NH_Q6_K.  NULL: every matrix is `matrix_element`.
     * attn_{q,k,v}_bias: byte offsets of f32 [rows] vectors per layer, UINT64_MAX = none, added to the projection before the
     * rotation.  Qwen2 checkpoints carry them (blk.N.attn_q.bias ...); the reference's own qwen example has none
     * (examples/qwen/attention.rs:98-154), so they have no counterpart there. */
    const int32_t *matrix_elements;
    const uint64_t *attn_q_bias, *attn_k_bias, *attn_v_bias;
} nh_tensor_table;

/* Batch::new (crates/neura-generate/src/batch.rs:279-465): allocates fp16 K/V caches of
 * capacity = (window, or context without one) + max_rows per (layer, kv head, plane) and every activation buffer. */
nh_model *nh_model_create(nh_device *device, const nh_model_config *config, nh_weights *weights, const nh_tensor_table *table);
void nh_model_destroy(nh_model *model);
/* the answer program (crates/neura-generate/src/batch.rs:1716-1725): one token per plane.
 * host arrays of `batch` entries; mask 0 = inactive plane.  chosen_out[b] = argmax of the logits. */
int32_t nh_decode_step(nh_model *model, const uint32_t *tokens, const uint32_t *cursors, const uint8_t *mask, uint32_t batch,
                       uint32_t *chosen_out);
/* the answer program of a sampled batch (crates/neura-generate/src/batch.rs:330-398, sampling.rs:69-94): as nh_decode_step,
 * with chosen_out[b] drawn from plane b's logits as nh_sample draws it with host_draws[b]. */
int32_t nh_decode_step_sampled(nh_model *model, const uint32_t *tokens, const uint32_t *cursors, const uint8_t *mask, uint32_t batch,
                               const nh_draw *host_draws, uint32_t *chosen_out);
/* a fill program (crates/neura-generate/src/batch.rs:1434-1517): `rows` tokens per plane,
 * tokens[row * batch + plane]; no logits, no readback. */
int32_t nh_prefill(nh_model *model, const uint32_t *tokens, uint32_t rows, const uint32_t *cursors, const uint8_t *mask, uint32_t batch);
/* Runtime::measure restricted to the products (crates/neura-runtime/src/runtime.rs:807-816,
 * examples/benchmark/product.rs:19-107): launches every narrow product of one decode step
 * (same matrices, shapes and buffers, nothing else) `steps` times back to back on the device's
 * stream between one pair of HIP events.  Returns the device seconds, the number of product
 * launches and the weight payload bytes they walked. */
int32_t nh_model_time_products(nh_model *model, uint32_t steps, double *seconds_out, uint64_t *launches_out, uint64_t *bytes_out);
/* the reset program (crates/neura-generate/src/batch.rs:1094-1100): zero the caches of planes
 * whose reset byte is non-zero */
int32_t nh_model_reset(nh_model *model, const uint8_t *reset, uint32_t batch);
/* Runtime::read of the logits value (crates/neura-runtime/src/runtime.rs:1064-1067): logits of
 * the last decode step, [batch][vocab] */
int32_t nh_model_logits(nh_model *model, float *host_out);
/* Runtime::restore_state / save_state of "blk.{i}.cache.key|value"
 * (crates/neura-decoder/src/cache.rs:135-137): [kv_heads][batch][capacity][head_dim] numbers of the config's cache_element,
 * as they lie (2 bytes each for NH_F16 and NH_BF16, 4 for NH_F32) */
int32_t nh_model_cache_write(nh_model *model, uint32_t layer, int32_t value_not_key, const void *host_src);
int32_t nh_model_cache_read(nh_model *model, uint32_t layer, int32_t value_not_key, void *host_dst);
uint32_t nh_model_capacity(const nh_model *model);
/* A decode step of one plane runs the products between two attentions as one launch with seams between them, the way the
 * reference runs a whole program as one persistent kernel (crates/neura-kernel/src/scheduler.rs:110-166).  A seam's wait is
 * bounded; where one gave up, the step was run again one launch a product and the model stays on that path.  This counts
 * those steps (0 in a healthy process). */
uint32_t nh_model_seam_fallbacks(const nh_model *model);
/* The shared prefix of a batch that declares one (Cache::with_shared / Cache::shared, crates/neura-decoder/src/cache.rs:71-90,
 * :138-161; Batch::prefix, crates/neura-generate/src/batch.rs:885-994): one more plane of keys and values per layer,
 * fp16 [kv_heads][1][capacity][head_dim], zero until kept.
 * nh_model_keep_prefix: the shared plane becomes a copy of plane `plane` -- the prefix program's result, once the caller has
 *   fed the prefix to that plane with nh_prefill / nh_decode_step while no plane holds a sequence.
 * nh_model_reset_shared: the reset program with its share input (cache.rs:223-250, batch.rs:1094-1100): a plane whose share
 *   byte is set becomes a copy of the shared plane, else a plane whose reset byte is set is zeroed.
 * nh_model_shared_write / _read: Runtime::restore_state / save_state of "blk.{i}.cache.shared.key|value". */
int32_t nh_model_keep_prefix(nh_model *model, uint32_t plane);
int32_t nh_model_reset_shared(nh_model *model, const uint8_t *reset, const uint8_t *share, uint32_t batch);
int32_t nh_model_shared_write(nh_model *model, uint32_t layer, int32_t value_not_key, const void *host_src);
int32_t nh_model_shared_read(nh_model *model, uint32_t layer, int32_t value_not_key, void *host_dst);

#ifdef __cplusplus
}
#endif
#endif /* NEURA_HIP_H */
