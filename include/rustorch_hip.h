/*
 * rustorch_hip.h -- C ABI of the MI355X (gfx950) backend for RusTorch's GGUF
 * quantized-inference path.
 *
 * The reference has no native FFI for GPUs (its CUDA / Metal / OpenCL backends
 * are Rust crates), so this ABI is shaped by the Rust signatures it sits under.
 * Each group below names the reference interface it replaces or extends
 * (paths relative to the reference checkout).
 *
 * Conventions
 *   - every function returns an rt_hip_status (0 = ok); it never aborts and no
 *     C++ exception crosses the boundary.  rt_hip_last_error() gives the text.
 *     The Rust shim maps the codes 1:1 onto RusTorchError variants
 *     (src/error.rs:15-300): INVALID_ARG -> InvalidParameters, SHAPE ->
 *     ShapeMismatch, NO_DEVICE -> DeviceNotAvailable, OOM -> OutOfMemory,
 *     HIP -> Gpu, UNSUPPORTED_TYPE -> BackendUnavailable/UnsupportedOperation.
 *     A GPU failure is an error, never a silent CPU fallback
 *     (policy of src/gpu/matrix_ops.rs:408-425).
 *   - `const` pointer arguments are borrowed until the call returns.
 *   - names ending in _dev take device pointers obtained from rt_hip_malloc and
 *     only enqueue work on the context's stream; the other entry points take
 *     host pointers and block until the result is in host memory (the contract
 *     of CudaKernelExecutor::matmul_f32, src/gpu/cuda_kernels.rs:231-283).
 *   - a context may be moved between threads; calls on one context are
 *     serialised internally; distinct contexts are independent.  There is no
 *     global mutable state (contrast src/gpu/mod.rs:757-772) apart from atomic
 *     per-device flags that record that a kernel's LDS limit has been raised
 *     (setting it twice is harmless, so they need no lock) and the atomic
 *     code-path switches of rt_hip_set_option.
 */
#ifndef RUSTORCH_HIP_H
#define RUSTORCH_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RT_HIP_API __attribute__((visibility("default")))

typedef enum {
    RT_HIP_OK = 0,
    RT_HIP_ERR_INVALID_ARG = 1,
    RT_HIP_ERR_SHAPE = 2,
    RT_HIP_ERR_NO_DEVICE = 3,
    RT_HIP_ERR_OOM = 4,
    RT_HIP_ERR_HIP = 5,
    RT_HIP_ERR_UNSUPPORTED_TYPE = 6
} rt_hip_status;

/* GGML type ids, the values of GGMLType (example-cli/src/model/formats/gguf.rs:78-99).  The ids listed here have the exact
 * dequantization and a GEMV kernel; Q4_K and Q6_K also have the fused matrix-core contraction, the others reach the matrix
 * cores through an fp16 copy.  Any other id is refused with RT_HIP_ERR_UNSUPPORTED_TYPE. */
typedef enum {
    RT_GGML_F32 = 0,
    RT_GGML_F16 = 1,
    RT_GGML_Q4_0 = 2,
    RT_GGML_Q4_1 = 3,
    RT_GGML_Q5_0 = 6,
    RT_GGML_Q5_1 = 7,
    RT_GGML_Q8_0 = 8,
    RT_GGML_Q8_1 = 9,
    RT_GGML_Q2_K = 10,
    RT_GGML_Q3_K = 11,
    RT_GGML_Q4_K = 12,
    RT_GGML_Q5_K = 13,
    RT_GGML_Q6_K = 14
} rt_ggml_type;

typedef struct rt_hip_ctx rt_hip_ctx;         /* executor: device, stream, scratch */
typedef struct rt_hip_qweight rt_hip_qweight; /* raw GGUF blocks resident in HBM */
typedef struct rt_hip_llama rt_hip_llama;     /* weights + KV cache + decode-step state */
typedef struct rt_hip_llama_batch rt_hip_llama_batch; /* KV caches and activations of several sequences decoded against one model */
typedef struct rt_hip_event rt_hip_event;     /* timing marker on the context's stream */

typedef struct {
    char name[128];
    char arch[64];
    int compute_units;
    int wavefront_size;
    size_t hbm_bytes;
    size_t lds_bytes_per_block;
} rt_hip_devinfo;

/* ---- device identity: DeviceType / is_available / GpuContext::new
 *      (src/gpu/mod.rs:227-258,429-486,511-599).  Rust adds DeviceType::Hip(usize). */
RT_HIP_API int rt_hip_device_count(void);
RT_HIP_API int rt_hip_device_info(int device, rt_hip_devinfo *out);

/* ---- executor object: CudaKernelExecutor::new(device_id) and its Drop
 *      (src/gpu/cuda_kernels.rs:211-227, src/gpu/cuda_enhanced.rs:30-60). */
RT_HIP_API int rt_hip_create(int device, rt_hip_ctx **out);
RT_HIP_API int rt_hip_destroy(rt_hip_ctx *ctx);
/* GpuDevice::synchronize (src/gpu/device.rs:9-48). */
RT_HIP_API int rt_hip_synchronize(rt_hip_ctx *ctx);
/* Text of the last failure on this context (thread-local text when ctx is NULL). */
RT_HIP_API const char *rt_hip_last_error(rt_hip_ctx *ctx);
/* bytes per block / elements per block of a GGML type: GGMLType::type_size (gguf.rs:125-144); 0 if unsupported. */
RT_HIP_API size_t rt_hip_type_block_bytes(int ggml_type);
RT_HIP_API size_t rt_hip_type_block_elems(int ggml_type);

/* ---- code-path switches (no reference counterpart; the nearest thing is the cargo feature set that picks a backend,
 *      Cargo.toml:166).  Where two kernels serve one call, the one with the longer record on the device is the default and
 *      the other is opt-in: process-wide, atomic, read at every launch, so a caller can run one call each way and compare.
 *      Initial values come from the environment (RUSTORCH_HIP_GEMV_LEAN, RUSTORCH_HIP_DENSE_MFMA: the value as one digit).
 *      Unknown options and values are refused with RT_HIP_ERR_INVALID_ARG. */
typedef enum {
    RT_HIP_OPT_GEMV_LEAN = 1,  /* 1: decode GEMV launches whose problems are all Q4_K / Q6_K / Q8_0 / Q4_0 take the lean kernel; 2: the same, and
                                * launches without a gate / up pair problem run it with five waves per SIMD (640-thread workgroups);
                                * 0 (default): the general kernel */
    RT_HIP_OPT_DENSE_MFMA = 2  /* 1: dense f32 products in whole 16-byte pieces take the f32 matrix-core kernel; 0 (default): the LDS-tiled one */
} rt_hip_option;
RT_HIP_API int rt_hip_set_option(rt_hip_ctx *ctx, int option, int value);
RT_HIP_API int rt_hip_get_option(rt_hip_ctx *ctx, int option, int *value);

/* ---- resident buffers: the GpuBuffer<T> idiom (src/gpu/memory_ops/buffer.rs:22-48). */
RT_HIP_API int rt_hip_malloc(rt_hip_ctx *ctx, size_t nbytes, void **out_dev);
RT_HIP_API int rt_hip_free(rt_hip_ctx *ctx, void *dev);
RT_HIP_API int rt_hip_memcpy_h2d(rt_hip_ctx *ctx, void *dst_dev, const void *src_host, size_t nbytes);
RT_HIP_API int rt_hip_memcpy_d2h(rt_hip_ctx *ctx, void *dst_host, const void *src_dev, size_t nbytes);
RT_HIP_API int rt_hip_memset_dev(rt_hip_ctx *ctx, void *dst_dev, int byte, size_t nbytes);

/* ---- timing markers on the context's stream (used by the bench; no reference counterpart). */
RT_HIP_API int rt_hip_event_create(rt_hip_ctx *ctx, rt_hip_event **out);
RT_HIP_API int rt_hip_event_record(rt_hip_ctx *ctx, rt_hip_event *ev);
RT_HIP_API int rt_hip_event_elapsed_ms(rt_hip_ctx *ctx, rt_hip_event *start, rt_hip_event *stop, float *ms);
RT_HIP_API int rt_hip_event_destroy(rt_hip_ctx *ctx, rt_hip_event *ev);

/* Measurement aid (used by the bench; no reference counterpart): read the first nbytes / 2048 * 2048 bytes of a device
 * buffer once, in the access shape of the decode GEMV's weight stream, and discard them.  The rate it reaches is the
 * practical read ceiling of the device that the GEMV's achieved rate is reported beside. */
RT_HIP_API int rt_hip_stream_read_dev(rt_hip_ctx *ctx, const void *dev, size_t nbytes);

/* ---- dense f32 matmul: CudaKernelExecutor::matmul_f32(a,b,c,m,n,k)
 *      (src/gpu/cuda_kernels.rs:231-239; callers src/gpu/kernels.rs:316,
 *      src/gpu/matrix_ops.rs:378-386).  Row-major a[m,k] . b[k,n] -> c[m,n], host slices, blocking. */
RT_HIP_API int rt_hip_matmul_f32(rt_hip_ctx *ctx, const float *a, const float *b, float *c, size_t m, size_t n,
                                 size_t k);

/* The same product on resident buffers (the GpuBuffer idiom, src/gpu/memory_ops/buffer.rs:22-48), enqueue only, and for a
 * batch of products laid out one after the other: c_dev[i] = a_dev[i] . b_dev[i], i < batch -- what
 * GpuLinearAlgebra::{gpu_matmul, gpu_batch_matmul, gpu_matvec} (src/gpu/matrix_ops.rs:562-595) and
 * GpuBatchMatrixExecutor::batch_matmul (:308-343) ask of a device; a matrix-vector product is n = 1.
 * Both forms run the f32 matrix-core kernel when m, n >= 64, k >= 16, n and k are multiples of 4 and the bases are
 * 16-byte aligned (f32 in, f32 accumulate; the order of the k additions is the hardware's), and a plain tiled kernel
 * that adds k in ascending order otherwise. */
RT_HIP_API int rt_hip_matmul_f32_dev(rt_hip_ctx *ctx, const float *a_dev, const float *b_dev, float *c_dev, size_t m,
                                     size_t n, size_t k, size_t batch);

/* ---- per-tensor affine int8 matmul: QuantizedOps::qmatmul
 *      (src/quantization/operations.rs:195-260), which OptimizedOps::qmatmul
 *      (src/quantization/hardware/mod.rs:25-46) reaches on every device through
 *      qmatmul_cuda / qmatmul_cpu (hardware/cuda.rs:12-26, hardware/cpu.rs:281-288).
 *      Row-major a[m,k] . b[k,n] with zero points removed, summed exactly; the
 *      result is re-quantized to int8 with scale scale_a*scale_b (returned in
 *      *out_scale) and zero point 0 (*out_zero_point).  Host slices, blocking.
 *      Zero points beyond +-1024 are refused (RT_HIP_ERR_INVALID_ARG). */
RT_HIP_API int rt_hip_qmatmul_i8(rt_hip_ctx *ctx, const int8_t *a, float scale_a, int zero_point_a, const int8_t *b,
                                 float scale_b, int zero_point_b, size_t m, size_t n, size_t k, int8_t *out,
                                 float *out_scale, int *out_zero_point);

/* ---- quantized weights under Linear / qmatmul: the device arm of
 *      OptimizedOps::qmatmul (src/quantization/hardware/mod.rs:25-46) and the
 *      weight side of Linear::forward (src/nn/linear.rs:150-182, W stored [out,in]).
 *      raw_blocks is the tensor payload exactly as it sits in the GGUF file:
 *      n_rows rows (output features) of n_cols/block_elems blocks; it is copied
 *      to HBM byte for byte.  nbytes must equal n_rows*(n_cols/block_elems)*block_bytes. */
RT_HIP_API int rt_hip_qweight_upload(rt_hip_ctx *ctx, int ggml_type, size_t n_rows, size_t n_cols,
                                     const void *raw_blocks, size_t nbytes, rt_hip_qweight **out);
/* Wrap blocks that are already in device memory (no copy; the caller keeps ownership of dev_blocks).  The kernels read
 * rows with 16-byte loads that may start inside a row's last block: dev_blocks must be 16-byte aligned and be followed by
 * at least 64 readable bytes beyond nbytes (rt_hip_qweight_upload allocates that slack itself). */
RT_HIP_API int rt_hip_qweight_wrap_dev(rt_hip_ctx *ctx, int ggml_type, size_t n_rows, size_t n_cols,
                                       const void *dev_blocks, size_t nbytes, rt_hip_qweight **out);
RT_HIP_API int rt_hip_qweight_free(rt_hip_ctx *ctx, rt_hip_qweight *w);
/* Decode the whole tensor to f32 [n_rows, n_cols]: TensorLoader::load_tensor / dequantize_tensor
 * (example-cli/src/model/formats/tensor_loader.rs:41-67,125-141) with real block decode; bit-exact. */
RT_HIP_API int rt_hip_dequant(rt_hip_ctx *ctx, const rt_hip_qweight *w, float *out_host);
RT_HIP_API int rt_hip_dequant_dev(rt_hip_ctx *ctx, const rt_hip_qweight *w, float *out_dev);
/* y[batch, n_rows] = x[batch, n_cols] . dequant(W)^T, batch 1..8 (decode): Linear::forward without bias.
 * Q4_K / Q6_K weights with batch >= 3 are read once for the whole batch (integer matrix-core kernel, rows quantized by a
 * small launch ahead of it); other formats and batch 2 run the one-row kernel per row. */
RT_HIP_API int rt_hip_qgemv(rt_hip_ctx *ctx, const rt_hip_qweight *w, const float *x, float *y, int batch);
RT_HIP_API int rt_hip_qgemv_dev(rt_hip_ctx *ctx, const rt_hip_qweight *w, const float *x_dev, float *y_dev,
                                int batch);
/* n weight matrices with the same n_cols against ONE activation batch x_dev[batch][n_cols] (the q / k / v projections of
 * an attention block, gate / up of a feed-forward block: example-cli/src/model/architectures/gpt.rs:192-215 calls
 * Linear::forward on the same input for each): ys_dev[i] is [batch][n_rows_i].  For Q4_K / Q6_K weights and batch >= 3 the
 * rows are quantized once and up to four matrices of one format share a launch; the other weights (another format, fewer
 * rows) are the problems of one launch of the one-row kernel.  n in 1..8. */
RT_HIP_API int rt_hip_qgemv_shared_x_dev(rt_hip_ctx *ctx, int n, const rt_hip_qweight *const *ws, const float *x_dev,
                                         float *const *ys_dev, int batch);
/* n independent GEMVs (batch 1 each) in one launch: ws[i], xs_dev[i] (n_cols_i floats), ys_dev[i] (n_rows_i floats). */
RT_HIP_API int rt_hip_qgemv_grouped_dev(rt_hip_ctx *ctx, int n, const rt_hip_qweight *const *ws,
                                        const float *const *xs_dev, float *const *ys_dev);
/* The two halves of rt_hip_qgemv_grouped_dev, for callers that keep activations in the kernels' own
 * quantized form (16-bit block-scaled integers split into two int8 planes, see rt_hip_xq_bytes):
 * quantize n vectors of n_cols[i] floats (each a multiple of 32) into xqs_dev[i] (rt_hip_xq_bytes(n_cols[i]) bytes,
 * 16-byte aligned), then run the n GEMVs on them in one launch. */
RT_HIP_API size_t rt_hip_xq_bytes(size_t n_cols);
RT_HIP_API int rt_hip_quantize_act_dev(rt_hip_ctx *ctx, int n, const float *const *xs_dev, const size_t *n_cols,
                                       void *const *xqs_dev);
RT_HIP_API int rt_hip_qgemv_xq_grouped_dev(rt_hip_ctx *ctx, int n, const rt_hip_qweight *const *ws,
                                           const void *const *xqs_dev, float *const *ys_dev);
/* Report aid (no reference counterpart): which kernel the grouped launches above would run for these n weights at this
 * batch size, and how the launch would be cut, as text in out (at most out_bytes - 1 characters and a NUL).  Launches
 * nothing.  The bench names the kernel it measured with this instead of assuming one. */
RT_HIP_API int rt_hip_qgemv_describe(rt_hip_ctx *ctx, int n, const rt_hip_qweight *const *ws, int batch, char *out,
                                     size_t out_bytes);
/* Y[M, n_rows] = X[M, n_cols] . dequant(W)^T for prefill (any M >= 1; MFMA path for M >= 16). */
RT_HIP_API int rt_hip_qgemm(rt_hip_ctx *ctx, const rt_hip_qweight *w, const float *X, size_t M, float *Y);
RT_HIP_API int rt_hip_qgemm_dev(rt_hip_ctx *ctx, const rt_hip_qweight *w, const float *X_dev, size_t M,
                                float *Y_dev);

/* ---- decode-loop steps (device pointers, enqueue only).
 *      RMSNorm::forward (src/nn/normalization.rs:612-701): y = gamma * x / sqrt(mean(x^2) + eps), rows of n. */
RT_HIP_API int rt_hip_rmsnorm_dev(rt_hip_ctx *ctx, const float *x, const float *gamma, float *y, size_t rows,
                                  size_t n, float eps);
/* swiglu (src/nn/activation.rs:378-419) with a = up, b = gate: out = up * gate * sigmoid(gate). */
RT_HIP_API int rt_hip_swiglu_dev(rt_hip_ctx *ctx, const float *gate, const float *up, float *out, size_t n);
/* Rotary embedding, interleaved pairs, in place on x[n_heads, head_dim] (no reference counterpart). */
RT_HIP_API int rt_hip_rope_dev(rt_hip_ctx *ctx, float *x, int n_heads, int head_dim, int pos, float theta);
/* Append one position to an fp16 cache laid out [max_pos][row_elems]: the append KVCache::update
 * (example-cli/src/model/transformer.rs:221-270) was meant to be. */
RT_HIP_API int rt_hip_kv_append_dev(rt_hip_ctx *ctx, uint16_t *cache, const float *v, size_t pos, size_t row_elems);
/* One query over positions [0, n_pos): softmax(q.K^T / sqrt(head_dim)) . V per head
 * (example-cli/src/model/architectures/attention.rs:233-338 for a single query row). */
RT_HIP_API int rt_hip_attn_decode_dev(rt_hip_ctx *ctx, const float *q, const uint16_t *kcache,
                                      const uint16_t *vcache, int n_pos, int n_heads, int head_dim, float *out);
/* A batch of consecutive positions with the causal mask: row m of q[n_queries][n_heads * head_dim] (position
 * pos0 + m) attends cache rows [0, pos0 + m] (the masked scores / softmax / weighted sum of
 * example-cli/src/model/architectures/attention.rs:233-338 over the cache).  Cache rows hold n_kv_heads heads
 * (0 = n_heads); query head h reads head h / (n_heads / n_kv_heads).  All pointers 16-byte aligned. */
RT_HIP_API int rt_hip_attn_causal_dev(rt_hip_ctx *ctx, const float *q, const uint16_t *kcache, const uint16_t *vcache,
                                      int pos0, int n_queries, int n_heads, int n_kv_heads, int head_dim, float *out);
/* x += y : the residual adds of GPTBlock::forward (example-cli/src/model/architectures/gpt.rs:43-55). */
RT_HIP_API int rt_hip_add_dev(rt_hip_ctx *ctx, float *x, const float *y, size_t n);
/* Greedy pick (SamplingConfig::greedy, example-cli/src/model/sampling.rs:28-35); ties -> lowest index. */
RT_HIP_API int rt_hip_argmax_dev(rt_hip_ctx *ctx, const float *v, size_t n, int *out_index_dev);

/* ---- the model object the CLI's InferenceEngine loop drives once per token
 *      (example-cli/src/model/inference.rs:91-211; GPTModel::forward, gpt.rs:192-263). */
typedef struct {
    int n_layers, hidden, n_heads, ffn, vocab, max_pos;
    float rms_eps, rope_theta;
    int n_kv_heads;   /* key / value heads (grouped-query attention); 0 means n_heads */
} rt_hip_llama_config;

typedef enum {
    RT_LLAMA_TOK_EMBD = 0,
    RT_LLAMA_OUTPUT = 1,
    RT_LLAMA_OUTPUT_NORM = 2,
    RT_LLAMA_ATTN_Q = 10,
    RT_LLAMA_ATTN_K = 11,
    RT_LLAMA_ATTN_V = 12,
    RT_LLAMA_ATTN_OUT = 13,
    RT_LLAMA_FFN_GATE = 14,
    RT_LLAMA_FFN_UP = 15,
    RT_LLAMA_FFN_DOWN = 16,
    RT_LLAMA_ATTN_NORM = 17,
    RT_LLAMA_FFN_NORM = 18
} rt_hip_llama_slot;

RT_HIP_API int rt_hip_llama_create(rt_hip_ctx *ctx, const rt_hip_llama_config *cfg, rt_hip_llama **out);
RT_HIP_API int rt_hip_llama_destroy(rt_hip_ctx *ctx, rt_hip_llama *m);
/* Upload one tensor's raw GGUF payload (norm vectors: F32). layer is ignored for the three global slots. */
RT_HIP_API int rt_hip_llama_upload_tensor(rt_hip_ctx *ctx, rt_hip_llama *m, int slot, int layer, int ggml_type,
                                          size_t n_rows, size_t n_cols, const void *raw, size_t nbytes);
/* How a decode step is issued: 1 (default) = one launch per operator group; 2 = the same launches, captured
 * into a HIP graph at the second step and replayed from then on (every argument of a step is a device
 * pointer or a model constant, so one capture serves all later tokens; measured no faster than mode 1 on
 * MI355X, where the cost of a launch is on the device side); 0 = one persistent launch per
 * token (one workgroup per CU, phases separated by a software grid barrier). Mode 0 is switched off in this
 * build and asking for it returns RT_HIP_ERR_UNSUPPORTED_TYPE. */
RT_HIP_API int rt_hip_llama_set_mode(rt_hip_ctx *ctx, rt_hip_llama *m, int mode);
/* Forget the KV cache (KVCache::clear). */
RT_HIP_API int rt_hip_llama_reset(rt_hip_ctx *ctx, rt_hip_llama *m);
/* Feed `token` at position `pos` (must equal the number of tokens fed so far); logits stay on the device.
 * next_token (may be NULL) receives the greedy pick. Blocks only when next_token is given. */
RT_HIP_API int rt_hip_llama_step(rt_hip_ctx *ctx, rt_hip_llama *m, int token, int pos, int *next_token);
/* Feed n_tok tokens starting at pos0; logits of the last one stay on the device. */
RT_HIP_API int rt_hip_llama_prefill(rt_hip_ctx *ctx, rt_hip_llama *m, const int *tokens, int n_tok, int pos0);
/* Copy the logits of the most recently fed token to host (vocab floats); blocks. */
RT_HIP_API int rt_hip_llama_logits(rt_hip_ctx *ctx, rt_hip_llama *m, float *logits_host);
/* Run n_steps greedy decode steps back to back without a host round trip per token, starting from
 * `first_token` at position pos0 (each step feeds the previous step's pick, or forced[i] when forced
 * is not NULL -- teacher forcing).  out_tokens receives the n_steps picks.  Blocks at the end. */
RT_HIP_API int rt_hip_llama_decode(rt_hip_ctx *ctx, rt_hip_llama *m, int first_token, int pos0, int n_steps,
                                   const int *forced, int *out_tokens);

/* ---- several sequences at once: the generate loop (InferenceEngine::generate_with_gpt,
 *      example-cli/src/model/inference.rs:135-192) run for up to 8 prompts side by side against one model's weights.  A
 *      batch owns a cache of max_pos (1..8192) rows per sequence and the activations of one step; the model must outlive
 *      it and must not change tensors while it exists.  One step feeds one token per sequence -- sequence i's token at
 *      positions[i], which must equal the number of tokens fed to that sequence so far (sequences need not be at the same
 *      position) -- and runs every weight matrix once for all sequences.  tokens[i] < 0 leaves sequence i idle for the
 *      step (nothing is fed, its pick is reported as -1, its row of the logits is meaningless); at least one sequence must
 *      be fed.  next_tokens (may be NULL; n_seq ints) receives the greedy picks (ties: lowest id) and makes the call block;
 *      rt_hip_llama_batch_logits copies the [n_seq][vocab] logits of the last step to host.  reset forgets the cache of
 *      sequence seq, or of every sequence when seq is -1 (a finished sequence's slot then takes a new prompt). */
RT_HIP_API int rt_hip_llama_batch_create(rt_hip_ctx *ctx, rt_hip_llama *m, int n_seq, int max_pos, rt_hip_llama_batch **out);
RT_HIP_API int rt_hip_llama_batch_destroy(rt_hip_ctx *ctx, rt_hip_llama_batch *b);
RT_HIP_API int rt_hip_llama_batch_reset(rt_hip_ctx *ctx, rt_hip_llama_batch *b, int seq);
RT_HIP_API int rt_hip_llama_batch_step(rt_hip_ctx *ctx, rt_hip_llama_batch *b, const int *tokens, const int *positions,
                                       int *next_tokens);
/* Feed n_tok (3 or more) tokens of sequence seq starting at pos0 (= the tokens fed to it so far) through the model's batched
 * prefill passes (dense contractions on the matrix cores), into that sequence's cache; the other sequences are untouched.
 * Its row of the logits then holds the last token's.  Blocks.  The call borrows the model's prefill workspace. */
RT_HIP_API int rt_hip_llama_batch_prefill(rt_hip_ctx *ctx, rt_hip_llama_batch *b, int seq, const int *tokens, int n_tok,
                                          int pos0);
RT_HIP_API int rt_hip_llama_batch_logits(rt_hip_ctx *ctx, rt_hip_llama_batch *b, float *logits_host);

/* ---- synthetic GGUF payloads (host only, no GPU needed): seeded, counter-based, so a tensor is a pure
 *      function of (seed, tensor_id).  Used by the tests, the bench and offline exercise of the CLI path. */
RT_HIP_API int rt_synth_blocks(int ggml_type, uint64_t seed, uint64_t tensor_id, size_t n_blocks, float d_lo,
                               float d_hi, void *out);
RT_HIP_API int rt_synth_normal_f32(uint64_t seed, uint64_t tensor_id, size_t n, float mean, float std, float *out);
RT_HIP_API int rt_synth_tokens(uint64_t seed, uint64_t tensor_id, size_t n, int vocab, int *out);

#ifdef __cplusplus
}
#endif
#endif /* RUSTORCH_HIP_H */
