// Internal declarations shared by the host-side C ABI (rt_api.hip) and the
// kernel launchers (rt_kernels.hip, rt_gemm.hip).  Not installed; the public
// surface is include/rustorch_hip.h.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <mutex>
#include <string>

#include "../../include/rustorch_hip.h"

namespace rt {

// Denominators every reported fraction is priced against (MI355X, gfx950 / CDNA4).
constexpr double kHbmPeakBytesPerSec = 8.0e12;
constexpr double kMfmaF16PeakFlops = 2.5e15;
constexpr int kWave = 64;

// ---- quantized activation vector ("xq"): what the GEMV kernels consume.
// A vector of K floats (K % 32 == 0) is stored per 32-element block as
//   q = rint(x * 16383 / amax_block)  in [-16383, 16383],   q = 128 * qh + ql,
//   qh in [-128,127] (int8), ql in [0,127] (int8), scale s = amax_block / 16383,
// so that an integer dot with int8 weights is exact:  sum w*q = 128*sum w*qh + sum w*ql.
// Byte layout of one vector:
//   [0, K)            qh   int8[K]
//   [K, 2K)           ql   int8[K]
//   [2K, 2K+K/8)      s    f32[K/32]
//   [.., +K/4)        bsum f32[K/16] = s * (sum of q over each 16-element run)  (for the -8 / -32 / -min terms)
// padded to a multiple of 16 bytes.
__host__ __device__ inline size_t xq_stride(size_t K) { return (2 * K + K / 8 + K / 4 + 15) & ~(size_t)15; }
// Unquantized weight matrices (F16 / F32) meet x as plain f32 in LDS; the block formats meet the two-plane integer form.
__host__ __device__ inline bool gemv_float_weights(int type) { return type == 0 /* F32 */ || type == 1 /* F16 */; }
__host__ __device__ inline size_t gemv_lds_bytes(int type, size_t K) { return gemv_float_weights(type) ? 4 * K : xq_stride(K); }
// most LDS a GEMV workgroup may ask for x: the CU's 160 KB less the kernel's own few static bytes, with room to spare
constexpr size_t kGemvLdsMax = 144 * 1024;

// How a GEMV workgroup obtains the activation vector it stages into LDS.
enum : int {
    kStageXq = 0,   // x points at a ready xq vector (batch stride xq_stride(K))
    kStageF32 = 1,  // x points at f32 (batch stride K); quantized while staging
    kStageRms = 2,  // x points at f32; RMS-normalised with gamma / eps, then quantized
};
enum : int {
    kEpiStore = 0,   // y = W x (+ res when res != nullptr)
    kEpiSwiglu = 1,  // y = (W2 x) * silu(W x): W = gate rows, W2 = up rows of the same shape and type
};

struct GemvProb {
    const uint8_t *w;    // raw GGUF blocks, row r at w + r * row_bytes
    const uint8_t *w2;   // second matrix for kEpiSwiglu
    const void *x;       // activations, see kStage*
    const float *gamma;  // kStageRms
    float *y;            // [batch, N]
    const float *res;    // optional residual added to y (same shape), may alias y
    size_t row_bytes;
    float eps;           // kStageRms
    int type, N, K;
    int stage, epi;
    int tile0;           // index of this problem's first tile in the launch
    int rows_per_tile;
    int ksplit;          // set by the planner (lean path, rows of more than one pass): a wave's unit of work is one pass of one
                         // row, the passes of a row are summed through LDS at the end of the workgroup
};
constexpr int kMaxGemvProbs = 8;
struct GemvArgs {
    GemvProb p[kMaxGemvProbs];
    int n;
};

struct QuantGroupArgs {
    const float *x[kMaxGemvProbs];
    uint8_t *xq[kMaxGemvProbs];
    int K[kMaxGemvProbs];
    int n;
};

// ---- code-path switches (rt_hip_set_option): process-wide atomics, initial value from the environment.
// index = rt_hip_option; value -1 until first read.
int path_option(int option);
bool set_path_option(int option, int value);

// ---- launchers (all enqueue on `s`, return hipError_t of the launch)
hipError_t launch_set_state(hipStream_t s, int *state, int pos, int token, int step);
hipError_t launch_quantize_x(hipStream_t s, const float *x, uint8_t *xq, size_t K, size_t batch);
hipError_t launch_quantize_group(hipStream_t s, const QuantGroupArgs &a);
hipError_t launch_qgemv(hipStream_t s, GemvArgs &args, int batch);  // fills tile0 / rows_per_tile
bool describe_qgemv(GemvArgs &args, int batch, char *out, size_t out_bytes);   // the kernel and cut launch_qgemv would choose, as text

// 2..8 activation rows against Q4_K / Q6_K weights in one pass over the weights, on the integer matrix cores
// (rt_gemv_mb.hip).  work: qgemv_mb_scratch_bytes(K) bytes, 256-byte aligned; res (optional) is added to y.
constexpr int kGemvMbMinBatch = 3;       // two rows are faster as two passes of the one-row kernel
bool qgemv_mb_serves(int type, size_t N, size_t K, int batch);
size_t qgemv_mb_scratch_bytes(size_t K);
hipError_t launch_qgemv_mb(hipStream_t s, int type, const void *w, size_t row_bytes, size_t N, size_t K, const float *x, int batch,
                           float *y, const float *res, void *work);
// The two halves of it: quantize the rows into `work` once, then up to 4 matrices of one format against them per launch.
struct MbProb {
    const void *w;
    size_t row_bytes, N;
    float *y;                  // [batch][N]
    const float *res;          // optional, added to y; may alias y
};
hipError_t launch_qgemv_mb_prep(hipStream_t s, const float *x, int batch, size_t K, void *work);
hipError_t launch_qgemv_mb_group(hipStream_t s, int type, const MbProb *probs, int n, size_t K, int batch, const void *work);
hipError_t launch_dequant(hipStream_t s, int type, const uint8_t *w, size_t n_rows, size_t n_cols, float *out);
hipError_t launch_rmsnorm(hipStream_t s, const float *x, const float *gamma, float *y, uint8_t *xq, size_t rows,
                          size_t n, float eps);
hipError_t launch_swiglu(hipStream_t s, const float *gate, const float *up, float *out, uint8_t *xq, size_t n);
hipError_t launch_rope(hipStream_t s, float *x, int n_heads, int head_dim, const int *pos_dev, int pos,
                       const float *inv_freq_dev, float theta);
hipError_t launch_kv_append(hipStream_t s, uint16_t *cache, const float *v, const int *pos_dev, size_t pos,
                            size_t row_elems);
hipError_t launch_rope_kv(hipStream_t s, float *q, const float *k, const float *v, uint16_t *kcache,
                          uint16_t *vcache, const int *pos_dev, int n_heads, int head_dim,
                          const float *inv_freq_dev);
// fused = rotate q / k of the step, append k / v at *pos_dev, then attend over [0, *pos_dev]; otherwise attend over [0, n_pos)
hipError_t launch_attn_decode(hipStream_t s, float *q, const float *k, const float *v, uint16_t *kc, uint16_t *vc,
                              const int *pos_dev, int n_pos, int n_heads, int n_kv_heads, int head_dim, const float *inv_freq_dev,
                              float *out, uint8_t *xq, bool fused);
hipError_t launch_attn_decode_split(hipStream_t s, const float *q, const float *k, const float *v, uint16_t *kc, uint16_t *vc,
                                    const int *pos_dev, int max_pos, int n_splits, int n_heads, int n_kv_heads, int head_dim,
                                    const float *inv_freq_dev, float *partials, float *out, uint8_t *xq);
hipError_t launch_rope_kv_batch(hipStream_t s, float *q, const float *k, const float *v, uint16_t *kcache, uint16_t *vcache,
                                int pos0, size_t n_tok, int n_heads, int n_kv_heads, int head_dim, const float *inv_freq_dev);
// several sequences in one step: row m of q / k / v is sequence m at position pos_rows_dev[m]; its cache starts m * seq_stride
// elements into kcache / vcache
hipError_t launch_rope_kv_rows(hipStream_t s, float *q, const float *k, const float *v, uint16_t *kcache, uint16_t *vcache, const int *pos_rows_dev,
                               size_t seq_stride, size_t n_rows, int n_heads, int n_kv_heads, int head_dim, const float *inv_freq_dev);
hipError_t launch_attn_rows(hipStream_t s, const float *q, uint16_t *kc, uint16_t *vc, const int *pos_rows_dev, size_t seq_stride, int max_pos,
                            size_t n_rows, int n_heads, int n_kv_heads, int head_dim, float *out, void *xq8_work_buf, const float *k_new,
                            const float *v_new, const float *inv_freq_dev);
// producers that write the operand form of the small-batch matrix-core GEMV (launch_qgemv_mb_group's `work`) directly:
// rows <= 8, n a multiple of 256; launch_attn_rows does the same with out == nullptr (and then rotates and appends itself)
hipError_t launch_rmsnorm_xq8(hipStream_t s, const float *x, const float *gamma, size_t rows, size_t n, float eps, void *work);
hipError_t launch_swiglu_xq8(hipStream_t s, const float *gate, const float *up, size_t rows, size_t n, void *work);
hipError_t launch_attn_batch(hipStream_t s, float *q, const float *k, const float *v, uint16_t *kc, uint16_t *vc,
                             const int *pos_dev, int n_pos, size_t n_queries, int n_heads, int n_kv_heads, int head_dim,
                             const float *inv_freq_dev, float *out, uint8_t *xq, bool fused);
// rows m = 0 .. n_queries-1 of q (position pos0 + m) attend cache rows [0, pos0 + m]; matrix-core kernel, one wave per 32 queries of a head
hipError_t launch_attn_causal(hipStream_t s, const float *q, const uint16_t *kc, const uint16_t *vc, int pos0, size_t n_queries,
                              int n_heads, int n_kv_heads, int head_dim, float *out);
hipError_t launch_embed_rows(hipStream_t s, int type, const uint8_t *w, size_t row_bytes, size_t n_cols,
                             const int *tokens_dev, size_t n_tok, int vocab, float *out);
hipError_t launch_add(hipStream_t s, float *x, const float *y, size_t n);
hipError_t launch_stream_read(hipStream_t s, const void *p, size_t nbytes, unsigned *sink);
hipError_t launch_argmax_rows(hipStream_t s, const float *v, size_t rows, size_t n, int *out_dev);     // out_dev[row] = pick of v[row][0..n)
hipError_t launch_argmax(hipStream_t s, const float *v, size_t n, int *out_dev);
// the greedy pick and the end of the decode step (as launch_step_advance) in one launch
hipError_t launch_argmax_advance(hipStream_t s, const float *v, size_t n, int *pick_dev, int *pos_dev, int *token_dev, const int *forced_dev,
                                 int *out_tokens_dev, int *step_dev);
hipError_t launch_embed_row(hipStream_t s, int type, const uint8_t *w, size_t row_bytes, size_t n_cols,
                            const int *token_dev, int vocab, float *out);
hipError_t launch_matmul_f32(hipStream_t s, const float *a, const float *b, float *c, size_t m, size_t n, size_t k, size_t batch = 1);
hipError_t launch_qmatmul_i8(hipStream_t s, const int8_t *a, const int8_t *b, int8_t *out, size_t m, size_t n, size_t k, int za, int zb,
                             float scale);
hipError_t launch_set_int(hipStream_t s, int *dst, int value);
hipError_t launch_step_advance(hipStream_t s, int *pos_dev, int *token_dev, const int *pick_dev,
                               const int *forced_dev, int *out_tokens_dev, int *step_dev);
// prefill GEMM (rt_gemm.hip)
hipError_t launch_qgemm(hipStream_t s, int type, const uint8_t *w, size_t N, size_t K, size_t row_bytes,
                        const float *X, size_t M, float *Y, const float *res, void *scratch, size_t scratch_bytes,
                        bool x_prepared = false);
size_t qgemm_scratch_bytes(int type, size_t M, size_t N, size_t K);
// true: launch_qgemm runs the matrix-core contraction (with its pre-pass of X); false: the GEMV kernel, one grid slice per row of X
bool qgemm_on_matrix_cores(int type, size_t M, size_t N, size_t K);

// fp16 contraction for the formats without a fused dequantizing kernel (rt_hgemm.hip): unquantized F16 weights as they
// are, the others through an fp16 copy in the workspace.  res may be Y.
bool hgemm_serves(int type, size_t M, size_t N, size_t K);
size_t hgemm_scratch_bytes(int type, size_t M, size_t N, size_t K);
hipError_t launch_hgemm(hipStream_t s, int type, const uint8_t *w, size_t N, size_t K, size_t row_bytes, const float *X, size_t M, float *Y,
                        const float *res, void *scratch, size_t scratch_bytes, const _Float16 *w_f16 = nullptr);
hipError_t launch_weights_f16(hipStream_t s, int type, const uint8_t *w, size_t N, size_t K, size_t row_bytes, _Float16 *out);

// A matrix held as n partial planes: element i is base[i] + base[stride + i] + ... (summed in that order).
// What a k-split contraction leaves behind; n = 1 is an ordinary matrix.
struct PlaneSum {
    const float *base;
    size_t stride;
    int n;
};
// The pieces of launch_qgemm for a caller that chains contractions: the pre-pass on its own (plain, or fused with the
// operation that produces the activation matrix), the contraction without the reduction of its k splits, and consumers
// that read plane sums.  Xp: M x K fp16 (scaled, k-permuted), inv_scale: M floats; K a multiple of 256.
size_t qgemm_planes_bytes(int type, size_t M, size_t N, size_t K);             // planes a contraction of this shape may write
constexpr size_t kXprepFusedMaxK = 49152;                                       // longest row the fused producers keep in registers
hipError_t launch_xprep(hipStream_t s, const float *X, size_t M, size_t K, _Float16 *Xp, float *inv_scale);
// x = in (+ res), stored to x_out when given; prepared matrix = gamma * x / sqrt(mean(x^2) + eps)
hipError_t launch_xprep_rmsnorm(hipStream_t s, PlaneSum in, const float *res, float *x_out, const float *gamma, float eps, size_t M, size_t K,
                                _Float16 *Xp, float *inv_scale);
// prepared matrix = up * gate * sigmoid(gate)
hipError_t launch_xprep_swiglu(hipStream_t s, PlaneSum gate, PlaneSum up, size_t M, size_t K, _Float16 *Xp, float *inv_scale);
hipError_t launch_qgemm_planes(hipStream_t s, int type, const uint8_t *w, size_t N, size_t K, size_t row_bytes, const _Float16 *Xp,
                               const float *inv_scale, size_t M, float *planes, size_t planes_bytes, PlaneSum *out);
// the same for two weight matrices of one shape and format in one launch
hipError_t launch_qgemm_planes2(hipStream_t s, int type, const uint8_t *wa, const uint8_t *wb, size_t N, size_t K, size_t row_bytes,
                                const _Float16 *Xp, const float *inv_scale, size_t M, float *planes_a, float *planes_b, size_t planes_bytes,
                                PlaneSum *out_a, PlaneSum *out_b);
// Y = in (+ res), n elements (a multiple of 4)
hipError_t launch_plane_sum(hipStream_t s, PlaneSum in, const float *res, float *Y, size_t n);
// rope_kv_batch with q, k, v given as plane sums; the rotated q goes to q_out
hipError_t launch_rope_kv_planes(hipStream_t s, PlaneSum q, PlaneSum k, PlaneSum v, float *q_out, uint16_t *kcache, uint16_t *vcache,
                                 int pos0, size_t n_tok, int n_heads, int n_kv_heads, int head_dim, const float *inv_freq_dev);

inline size_t type_block_bytes(int t) {
    switch (t) {
    case RT_GGML_F32: return 4;
    case RT_GGML_F16: return 2;
    case RT_GGML_Q4_0: return 18;
    case RT_GGML_Q4_1: return 20;
    case RT_GGML_Q5_0: return 22;
    case RT_GGML_Q5_1: return 24;
    case RT_GGML_Q8_0: return 34;
    case RT_GGML_Q8_1: return 36;
    case RT_GGML_Q2_K: return 84;      // 16 scale bytes + 64 + two f16: the public ggml block (the reference's size table lists 82)
    case RT_GGML_Q3_K: return 110;
    case RT_GGML_Q4_K: return 144;
    case RT_GGML_Q5_K: return 176;
    case RT_GGML_Q6_K: return 210;
    default: return 0;
    }
}
inline size_t type_block_elems(int t) {
    switch (t) {
    case RT_GGML_F32: case RT_GGML_F16: return 1;
    case RT_GGML_Q4_0: case RT_GGML_Q4_1: case RT_GGML_Q5_0: case RT_GGML_Q5_1: case RT_GGML_Q8_0: case RT_GGML_Q8_1: return 32;
    case RT_GGML_Q2_K: case RT_GGML_Q3_K: case RT_GGML_Q4_K: case RT_GGML_Q5_K: case RT_GGML_Q6_K: return 256;
    default: return 0;
    }
}

}  // namespace rt

struct rt_hip_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    std::mutex mu;
    std::string err;
    // scratch owned by the context for the host-pointer entry points and the xq of *_dev GEMV calls
    void *scratch = nullptr;
    size_t scratch_bytes = 0;
};

struct rt_hip_qweight {
    int type = 0;
    size_t n_rows = 0, n_cols = 0, nbytes = 0, row_bytes = 0;
    uint8_t *dev = nullptr;
    bool owns = false;
};

struct rt_hip_event {
    hipEvent_t ev = nullptr;
};

// ---- host-side helpers shared by the C-ABI translation units
namespace rt {
int fail(rt_hip_ctx *ctx, int code, const char *fmt, ...) __attribute__((format(printf, 3, 4)));
int hip_fail(rt_hip_ctx *ctx, hipError_t e, const char *what);
int ensure_scratch(rt_hip_ctx *ctx, size_t bytes);

// Serialises calls on one context and makes its device current.
struct Guard {
    rt_hip_ctx *c;
    explicit Guard(rt_hip_ctx *ctx) : c(ctx) {
        c->mu.lock();
        (void)hipSetDevice(c->device);
    }
    ~Guard() { c->mu.unlock(); }
    Guard(const Guard &) = delete;
    Guard &operator=(const Guard &) = delete;
};
}  // namespace rt

#define RT_TRY_HIP(ctx, expr)                                        \
    do {                                                             \
        hipError_t e__ = (expr);                                     \
        if (e__ != hipSuccess) return rt::hip_fail(ctx, e__, #expr); \
    } while (0)

#define RT_REQUIRE(ctx, cond, code, ...)                      \
    do {                                                      \
        if (!(cond)) return rt::fail(ctx, code, __VA_ARGS__); \
    } while (0)
