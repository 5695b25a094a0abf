// Decode-path kernels for gfx950 (wave64): block decode, activation
// quantization, dequant-fused GEMV, RMSNorm, RoPE, KV append, single-query
// attention, SwiGLU, residual add, argmax, embedding row, dense f32 matmul.
//
// Block layouts are the public ggml ones (byte sizes as in
// example-cli/src/model/formats/gguf.rs:125-144):
//   Q8_0 34 B / 32 el : f16 d; i8 qs[32]
//   Q4_0 18 B / 32 el : f16 d; u8 qs[16]        (low nibbles = el 0..15, high = 16..31)
//   Q4_1 20 B / 32 el : f16 d; f16 m; u8 qs[16]                 (q * d + m)
//   Q5_0 22 B / 32 el : f16 d; u8 qh[4]; u8 qs[16]              (bit j of qh = fifth bit of element j; (q - 16) * d)
//   Q5_1 24 B / 32 el : f16 d; f16 m; u8 qh[4]; u8 qs[16]
//   Q2_K 84 B / 256   : u8 scales[16]; u8 qs[64]; f16 d; f16 dmin
//   Q3_K 110 B / 256  : u8 hmask[32]; u8 qs[64]; u8 scales[12]; f16 d
//   Q4_K 144 B / 256  : f16 d; f16 dmin; u8 scales[12]; u8 qs[128]
//   Q5_K 176 B / 256  : f16 d; f16 dmin; u8 scales[12]; u8 qh[32]; u8 qs[128]
//   Q6_K 210 B / 256  : u8 ql[128]; u8 qh[64]; i8 scales[16]; f16 d
#include "rt_device.h"

namespace rt {

#pragma clang fp contract(off)
__global__ void dequant_kernel(int type, const uint8_t *w, size_t row_bytes, size_t n_rows, size_t n_cols, float *out) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t total = n_rows * n_cols;
    for (; i < total; i += (size_t)gridDim.x * blockDim.x) {
        size_t r = i / n_cols, c = i - r * n_cols;
        out[i] = deq_elem(type, w + r * row_bytes, c);
    }
}

__global__ void embed_row_kernel(int type, const uint8_t *w, size_t row_bytes, size_t n_cols, const int *token_dev,
                                 int vocab, float *out) {
    int tok = token_dev[blockIdx.y];          // grid.y tokens, one output row each
    if (tok < 0) tok = 0;
    if (tok >= vocab) tok = vocab - 1;
    size_t c = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c < n_cols) out[(size_t)blockIdx.y * n_cols + c] = deq_elem(type, w + (size_t)tok * row_bytes, c);
}
#pragma clang fp contract(fast)

// ----------------------------------------------------- activation quantization
// Quantize 4 consecutive elements (e % 4 == 0) of a K-vector into xq.  The 8 lanes that
// hold one 32-element block must be consecutive lanes of one wave and all active.
__device__ __forceinline__ void quantize_store4(float4 v, size_t e, uint8_t *xq, size_t K) {
    Q4Pack p = quantize4(v);
    *reinterpret_cast<uint32_t *>(xq + e) = p.hi;
    *reinterpret_cast<uint32_t *>(xq + K + e) = p.lo;
    float *sp = reinterpret_cast<float *>(xq + 2 * K);
    float *bp = sp + K / 32;
    if ((e & 15) == 0) bp[e >> 4] = p.s * (float)p.sum16;
    if ((e & 31) == 0) sp[e >> 5] = p.s;
}

__global__ __launch_bounds__(256) void quantize_x_kernel(const float *x, uint8_t *xq, size_t K) {
    size_t m = blockIdx.y;
    size_t i4 = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i4 * 4 >= K) return;  // whole 8-lane groups leave together because K % 32 == 0
    float4 v = reinterpret_cast<const float4 *>(x + m * K)[i4];
    quantize_store4(v, i4 * 4, xq + m * xq_stride(K), K);
}

// Several independent vectors in one launch (grid.y = vector index).
__global__ __launch_bounds__(256) void quantize_group_kernel(QuantGroupArgs a) {
    int p = blockIdx.y;
    size_t K = (size_t)a.K[p];
    size_t i4 = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i4 * 4 >= K) return;
    float4 v = reinterpret_cast<const float4 *>(a.x[p])[i4];
    quantize_store4(v, i4 * 4, a.xq[p], K);
}

// ------------------------------------------------------------------ RMSNorm
// One block per row.  y = gamma * (x / sqrt(mean(x^2) + eps))  (src/nn/normalization.rs:682-696).
// Writes f32 y when y != nullptr and the xq form when xq != nullptr (needs n % 32 == 0).
__global__ __launch_bounds__(1024) void rmsnorm_kernel(const float *x, const float *gamma, float *y, uint8_t *xq,
                                                       size_t n, float eps) {
    __shared__ float red[16];
    size_t m = blockIdx.x;
    const float *xr = x + m * n;
    float ss = 0.f;
    if ((n & 3) == 0) {
        const float4 *x4 = reinterpret_cast<const float4 *>(xr);
        for (size_t i = threadIdx.x; i < n / 4; i += blockDim.x) {
            float4 v = x4[i];
            ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
        }
    } else {
        for (size_t i = threadIdx.x; i < n; i += blockDim.x) ss += xr[i] * xr[i];
    }
    ss = block_sum(ss, red);
    float rms = sqrtf(ss / (float)n + eps);
    if ((n & 3) == 0) {
        const float4 *x4 = reinterpret_cast<const float4 *>(xr);
        const float4 *g4 = reinterpret_cast<const float4 *>(gamma);
        for (size_t i = threadIdx.x; i < n / 4; i += blockDim.x) {
            float4 v = x4[i], g = g4[i];
            float4 o = make_float4(g.x * (v.x / rms), g.y * (v.y / rms), g.z * (v.z / rms), g.w * (v.w / rms));
            if (y) reinterpret_cast<float4 *>(y + m * n)[i] = o;
            if (xq) quantize_store4(o, i * 4, xq + m * xq_stride(n), n);
        }
    } else {
        for (size_t i = threadIdx.x; i < n; i += blockDim.x) y[m * n + i] = gamma[i] * (xr[i] / rms);
    }
}

// ------------------------------------------------------------------- SwiGLU
// out = up * (gate * 1/(1+exp(-gate)))  (src/nn/activation.rs:404-414 with a = up, b = gate).
__global__ __launch_bounds__(256) void swiglu_kernel(const float *gate, const float *up, float *out, uint8_t *xq,
                                                     size_t n) {
    size_t i4 = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if ((n & 3) == 0) {
        if (i4 * 4 >= n) return;
        float4 g = reinterpret_cast<const float4 *>(gate)[i4], u = reinterpret_cast<const float4 *>(up)[i4];
        float4 o;
        o.x = u.x * (g.x * (1.0f / (1.0f + expf(-g.x))));
        o.y = u.y * (g.y * (1.0f / (1.0f + expf(-g.y))));
        o.z = u.z * (g.z * (1.0f / (1.0f + expf(-g.z))));
        o.w = u.w * (g.w * (1.0f / (1.0f + expf(-g.w))));
        if (out) reinterpret_cast<float4 *>(out)[i4] = o;
        if (xq) quantize_store4(o, i4 * 4, xq, n);
    } else {
        for (size_t i = i4 * 4; i < n && i < i4 * 4 + 4; i++) {
            float b = gate[i];
            out[i] = up[i] * (b * (1.0f / (1.0f + expf(-b))));
        }
    }
}

// ---- the same two operations writing the operand form of the small-batch matrix-core GEMV (xq8_store4) instead of f32:
// the step of several sequences runs them in front of q / k / v, gate / up and the down-projection, which saves those
// contractions their quantizing launch.  Arithmetic as in rmsnorm_kernel / swiglu_kernel, then the quantization step the
// stand-alone pre-pass applies to their f32 result.  n % 32 == 0.  All 8 rows of the operand are written: zeros from row
// `batch` on.
__global__ __launch_bounds__(1024) void rmsnorm_xq8_kernel(const float *x, const float *gamma, size_t n, float eps, int batch, Xq8Work w) {
    __shared__ float red[16];
    const int m = blockIdx.x;
    const size_t n4 = n / 4;
    if (m >= batch) {
        for (size_t i = threadIdx.x; i < n4; i += blockDim.x) xq8_store4(make_float4(0.f, 0.f, 0.f, 0.f), (int)i, m, w);
        return;
    }
    const float4 *x4 = reinterpret_cast<const float4 *>(x + (size_t)m * n);
    const float4 *g4 = reinterpret_cast<const float4 *>(gamma);
    float ss = 0.f;
    for (size_t i = threadIdx.x; i < n4; i += blockDim.x) {
        float4 v = x4[i];
        ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
    }
    ss = block_sum(ss, red);
    float rms = sqrtf(ss / (float)n + eps);
    for (size_t i = threadIdx.x; i < n4; i += blockDim.x) {
        float4 v = x4[i], g = g4[i];
        xq8_store4(make_float4(g.x * (v.x / rms), g.y * (v.y / rms), g.z * (v.z / rms), g.w * (v.w / rms)), (int)i, m, w);
    }
}

// grid (n / 4 / 256 rounded up, 8): blockIdx.y = row
__global__ __launch_bounds__(256) void swiglu_xq8_kernel(const float *gate, const float *up, size_t n, int batch, Xq8Work w) {
    const int t = blockIdx.y;
    const size_t i4 = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i4 * 4 >= n) return;          // whole 8-lane groups leave together because n % 32 == 0
    float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
    if (t < batch) {
        float4 g = reinterpret_cast<const float4 *>(gate + (size_t)t * n)[i4], u = reinterpret_cast<const float4 *>(up + (size_t)t * n)[i4];
        o.x = u.x * (g.x * (1.0f / (1.0f + expf(-g.x))));
        o.y = u.y * (g.y * (1.0f / (1.0f + expf(-g.y))));
        o.z = u.z * (g.z * (1.0f / (1.0f + expf(-g.z))));
        o.w = u.w * (g.w * (1.0f / (1.0f + expf(-g.w))));
    }
    xq8_store4(o, (int)i4, t, w);
}

// --------------------------------------------------------------------- RoPE
// Interleaved pairs: (x[2i], x[2i+1]) turned by pos * inv_freq[i].  One thread per pair.
__global__ void rope_kernel(float *x, int n_heads, int head_dim, const int *pos_dev, int pos, const float *inv_freq,
                            float theta) {
    int half = head_dim / 2;
    int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_heads * half) return;
    int i = t % half;
    int p = pos_dev ? *pos_dev : pos;
    float f = inv_freq ? inv_freq[i] : (float)pow((double)theta, -2.0 * (double)i / (double)head_dim);
    float ang = (float)p * f;
    float s, c;
    sincosf(ang, &s, &c);
    float2 v = reinterpret_cast<float2 *>(x)[t];
    reinterpret_cast<float2 *>(x)[t] = make_float2(v.x * c - v.y * s, v.x * s + v.y * c);
}

__global__ void kv_append_kernel(uint16_t *cache, const float *v, const int *pos_dev, size_t pos, size_t row_elems) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t p = pos_dev ? (size_t)*pos_dev : pos;
    if (i < row_elems) cache[p * row_elems + i] = f2h_rne(v[i]);
}

// Fused decode-step form: rotate q in place, rotate k and store it and v as fp16 at row *pos_dev.
__global__ void rope_kv_kernel(float *q, const float *k, const float *v, uint16_t *kcache, uint16_t *vcache,
                               const int *pos_dev, int n_heads, int head_dim, const float *inv_freq) {
    int half = head_dim / 2;
    int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_heads * half) return;
    int i = t % half;
    int p = *pos_dev;
    size_t row = (size_t)n_heads * head_dim;
    float ang = (float)p * inv_freq[i];
    float s, c;
    sincosf(ang, &s, &c);
    float2 qv = reinterpret_cast<float2 *>(q)[t];
    reinterpret_cast<float2 *>(q)[t] = make_float2(qv.x * c - qv.y * s, qv.x * s + qv.y * c);
    float2 kv = reinterpret_cast<const float2 *>(k)[t];
    float k0 = kv.x * c - kv.y * s, k1 = kv.x * s + kv.y * c;
    float2 vv = reinterpret_cast<const float2 *>(v)[t];
    uint32_t kp = (uint32_t)f2h_rne(k0) | ((uint32_t)f2h_rne(k1) << 16);
    uint32_t vp = (uint32_t)f2h_rne(vv.x) | ((uint32_t)f2h_rne(vv.y) << 16);
    reinterpret_cast<uint32_t *>(kcache + (size_t)p * row)[t] = kp;
    reinterpret_cast<uint32_t *>(vcache + (size_t)p * row)[t] = vp;
}

// Prefill form: blockIdx.y = token m of the batch at position pos0 + m; q [M][row] is rotated in place,
// rotated k and v go to the fp16 cache rows pos0 + m.
__global__ void rope_kv_batch_kernel(float *q, const float *k, const float *v, uint16_t *kcache, uint16_t *vcache,
                                     int pos0, int n_heads, int n_kv_heads, int head_dim, const float *inv_freq) {
    int half = head_dim / 2;
    int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_heads * half) return;
    int i = t % half;
    const size_t row = (size_t)n_heads * head_dim, rowkv = (size_t)n_kv_heads * head_dim, m = blockIdx.y;
    const int p = pos0 + (int)m;
    float s, c;
    sincosf((float)p * inv_freq[i], &s, &c);
    float2 *qr = reinterpret_cast<float2 *>(q + m * row);
    float2 qv = qr[t];
    qr[t] = make_float2(qv.x * c - qv.y * s, qv.x * s + qv.y * c);
    if (t >= n_kv_heads * half) return;          // fewer key / value heads than query heads
    float2 kv = reinterpret_cast<const float2 *>(k + m * rowkv)[t];
    float k0 = kv.x * c - kv.y * s, k1 = kv.x * s + kv.y * c;
    float2 vv = reinterpret_cast<const float2 *>(v + m * rowkv)[t];
    reinterpret_cast<uint32_t *>(kcache + (size_t)p * rowkv)[t] = (uint32_t)f2h_rne(k0) | ((uint32_t)f2h_rne(k1) << 16);
    reinterpret_cast<uint32_t *>(vcache + (size_t)p * rowkv)[t] = (uint32_t)f2h_rne(vv.x) | ((uint32_t)f2h_rne(vv.y) << 16);
}

// The same with q, k, v given as the partial planes of k-split contractions: the planes are summed on the way in and
// the rotated q goes to q_out.
__device__ __forceinline__ float2 plane_pair(const PlaneSum &p, size_t pair) {
    float2 a = reinterpret_cast<const float2 *>(p.base)[pair];
    for (int z = 1; z < p.n; z++) {
        const float2 b = reinterpret_cast<const float2 *>(p.base + (size_t)z * p.stride)[pair];
        a.x += b.x;
        a.y += b.y;
    }
    return a;
}
__global__ void rope_kv_planes_kernel(PlaneSum q, PlaneSum k, PlaneSum v, float *q_out, uint16_t *kcache, uint16_t *vcache,
                                      int pos0, int n_heads, int n_kv_heads, int head_dim, const float *inv_freq) {
    int half = head_dim / 2;
    int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_heads * half) return;
    int i = t % half;
    const size_t prow = (size_t)n_heads * half, prowkv = (size_t)n_kv_heads * half, m = blockIdx.y;     // float2 pairs per row
    const int p = pos0 + (int)m;
    float s, c;
    sincosf((float)p * inv_freq[i], &s, &c);
    const float2 qv = plane_pair(q, m * prow + t);
    reinterpret_cast<float2 *>(q_out)[m * prow + t] = make_float2(qv.x * c - qv.y * s, qv.x * s + qv.y * c);
    if (t >= n_kv_heads * half) return;          // fewer key / value heads than query heads
    const float2 kv = plane_pair(k, m * prowkv + t), vv = plane_pair(v, m * prowkv + t);
    float k0 = kv.x * c - kv.y * s, k1 = kv.x * s + kv.y * c;
    reinterpret_cast<uint32_t *>(kcache + (size_t)p * 2 * prowkv)[t] = (uint32_t)f2h_rne(k0) | ((uint32_t)f2h_rne(k1) << 16);
    reinterpret_cast<uint32_t *>(vcache + (size_t)p * 2 * prowkv)[t] = (uint32_t)f2h_rne(vv.x) | ((uint32_t)f2h_rne(vv.y) << 16);
}

// -------------------------------------------------------- decode attention
// One block (256 threads) per query head; cache layout [pos][kv head][dim], fp16.  With fewer key / value heads
// than query heads, query head h reads kv head h / (n_heads / n_kv_heads) and the first query head of each
// group is the one that appends the new row.
//   scores_j = (q . k_j) / sqrt(dim);  p = softmax(scores) with max subtraction;  out = sum_j p_j v_j
// (example-cli/src/model/architectures/attention.rs:233-338 for one query row).
// FUSED: the block first rotates its head's q and k (interleaved pairs, angle pos * inv_freq[i]), stores
// fp16(k), fp16(v) as cache row pos and attends over [0, pos]; the fresh row is taken from LDS, not re-read.
// Scores: one thread per position, the whole head_dim dot in that thread (16-byte loads of 8 halves).
// Values: 16-byte column chunks x position groups, combined through LDS.
// Dynamic LDS: n_pos floats.
__device__ __forceinline__ void unpack8(uint4 v, float *f) {
    const uint32_t w[4] = { v.x, v.y, v.z, v.w };
#pragma unroll
    for (int i = 0; i < 4; i++) {
        f[2 * i] = h2f(w[i] & 0xFFFF);
        f[2 * i + 1] = h2f(w[i] >> 16);
    }
}

// One workgroup per head.  The cache rows of the positions already stored do not depend on this step's
// q, k, v, so their loads are issued first -- the key row of the thread's position and the value chunks of
// the thread's first kVPre positions -- and the rope/append of the new token, the scores and the softmax run
// while they are in flight: one memory round trip instead of three dependent ones.
template <int HD, bool FUSED>
__global__ __launch_bounds__(256) void attn_decode_kernel(float *q, const float *k, const float *v, uint16_t *kc,
                                                          uint16_t *vc, const int *pos_dev, int n_pos_arg, int n_heads, int n_kv_heads,
                                                          const float *inv_freq, float *out, uint8_t *xq) {
    RT_DYN_LDS(float, sc);
    __shared__ float red[4];
    __shared__ __align__(16) float qs[HD];
    __shared__ __align__(16) float kcur[HD];
    __shared__ __align__(16) float vcur[HD];
    __shared__ __align__(16) float part[2048];
    constexpr int CH = HD / 8;          // 16-byte chunks per cache row of this head
    constexpr int NG = 256 / CH;        // position groups in the value phase
    constexpr int kVPre = 16;           // value chunks a thread requests ahead (covers NG * kVPre positions)
    const int h = blockIdx.x, tid = threadIdx.x;
    const size_t row = (size_t)n_heads * HD, rowkv = (size_t)n_kv_heads * HD;
    const int group = n_heads / n_kv_heads, kvh = h / group;
    const bool appends = h % group == 0;
    const int cur = FUSED ? *pos_dev : -1;
    // not fused: blockIdx.y = query m of a causal batch; query m sees n_pos_arg + m positions
    const int n_pos = FUSED ? cur + 1 : n_pos_arg + (int)blockIdx.y;
    if (!FUSED) {
        q += (size_t)blockIdx.y * row;
        if (out) out += (size_t)blockIdx.y * row;
    }
    const float scale = 1.0f / sqrtf((float)HD);
    const int c = tid % CH, g = tid / CH;

    // ---- requests that do not depend on the new token
    uint4 kreg[CH], vreg[kVPre];
    const bool k_pre = tid < n_pos && tid != cur;
    if (k_pre) {
        const uint4 *kr = reinterpret_cast<const uint4 *>(kc + (size_t)tid * rowkv + (size_t)kvh * HD);
#pragma unroll
        for (int i = 0; i < CH; i++) kreg[i] = kr[i];
    }
#pragma unroll
    for (int i = 0; i < kVPre; i++) {
        const int j = g + NG * i;
        if (j < n_pos && j != cur) vreg[i] = reinterpret_cast<const uint4 *>(vc + (size_t)j * rowkv + (size_t)kvh * HD)[c];
    }

    if (FUSED) {
        if (tid < HD / 2) {
            int i = tid;
            float sn, cs;
            sincosf((float)cur * inv_freq[i], &sn, &cs);
            float2 qv = reinterpret_cast<const float2 *>(q + (size_t)h * HD)[i];
            float2 kv = reinterpret_cast<const float2 *>(k + (size_t)kvh * HD)[i];
            float q0 = qv.x * cs - qv.y * sn, q1 = qv.x * sn + qv.y * cs;
            float k0 = kv.x * cs - kv.y * sn, k1 = kv.x * sn + kv.y * cs;
            qs[2 * i] = q0;
            qs[2 * i + 1] = q1;
            reinterpret_cast<float2 *>(q + (size_t)h * HD)[i] = make_float2(q0, q1);
            uint16_t a = f2h_rne(k0), b = f2h_rne(k1);
            kcur[2 * i] = h2f(a);
            kcur[2 * i + 1] = h2f(b);
            if (appends) reinterpret_cast<uint32_t *>(kc + (size_t)cur * rowkv + (size_t)kvh * HD)[i] = (uint32_t)a | ((uint32_t)b << 16);
        } else if (tid < HD) {
            int i = tid - HD / 2;
            float2 vv = reinterpret_cast<const float2 *>(v + (size_t)kvh * HD)[i];
            uint16_t a = f2h_rne(vv.x), b = f2h_rne(vv.y);
            vcur[2 * i] = h2f(a);
            vcur[2 * i + 1] = h2f(b);
            if (appends) reinterpret_cast<uint32_t *>(vc + (size_t)cur * rowkv + (size_t)kvh * HD)[i] = (uint32_t)a | ((uint32_t)b << 16);
        }
    } else if (tid < HD) {
        qs[tid] = q[(size_t)h * HD + tid];
    }
    __syncthreads();
    // ---- scores
    float mx = -INFINITY;
    for (int j = tid; j < n_pos; j += 256) {
        float s = 0.f;
        if (j == cur) {
#pragma unroll 8
            for (int d = 0; d < HD; d++) s += qs[d] * kcur[d];
        } else {
            const uint4 *kr = reinterpret_cast<const uint4 *>(kc + (size_t)j * rowkv + (size_t)kvh * HD);
#pragma unroll
            for (int cc = 0; cc < CH; cc++) {
                float f[8];
                unpack8(j == tid ? kreg[cc] : kr[cc], f);
#pragma unroll
                for (int e = 0; e < 8; e++) s += qs[8 * cc + e] * f[e];
            }
        }
        s *= scale;
        sc[j] = s;
        mx = fmaxf(mx, s);
    }
    mx = block_max(mx, red);
    float sum = 0.f;
    for (int j = tid; j < n_pos; j += 256) {
        float e = expf(sc[j] - mx);
        sc[j] = e;
        sum += e;
    }
    sum = block_sum(sum, red);
    for (int j = tid; j < n_pos; j += 256) sc[j] = sc[j] / sum;
    __syncthreads();
    // ---- values
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; e++) acc[e] = 0.f;
#pragma unroll
    for (int i = 0; i < kVPre; i++) {
        const int j = g + NG * i;
        if (j < n_pos) {
            float f[8];
            if (j == cur) {
#pragma unroll
                for (int e = 0; e < 8; e++) f[e] = vcur[8 * c + e];
            } else {
                unpack8(vreg[i], f);
            }
            float p = sc[j];
#pragma unroll
            for (int e = 0; e < 8; e++) acc[e] += p * f[e];
        }
    }
    for (int j = g + NG * kVPre; j < n_pos; j += NG) {
        float f[8];
        if (j == cur) {
#pragma unroll
            for (int e = 0; e < 8; e++) f[e] = vcur[8 * c + e];
        } else {
            unpack8(reinterpret_cast<const uint4 *>(vc + (size_t)j * rowkv + (size_t)kvh * HD)[c], f);
        }
        float p = sc[j];
#pragma unroll
        for (int e = 0; e < 8; e++) acc[e] += p * f[e];
    }
#pragma unroll
    for (int e = 0; e < 8; e++) part[g * HD + 8 * c + e] = acc[e];
    __syncthreads();
    float o = 0.f;
    if (tid < HD) {
        for (int gg = 0; gg < NG; gg++) o += part[gg * HD + tid];
    }
    __syncthreads();
    if (tid < HD) {
        part[tid] = o;
        if (out) out[(size_t)h * HD + tid] = o;
    }
    if (xq) {
        __syncthreads();
        if (tid < HD / 4) {
            float4 vq = reinterpret_cast<const float4 *>(part)[tid];
            quantize_store4(vq, (size_t)h * HD + tid * 4, xq, row);
        }
    }
}

// ---- several sequences in one step: row m of q / k / v belongs to sequence m, which has a position of its own
// (pos_rows[m]) and a cache of its own (seq_stride elements after the one before it).
// Rotate q in place, rotate k and store it and v as fp16 cache row pos_rows[m] of sequence m.  blockIdx.y = m.
__global__ void rope_kv_rows_kernel(float *q, const float *k, const float *v, uint16_t *kcache, uint16_t *vcache, const int *pos_rows,
                                    size_t seq_stride, int n_heads, int n_kv_heads, int head_dim, const float *inv_freq) {
    int half = head_dim / 2;
    int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n_heads * half) return;
    int i = t % half;
    const size_t row = (size_t)n_heads * head_dim, rowkv = (size_t)n_kv_heads * head_dim, m = blockIdx.y;
    const int p = pos_rows[m];
    float s, c;
    sincosf((float)p * inv_freq[i], &s, &c);
    float2 *qr = reinterpret_cast<float2 *>(q + m * row);
    float2 qv = qr[t];
    qr[t] = make_float2(qv.x * c - qv.y * s, qv.x * s + qv.y * c);
    if (t >= n_kv_heads * half) return;          // fewer key / value heads than query heads
    float2 kv = reinterpret_cast<const float2 *>(k + m * rowkv)[t];
    float k0 = kv.x * c - kv.y * s, k1 = kv.x * s + kv.y * c;
    float2 vv = reinterpret_cast<const float2 *>(v + m * rowkv)[t];
    reinterpret_cast<uint32_t *>(kcache + m * seq_stride + (size_t)p * rowkv)[t] = (uint32_t)f2h_rne(k0) | ((uint32_t)f2h_rne(k1) << 16);
    reinterpret_cast<uint32_t *>(vcache + m * seq_stride + (size_t)p * rowkv)[t] = (uint32_t)f2h_rne(vv.x) | ((uint32_t)f2h_rne(vv.y) << 16);
}

// One workgroup (256 threads) per (query head, sequence): the rotated query row m against rows [0, pos_rows[m]] of sequence
// m's cache (the row of the step itself was stored by rope_kv_rows_kernel before).  Same arithmetic as the decode step's
// kernel in its plain form: a thread per position for the scores (the whole dot in the thread), max-subtracted softmax over
// the workgroup, values as 16-byte column chunks x position groups folded through LDS.  Dynamic LDS: max_pos floats.
// With xw.xq set the kernel is the whole attention block of the step of several sequences: q, k_new and v_new are the
// projections as the contractions left them; the workgroup rotates its query head and the step's key row by the sequence's
// position (rope_kv_rows_kernel's arithmetic), the first query head of a key / value group stores the rotated key and the
// value as the cache's row of that position, and every workgroup takes that row from its own LDS copy (rounded to fp16 as the
// cache holds it) instead of waiting for the store of another workgroup.  The result goes out in the operand form of the
// small-batch matrix-core GEMV (the o-projection's input; out is not written) and the grid has 8 rows: the rows from
// n_rows on are stored as zeros.
template <int HD>
__global__ __launch_bounds__(256) void attn_rows_kernel(const float *q, uint16_t *kc, uint16_t *vc, const int *pos_rows, size_t seq_stride,
                                                        int n_heads, int n_kv_heads, float *out, Xq8Work xw, int n_rows, const float *k_new,
                                                        const float *v_new, const float *inv_freq) {
    RT_DYN_LDS(float, sc);
    __shared__ float red[4];
    __shared__ __align__(16) float qs[HD];
    __shared__ __align__(16) float knew[HD], vnew[HD];
    __shared__ __align__(16) float part[2048];
    constexpr int CH = HD / 8;          // 16-byte chunks per cache row of this head
    constexpr int NG = 256 / CH;        // position groups in the value phase
    const int h = blockIdx.x, tid = threadIdx.x;
    const size_t m = blockIdx.y, row = (size_t)n_heads * HD, rowkv = (size_t)n_kv_heads * HD;
    const bool whole = xw.xq != nullptr;
    if ((int)m >= n_rows) {             // only in the operand form: a row without a sequence
        if (tid < HD / 4) xq8_store4(make_float4(0.f, 0.f, 0.f, 0.f), h * (HD / 4) + tid, (int)m, xw);
        return;
    }
    const int group = n_heads / n_kv_heads, kvh = h / group;
    const int last = pos_rows[m], n_pos = last + 1;
    kc += m * seq_stride + (size_t)kvh * HD;
    vc += m * seq_stride + (size_t)kvh * HD;
    const float scale = 1.0f / sqrtf((float)HD);
    if (whole) {
        if (tid < HD / 2) {
            float s, c;
            sincosf((float)last * inv_freq[tid], &s, &c);
            const float2 qv = reinterpret_cast<const float2 *>(q + m * row + (size_t)h * HD)[tid];
            qs[2 * tid] = qv.x * c - qv.y * s;
            qs[2 * tid + 1] = qv.x * s + qv.y * c;
            const float2 kv = reinterpret_cast<const float2 *>(k_new + m * rowkv + (size_t)kvh * HD)[tid];
            const float k0 = kv.x * c - kv.y * s, k1 = kv.x * s + kv.y * c;
            const float2 vv = reinterpret_cast<const float2 *>(v_new + m * rowkv + (size_t)kvh * HD)[tid];
            const uint32_t kh = (uint32_t)f2h_rne(k0) | ((uint32_t)f2h_rne(k1) << 16), vh = (uint32_t)f2h_rne(vv.x) | ((uint32_t)f2h_rne(vv.y) << 16);
            knew[2 * tid] = h2f(kh & 0xFFFF);
            knew[2 * tid + 1] = h2f(kh >> 16);
            vnew[2 * tid] = h2f(vh & 0xFFFF);
            vnew[2 * tid + 1] = h2f(vh >> 16);
            if (h == kvh * group) {
                reinterpret_cast<uint32_t *>(kc + (size_t)last * rowkv)[tid] = kh;
                reinterpret_cast<uint32_t *>(vc + (size_t)last * rowkv)[tid] = vh;
            }
        }
    } else if (tid < HD) {
        qs[tid] = q[m * row + (size_t)h * HD + tid];
    }
    __syncthreads();
    float mx = -INFINITY;
    for (int j = tid; j < n_pos; j += 256) {
        const uint4 *kr = reinterpret_cast<const uint4 *>(kc + (size_t)j * rowkv);
        const bool own = whole && j == last;      // this step's row: from LDS, the cache's copy may not be there yet
        float s = 0.f;
#pragma unroll
        for (int cc = 0; cc < CH; cc++) {
            float f[8];
            if (own) {
#pragma unroll
                for (int e = 0; e < 8; e++) f[e] = knew[8 * cc + e];
            } else {
                unpack8(kr[cc], f);
            }
#pragma unroll
            for (int e = 0; e < 8; e++) s += qs[8 * cc + e] * f[e];
        }
        s *= scale;
        sc[j] = s;
        mx = fmaxf(mx, s);
    }
    mx = block_max(mx, red);
    float sum = 0.f;
    for (int j = tid; j < n_pos; j += 256) {
        float e = expf(sc[j] - mx);
        sc[j] = e;
        sum += e;
    }
    sum = block_sum(sum, red);
    for (int j = tid; j < n_pos; j += 256) sc[j] = sc[j] / sum;
    __syncthreads();
    const int c = tid % CH, g = tid / CH;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; e++) acc[e] = 0.f;
    for (int j = g; j < n_pos; j += NG) {
        float f[8];
        if (whole && j == last) {
#pragma unroll
            for (int e = 0; e < 8; e++) f[e] = vnew[8 * c + e];
        } else {
            unpack8(reinterpret_cast<const uint4 *>(vc + (size_t)j * rowkv)[c], f);
        }
        const float p = sc[j];
#pragma unroll
        for (int e = 0; e < 8; e++) acc[e] += p * f[e];
    }
#pragma unroll
    for (int e = 0; e < 8; e++) part[g * HD + 8 * c + e] = acc[e];
    __syncthreads();
    if (tid < HD) {
        float o = 0.f;
        for (int gg = 0; gg < NG; gg++) o += part[gg * HD + tid];
        if (xw.xq) qs[tid] = o;         // the query row has done its work
        else out[m * row + (size_t)h * HD + tid] = o;
    }
    if (xw.xq) {
        __syncthreads();
        if (tid < HD / 4) xq8_store4(reinterpret_cast<const float4 *>(qs)[tid], h * (HD / 4) + tid, (int)m, xw);
    }
}

// ---- long contexts: the positions of a head are split over several workgroups
// Workgroup (h, s) of the fused decode step covers positions [s * chunk, (s + 1) * chunk) of query head h and leaves
// a partial result {m = max score, l = sum of exp(score - m), acc[HD] = sum of exp(score - m) * v} in
// partials[(h * n_splits + s) * (HD + 2)]; attn_combine_kernel folds the splits of a head:
//   M = max m_s,  out = sum_s acc_s * exp(m_s - M) / sum_s l_s * exp(m_s - M).
// The workgroup whose range holds the current position rotates k, stores the new cache row (first query head of
// a kv group only) and takes that row from LDS.  Splits past the current position report l = 0.
// Dynamic LDS: chunk floats.
template <int HD>
__global__ __launch_bounds__(256) void attn_split_kernel(const float *q, const float *k, const float *v, uint16_t *kc, uint16_t *vc,
                                                         const int *pos_dev, int chunk, int n_heads, int n_kv_heads,
                                                         const float *inv_freq, float *partials) {
    RT_DYN_LDS(float, sc);
    __shared__ float red[4];
    __shared__ __align__(16) float qs[HD];
    __shared__ __align__(16) float kcur[HD];
    __shared__ __align__(16) float vcur[HD];
    __shared__ __align__(16) float part[2048];
    constexpr int CH = HD / 8, NG = 256 / CH;
    const int h = blockIdx.x, sp = blockIdx.y, n_splits = gridDim.y, tid = threadIdx.x;
    const size_t rowkv = (size_t)n_kv_heads * HD;
    const int group = n_heads / n_kv_heads, kvh = h / group;
    const int cur = *pos_dev, n_pos = cur + 1;
    const int j0 = sp * chunk, j1 = min(n_pos, j0 + chunk);
    float *P = partials + ((size_t)h * n_splits + sp) * (HD + 2);
    if (j0 >= n_pos) {                        // nothing stored in this range yet
        if (tid == 0) { P[0] = -INFINITY; P[1] = 0.f; }
        return;
    }
    const bool owns_cur = cur >= j0 && cur < j1;
    const float scale = 1.0f / sqrtf((float)HD);
    const int c = tid % CH, g = tid / CH;
    // the thread's first key row does not depend on the new token: request it before the rotation
    uint4 kreg[CH];
    const int jt = j0 + tid;
    const bool k_pre = jt < j1 && jt != cur;
    if (k_pre) {
        const uint4 *kr = reinterpret_cast<const uint4 *>(kc + (size_t)jt * rowkv + (size_t)kvh * HD);
#pragma unroll
        for (int i = 0; i < CH; i++) kreg[i] = kr[i];
    }
    if (tid < HD / 2) {
        const int i = tid;
        float sn, cs;
        sincosf((float)cur * inv_freq[i], &sn, &cs);
        const float2 qv = reinterpret_cast<const float2 *>(q + (size_t)h * HD)[i];
        qs[2 * i] = qv.x * cs - qv.y * sn;
        qs[2 * i + 1] = qv.x * sn + qv.y * cs;
        if (owns_cur) {
            const float2 kv = reinterpret_cast<const float2 *>(k + (size_t)kvh * HD)[i];
            const uint16_t a = f2h_rne(kv.x * cs - kv.y * sn), b = f2h_rne(kv.x * sn + kv.y * cs);
            kcur[2 * i] = h2f(a);
            kcur[2 * i + 1] = h2f(b);
            if (h % group == 0) reinterpret_cast<uint32_t *>(kc + (size_t)cur * rowkv + (size_t)kvh * HD)[i] = (uint32_t)a | ((uint32_t)b << 16);
        }
    } else if (tid < HD && owns_cur) {
        const int i = tid - HD / 2;
        const float2 vv = reinterpret_cast<const float2 *>(v + (size_t)kvh * HD)[i];
        const uint16_t a = f2h_rne(vv.x), b = f2h_rne(vv.y);
        vcur[2 * i] = h2f(a);
        vcur[2 * i + 1] = h2f(b);
        if (h % group == 0) reinterpret_cast<uint32_t *>(vc + (size_t)cur * rowkv + (size_t)kvh * HD)[i] = (uint32_t)a | ((uint32_t)b << 16);
    }
    __syncthreads();
    float mx = -INFINITY;
    for (int j = jt; j < j1; j += 256) {
        float sum = 0.f;
        if (j == cur) {
#pragma unroll 8
            for (int d = 0; d < HD; d++) sum += qs[d] * kcur[d];
        } else {
            const uint4 *kr = reinterpret_cast<const uint4 *>(kc + (size_t)j * rowkv + (size_t)kvh * HD);
#pragma unroll
            for (int cc = 0; cc < CH; cc++) {
                float f[8];
                unpack8(j == jt ? kreg[cc] : kr[cc], f);
#pragma unroll
                for (int e = 0; e < 8; e++) sum += qs[8 * cc + e] * f[e];
            }
        }
        sum *= scale;
        sc[j - j0] = sum;
        mx = fmaxf(mx, sum);
    }
    mx = block_max(mx, red);
    float l = 0.f;
    for (int j = jt; j < j1; j += 256) {
        const float e = expf(sc[j - j0] - mx);
        sc[j - j0] = e;
        l += e;
    }
    l = block_sum(l, red);          // ends with a barrier: the weights are visible to every thread
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; e++) acc[e] = 0.f;
    for (int j = j0 + g; j < j1; j += NG) {
        float f[8];
        if (j == cur) {
#pragma unroll
            for (int e = 0; e < 8; e++) f[e] = vcur[8 * c + e];
        } else {
            unpack8(reinterpret_cast<const uint4 *>(vc + (size_t)j * rowkv + (size_t)kvh * HD)[c], f);
        }
        const float w = sc[j - j0];
#pragma unroll
        for (int e = 0; e < 8; e++) acc[e] += w * f[e];
    }
#pragma unroll
    for (int e = 0; e < 8; e++) part[g * HD + 8 * c + e] = acc[e];
    __syncthreads();
    if (tid < HD) {
        float o = 0.f;
        for (int gg = 0; gg < NG; gg++) o += part[gg * HD + tid];
        P[2 + tid] = o;
    }
    if (tid == 0) { P[0] = mx; P[1] = l; }
}

// One workgroup of HD threads per query head: fold the partial results of its splits, write the head's slice of the
// attention output (f32 when out != NULL) and its quantized form for the o-projection (when xq != NULL).
template <int HD>
__global__ __launch_bounds__(HD) void attn_combine_kernel(const float *partials, int n_splits, int n_heads, float *out, uint8_t *xq) {
    __shared__ __align__(16) float res[HD];
    const int h = blockIdx.x, tid = threadIdx.x;
    const float *P = partials + (size_t)h * n_splits * (HD + 2);
    float M = -INFINITY;
    for (int s = 0; s < n_splits; s++) M = fmaxf(M, P[(size_t)s * (HD + 2)]);
    float num = 0.f, den = 0.f;
    for (int s = 0; s < n_splits; s++) {
        const float *Ps = P + (size_t)s * (HD + 2);
        if (Ps[1] > 0.f) {                     // a split past the current position holds nothing (its acc is not written)
            const float w = expf(Ps[0] - M);
            num += Ps[2 + tid] * w;
            den += Ps[1] * w;
        }
    }
    const float o = num / den;
    res[tid] = o;
    if (out) out[(size_t)h * HD + tid] = o;
    if (xq) {
        __syncthreads();
        if (tid < HD / 4) quantize_store4(reinterpret_cast<const float4 *>(res)[tid], (size_t)h * HD + tid * 4, xq, (size_t)n_heads * HD);
    }
}

// ------------------------------------------------------------- small pieces
__global__ void add_kernel(float *x, const float *y, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] = x[i] + y[i];
}

// Measurement aid: reads n_chunks pieces of 2 KB once and throws them away, in the shape the decode GEMV reads its weights
// (persistent waves take pieces round-robin, the next piece requested before the current one is used, lanes on
// consecutive 16 bytes).  What this reaches is the practical ceiling a weight-streaming kernel is measured against.
__global__ __launch_bounds__(512) void stream_read_kernel(const uint4 *__restrict__ p, size_t n_chunks, unsigned *sink) {
    const int lane = (int)(threadIdx.x & 63);
    size_t c = (size_t)blockIdx.x * 8 + (threadIdx.x >> 6);
    const size_t n_gw = (size_t)gridDim.x * 8;
    unsigned acc = 0;
    uint4 a[2], b[2];
    if (c < n_chunks) { a[0] = p[c * 128 + lane]; a[1] = p[c * 128 + 64 + lane]; }
    while (c < n_chunks) {
        size_t c2 = c + n_gw;
        if (c2 < n_chunks) { b[0] = p[c2 * 128 + lane]; b[1] = p[c2 * 128 + 64 + lane]; }
        acc += a[0].x ^ a[0].y ^ a[0].z ^ a[0].w ^ a[1].x ^ a[1].y ^ a[1].z ^ a[1].w;
        c = c2;
        if (c >= n_chunks) break;
        c2 = c + n_gw;
        if (c2 < n_chunks) { a[0] = p[c2 * 128 + lane]; a[1] = p[c2 * 128 + 64 + lane]; }
        acc += b[0].x ^ b[0].y ^ b[0].z ^ b[0].w ^ b[1].x ^ b[1].y ^ b[1].z ^ b[1].w;
        c = c2;
    }
    if (acc == 0x12345678u) sink[0] = acc;      // keeps the loads alive; practically never taken
}

// Greedy pick; ties resolve to the lowest index.
// A thread's candidates are loaded eight at a time before they are compared (independent loads, one round trip per
// eight).  With `adv` the same launch ends the decode step: record the pick, choose the next input token, advance.
struct StepAdvance {
    int *pos_dev, *token_dev, *out_tokens_dev, *step_dev;
    const int *forced_dev;
    int enabled;
};
// The pick of one workgroup of 1024 threads over v[0..n); valid in thread 0.
__device__ __forceinline__ int block_argmax(const float *v, size_t n, float *bv, int *bi) {
    float best = -INFINITY;
    int idx = 0x7fffffff;
    for (size_t i0 = threadIdx.x; i0 < n; i0 += 8 * (size_t)blockDim.x) {
        float f[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const size_t i = i0 + (size_t)u * blockDim.x;
            f[u] = i < n ? v[i] : -INFINITY;
        }
#pragma unroll
        for (int u = 0; u < 8; u++)
            if (f[u] > best) { best = f[u]; idx = (int)(i0 + (size_t)u * blockDim.x); }      // ascending index: the first of equals stays
    }
    bv[threadIdx.x] = best;
    bi[threadIdx.x] = idx;
    __syncthreads();
    for (int s = blockDim.x / 2; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) {
            float o = bv[threadIdx.x + s];
            int oi = bi[threadIdx.x + s];
            if (o > bv[threadIdx.x] || (o == bv[threadIdx.x] && oi < bi[threadIdx.x])) {
                bv[threadIdx.x] = o;
                bi[threadIdx.x] = oi;
            }
        }
        __syncthreads();
    }
    return bi[0] == 0x7fffffff ? 0 : bi[0];
}

// One workgroup per row of v[rows][n]: out[row] = its pick (the step of several sequences).
__global__ __launch_bounds__(1024) void argmax_rows_kernel(const float *v, size_t n, int *out) {
    __shared__ float bv[1024];
    __shared__ int bi[1024];
    const int pick = block_argmax(v + (size_t)blockIdx.x * n, n, bv, bi);
    if (threadIdx.x == 0) out[blockIdx.x] = pick;
}

__global__ __launch_bounds__(1024) void argmax_kernel(const float *v, size_t n, int *out, StepAdvance adv) {
    __shared__ float bv[1024];
    __shared__ int bi[1024];
    const int pick = block_argmax(v, n, bv, bi);
    if (threadIdx.x == 0) {
        *out = pick;
        if (adv.enabled) {
            const int step = *adv.step_dev;
            if (adv.out_tokens_dev) adv.out_tokens_dev[step] = pick;
            *adv.token_dev = adv.forced_dev ? adv.forced_dev[step] : pick;
            *adv.pos_dev = *adv.pos_dev + 1;
            *adv.step_dev = step + 1;
        }
    }
}

__global__ void set_int_kernel(int *dst, int value) { *dst = value; }
__global__ void set_state_kernel(int *state, int pos, int token, int step) {
    state[0] = pos;
    state[1] = token;
    state[3] = step;
}

// End of a decode step: record the pick, choose the next input token, advance the position.
__global__ void step_advance_kernel(int *pos_dev, int *token_dev, const int *pick_dev, const int *forced_dev,
                                    int *out_tokens_dev, int *step_dev) {
    int step = *step_dev;
    int pick = *pick_dev;
    if (out_tokens_dev) out_tokens_dev[step] = pick;
    *token_dev = forced_dev ? forced_dev[step] : pick;
    *pos_dev = *pos_dev + 1;
    *step_dev = step + 1;
}

// Dense row-major f32 C[m,n] = A[m,k] . B[k,n], 32x32 tiles through LDS, k summed in ascending order; grid.z walks a batch
// of such products laid out one after the other (batch_matmul: src/gpu/matrix_ops.rs:308-343).  The kernel of small and
// odd-shaped products; larger ones go to the matrix cores (below).
__global__ __launch_bounds__(1024) void matmul_f32_kernel(const float *a, const float *b, float *c, size_t m, size_t n,
                                                          size_t k) {
    __shared__ float as[32][33];
    __shared__ float bs[32][33];
    a += (size_t)blockIdx.z * m * k;
    b += (size_t)blockIdx.z * k * n;
    c += (size_t)blockIdx.z * m * n;
    size_t row = (size_t)blockIdx.y * 32 + threadIdx.y, col = (size_t)blockIdx.x * 32 + threadIdx.x;
    float acc = 0.f;
    for (size_t k0 = 0; k0 < k; k0 += 32) {
        as[threadIdx.y][threadIdx.x] = (row < m && k0 + threadIdx.x < k) ? a[row * k + k0 + threadIdx.x] : 0.f;
        bs[threadIdx.y][threadIdx.x] = (col < n && k0 + threadIdx.y < k) ? b[(k0 + threadIdx.y) * n + col] : 0.f;
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 32; kk++) acc += as[threadIdx.y][kk] * bs[kk][threadIdx.x];
        __syncthreads();
    }
    if (row < m && col < n) c[row * n + col] = acc;
}

// The same product on the matrix cores, for operands whose rows are whole 16-byte pieces (n % 4 == 0, k % 4 == 0, 16-byte
// aligned bases): v_mfma_f32_32x32x2f32, f32 in and out.  Workgroup = 4 waves = a 128 x 128 tile of C, a wave a 64 x 64
// quarter of it as 2 x 2 blocks of 32 x 32 (64 accumulator registers).  k goes by in slices of 16 through a double-buffered
// LDS pair: A transposed to [k][m] (rows padded to 132 floats: a lane reads 32 consecutive m of one k), B as it lies,
// [k][n].  The slice after the current one is in flight in registers while the 32 matrix instructions of the current one
// run; a slice is 16 KB of global reads per 128 x 128 x 16 x 2 flop, so the kernel is bound by the matrix pipe
// (157 TFLOP/s dense f32), not by HBM.  Lane l of a wave gives A[l % 32][l / 32] and B[l / 32][l % 32] of a k pair;
// accumulator r holds C[8 (r / 4) + 4 (l / 32) + r % 4][l % 32] of the block.  Rows and columns past the matrix are
// loaded as zeros and not stored.
typedef float float16v __attribute__((ext_vector_type(16)));
constexpr int kMmTile = 128, kMmK = 16, kMmLda = kMmTile + 4;
__global__ __launch_bounds__(256) void matmul_f32_mfma_kernel(const float *a, const float *b, float *c, size_t m, size_t n, size_t k) {
    __shared__ __align__(16) float as[2][kMmK][kMmLda];
    __shared__ __align__(16) float bs[2][kMmK][kMmTile];
    a += (size_t)blockIdx.z * m * k;
    b += (size_t)blockIdx.z * k * n;
    c += (size_t)blockIdx.z * m * n;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1, l32 = lane & 31, lh = lane >> 5;
    const size_t m0 = (size_t)blockIdx.y * kMmTile, n0 = (size_t)blockIdx.x * kMmTile;
    float16v acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
    // a thread's two 16-byte pieces of each operand's slice: A piece (row, 4 k), B piece (k row, 4 columns)
    float4 ra[2], rb[2];
    auto fetch = [&](size_t k0) {
#pragma unroll
        for (int p = 0; p < 2; p++) {
            const int idx = tid + 256 * p;
            const size_t row = m0 + (size_t)(idx >> 2), ka = k0 + 4 * (size_t)(idx & 3);
            ra[p] = (row < m && ka < k) ? *reinterpret_cast<const float4 *>(a + row * k + ka) : make_float4(0.f, 0.f, 0.f, 0.f);
            const size_t kb = k0 + (size_t)(idx >> 5), col = n0 + 4 * (size_t)(idx & 31);
            rb[p] = (kb < k && col < n) ? *reinterpret_cast<const float4 *>(b + kb * n + col) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    auto park = [&](int buf) {
#pragma unroll
        for (int p = 0; p < 2; p++) {
            const int idx = tid + 256 * p, row = idx >> 2, kq = 4 * (idx & 3);
            as[buf][kq + 0][row] = ra[p].x;
            as[buf][kq + 1][row] = ra[p].y;
            as[buf][kq + 2][row] = ra[p].z;
            as[buf][kq + 3][row] = ra[p].w;
            *reinterpret_cast<float4 *>(&bs[buf][idx >> 5][4 * (idx & 31)]) = rb[p];
        }
    };
    fetch(0);
    park(0);
    __syncthreads();
    int buf = 0;
    for (size_t k0 = 0; k0 < k; k0 += kMmK) {
        const bool more = k0 + kMmK < k;
        if (more) fetch(k0 + kMmK);
#pragma unroll
        for (int kp = 0; kp < kMmK / 2; kp++) {
            const int kk = 2 * kp + lh;
            const float a0 = as[buf][kk][wm * 64 + l32], a1 = as[buf][kk][wm * 64 + 32 + l32];
            const float b0 = bs[buf][kk][wn * 64 + l32], b1 = bs[buf][kk][wn * 64 + 32 + l32];
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
        }
        if (more) park(buf ^ 1);      // the other buffer: its last readers passed the barrier at the end of the previous slice
        __syncthreads();
        buf ^= 1;
    }
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const size_t col = n0 + (size_t)(wn * 64 + j * 32 + l32);
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const size_t row = m0 + (size_t)(wm * 64 + i * 32 + 8 * (r / 4) + 4 * lh + r % 4);
                if (row < m && col < n) c[row * n + col] = acc[i][j][r];
            }
        }
}

// Per-tensor affine int8 matmul (QuantizedOps::qmatmul, src/quantization/operations.rs:195-260):
// out[i][j] = clamp_i8(round(((float)sum * scale) / scale)), sum = sum_l (a[i][l] - za)(b[l][j] - zb), scale = sa * sb.
// 64x64 output tile per workgroup of 256 threads (4x4 outputs each), 64-deep k slices through LDS; a slice is
// summed in 32-bit (|term| <= 383^2, 64 terms) and added to a 64-bit total, so the sum is exact as in the
// reference's i64.  The float tail is kept free of contraction: its two roundings are part of the result.
#pragma clang fp contract(off)
__global__ __launch_bounds__(256) void qmatmul_i8_kernel(const int8_t *a, const int8_t *b, int8_t *out, size_t m, size_t n, size_t k,
                                                         int za, int zb, float scale) {
    __shared__ int16_t as[64][64 + 2];     // [row][l], zero point already removed
    __shared__ int16_t bs[64][64 + 2];     // [l][col]
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const size_t row0 = (size_t)blockIdx.y * 64, col0 = (size_t)blockIdx.x * 64;
    long long acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = 0;
    for (size_t k0 = 0; k0 < k; k0 += 64) {
        for (int e = threadIdx.x; e < 64 * 64; e += 256) {
            const int r = e >> 6, c = e & 63;
            as[r][c] = (row0 + r < m && k0 + c < k) ? (int16_t)((int)a[(row0 + r) * k + k0 + c] - za) : (int16_t)0;
            bs[r][c] = (k0 + r < k && col0 + c < n) ? (int16_t)((int)b[(k0 + r) * n + col0 + c] - zb) : (int16_t)0;
        }
        __syncthreads();
        int part[4][4];
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) part[i][j] = 0;
#pragma unroll 8
        for (int l = 0; l < 64; l++) {
            int av[4], bv[4];
#pragma unroll
            for (int i = 0; i < 4; i++) av[i] = as[ty + 16 * i][l];
#pragma unroll
            for (int j = 0; j < 4; j++) bv[j] = bs[l][tx + 16 * j];
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) part[i][j] += av[i] * bv[j];
        }
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) acc[i][j] += part[i][j];
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const size_t r = row0 + ty + 16 * i, c = col0 + tx + 16 * j;
            if (r >= m || c >= n) continue;
            const float fp = (float)acc[i][j] * scale;
            const float q = roundf(fp / scale);
            int v;
            if (q != q) v = 0;                                   // Rust's float -> int cast: NaN -> 0, saturating
            else if (q >= 2147483648.0f) v = 2147483647;
            else if (q <= -2147483648.0f) v = -2147483647 - 1;
            else v = (int)q;
            out[r * n + c] = (int8_t)(v > 127 ? 127 : (v < -128 ? -128 : v));
        }
}
#pragma clang fp contract(fast)

// ================================================================ launchers

hipError_t launch_qmatmul_i8(hipStream_t s, const int8_t *a, const int8_t *b, int8_t *out, size_t m, size_t n, size_t k, int za, int zb,
                             float scale) {
    dim3 grid((unsigned)((n + 63) / 64), (unsigned)((m + 63) / 64));
    qmatmul_i8_kernel<<<grid, 256, 0, s>>>(a, b, out, m, n, k, za, zb, scale);
    return hipGetLastError();
}

hipError_t launch_quantize_x(hipStream_t s, const float *x, uint8_t *xq, size_t K, size_t batch) {
    dim3 grid((unsigned)((K / 4 + 255) / 256), (unsigned)batch);
    quantize_x_kernel<<<grid, 256, 0, s>>>(x, xq, K);
    return hipGetLastError();
}

hipError_t launch_quantize_group(hipStream_t s, const QuantGroupArgs &a) {
    size_t maxK = 0;
    for (int i = 0; i < a.n; i++) maxK = (size_t)a.K[i] > maxK ? (size_t)a.K[i] : maxK;
    if (a.n == 0 || maxK == 0) return hipSuccess;
    dim3 grid((unsigned)((maxK / 4 + 255) / 256), (unsigned)a.n);
    quantize_group_kernel<<<grid, 256, 0, s>>>(a);
    return hipGetLastError();
}

hipError_t launch_dequant(hipStream_t s, int type, const uint8_t *w, size_t n_rows, size_t n_cols, float *out) {
    size_t total = n_rows * n_cols;
    size_t rb = n_cols / type_block_elems(type) * type_block_bytes(type);
    size_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (blocks == 0) return hipSuccess;
    dequant_kernel<<<dim3((unsigned)blocks), 256, 0, s>>>(type, w, rb, n_rows, n_cols, out);
    return hipGetLastError();
}

hipError_t launch_rmsnorm(hipStream_t s, const float *x, const float *gamma, float *y, uint8_t *xq, size_t rows,
                          size_t n, float eps) {
    if (rows == 0) return hipSuccess;
    rmsnorm_kernel<<<dim3((unsigned)rows), 1024, 0, s>>>(x, gamma, y, xq, n, eps);
    return hipGetLastError();
}

hipError_t launch_swiglu(hipStream_t s, const float *gate, const float *up, float *out, uint8_t *xq, size_t n) {
    if (n == 0) return hipSuccess;
    size_t n4 = (n + 3) / 4;
    swiglu_kernel<<<dim3((unsigned)((n4 + 255) / 256)), 256, 0, s>>>(gate, up, out, xq, n);
    return hipGetLastError();
}

hipError_t launch_rope(hipStream_t s, float *x, int n_heads, int head_dim, const int *pos_dev, int pos,
                       const float *inv_freq_dev, float theta) {
    int pairs = n_heads * head_dim / 2;
    if (pairs == 0) return hipSuccess;
    rope_kernel<<<dim3((unsigned)((pairs + 255) / 256)), 256, 0, s>>>(x, n_heads, head_dim, pos_dev, pos, inv_freq_dev,
                                                                      theta);
    return hipGetLastError();
}

hipError_t launch_kv_append(hipStream_t s, uint16_t *cache, const float *v, const int *pos_dev, size_t pos,
                            size_t row_elems) {
    if (row_elems == 0) return hipSuccess;
    kv_append_kernel<<<dim3((unsigned)((row_elems + 255) / 256)), 256, 0, s>>>(cache, v, pos_dev, pos, row_elems);
    return hipGetLastError();
}

hipError_t launch_rope_kv(hipStream_t s, float *q, const float *k, const float *v, uint16_t *kcache,
                          uint16_t *vcache, const int *pos_dev, int n_heads, int head_dim,
                          const float *inv_freq_dev) {
    int pairs = n_heads * head_dim / 2;
    rope_kv_kernel<<<dim3((unsigned)((pairs + 255) / 256)), 256, 0, s>>>(q, k, v, kcache, vcache, pos_dev, n_heads,
                                                                         head_dim, inv_freq_dev);
    return hipGetLastError();
}

hipError_t launch_rope_kv_batch(hipStream_t s, float *q, const float *k, const float *v, uint16_t *kcache, uint16_t *vcache,
                                int pos0, size_t n_tok, int n_heads, int n_kv_heads, int head_dim, const float *inv_freq_dev) {
    if (n_kv_heads <= 0 || n_heads % n_kv_heads != 0) return hipErrorInvalidValue;
    int pairs = n_heads * head_dim / 2;
    rope_kv_batch_kernel<<<dim3((unsigned)((pairs + 255) / 256), (unsigned)n_tok), 256, 0, s>>>(q, k, v, kcache, vcache, pos0, n_heads,
                                                                                                n_kv_heads, head_dim, inv_freq_dev);
    return hipGetLastError();
}

hipError_t launch_rope_kv_rows(hipStream_t s, float *q, const float *k, const float *v, uint16_t *kcache, uint16_t *vcache, const int *pos_rows_dev,
                               size_t seq_stride, size_t n_rows, int n_heads, int n_kv_heads, int head_dim, const float *inv_freq_dev) {
    if (n_kv_heads <= 0 || n_heads % n_kv_heads != 0 || n_rows == 0 || n_rows > 65535) return hipErrorInvalidValue;
    int pairs = n_heads * head_dim / 2;
    rope_kv_rows_kernel<<<dim3((unsigned)((pairs + 255) / 256), (unsigned)n_rows), 256, 0, s>>>(q, k, v, kcache, vcache, pos_rows_dev, seq_stride,
                                                                                                n_heads, n_kv_heads, head_dim, inv_freq_dev);
    return hipGetLastError();
}

// Two forms.  (1) out set: q rotated, the caches hold the step's rows (launch_rope_kv_rows before); result [n_rows][n_heads *
// head_dim] f32.  (2) out == nullptr, xq8_work_buf, k_new, v_new and inv_freq_dev set: q, k_new, v_new as projected; the launch
// rotates, appends to the caches and leaves the result in the operand form of the small-batch matrix-core GEMV in that
// workspace (n_rows <= 8, n_heads * head_dim a multiple of 256).
hipError_t launch_attn_rows(hipStream_t s, const float *q, uint16_t *kc, uint16_t *vc, const int *pos_rows_dev, size_t seq_stride, int max_pos,
                            size_t n_rows, int n_heads, int n_kv_heads, int head_dim, float *out, void *xq8_work_buf, const float *k_new,
                            const float *v_new, const float *inv_freq_dev) {
    if (n_kv_heads <= 0 || n_heads % n_kv_heads != 0 || n_rows == 0 || n_rows > 65535 || max_pos <= 0 || max_pos > 8192) return hipErrorInvalidValue;
    if ((out == nullptr) == (xq8_work_buf == nullptr)) return hipErrorInvalidValue;
    const size_t H = (size_t)n_heads * (size_t)head_dim;
    if (xq8_work_buf && (n_rows > 8 || H % 256 != 0 || ((uintptr_t)xq8_work_buf & 255) || !k_new || !v_new || !inv_freq_dev)) return hipErrorInvalidValue;
    const size_t lds = (size_t)max_pos * sizeof(float);      // at most 32 KB beside the 10 KB of static arrays: inside the default 64 KB
    const Xq8Work xw = xq8_work_buf ? xq8_work(xq8_work_buf, H) : Xq8Work{ nullptr, nullptr, nullptr };
    dim3 grid((unsigned)n_heads, xq8_work_buf ? 8u : (unsigned)n_rows);
    if (head_dim == 128)
        attn_rows_kernel<128><<<grid, 256, lds, s>>>(q, kc, vc, pos_rows_dev, seq_stride, n_heads, n_kv_heads, out, xw, (int)n_rows, k_new, v_new, inv_freq_dev);
    else if (head_dim == 64)
        attn_rows_kernel<64><<<grid, 256, lds, s>>>(q, kc, vc, pos_rows_dev, seq_stride, n_heads, n_kv_heads, out, xw, (int)n_rows, k_new, v_new, inv_freq_dev);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

// RMSNorm / SwiGLU of `rows` <= 8 rows of n elements (n % 256 == 0) into the operand form of the small-batch matrix-core GEMV
hipError_t launch_rmsnorm_xq8(hipStream_t s, const float *x, const float *gamma, size_t rows, size_t n, float eps, void *work) {
    if (!x || !gamma || !work || rows < 1 || rows > 8 || n < 256 || n % 256 != 0) return hipErrorInvalidValue;
    if (((uintptr_t)x & 15) || ((uintptr_t)gamma & 15) || ((uintptr_t)work & 255)) return hipErrorInvalidValue;
    rmsnorm_xq8_kernel<<<8, 1024, 0, s>>>(x, gamma, n, eps, (int)rows, xq8_work(work, n));
    return hipGetLastError();
}

hipError_t launch_swiglu_xq8(hipStream_t s, const float *gate, const float *up, size_t rows, size_t n, void *work) {
    if (!gate || !up || !work || rows < 1 || rows > 8 || n < 256 || n % 256 != 0) return hipErrorInvalidValue;
    if (((uintptr_t)gate & 15) || ((uintptr_t)up & 15) || ((uintptr_t)work & 255)) return hipErrorInvalidValue;
    swiglu_xq8_kernel<<<dim3((unsigned)((n / 4 + 255) / 256), 8), 256, 0, s>>>(gate, up, n, (int)rows, xq8_work(work, n));
    return hipGetLastError();
}

hipError_t launch_rope_kv_planes(hipStream_t s, PlaneSum q, PlaneSum k, PlaneSum v, float *q_out, uint16_t *kcache, uint16_t *vcache,
                                 int pos0, size_t n_tok, int n_heads, int n_kv_heads, int head_dim, const float *inv_freq_dev) {
    if (n_kv_heads <= 0 || n_heads % n_kv_heads != 0 || n_tok == 0 || n_tok > 65535 || q.n < 1 || k.n < 1 || v.n < 1) return hipErrorInvalidValue;
    int pairs = n_heads * head_dim / 2;
    rope_kv_planes_kernel<<<dim3((unsigned)((pairs + 255) / 256), (unsigned)n_tok), 256, 0, s>>>(q, k, v, q_out, kcache, vcache, pos0, n_heads,
                                                                                                 n_kv_heads, head_dim, inv_freq_dev);
    return hipGetLastError();
}

hipError_t launch_attn_decode(hipStream_t s, float *q, const float *k, const float *v, uint16_t *kc, uint16_t *vc,
                              const int *pos_dev, int n_pos, int n_heads, int n_kv_heads, int head_dim, const float *inv_freq_dev,
                              float *out, uint8_t *xq, bool fused) {
    return launch_attn_batch(s, q, k, v, kc, vc, pos_dev, n_pos, 1, n_heads, n_kv_heads, head_dim, inv_freq_dev, out, xq, fused);
}

// n_queries > 1 (not fused, xq == NULL): query m of q [n_queries][row] attends over the first n_pos + m cache rows
hipError_t launch_attn_batch(hipStream_t s, float *q, const float *k, const float *v, uint16_t *kc, uint16_t *vc,
                             const int *pos_dev, int n_pos, size_t n_queries, int n_heads, int n_kv_heads, int head_dim,
                             const float *inv_freq_dev, float *out, uint8_t *xq, bool fused) {
    if (n_queries > 1 && (fused || xq)) return hipErrorInvalidValue;
    if (n_kv_heads <= 0 || n_heads % n_kv_heads != 0) return hipErrorInvalidValue;
    size_t lds = ((size_t)n_pos + n_queries - 1) * sizeof(float);  // fused: n_pos is the upper bound (max_pos)
    dim3 grid((unsigned)n_heads, (unsigned)n_queries);
    if (head_dim == 128 && fused)
        attn_decode_kernel<128, true><<<grid, 256, lds, s>>>(q, k, v, kc, vc, pos_dev, n_pos, n_heads, n_kv_heads, inv_freq_dev, out, xq);
    else if (head_dim == 128)
        attn_decode_kernel<128, false><<<grid, 256, lds, s>>>(q, k, v, kc, vc, pos_dev, n_pos, n_heads, n_kv_heads, inv_freq_dev, out, xq);
    else if (head_dim == 64 && fused)
        attn_decode_kernel<64, true><<<grid, 256, lds, s>>>(q, k, v, kc, vc, pos_dev, n_pos, n_heads, n_kv_heads, inv_freq_dev, out, xq);
    else if (head_dim == 64)
        attn_decode_kernel<64, false><<<grid, 256, lds, s>>>(q, k, v, kc, vc, pos_dev, n_pos, n_heads, n_kv_heads, inv_freq_dev, out, xq);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

// Fused decode step over a long context: n_splits workgroups per head (positions in chunks of ceil(max_pos / n_splits)),
// then the fold.  partials: n_heads * n_splits * (head_dim + 2) floats.
hipError_t launch_attn_decode_split(hipStream_t s, const float *q, const float *k, const float *v, uint16_t *kc, uint16_t *vc,
                                    const int *pos_dev, int max_pos, int n_splits, int n_heads, int n_kv_heads, int head_dim,
                                    const float *inv_freq_dev, float *partials, float *out, uint8_t *xq) {
    if (n_kv_heads <= 0 || n_heads % n_kv_heads != 0 || n_splits < 1) return hipErrorInvalidValue;
    const int chunk = (max_pos + n_splits - 1) / n_splits;
    const size_t lds = (size_t)chunk * sizeof(float);
    dim3 grid((unsigned)n_heads, (unsigned)n_splits);
    if (head_dim == 128) {
        attn_split_kernel<128><<<grid, 256, lds, s>>>(q, k, v, kc, vc, pos_dev, chunk, n_heads, n_kv_heads, inv_freq_dev, partials);
        attn_combine_kernel<128><<<dim3((unsigned)n_heads), 128, 0, s>>>(partials, n_splits, n_heads, out, xq);
    } else if (head_dim == 64) {
        attn_split_kernel<64><<<grid, 256, lds, s>>>(q, k, v, kc, vc, pos_dev, chunk, n_heads, n_kv_heads, inv_freq_dev, partials);
        attn_combine_kernel<64><<<dim3((unsigned)n_heads), 64, 0, s>>>(partials, n_splits, n_heads, out, xq);
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_add(hipStream_t s, float *x, const float *y, size_t n) {
    if (n == 0) return hipSuccess;
    add_kernel<<<dim3((unsigned)((n + 255) / 256)), 256, 0, s>>>(x, y, n);
    return hipGetLastError();
}

hipError_t launch_stream_read(hipStream_t s, const void *p, size_t nbytes, unsigned *sink) {
    const size_t n_chunks = nbytes / 2048;       // whole pieces only: nothing past p + nbytes is touched
    if (n_chunks == 0) return hipSuccess;
    stream_read_kernel<<<512, 512, 0, s>>>(reinterpret_cast<const uint4 *>(p), n_chunks, sink);
    return hipGetLastError();
}

hipError_t launch_argmax_rows(hipStream_t s, const float *v, size_t rows, size_t n, int *out_dev) {
    if (rows == 0 || rows > 65535) return hipErrorInvalidValue;
    argmax_rows_kernel<<<(unsigned)rows, 1024, 0, s>>>(v, n, out_dev);
    return hipGetLastError();
}

hipError_t launch_argmax(hipStream_t s, const float *v, size_t n, int *out_dev) {
    argmax_kernel<<<1, 1024, 0, s>>>(v, n, out_dev, StepAdvance{ nullptr, nullptr, nullptr, nullptr, nullptr, 0 });
    return hipGetLastError();
}

hipError_t launch_argmax_advance(hipStream_t s, const float *v, size_t n, int *pick_dev, int *pos_dev, int *token_dev, const int *forced_dev,
                                 int *out_tokens_dev, int *step_dev) {
    argmax_kernel<<<1, 1024, 0, s>>>(v, n, pick_dev, StepAdvance{ pos_dev, token_dev, out_tokens_dev, step_dev, forced_dev, 1 });
    return hipGetLastError();
}

hipError_t launch_embed_row(hipStream_t s, int type, const uint8_t *w, size_t row_bytes, size_t n_cols,
                            const int *token_dev, int vocab, float *out) {
    return launch_embed_rows(s, type, w, row_bytes, n_cols, token_dev, 1, vocab, out);
}

hipError_t launch_embed_rows(hipStream_t s, int type, const uint8_t *w, size_t row_bytes, size_t n_cols,
                             const int *tokens_dev, size_t n_tok, int vocab, float *out) {
    embed_row_kernel<<<dim3((unsigned)((n_cols + 255) / 256), (unsigned)n_tok), 256, 0, s>>>(type, w, row_bytes, n_cols, tokens_dev,
                                                                                             vocab, out);
    return hipGetLastError();
}

hipError_t launch_matmul_f32(hipStream_t s, const float *a, const float *b, float *c, size_t m, size_t n, size_t k, size_t batch) {
    if (m == 0 || n == 0 || batch == 0) return hipSuccess;
    if (batch > 65535 || (m + 31) / 32 > 65535) return hipErrorInvalidValue;
    // the matrix cores take products large enough to fill tiles and laid out in whole 16-byte pieces; the rest (the
    // reference's 2 x 2 known answer, odd widths, matrix-vector products) goes through the plain kernel
    const bool pieces = n % 4 == 0 && k % 4 == 0 && (((uintptr_t)a | (uintptr_t)b) & 15) == 0;
    if (pieces && m >= 64 && n >= 64 && k >= kMmK && path_option(RT_HIP_OPT_DENSE_MFMA) == 1) {      // opt-in (rt_hip_set_option)
        dim3 grid((unsigned)((n + kMmTile - 1) / kMmTile), (unsigned)((m + kMmTile - 1) / kMmTile), (unsigned)batch);
        matmul_f32_mfma_kernel<<<grid, 256, 0, s>>>(a, b, c, m, n, k);
        return hipGetLastError();
    }
    dim3 grid((unsigned)((n + 31) / 32), (unsigned)((m + 31) / 32), (unsigned)batch);
    matmul_f32_kernel<<<grid, dim3(32, 32), 0, s>>>(a, b, c, m, n, k);
    return hipGetLastError();
}

hipError_t launch_set_state(hipStream_t s, int *state, int pos, int token, int step) {
    set_state_kernel<<<1, 1, 0, s>>>(state, pos, token, step);
    return hipGetLastError();
}

hipError_t launch_set_int(hipStream_t s, int *dst, int value) {
    set_int_kernel<<<1, 1, 0, s>>>(dst, value);
    return hipGetLastError();
}

hipError_t launch_step_advance(hipStream_t s, int *pos_dev, int *token_dev, const int *pick_dev,
                               const int *forced_dev, int *out_tokens_dev, int *step_dev) {
    step_advance_kernel<<<1, 1, 0, s>>>(pos_dev, token_dev, pick_dev, forced_dev, out_tokens_dev, step_dev);
    return hipGetLastError();
}

}  // namespace rt
