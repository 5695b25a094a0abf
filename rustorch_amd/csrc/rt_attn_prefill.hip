// Causal attention of a batch of consecutive query rows over the fp16 cache, on the matrix cores.
//   row m (position pos0 + m) attends cache rows [0, pos0 + m]:
//   scores_k = (q_m . k_k) / sqrt(head_dim);  p = softmax(scores) with max subtraction;  out_m = sum_k p_k v_k
// (example-cli/src/model/architectures/attention.rs:233-338: the masked scores, softmax and weighted sum of a
// whole sequence; here the keys and values are the cache rows, as in the decode step).
//
// One workgroup per 32 consecutive queries of one head, against tiles of 32 cache rows, flash style (running maximum
// and sum per query, accumulated output rescaled when the maximum moves).  The four waves of the workgroup take the
// tiles in turn (wave w: tiles w, w + 4, ...), each with its own running state and its own LDS tile, and never meet
// before the end, where the four partial results {max, sum, output} are folded through LDS.  Both products run on
// v_mfma_f32_32x32x16_f16 with the f32 operand split into two fp16 terms (value = hi + lo, both exact in the f32
// accumulation), so the result keeps f32-level accuracy:
//   S^T[key][query] = K . (Qhi + Qlo)^T    the lane's 16 scores belong to ONE query (lane % 32): its maximum and sum
//                                          are an in-lane reduction plus one exchange with lane ^ 32
//   O^T[d][query]   = V^T . (Phi + Plo)^T  the 16 probabilities of a lane are, as they stand, the second operand
//                                          (keys permuted, the same permutation picks the V elements from LDS)
// q is scaled per query by a power of two that brings its largest magnitude into [2^13, 2^14) and p by 2^14, so
// the lo terms stay normal fp16 numbers; both factors leave with the final scaling.
#include "rt_device.h"
#include "rt_internal.h"

namespace rt {
namespace {

typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kAttnWaves = 4;

// Orders the LDS traffic of ONE wave (a tile written by all its lanes, then read across lanes).  The hardware runs a
// wave's LDS instructions in order; this keeps the compiler from moving them across the point.  Not a workgroup
// barrier: the waves of a workgroup run different numbers of tiles.
__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

template <int HD>
__global__ __launch_bounds__(64 * kAttnWaves) void attn_causal_kernel(const float *q, const uint16_t *kc, const uint16_t *vc, int pos0, int M,
                                                         int n_heads, int n_kv_heads, float *out) {
    constexpr int KK = HD / 16;           // 16-wide steps of the score product
    constexpr int DB = HD / 32;           // 32-row blocks of the head dimension in the output product
    constexpr int VS = HD + 8;            // halves per value row in LDS (16-byte aligned, rows 4 apart fall on different banks)
    constexpr int CPR = HD / 8;           // 16-byte chunks per cache row of one head
    constexpr int VL = 32 * CPR / 64;     // 16-byte loads per lane for a tile of 32 value rows
    constexpr int W = kAttnWaves;
    constexpr int PS = 2 * 16 + 4;        // floats per lane of a fold round: two accumulator blocks, max, sum (padded to 16 bytes)
    constexpr int kTileBytes = W * 32 * VS * 2, kPartBytes = W * 64 * PS * 4;
    __shared__ __align__(16) uint8_t lds[kTileBytes > kPartBytes ? kTileBytes : kPartBytes];    // the partials reuse the tiles' space

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), j = lane & 31, hh = lane >> 5;
    uint16_t *vs = reinterpret_cast<uint16_t *>(lds) + wave * 32 * VS;
    const int h = blockIdx.x, qb = blockIdx.y;
    const int group = n_heads / n_kv_heads, kvh = h / group;
    const size_t row = (size_t)n_heads * HD, rowkv = (size_t)n_kv_heads * HD;
    const int m = qb * 32 + j;                       // the lane's query
    const int mq = min(m, M - 1);                    // lanes past the batch repeat its last query and store nothing
    const int last_key = pos0 + mq;
    const int n_keys = pos0 + min(qb * 32 + 31, M - 1) + 1;     // cache rows any query of this workgroup sees
    const int T = (n_keys + 31) / 32;

    // ---- the query fragments: lane (j, hh) holds elements 16 kk + 8 hh .. + 7 of query j for every kk
    float qf[KK][8];
    float amax = 0.f;
    {
        const float *qp = q + (size_t)mq * row + (size_t)h * HD + 8 * hh;
#pragma unroll
        for (int kk = 0; kk < KK; kk++) {
            const float4 a = *reinterpret_cast<const float4 *>(qp + 16 * kk), b = *reinterpret_cast<const float4 *>(qp + 16 * kk + 4);
            qf[kk][0] = a.x; qf[kk][1] = a.y; qf[kk][2] = a.z; qf[kk][3] = a.w;
            qf[kk][4] = b.x; qf[kk][5] = b.y; qf[kk][6] = b.z; qf[kk][7] = b.w;
#pragma unroll
            for (int e = 0; e < 8; e++) amax = fmaxf(amax, fabsf(qf[kk][e]));
        }
    }
    amax = fmaxf(amax, __shfl_xor(amax, 32));
    int ex = 0;
    if (amax > 0.f) frexpf(amax, &ex);               // amax = f * 2^ex, f in [0.5, 1)
    ex = max(ex, -100);
    const float qscale = ldexpf(1.0f, 14 - ex);
    const float sscale = ldexpf(1.0f, ex - 14) * (1.0f / sqrtf((float)HD));
    half8v qhi[KK], qlo[KK];
#pragma unroll
    for (int kk = 0; kk < KK; kk++)
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float v = qf[kk][e] * qscale;
            const _Float16 hi = (_Float16)v;
            qhi[kk][e] = hi;
            qlo[kk][e] = (_Float16)(v - (float)hi);
        }

    // ---- tiles of 32 cache rows; the next tile's rows are requested before the current one is used
    const uint16_t *kbase = kc + (size_t)kvh * HD + 8 * hh;
    const uint16_t *vbase = vc + (size_t)kvh * HD;
    half8v kn[KK];
    u32x4 vn[VL];
    auto request = [&](int t) {
        const int key = min(32 * t + j, n_keys - 1);          // rows past the last visible one repeat it (their scores are masked)
        const uint16_t *kp = kbase + (size_t)key * rowkv;
#pragma unroll
        for (int kk = 0; kk < KK; kk++) kn[kk] = *reinterpret_cast<const half8v *>(kp + 16 * kk);
#pragma unroll
        for (int i = 0; i < VL; i++) {
            const int c = i * 64 + lane, vkey = min(32 * t + c / CPR, n_keys - 1);
            vn[i] = *reinterpret_cast<const u32x4 *>(vbase + (size_t)vkey * rowkv + 8 * (c % CPR));
        }
    };
    request(min(wave, T - 1));

    float16v acc[DB];
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[db][r] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;
    const _Float16 *vsh = reinterpret_cast<const _Float16 *>(vs);

    for (int t = wave; t < T; t += W) {
        half8v kcur[KK];
#pragma unroll
        for (int kk = 0; kk < KK; kk++) kcur[kk] = kn[kk];
        wave_lds_fence();                                     // the previous tile's value reads come first
#pragma unroll
        for (int i = 0; i < VL; i++) {
            const int c = i * 64 + lane;
            *reinterpret_cast<u32x4 *>(vs + (c / CPR) * VS + 8 * (c % CPR)) = vn[i];
        }
        request(min(t + W, T - 1));                          // past the end a tile is requested again: no branch around the loads
        wave_lds_fence();

        // scores: register r of lane (j, hh) is key 8 (r / 4) + 4 hh + r % 4 of the tile against query j
        float16v s;
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = 0.f;
#pragma unroll
        for (int kk = 0; kk < KK; kk++) {
            s = __builtin_amdgcn_mfma_f32_32x32x16_f16(kcur[kk], qhi[kk], s, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_32x32x16_f16(kcur[kk], qlo[kk], s, 0, 0, 0);
        }
        float mt = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int key = 32 * t + 8 * (r >> 2) + 4 * hh + (r & 3);
            s[r] = key <= last_key ? s[r] * sscale : -INFINITY;
            mt = fmaxf(mt, s[r]);
        }
        mt = fmaxf(mt, __shfl_xor(mt, 32));
        // Finite from wave 0's first tile on (key 0 is visible to every query), but not in every wave: with pos0 off a
        // multiple of 32 the first tile of a later wave can lie wholly beyond an early query.  Such a query keeps
        // max = -inf, sum = 0 and a zero accumulator in that wave (exp(-inf - (-inf)) would make them NaN), and the
        // fold below gives the wave the factor 0.
        const float m_new = fmaxf(m_run, mt);
        const float m_ref = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = expf(m_run - m_ref);
        float psum = 0.f;
        half8v phi[2], plo[2];
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const float p = expf(s[r] - m_ref);
            psum += p;
            const float ps = p * 16384.0f;
            const _Float16 hi = (_Float16)ps;
            phi[r >> 3][r & 7] = hi;
            plo[r >> 3][r & 7] = (_Float16)(ps - (float)hi);
        }
        psum += __shfl_xor(psum, 32);
        l_run = l_run * alpha + psum;
        m_run = m_new;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[db][r] *= alpha;

        // output: slot e of product mm stands for the key of score register 8 mm + e, i.e. row 16 mm + 8 (e / 4) + 4 hh + e % 4
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int mm = 0; mm < 2; mm++) {
                half8v av;
#pragma unroll
                for (int e = 0; e < 8; e++) av[e] = vsh[(16 * mm + 8 * (e >> 2) + 4 * hh + (e & 3)) * VS + 32 * db + j];
                acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, phi[mm], acc[db], 0, 0, 0);
                acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, plo[mm], acc[db], 0, 0, 0);
            }
    }

    // ---- fold the waves' partial results, two 32-element blocks of the head dimension per round; in a round wave w
    // finishes half of block (w & 1).  Register r of lane (j, hh) is element 32 db + 8 (r / 4) + 4 hh + r % 4 of query j.
    float *part = reinterpret_cast<float *>(lds);
    float *mine = part + (size_t)(wave * 64 + lane) * PS;
    float fw[W], inv = 0.f;
#pragma unroll
    for (int c = 0; c < DB / 2; c++) {
        __syncthreads();                                      // the tiles (first round) or the previous round's reads are done
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int g = 0; g < 4; g++)
                *reinterpret_cast<float4 *>(mine + 16 * b + 4 * g) =
                    make_float4(acc[2 * c + b][4 * g], acc[2 * c + b][4 * g + 1], acc[2 * c + b][4 * g + 2], acc[2 * c + b][4 * g + 3]);
        if (c == 0) *reinterpret_cast<float2 *>(mine + 32) = make_float2(m_run, l_run);
        __syncthreads();
        if (c == 0) {
            float lw[W], m_all = -INFINITY;
#pragma unroll
            for (int w = 0; w < W; w++) {
                const float2 ml = *reinterpret_cast<const float2 *>(part + (size_t)(w * 64 + lane) * PS + 32);
                fw[w] = ml.x;
                lw[w] = ml.y;
                m_all = fmaxf(m_all, ml.x);                   // finite: wave 0 always has tile 0
            }
            float l_all = 0.f;
#pragma unroll
            for (int w = 0; w < W; w++) {
                fw[w] = expf(fw[w] - m_all);                  // a wave without tiles reports max = -inf: factor 0
                l_all += lw[w] * fw[w];
            }
            inv = 1.0f / (l_all * 16384.0f);
        }
        const int b = wave & 1, db = 2 * c + b;
#pragma unroll
        for (int gi = 0; gi < 2; gi++) {
            const int g = 2 * (wave >> 1) + gi;
            float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int w = 0; w < W; w++) {
                const float4 a = *reinterpret_cast<const float4 *>(part + (size_t)(w * 64 + lane) * PS + 16 * b + 4 * g);
                o.x += a.x * fw[w]; o.y += a.y * fw[w]; o.z += a.z * fw[w]; o.w += a.w * fw[w];
            }
            if (m < M)
                *reinterpret_cast<float4 *>(out + (size_t)m * row + (size_t)h * HD + 4 * hh + 32 * db + 8 * g) =
                    make_float4(o.x * inv, o.y * inv, o.z * inv, o.w * inv);
        }
    }
}

}  // namespace

hipError_t launch_attn_causal(hipStream_t s, const float *q, const uint16_t *kc, const uint16_t *vc, int pos0, size_t n_queries,
                              int n_heads, int n_kv_heads, int head_dim, float *out) {
    if (n_queries == 0) return hipSuccess;
    if ((head_dim != 64 && head_dim != 128) || pos0 < 0 || n_heads <= 0 || n_kv_heads <= 0 || n_heads % n_kv_heads != 0 ||
        n_queries > (size_t)65535 * 32 || (size_t)pos0 + n_queries > (size_t)INT32_MAX / 2)
        return hipErrorInvalidValue;
    // 16-byte accesses to every operand
    if (((uintptr_t)q | (uintptr_t)kc | (uintptr_t)vc | (uintptr_t)out) & 15) return hipErrorInvalidValue;
    const dim3 grid((unsigned)n_heads, (unsigned)((n_queries + 31) / 32));
    if (head_dim == 128)
        attn_causal_kernel<128><<<grid, 64 * kAttnWaves, 0, s>>>(q, kc, vc, pos0, (int)n_queries, n_heads, n_kv_heads, out);
    else
        attn_causal_kernel<64><<<grid, 64 * kAttnWaves, 0, s>>>(q, kc, vc, pos0, (int)n_queries, n_heads, n_kv_heads, out);
    return hipGetLastError();
}

}  // namespace rt
