// One decode step of a Llama model as a single persistent launch: 1 workgroup of 1024 threads per CU,
// all of a token's GEMVs, the attention and the greedy pick run as phases of one kernel separated by a
// software grid barrier.
//
// Why: a decode step streams ~130 MB of weights per layer in five dependent pieces of 9..51 MB.  As
// separate launches each piece pays a kernel boundary (drain, cache write-back, ramp-up) that is as long
// as the piece's own transfer time.  Inside one launch the workgroups keep their weight loads in flight
// across phase boundaries: the first weight slices of the next phase are requested before the barrier
// wait and before the input vector is staged, because weights do not depend on activations.
//
// Coherence: workgroups on different XCDs do not share an L2, so every activation that crosses a phase
// (x, q, k, v, attention output, f, logits) is written and read with device-scope relaxed atomics, which
// go around the per-XCD L2.  That keeps the barrier free of cache write-backs and invalidations: it only
// drains the workgroup's own stores and then synchronises on counters.  Weights and the KV cache of
// earlier tokens are read-only during a launch and use the normal cached path.
//
// State of this code: NOT part of the library.  Its one run on the GPU ended in a memory fault whose cause has not been
// found, so no translation unit of the product includes this header and rt_hip_llama_set_mode refuses mode 0; what
// remains is the device code and its CPU run as fibers under AddressSanitizer (tests/emu/emu_main.cpp).
//
// Barrier: two levels (8 group counters on separate cache lines, one top counter, one generation flag);
// every spin is bounded, a time-out raises an error flag that makes all workgroups leave the kernel.
#pragma once

#include "rt_gemv_device.h"

namespace rt {

// ---- arguments of the step kernel
struct MegaLayer {
    const uint8_t *wq, *wk, *wv, *wo, *wgate, *wup, *wdown;
    size_t rb_q, rb_k, rb_v, rb_o, rb_g, rb_d;
    int t_q, t_k, t_v, t_o, t_g, t_d;
    const float *attn_norm, *ffn_norm;
    uint16_t *kc, *vc;  // this layer's fp16 cache rows [max_pos][hidden]
};
struct MegaArgs {
    const MegaLayer *layers;  // device array
    int n_layers, hidden, n_heads, head_dim, ffn, vocab, max_pos;
    float eps;
    const uint8_t *embd; size_t rb_embd; int t_embd;
    const uint8_t *wout; size_t rb_out; int t_out;
    const float *out_norm;
    float *x, *q, *k, *v, *a, *f, *logits;
    const float *inv_freq;
    int *state;          // [0] pos, [1] token, [2] pick, [3] step
    const int *forced;   // optional: token fed at the next step
    int *out_tokens;     // optional: picks by step
    unsigned *bar;       // kMegaBarBytes of barrier words, zeroed by the launcher
    int wg_q, wg_k;      // workgroups given to the q and k matrices in the q/k/v phase (v takes the rest)
    int want_logits, do_advance;
};
constexpr size_t kMegaBarBytes = 4096;
constexpr size_t kMegaErrWord = 32 * 24;  // index of the time-out flag inside the barrier words
constexpr int kMegaThreads = 1024;
// Launch-sized LDS of the step kernel: the larger of the GEMV staging area, the attention phase
// (q / k / v of the step, per-group partial outputs, scores) and the greedy-pick scratch.
inline size_t mega_lds_bytes(int hidden, int ffn, int head_dim, int max_pos) {
    size_t g = xq_stride((size_t)(hidden > ffn ? hidden : ffn));
    size_t a = ((size_t)3 * head_dim + (size_t)(kMegaThreads / (head_dim / 8)) * head_dim + (size_t)max_pos) * sizeof(float);
    size_t m = g > a ? g : a;
    size_t am = (size_t)2 * kMegaThreads * sizeof(float);
    return m > am ? m : am;
}


constexpr unsigned kSpinLimit = 1u << 21;
constexpr unsigned kBarGroups = 8;

struct Bar {
    unsigned *mem;   // [0] generation flag, [32*(1+g)] group counters, [32*20] top counter, [32*24] error flag
    unsigned gen;
    unsigned nwg;
};

__device__ __forceinline__ bool grid_barrier(Bar &B) {
    __builtin_amdgcn_s_waitcnt(0);  // this wave's coherent stores have been acknowledged
    __syncthreads();
    __shared__ int ok;
    if (threadIdx.x == 0) {
        int good = 1;
        unsigned spins = 0;
        B.gen += 1;
        unsigned *flag = B.mem, *err = B.mem + 32 * 24;
        unsigned grp = blockIdx.x % kBarGroups, per = B.nwg / kBarGroups;
        unsigned prev = __hip_atomic_fetch_add(B.mem + 32 * (1 + grp), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (prev + 1 == B.gen * per) {
            unsigned p2 = __hip_atomic_fetch_add(B.mem + 32 * 20, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (p2 + 1 == B.gen * kBarGroups) __hip_atomic_store(flag, B.gen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < B.gen) {
            __builtin_amdgcn_s_sleep(1);
            ++spins;
            // bounded wait: give up after kSpinLimit polls, or as soon as another workgroup has given up
            if (spins > kSpinLimit || ((spins & 255u) == 0 && __hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
                __hip_atomic_store(err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                good = 0;
                break;
            }
        }
        ok = good;
    }
    __syncthreads();
    return ok != 0;
}

__device__ __forceinline__ GemvProb mk_prob(const uint8_t *w, size_t rb, int type, int N, int K, const void *x, int stage,
                                            float *y, const float *res) {
    GemvProb p;
    p.w = w; p.w2 = nullptr; p.x = x; p.gamma = nullptr; p.y = y; p.res = res; p.row_bytes = rb; p.eps = 0.f;
    p.type = type; p.N = N; p.K = K; p.stage = stage; p.epi = kEpiStore; p.tile0 = 0; p.rows_per_tile = 0;
    return p;
}

__device__ __forceinline__ void unpack8h(uint4 v, float *f) {
    const uint32_t w[4] = { v.x, v.y, v.z, v.w };
#pragma unroll
    for (int i = 0; i < 4; i++) {
        f[2 * i] = h2f(w[i] & 0xFFFF);
        f[2 * i + 1] = h2f(w[i] >> 16);
    }
}

// Head h of the attention phase with all 1024 threads of the workgroup: rotate q / k of this step, append
// fp16 k / v at row pos, attend over [0, pos] (example-cli/src/model/architectures/attention.rs:233-338 for
// one query row).  LDS (floats): qs[HD] kcur[HD] vcur[HD] | part[(1024 / (HD/8)) * HD] | sc[pos + 1].
template <int HD>
__device__ __forceinline__ void attn_head(const MegaArgs &A, const MegaLayer &L, int h, int pos, float *ldsf, float *red) {
    constexpr int CH = HD / 8, NG = kMegaThreads / CH;
    float *qs = ldsf, *kcur = ldsf + HD, *vcur = ldsf + 2 * HD, *part = ldsf + 3 * HD, *sc = part + NG * HD;
    const int tid = threadIdx.x, n_pos = pos + 1;
    const size_t row = (size_t)A.n_heads * HD;
    const float scale = 1.0f / sqrtf((float)HD);
    if (tid < HD / 2) {
        int i = tid;
        float sn, cs;
        sincosf((float)pos * A.inv_freq[i], &sn, &cs);
        float qx = ld_f<true>(A.q + (size_t)h * HD + 2 * i), qy = ld_f<true>(A.q + (size_t)h * HD + 2 * i + 1);
        float kx = ld_f<true>(A.k + (size_t)h * HD + 2 * i), ky = ld_f<true>(A.k + (size_t)h * HD + 2 * i + 1);
        qs[2 * i] = qx * cs - qy * sn;
        qs[2 * i + 1] = qx * sn + qy * cs;
        uint16_t a = f2h_rne(kx * cs - ky * sn), b = f2h_rne(kx * sn + ky * cs);
        kcur[2 * i] = h2f(a);
        kcur[2 * i + 1] = h2f(b);
        reinterpret_cast<uint32_t *>(L.kc + (size_t)pos * row + (size_t)h * HD)[i] = (uint32_t)a | ((uint32_t)b << 16);
    } else if (tid < HD) {
        int i = tid - HD / 2;
        float vx = ld_f<true>(A.v + (size_t)h * HD + 2 * i), vy = ld_f<true>(A.v + (size_t)h * HD + 2 * i + 1);
        uint16_t a = f2h_rne(vx), b = f2h_rne(vy);
        vcur[2 * i] = h2f(a);
        vcur[2 * i + 1] = h2f(b);
        reinterpret_cast<uint32_t *>(L.vc + (size_t)pos * row + (size_t)h * HD)[i] = (uint32_t)a | ((uint32_t)b << 16);
    }
    __syncthreads();
    float mx = -INFINITY;
    for (int j = tid; j < n_pos; j += kMegaThreads) {
        float s = 0.f;
        if (j == pos) {
#pragma unroll 8
            for (int d = 0; d < HD; d++) s += qs[d] * kcur[d];
        } else {
            const uint4 *kr = reinterpret_cast<const uint4 *>(L.kc + (size_t)j * row + (size_t)h * HD);
#pragma unroll
            for (int c = 0; c < CH; c++) {
                float f[8];
                unpack8h(kr[c], f);
#pragma unroll
                for (int e = 0; e < 8; e++) s += qs[8 * c + e] * f[e];
            }
        }
        s *= scale;
        sc[j] = s;
        mx = fmaxf(mx, s);
    }
    mx = block_max(mx, red);
    float sum = 0.f;
    for (int j = tid; j < n_pos; j += kMegaThreads) {
        float e = expf(sc[j] - mx);
        sc[j] = e;
        sum += e;
    }
    sum = block_sum(sum, red);
    for (int j = tid; j < n_pos; j += kMegaThreads) sc[j] = sc[j] / sum;
    __syncthreads();
    const int c = tid % CH, g = tid / CH;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; e++) acc[e] = 0.f;
    for (int j = g; j < n_pos; j += NG) {
        float f[8];
        if (j == pos) {
#pragma unroll
            for (int e = 0; e < 8; e++) f[e] = vcur[8 * c + e];
        } else {
            unpack8h(reinterpret_cast<const uint4 *>(L.vc + (size_t)j * row + (size_t)h * HD)[c], f);
        }
        float p = sc[j];
#pragma unroll
        for (int e = 0; e < 8; e++) acc[e] += p * f[e];
    }
#pragma unroll
    for (int e = 0; e < 8; e++) part[g * HD + 8 * c + e] = acc[e];
    __syncthreads();
    if (tid < HD) {
        float o = 0.f;
        for (int gg = 0; gg < NG; gg++) o += part[gg * HD + tid];
        st_f<true>(A.a + (size_t)h * HD + tid, o);
    }
    __syncthreads();
}

__global__ __launch_bounds__(kMegaThreads) void llama_step_kernel(MegaArgs A) {
    RT_DYN_LDS(uint4, lds4);
    __shared__ float red[kMegaThreads / 64];
    uint32_t *lds = reinterpret_cast<uint32_t *>(lds4);
    const int wg = blockIdx.x, nwg = gridDim.x, tid = threadIdx.x;
    Bar B{ A.bar, 0u, (unsigned)nwg };
    const int pos = A.state[0];
    int tok = A.state[1];
    tok = tok < 0 ? 0 : (tok >= A.vocab ? A.vocab - 1 : tok);
    const int H = A.hidden, F = A.ffn;

    // embedding row -> x
    for (int c = wg * kMegaThreads + tid; c < H; c += nwg * kMegaThreads)
        st_f<true>(A.x + c, deq_elem(A.t_embd, A.embd + (size_t)tok * A.rb_embd, (size_t)c));
    if (!grid_barrier(B)) return;

    // Phases 0..4 of each layer, then the output head as one more phase; every GEMV goes through the same
    // call site so the compiler keeps one copy of the streaming loops.
    const int n_phase = 5 * A.n_layers + (A.want_logits ? 1 : 0);
    for (int ph = 0; ph < n_phase; ph++) {
        const int l = ph / 5, k = ph - 5 * l;
        const bool head = l == A.n_layers;
        const MegaLayer &L = A.layers[head ? 0 : l];
        if (!head && k == 1) {
            // rope + cache append + attention, one workgroup per head
            if (wg < A.n_heads) {
                if (A.head_dim == 128) attn_head<128>(A, L, wg, pos, reinterpret_cast<float *>(lds), red);
                else attn_head<64>(A, L, wg, pos, reinterpret_cast<float *>(lds), red);
            }
        } else {
            GemvProb P;
            int first = 0, n = nwg;
            if (head) {                 // logits = Wout . rmsnorm(x)
                P = mk_prob(A.wout, A.rb_out, A.t_out, A.vocab, H, A.x, kStageRms, A.logits, nullptr);
                P.gamma = A.out_norm; P.eps = A.eps;
            } else if (k == 0) {        // q, k, v = W . rmsnorm(x): workgroups split over the three matrices by bytes
                if (wg < A.wg_q) {
                    P = mk_prob(L.wq, L.rb_q, L.t_q, H, H, A.x, kStageRms, A.q, nullptr); n = A.wg_q;
                } else if (wg < A.wg_q + A.wg_k) {
                    P = mk_prob(L.wk, L.rb_k, L.t_k, H, H, A.x, kStageRms, A.k, nullptr); first = A.wg_q; n = A.wg_k;
                } else {
                    P = mk_prob(L.wv, L.rb_v, L.t_v, H, H, A.x, kStageRms, A.v, nullptr); first = A.wg_q + A.wg_k; n = nwg - first;
                }
                P.gamma = L.attn_norm; P.eps = A.eps;
            } else if (k == 2) {        // x += Wo . a
                P = mk_prob(L.wo, L.rb_o, L.t_o, H, H, A.a, kStageF32, A.x, A.x);
            } else if (k == 3) {        // f = up(h) * silu(gate(h)), h = rmsnorm(x)
                P = mk_prob(L.wgate, L.rb_g, L.t_g, F, H, A.x, kStageRms, A.f, nullptr);
                P.w2 = L.wup; P.epi = kEpiSwiglu; P.gamma = L.ffn_norm; P.eps = A.eps;
            } else {                    // x += Wdown . f
                P = mk_prob(L.wdown, L.rb_d, L.t_d, H, F, A.f, kStageF32, A.x, A.x);
            }
            gemv_dispatch<true, false>(P, wg - first, n, 0, false, lds, red);
        }
        if (!grid_barrier(B)) return;
    }
    if (!A.want_logits) {
        // prompt tokens other than the last: no output head; every workgroup read state[] before the first barrier
        if (wg == 0 && tid == 0 && A.do_advance) {
            int step = A.state[3];
            if (A.forced) A.state[1] = A.forced[step];
            A.state[0] = pos + 1;
            A.state[3] = step + 1;
        }
        return;
    }
    if (wg != 0) return;
    // greedy pick by workgroup 0 (ties -> lowest index), then advance the device-side state
    float *bv = reinterpret_cast<float *>(lds);
    int *bi = reinterpret_cast<int *>(lds) + kMegaThreads;
    float best = -INFINITY;
    int idx = 0x7fffffff;
    for (int i = tid; i < A.vocab; i += kMegaThreads) {
        float f = ld_f<true>(A.logits + i);
        if (f > best) { best = f; idx = i; }
    }
    bv[tid] = best;
    bi[tid] = idx;
    __syncthreads();
    for (int s = kMegaThreads / 2; s > 0; s >>= 1) {
        if (tid < s) {
            float o = bv[tid + s];
            int oi = bi[tid + s];
            if (o > bv[tid] || (o == bv[tid] && oi < bi[tid])) { bv[tid] = o; bi[tid] = oi; }
        }
        __syncthreads();
    }
    if (tid == 0) {
        int pick = bi[0] == 0x7fffffff ? 0 : bi[0];
        A.state[2] = pick;
        if (A.do_advance) {
            int step = A.state[3];
            if (A.out_tokens) A.out_tokens[step] = pick;
            A.state[1] = A.forced ? A.forced[step] : pick;
            A.state[0] = pos + 1;
            A.state[3] = step + 1;
        }
    }
}

}  // namespace rt
