// Llama-architecture decode loop on one GPU: weights stay in HBM as raw GGUF
// blocks, the KV cache is fp16 [layer][pos][head][dim], and one decode step is a
// fixed sequence of kernels driven by device-resident position / token state, so
// consecutive steps need no host round trip.
//
// Step order (pre-norm residual block of example-cli/src/model/architectures/gpt.rs:43-55,192-215
// with RMSNorm / RoPE / SwiGLU / causal cache in place of LayerNorm / sinusoidal PE / ReLU / full recompute):
//   x = embd[token]
//   per layer: h = rmsnorm(x); q,k,v = W h; rope(q,k); cache <- k,v; a = attn(q, cache);
//              x += Wo a; h = rmsnorm(x); x += Wdown (up(h) * silu(gate(h)))
//   logits = Wout rmsnorm(x)
#include "rt_internal.h"

#include <cmath>
#include <algorithm>
#include <cstring>
#include <new>
#include <vector>

using rt::ensure_scratch;
using rt::fail;
using rt::Guard;
using rt::hip_fail;

struct rt_hip_llama {
    struct T {
        int type = -1;
        size_t n_rows = 0, n_cols = 0, row_bytes = 0, nbytes = 0;
        uint8_t *dev = nullptr;
        _Float16 *f16 = nullptr;    // fp16 copy, made when a batched prefill first meets a matrix whose format has no fused contraction
    };
    rt_hip_llama_config cfg{};
    int head_dim = 0;
    int n_kv = 0;             // key / value heads; kv_dim = n_kv * head_dim is the width of k, v and of a cache row
    size_t kv_dim = 0;
    int attn_splits = 1;      // workgroups per head in the decode step's attention (long contexts), fixed by max_pos
    float *attn_part = nullptr;
    T tok_embd, output;
    float *out_norm = nullptr;
    std::vector<T> wq, wk, wv, wo, wgate, wup, wdown;
    std::vector<float *> attn_norm, ffn_norm;
    uint16_t *kcache = nullptr, *vcache = nullptr;
    // the cache the batched prefill passes write and attend: the model's own ([layer][max_pos][kv_dim]), or for the length of one
    // call a sequence of a batch object (rt_hip_llama_batch_prefill); layer l starts pf_layer_stride * l elements in
    uint16_t *pf_kcache = nullptr, *pf_vcache = nullptr;
    size_t pf_layer_stride = 0;
    float *x = nullptr, *q = nullptr, *k = nullptr, *v = nullptr, *g = nullptr, *u = nullptr, *logits = nullptr;
    uint8_t *xq_h = nullptr, *xq_a = nullptr, *xq_f = nullptr;
    float *inv_freq = nullptr;
    int *state = nullptr;  // [0] pos, [1] token, [2] pick, [3] step
    int *forced_dev = nullptr, *out_tokens_dev = nullptr;
    int n_fed = 0;
    // persistent step kernel
    int mode = 1;             // 1: separate launches (default), 2: the same launches replayed from a captured graph (0, a persistent step kernel, is refused)
    // mode 2: one graph per (want_logits, advance, use_forced); a combination runs eagerly once, is captured at its
    // second use and replayed from then on.  Every argument of a step is a device pointer or a model constant
    // (position and token live in `state`), so one capture serves every later token.
    struct StepGraph { int uses = 0; hipGraph_t graph = nullptr; hipGraphExec_t exec = nullptr; };
    StepGraph step_graphs[8];
    float *a = nullptr;       // attention output, f32
    // batched prefill (dense contraction path): activations of up to pf_cap tokens
    size_t pf_cap = 0;
    float *pf_x = nullptr, *pf_x2 = nullptr, *pf_n = nullptr, *pf_q = nullptr, *pf_k = nullptr, *pf_v = nullptr, *pf_a = nullptr;
    float *pf_g = nullptr, *pf_u = nullptr;
    int *pf_tok = nullptr;
    // chained form of the batched prefill: prepared activation matrix, its row scales, three areas of partial planes
    _Float16 *pf_xp = nullptr;
    float *pf_inv = nullptr, *pf_planes[3] = { nullptr, nullptr, nullptr };
    size_t pf_planes_bytes = 0;
    std::vector<void *> allocs;
};

// Several sequences decoded side by side against one model's weights (the model's own cache serves its own single
// sequence): every sequence has a position and a cache of its own, one step feeds one token per sequence and runs every
// matrix once for all of them.
struct rt_hip_llama_batch {
    rt_hip_llama *m = nullptr;
    int n_seq = 0, max_pos = 0;
    std::vector<int> fed;                     // tokens fed so far, per sequence
    uint16_t *kcache = nullptr, *vcache = nullptr;      // [layer][sequence][max_pos][kv_dim] fp16
    float *x = nullptr, *x2 = nullptr, *n = nullptr, *q = nullptr, *k = nullptr, *v = nullptr, *a = nullptr, *g = nullptr, *u = nullptr;
    float *logits = nullptr;                  // [sequence][vocab]
    int *tok = nullptr, *pos = nullptr, *pick = nullptr;
    std::vector<void *> allocs;
};

namespace {

#ifndef RT_ATTN_SPLIT_MIN
#define RT_ATTN_SPLIT_MIN 512
#endif

int dev_alloc(rt_hip_ctx *ctx, rt_hip_llama *m, void **p, size_t bytes) {
    RT_TRY_HIP(ctx, hipMalloc(p, bytes ? bytes : 1));
    m->allocs.push_back(*p);
    return RT_HIP_OK;
}

// Gives a buffer of the model back before the model itself goes (a replaced tensor, an outgrown workspace).  The stream is
// drained first: launches that still name the buffer may be in flight.
void dev_release(rt_hip_ctx *ctx, rt_hip_llama *m, void *p) {
    if (!p) return;
    for (size_t i = 0; i < m->allocs.size(); i++) {
        if (m->allocs[i] != p) continue;
        (void)hipStreamSynchronize(ctx->stream);
        (void)hipFree(p);
        m->allocs[i] = m->allocs.back();
        m->allocs.pop_back();
        return;
    }
}

// Captured steps name device pointers: drop them whenever a tensor or buffer they name may change.
void drop_step_graphs(rt_hip_llama *m) {
    for (auto &g : m->step_graphs) {
        if (g.exec) (void)hipGraphExecDestroy(g.exec);
        if (g.graph) (void)hipGraphDestroy(g.graph);
        g = rt_hip_llama::StepGraph();
    }
}

void free_all(rt_hip_llama *m) {
    drop_step_graphs(m);
    for (void *p : m->allocs) (void)hipFree(p);
    m->allocs.clear();
}

rt::GemvProb make_prob(const rt_hip_llama::T &t, const void *x, int stage, float *y, const float *res) {
    rt::GemvProb p;
    memset(&p, 0, sizeof p);
    p.w = t.dev; p.x = x; p.stage = stage; p.y = y; p.res = res; p.row_bytes = t.row_bytes;
    p.type = t.type; p.N = (int)t.n_rows; p.K = (int)t.n_cols;
    return p;
}

int check_complete(rt_hip_ctx *ctx, const rt_hip_llama *m) {
    RT_REQUIRE(ctx, m->tok_embd.dev && m->output.dev && m->out_norm, RT_HIP_ERR_INVALID_ARG,
               "llama: token embedding / output head / output norm not uploaded");
    for (int l = 0; l < m->cfg.n_layers; l++) {
        bool ok = m->wq[l].dev && m->wk[l].dev && m->wv[l].dev && m->wo[l].dev && m->wgate[l].dev && m->wup[l].dev &&
                  m->wdown[l].dev && m->attn_norm[l] && m->ffn_norm[l];
        RT_REQUIRE(ctx, ok, RT_HIP_ERR_INVALID_ARG, "llama: layer %d has tensors that were not uploaded", l);
    }
    return RT_HIP_OK;
}

// One decode step driven by state[0] (pos) and state[1] (token). Enqueue only.  Five launches per layer:
//   q,k,v = W . rmsnorm(x)         (norm + quantization fused into the GEMV's staging)
//   rope + cache append + attention (output in the GEMV's quantized form)
//   x += Wo . a
//   f = up(h) * silu(gate(h)), h = rmsnorm(x)   (norm in the staging, SwiGLU in the epilogue)
//   x += Wdown . f                  (quantization of f in the staging)
int enqueue_step(rt_hip_ctx *ctx, rt_hip_llama *m, bool want_logits) {
    hipStream_t s = ctx->stream;
    const rt_hip_llama_config &c = m->cfg;
    const size_t H = (size_t)c.hidden;
    int *pos_dev = m->state, *tok_dev = m->state + 1;
    RT_TRY_HIP(ctx, rt::launch_embed_row(s, m->tok_embd.type, m->tok_embd.dev, m->tok_embd.row_bytes, H, tok_dev, c.vocab, m->x));
    for (int l = 0; l < c.n_layers; l++) {
        uint16_t *kc = m->kcache + (size_t)l * (size_t)c.max_pos * m->kv_dim;
        uint16_t *vc = m->vcache + (size_t)l * (size_t)c.max_pos * m->kv_dim;
        rt::GemvArgs a;
        memset(&a, 0, sizeof a);
        a.n = 3;
        a.p[0] = make_prob(m->wq[l], m->x, rt::kStageRms, m->q, nullptr);
        a.p[1] = make_prob(m->wk[l], m->x, rt::kStageRms, m->k, nullptr);
        a.p[2] = make_prob(m->wv[l], m->x, rt::kStageRms, m->v, nullptr);
        for (int i = 0; i < 3; i++) { a.p[i].gamma = m->attn_norm[l]; a.p[i].eps = c.rms_eps; }
        RT_TRY_HIP(ctx, rt::launch_qgemv(s, a, 1));
        if (m->attn_splits > 1)
            RT_TRY_HIP(ctx, rt::launch_attn_decode_split(s, m->q, m->k, m->v, kc, vc, pos_dev, c.max_pos, m->attn_splits, c.n_heads, m->n_kv,
                                                         m->head_dim, m->inv_freq, m->attn_part, nullptr, m->xq_a));
        else
            RT_TRY_HIP(ctx, rt::launch_attn_decode(s, m->q, m->k, m->v, kc, vc, pos_dev, c.max_pos, c.n_heads, m->n_kv, m->head_dim, m->inv_freq,
                                                   nullptr, m->xq_a, true));
        memset(&a, 0, sizeof a);
        a.n = 1;
        a.p[0] = make_prob(m->wo[l], m->xq_a, rt::kStageXq, m->x, m->x);
        RT_TRY_HIP(ctx, rt::launch_qgemv(s, a, 1));
        memset(&a, 0, sizeof a);
        if (m->wgate[l].type == m->wup[l].type && m->wgate[l].type != RT_GGML_Q5_K && m->wgate[l].type != RT_GGML_Q3_K &&
            m->wgate[l].type != RT_GGML_Q2_K) {
            a.n = 1;
            a.p[0] = make_prob(m->wgate[l], m->x, rt::kStageRms, m->g, nullptr);
            a.p[0].w2 = m->wup[l].dev; a.p[0].epi = rt::kEpiSwiglu; a.p[0].gamma = m->ffn_norm[l]; a.p[0].eps = c.rms_eps;
            RT_TRY_HIP(ctx, rt::launch_qgemv(s, a, 1));
        } else {
            // gate and up of different block formats, or of one without the pair form: two problems in one launch, then SwiGLU
            a.n = 2;
            a.p[0] = make_prob(m->wgate[l], m->x, rt::kStageRms, m->g, nullptr);
            a.p[1] = make_prob(m->wup[l], m->x, rt::kStageRms, m->u, nullptr);
            for (int i = 0; i < 2; i++) { a.p[i].gamma = m->ffn_norm[l]; a.p[i].eps = c.rms_eps; }
            RT_TRY_HIP(ctx, rt::launch_qgemv(s, a, 1));
            RT_TRY_HIP(ctx, rt::launch_swiglu(s, m->g, m->u, m->g, nullptr, (size_t)c.ffn));
        }
        memset(&a, 0, sizeof a);
        a.n = 1;
        a.p[0] = make_prob(m->wdown[l], m->g, rt::kStageF32, m->x, m->x);
        RT_TRY_HIP(ctx, rt::launch_qgemv(s, a, 1));
    }
    if (want_logits) {
        rt::GemvArgs a;
        memset(&a, 0, sizeof a);
        a.n = 1;
        a.p[0] = make_prob(m->output, m->x, rt::kStageRms, m->logits, nullptr);
        a.p[0].gamma = m->out_norm; a.p[0].eps = c.rms_eps;
        RT_TRY_HIP(ctx, rt::launch_qgemv(s, a, 1));
    }
    return RT_HIP_OK;
}

bool gemv_type_ok(int t) {
    return t == RT_GGML_F32 || t == RT_GGML_F16 || t == RT_GGML_Q8_0 || t == RT_GGML_Q8_1 || t == RT_GGML_Q4_0 || t == RT_GGML_Q4_1 || t == RT_GGML_Q5_0 ||
           t == RT_GGML_Q5_1 || t == RT_GGML_Q2_K || t == RT_GGML_Q3_K || t == RT_GGML_Q4_K || t == RT_GGML_Q5_K || t == RT_GGML_Q6_K;
}

constexpr size_t kPrefillChunk = 512;     // tokens per pass of the batched prefill
constexpr int kPrefillMinRows = 3;        // fewer tokens go through the decode step; 3..15 run the contractions eight rows at a time

// The batched prefill serves every block format: Q4_K / Q6_K matrices go to the matrix cores, the others run the GEMV
// kernel with one grid slice per token (weights found in L2 / Infinity Cache after the first).
bool prefill_batchable(const rt_hip_llama *m) { return m->head_dim == 64 || m->head_dim == 128; }

int ensure_prefill_buffers(rt_hip_ctx *ctx, rt_hip_llama *m, size_t n_tok) {
    if (m->pf_cap >= n_tok) return RT_HIP_OK;
    const size_t H = (size_t)m->cfg.hidden, F = (size_t)m->cfg.ffn, cap = n_tok;
    int rc;
    float **hs[] = { &m->pf_x, &m->pf_x2, &m->pf_n, &m->pf_q, &m->pf_k, &m->pf_v, &m->pf_a };
    // a longer prompt than any before: the smaller set goes back first (prompts of rising length would otherwise pile up sets)
    for (float **p : hs) { dev_release(ctx, m, *p); *p = nullptr; }
    dev_release(ctx, m, m->pf_g); dev_release(ctx, m, m->pf_u); dev_release(ctx, m, m->pf_tok); dev_release(ctx, m, m->pf_xp); dev_release(ctx, m, m->pf_inv);
    m->pf_g = m->pf_u = nullptr; m->pf_tok = nullptr; m->pf_xp = nullptr; m->pf_inv = nullptr;
    for (float *&p : m->pf_planes) { dev_release(ctx, m, p); p = nullptr; }
    m->pf_cap = 0;
    for (float **p : hs)
        if ((rc = dev_alloc(ctx, m, (void **)p, cap * H * sizeof(float)))) return rc;
    if ((rc = dev_alloc(ctx, m, (void **)&m->pf_g, cap * F * sizeof(float)))) return rc;
    if ((rc = dev_alloc(ctx, m, (void **)&m->pf_u, cap * F * sizeof(float)))) return rc;
    if ((rc = dev_alloc(ctx, m, (void **)&m->pf_tok, cap * sizeof(int)))) return rc;
    // a k-split contraction writes at most 256 tiles of 128 x 256 results; without a split, one matrix of cap rows
    const size_t widest = std::max(std::max(H, F), m->kv_dim);
    m->pf_planes_bytes = std::max((size_t)256 * 128 * 256, cap * widest) * sizeof(float);
    for (float *&p : m->pf_planes)
        if ((rc = dev_alloc(ctx, m, (void **)&p, m->pf_planes_bytes))) return rc;
    if ((rc = dev_alloc(ctx, m, (void **)&m->pf_xp, cap * std::max(H, F) * sizeof(_Float16)))) return rc;
    if ((rc = dev_alloc(ctx, m, (void **)&m->pf_inv, (cap + 64) * sizeof(float)))) return rc;     // read four rows at a time, past the last
    m->pf_cap = cap;
    return RT_HIP_OK;
}

// The contractions of one prefill pass.  Consecutive weights that meet the same activation matrix on the matrix cores
// share its pre-pass, which stays in the workspace until another matrix is prepared.
struct PrefillGemm {
    rt_hip_ctx *ctx;
    rt_hip_llama *m;
    const float *prepared = nullptr;
    int operator()(rt_hip_llama::T &t, const float *X, size_t M, float *Y, const float *res) {
        if (rt::hgemm_serves(t.type, M, t.n_rows, t.n_cols)) {
            // 288 GB of HBM: the fp16 copy (2 bytes per weight) is made once and stays beside the blocks, so later
            // prompts skip the conversion
            if (t.type != RT_GGML_F16 && !t.f16) {
                void *p = nullptr;
                int rc = dev_alloc(ctx, m, &p, t.n_rows * t.n_cols * sizeof(_Float16));
                if (rc) return rc;
                RT_TRY_HIP(ctx, rt::launch_weights_f16(ctx->stream, t.type, t.dev, t.n_rows, t.n_cols, t.row_bytes, (_Float16 *)p));
                t.f16 = (_Float16 *)p;
            }
            RT_TRY_HIP(ctx, rt::launch_hgemm(ctx->stream, t.type, t.dev, t.n_rows, t.n_cols, t.row_bytes, X, M, Y, res, ctx->scratch,
                                             ctx->scratch_bytes, t.f16));
            prepared = nullptr;      // this contraction's own form of X now lies where the matrix-core pre-pass keeps its
            return RT_HIP_OK;
        }
        const bool mc = rt::qgemm_on_matrix_cores(t.type, M, t.n_rows, t.n_cols) && res != Y;
        RT_TRY_HIP(ctx, rt::launch_qgemm(ctx->stream, t.type, t.dev, t.n_rows, t.n_cols, t.row_bytes, X, M, Y, res, ctx->scratch, ctx->scratch_bytes,
                                         mc && prepared == X));
        prepared = mc ? X : nullptr;      // every other branch of launch_qgemm may use the workspace for something else
        return RT_HIP_OK;
    }
    // n matrices against the same rows of X (q, k, v; gate, up).  3..15 rows of Q4_K / Q6_K: the rows are quantized once
    // per eight and the matrices of one format share a launch; otherwise one contraction per matrix.
    int shared(rt_hip_llama::T *const *ts, float *const *Ys, int n, const float *X, size_t M) {
        const size_t K = ts[0]->n_cols;
        bool ok = n <= 4 && M >= (size_t)rt::kGemvMbMinBatch && M < 16 && (M <= 8 || M - 8 >= (size_t)rt::kGemvMbMinBatch) &&
                  ctx->scratch_bytes >= rt::qgemv_mb_scratch_bytes(K);
        for (int i = 0; i < n && ok; i++)
            ok = ts[i]->n_cols == K && rt::qgemv_mb_serves(ts[i]->type, ts[i]->n_rows, K, (int)std::min<size_t>(M, 8));
        if (!ok) {
            for (int i = 0; i < n; i++) {
                int rc = (*this)(*ts[i], X, M, Ys[i], nullptr);
                if (rc) return rc;
            }
            return RT_HIP_OK;
        }
        for (size_t m0 = 0; m0 < M; m0 += 8) {
            const int b = (int)std::min<size_t>(8, M - m0);
            RT_TRY_HIP(ctx, rt::launch_qgemv_mb_prep(ctx->stream, X + m0 * K, b, K, ctx->scratch));
            for (int type : { (int)RT_GGML_Q4_K, (int)RT_GGML_Q6_K }) {
                rt::MbProb probs[4];
                int k = 0;
                for (int i = 0; i < n; i++)
                    if (ts[i]->type == type) probs[k++] = rt::MbProb{ ts[i]->dev, ts[i]->row_bytes, ts[i]->n_rows, Ys[i] + m0 * ts[i]->n_rows, nullptr };
                if (k) RT_TRY_HIP(ctx, rt::launch_qgemv_mb_group(ctx->stream, type, probs, k, K, b, ctx->scratch));
            }
        }
        return RT_HIP_OK;
    }
};

// Every matrix of every layer goes to the matrix cores at this M, and the rows fit the fused pre-pass kernels.
bool prefill_chainable(const rt_hip_llama *m, size_t M) {
    const size_t H = (size_t)m->cfg.hidden, F = (size_t)m->cfg.ffn;
    if (H > rt::kXprepFusedMaxK || F > rt::kXprepFusedMaxK || H % 256 != 0 || F % 256 != 0) return false;
    for (int l = 0; l < m->cfg.n_layers; l++)
        for (const auto *t : { &m->wq[l], &m->wk[l], &m->wv[l], &m->wo[l], &m->wgate[l], &m->wup[l], &m->wdown[l] })
            if (!rt::qgemm_on_matrix_cores(t->type, M, t->n_rows, t->n_cols) ||
                rt::qgemm_planes_bytes(t->type, M, t->n_rows, t->n_cols) > m->pf_planes_bytes)
                return false;
    return true;
}

// The batched prefill as a chain without stand-alone reductions or pre-passes: a k-split contraction leaves its partial
// planes, and the kernel that consumes the result sums them on the way in; the operations that produce an activation
// matrix (RMSNorm of the residual stream, SwiGLU) write it directly in the contraction's prepared form.
// Per layer: [x += planes of the previous down-projection] RMSNorm -> q, k, v -> RoPE + cache append -> causal
// attention -> pre-pass -> o-projection -> [x += its planes] RMSNorm -> gate, up -> SwiGLU -> down-projection.
int enqueue_prefill_chain(rt_hip_ctx *ctx, rt_hip_llama *m, size_t M, int pos0) {
    hipStream_t s = ctx->stream;
    const rt_hip_llama_config &c = m->cfg;
    const size_t H = (size_t)c.hidden, F = (size_t)c.ffn;
    float *x = m->pf_x;                          // the residual stream, updated in place (a thread rewrites what it has read)
    float **P = m->pf_planes;
    auto mm = [&](const rt_hip_llama::T &t, float *planes, rt::PlaneSum *out) {
        return rt::launch_qgemm_planes(s, t.type, t.dev, t.n_rows, t.n_cols, t.row_bytes, m->pf_xp, m->pf_inv, M, planes, m->pf_planes_bytes, out);
    };
    // two matrices of one shape and format that meet the same prepared X (q and k without grouped-query attention, gate and up)
    // go out as one launch
    auto same_kind = [](const rt_hip_llama::T &a, const rt_hip_llama::T &b) {
        return a.type == b.type && a.n_rows == b.n_rows && a.n_cols == b.n_cols && a.row_bytes == b.row_bytes;
    };
    auto mm2 = [&](const rt_hip_llama::T &a, const rt_hip_llama::T &b, float *pa, float *pb, rt::PlaneSum *oa, rt::PlaneSum *ob) {
        return rt::launch_qgemm_planes2(s, a.type, a.dev, b.dev, a.n_rows, a.n_cols, a.row_bytes, m->pf_xp, m->pf_inv, M, pa, pb, m->pf_planes_bytes,
                                        oa, ob);
    };
    RT_TRY_HIP(ctx, rt::launch_embed_rows(s, m->tok_embd.type, m->tok_embd.dev, m->tok_embd.row_bytes, H, m->pf_tok, M, c.vocab, x));
    rt::PlaneSum pending{ x, 0, 1 };             // what the next RMSNorm reads: first the embeddings themselves,
    const float *pending_res = nullptr;          // later the planes of a down-projection, to be added to x
    for (int l = 0; l < c.n_layers; l++) {
        uint16_t *kc = m->pf_kcache + (size_t)l * m->pf_layer_stride;
        uint16_t *vc = m->pf_vcache + (size_t)l * m->pf_layer_stride;
        rt::PlaneSum q, k, v, o, g, u, d;
        RT_TRY_HIP(ctx, rt::launch_xprep_rmsnorm(s, pending, pending_res, pending_res ? x : nullptr, m->attn_norm[l], c.rms_eps, M, H, m->pf_xp, m->pf_inv));
        if (same_kind(m->wq[l], m->wk[l])) {
            RT_TRY_HIP(ctx, mm2(m->wq[l], m->wk[l], P[0], P[1], &q, &k));
        } else {
            RT_TRY_HIP(ctx, mm(m->wq[l], P[0], &q));
            RT_TRY_HIP(ctx, mm(m->wk[l], P[1], &k));
        }
        RT_TRY_HIP(ctx, mm(m->wv[l], P[2], &v));
        RT_TRY_HIP(ctx, rt::launch_rope_kv_planes(s, q, k, v, m->pf_q, kc, vc, pos0, M, c.n_heads, m->n_kv, m->head_dim, m->inv_freq));
        RT_TRY_HIP(ctx, rt::launch_attn_causal(s, m->pf_q, kc, vc, pos0, M, c.n_heads, m->n_kv, m->head_dim, m->pf_a));
        RT_TRY_HIP(ctx, rt::launch_xprep(s, m->pf_a, M, H, m->pf_xp, m->pf_inv));
        RT_TRY_HIP(ctx, mm(m->wo[l], P[0], &o));
        RT_TRY_HIP(ctx, rt::launch_xprep_rmsnorm(s, o, x, x, m->ffn_norm[l], c.rms_eps, M, H, m->pf_xp, m->pf_inv));      // x += o
        if (same_kind(m->wgate[l], m->wup[l])) {
            RT_TRY_HIP(ctx, mm2(m->wgate[l], m->wup[l], P[1], P[2], &g, &u));
        } else {
            RT_TRY_HIP(ctx, mm(m->wgate[l], P[1], &g));
            RT_TRY_HIP(ctx, mm(m->wup[l], P[2], &u));
        }
        RT_TRY_HIP(ctx, rt::launch_xprep_swiglu(s, g, u, M, F, m->pf_xp, m->pf_inv));
        RT_TRY_HIP(ctx, mm(m->wdown[l], P[0], &d));
        pending = d;                             // x += d happens in the next layer's RMSNorm launch
        pending_res = x;
    }
    // hidden state of the last token = its row of pending_res + pending
    const size_t last = (M - 1) * H;
    rt::PlaneSum row{ pending.base + last, pending.stride, pending.n };
    RT_TRY_HIP(ctx, rt::launch_plane_sum(s, row, pending_res ? pending_res + last : nullptr, m->x, H));
    return RT_HIP_OK;
}

// M tokens (already in pf_tok) at positions pos0 .. pos0+M-1 through all layers with the dense contraction:
// per layer rmsnorm rows -> q,k,v GEMMs -> rope + cache append -> causal attention (query m over pos0+m+1 rows)
// -> o-projection + residual -> rmsnorm -> gate, up GEMMs -> SwiGLU -> down-projection + residual.
// The hidden state of the last token ends in m->x.  Enqueue only.
int enqueue_prefill_batch(rt_hip_ctx *ctx, rt_hip_llama *m, size_t M, int pos0) {
    hipStream_t s = ctx->stream;
    const rt_hip_llama_config &c = m->cfg;
    const size_t H = (size_t)c.hidden, F = (size_t)c.ffn;
    size_t need = 0;      // formats may differ from layer to layer (the common 4-bit files alternate Q4_K and Q6_K for v and down)
    for (int l = 0; l < c.n_layers; l++)
        for (const auto *t : { &m->wq[l], &m->wk[l], &m->wv[l], &m->wo[l], &m->wgate[l], &m->wup[l], &m->wdown[l] })
            need = std::max(need, rt::qgemm_scratch_bytes(t->type, M, t->n_rows, t->n_cols));
    int rc = ensure_scratch(ctx, need);
    if (rc) return rc;
    float *x = m->pf_x, *x2 = m->pf_x2;
    PrefillGemm gemm{ ctx, m };
    RT_TRY_HIP(ctx, rt::launch_embed_rows(s, m->tok_embd.type, m->tok_embd.dev, m->tok_embd.row_bytes, H, m->pf_tok, M, c.vocab, x));
    for (int l = 0; l < c.n_layers; l++) {
        uint16_t *kc = m->pf_kcache + (size_t)l * m->pf_layer_stride;
        uint16_t *vc = m->pf_vcache + (size_t)l * m->pf_layer_stride;
        RT_TRY_HIP(ctx, rt::launch_rmsnorm(s, x, m->attn_norm[l], m->pf_n, nullptr, M, H, c.rms_eps));
        gemm.prepared = nullptr;          // pf_n has new contents
        rt_hip_llama::T *qkv[3] = { &m->wq[l], &m->wk[l], &m->wv[l] };
        float *qkv_y[3] = { m->pf_q, m->pf_k, m->pf_v };
        if ((rc = gemm.shared(qkv, qkv_y, 3, m->pf_n, M))) return rc;
        RT_TRY_HIP(ctx, rt::launch_rope_kv_batch(s, m->pf_q, m->pf_k, m->pf_v, kc, vc, pos0, M, c.n_heads, m->n_kv, m->head_dim, m->inv_freq));
        RT_TRY_HIP(ctx, rt::launch_attn_causal(s, m->pf_q, kc, vc, pos0, M, c.n_heads, m->n_kv, m->head_dim, m->pf_a));
        if ((rc = gemm(m->wo[l], m->pf_a, M, x2, x))) return rc;
        std::swap(x, x2);
        RT_TRY_HIP(ctx, rt::launch_rmsnorm(s, x, m->ffn_norm[l], m->pf_n, nullptr, M, H, c.rms_eps));
        gemm.prepared = nullptr;
        rt_hip_llama::T *gu[2] = { &m->wgate[l], &m->wup[l] };
        float *gu_y[2] = { m->pf_g, m->pf_u };
        if ((rc = gemm.shared(gu, gu_y, 2, m->pf_n, M))) return rc;
        RT_TRY_HIP(ctx, rt::launch_swiglu(s, m->pf_g, m->pf_u, m->pf_g, nullptr, M * F));
        gemm.prepared = nullptr;          // pf_g is rewritten in place
        if ((rc = gemm(m->wdown[l], m->pf_g, M, x2, x))) return rc;
        std::swap(x, x2);
    }
    RT_TRY_HIP(ctx, hipMemcpyAsync(m->x, x + (M - 1) * H, H * sizeof(float), hipMemcpyDeviceToDevice, s));
    return RT_HIP_OK;
}

// One token of each of b->n_seq sequences (tokens and positions already in b->tok / b->pos) through all layers.  The
// matrices see the sequences as rows of one activation matrix -- from three rows on, Q4_K / Q6_K weights are streamed once
// for all of them on the integer matrix cores (rt_gemv_mb.hip), q / k / v and gate / up sharing one quantization of the
// rows; RoPE, the cache append and the attention are per sequence.  Block order as in enqueue_step.  Enqueue only.
int enqueue_batch_step(rt_hip_ctx *ctx, rt_hip_llama_batch *b) {
    rt_hip_llama *m = b->m;
    hipStream_t s = ctx->stream;
    const rt_hip_llama_config &c = m->cfg;
    const size_t H = (size_t)c.hidden, F = (size_t)c.ffn, M = (size_t)b->n_seq;
    const size_t seq_stride = (size_t)b->max_pos * m->kv_dim;
    size_t need = rt::qgemv_mb_scratch_bytes(std::max(H, F));
    for (int l = 0; l < c.n_layers; l++)
        for (const auto *t : { &m->wq[l], &m->wk[l], &m->wv[l], &m->wo[l], &m->wgate[l], &m->wup[l], &m->wdown[l] })
            need = std::max(need, rt::qgemm_scratch_bytes(t->type, M, t->n_rows, t->n_cols));
    need = std::max(need, rt::qgemm_scratch_bytes(m->output.type, M, m->output.n_rows, m->output.n_cols));
    int rc = ensure_scratch(ctx, need);
    if (rc) return rc;
    float *x = b->x, *x2 = b->x2;
    PrefillGemm gemm{ ctx, m };
    RT_TRY_HIP(ctx, rt::launch_embed_rows(s, m->tok_embd.type, m->tok_embd.dev, m->tok_embd.row_bytes, H, b->tok, M, c.vocab, x));
    // Every matrix of a layer on the small-batch matrix-core GEMV (3..8 sequences, Q4_K / Q6_K): the kernel in front of
    // each contraction writes the GEMV's operand form itself -- RMSNorm for q / k / v and for gate / up, the attention (which
    // then also rotates and appends) for the o-projection, SwiGLU for the down-projection -- so no contraction needs a
    // quantizing launch of its own (five launches fewer per layer), and no f32 copy of those activations is written or read.
    auto mb = [&](const rt_hip_llama::T &t, size_t K) { return t.n_cols == K && rt::qgemv_mb_serves(t.type, t.n_rows, K, (int)M); };
    auto mb_group = [&](std::initializer_list<const rt_hip_llama::T *> ts, std::initializer_list<float *> ys, const float *res, size_t K) {
        for (int type : { (int)RT_GGML_Q4_K, (int)RT_GGML_Q6_K }) {
            rt::MbProb probs[4];
            int k = 0;
            auto y = ys.begin();
            for (const rt_hip_llama::T *t : ts) {
                if (t->type == type) probs[k++] = rt::MbProb{ t->dev, t->row_bytes, t->n_rows, *y, res };
                ++y;
            }
            if (k) RT_TRY_HIP(ctx, rt::launch_qgemv_mb_group(s, type, probs, k, K, (int)M, ctx->scratch));
        }
        return (int)RT_HIP_OK;
    };
    for (int l = 0; l < c.n_layers; l++) {
        uint16_t *kc = b->kcache + (size_t)l * M * seq_stride;
        uint16_t *vc = b->vcache + (size_t)l * M * seq_stride;
        const bool fused = M >= (size_t)rt::kGemvMbMinBatch && M <= 8 && ((uintptr_t)ctx->scratch & 255) == 0 &&
                           ctx->scratch_bytes >= rt::qgemv_mb_scratch_bytes(std::max(H, F)) && mb(m->wq[l], H) && mb(m->wk[l], H) &&
                           mb(m->wv[l], H) && mb(m->wo[l], H) && mb(m->wgate[l], H) && mb(m->wup[l], H) && mb(m->wdown[l], F);
        if (fused) {
            RT_TRY_HIP(ctx, rt::launch_rmsnorm_xq8(s, x, m->attn_norm[l], M, H, c.rms_eps, ctx->scratch));
            if ((rc = mb_group({ &m->wq[l], &m->wk[l], &m->wv[l] }, { b->q, b->k, b->v }, nullptr, H))) return rc;
            RT_TRY_HIP(ctx, rt::launch_attn_rows(s, b->q, kc, vc, b->pos, seq_stride, b->max_pos, M, c.n_heads, m->n_kv, m->head_dim, nullptr, ctx->scratch,
                                                 b->k, b->v, m->inv_freq));
            if ((rc = mb_group({ &m->wo[l] }, { x2 }, x, H))) return rc;
            std::swap(x, x2);
            RT_TRY_HIP(ctx, rt::launch_rmsnorm_xq8(s, x, m->ffn_norm[l], M, H, c.rms_eps, ctx->scratch));
            if ((rc = mb_group({ &m->wgate[l], &m->wup[l] }, { b->g, b->u }, nullptr, H))) return rc;
            RT_TRY_HIP(ctx, rt::launch_swiglu_xq8(s, b->g, b->u, M, F, ctx->scratch));
            if ((rc = mb_group({ &m->wdown[l] }, { x2 }, x, F))) return rc;
            std::swap(x, x2);
            continue;
        }
        RT_TRY_HIP(ctx, rt::launch_rmsnorm(s, x, m->attn_norm[l], b->n, nullptr, M, H, c.rms_eps));
        gemm.prepared = nullptr;
        rt_hip_llama::T *qkv[3] = { &m->wq[l], &m->wk[l], &m->wv[l] };
        float *qkv_y[3] = { b->q, b->k, b->v };
        if ((rc = gemm.shared(qkv, qkv_y, 3, b->n, M))) return rc;
        RT_TRY_HIP(ctx, rt::launch_rope_kv_rows(s, b->q, b->k, b->v, kc, vc, b->pos, seq_stride, M, c.n_heads, m->n_kv, m->head_dim, m->inv_freq));
        RT_TRY_HIP(ctx, rt::launch_attn_rows(s, b->q, kc, vc, b->pos, seq_stride, b->max_pos, M, c.n_heads, m->n_kv, m->head_dim, b->a, nullptr, nullptr, nullptr, nullptr));
        if ((rc = gemm(m->wo[l], b->a, M, x2, x))) return rc;
        std::swap(x, x2);
        RT_TRY_HIP(ctx, rt::launch_rmsnorm(s, x, m->ffn_norm[l], b->n, nullptr, M, H, c.rms_eps));
        gemm.prepared = nullptr;
        rt_hip_llama::T *gu[2] = { &m->wgate[l], &m->wup[l] };
        float *gu_y[2] = { b->g, b->u };
        if ((rc = gemm.shared(gu, gu_y, 2, b->n, M))) return rc;
        RT_TRY_HIP(ctx, rt::launch_swiglu(s, b->g, b->u, b->g, nullptr, M * F));
        gemm.prepared = nullptr;
        if ((rc = gemm(m->wdown[l], b->g, M, x2, x))) return rc;
        std::swap(x, x2);
    }
    if (M >= (size_t)rt::kGemvMbMinBatch && M <= 8 && ((uintptr_t)ctx->scratch & 255) == 0 && ctx->scratch_bytes >= rt::qgemv_mb_scratch_bytes(H) &&
        mb(m->output, H)) {
        RT_TRY_HIP(ctx, rt::launch_rmsnorm_xq8(s, x, m->out_norm, M, H, c.rms_eps, ctx->scratch));
        if ((rc = mb_group({ &m->output }, { b->logits }, nullptr, H))) return rc;
    } else {
        RT_TRY_HIP(ctx, rt::launch_rmsnorm(s, x, m->out_norm, b->n, nullptr, M, H, c.rms_eps));
        gemm.prepared = nullptr;
        if ((rc = gemm(m->output, b->n, M, b->logits, nullptr))) return rc;
    }
    RT_TRY_HIP(ctx, rt::launch_argmax_rows(s, b->logits, M, (size_t)c.vocab, b->pick));
    return RT_HIP_OK;
}

void free_batch(rt_hip_llama_batch *b) {
    for (void *p : b->allocs) (void)hipFree(p);
    b->allocs.clear();
}

}  // namespace

extern "C" {

int rt_hip_llama_create(rt_hip_ctx *ctx, const rt_hip_llama_config *cfg, rt_hip_llama **out) {
    if (!ctx || !cfg || !out) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_llama_create: NULL argument");
    *out = nullptr;
    RT_REQUIRE(ctx, cfg->n_layers > 0 && cfg->hidden > 0 && cfg->n_heads > 0 && cfg->ffn > 0 && cfg->vocab > 0 && cfg->max_pos > 0,
               RT_HIP_ERR_SHAPE, "llama config has a non-positive dimension");
    RT_REQUIRE(ctx, cfg->hidden % cfg->n_heads == 0, RT_HIP_ERR_SHAPE, "hidden=%d not divisible by n_heads=%d", cfg->hidden, cfg->n_heads);
    int hd = cfg->hidden / cfg->n_heads;
    RT_REQUIRE(ctx, hd == 64 || hd == 128, RT_HIP_ERR_SHAPE, "head_dim=%d (64 or 128 supported)", hd);
    const int n_kv = cfg->n_kv_heads == 0 ? cfg->n_heads : cfg->n_kv_heads;
    RT_REQUIRE(ctx, n_kv > 0 && cfg->n_heads % n_kv == 0, RT_HIP_ERR_SHAPE, "n_kv_heads=%d does not divide n_heads=%d", cfg->n_kv_heads, cfg->n_heads);
    RT_REQUIRE(ctx, cfg->hidden % 256 == 0 && cfg->ffn % 256 == 0, RT_HIP_ERR_SHAPE, "hidden=%d and ffn=%d must be multiples of 256", cfg->hidden, cfg->ffn);
    RT_REQUIRE(ctx, cfg->max_pos <= 16000, RT_HIP_ERR_SHAPE, "max_pos=%d exceeds 16000", cfg->max_pos);
    RT_REQUIRE(ctx, rt::xq_stride((size_t)cfg->ffn) <= rt::kGemvLdsMax && rt::xq_stride((size_t)cfg->hidden) <= rt::kGemvLdsMax, RT_HIP_ERR_SHAPE,
               "hidden / ffn exceed the GEMV staging limit");
    RT_REQUIRE(ctx, cfg->rms_eps >= 0.f && cfg->rope_theta > 0.f, RT_HIP_ERR_INVALID_ARG, "rms_eps=%g rope_theta=%g", (double)cfg->rms_eps,
               (double)cfg->rope_theta);
    Guard g(ctx);
    rt_hip_llama *m = new (std::nothrow) rt_hip_llama();
    if (!m) return fail(ctx, RT_HIP_ERR_OOM, "host allocation failed");
    m->cfg = *cfg;
    m->cfg.n_kv_heads = n_kv;
    m->head_dim = hd;
    m->n_kv = n_kv;
    m->kv_dim = (size_t)n_kv * (size_t)hd;
    size_t L = (size_t)cfg->n_layers, H = (size_t)cfg->hidden, F = (size_t)cfg->ffn, V = (size_t)cfg->vocab, P = (size_t)cfg->max_pos;
    m->wq.resize(L); m->wk.resize(L); m->wv.resize(L); m->wo.resize(L); m->wgate.resize(L); m->wup.resize(L); m->wdown.resize(L);
    m->attn_norm.assign(L, nullptr); m->ffn_norm.assign(L, nullptr);
    int rc = RT_HIP_OK;
    auto A = [&](void **p, size_t b) { if (rc == RT_HIP_OK) rc = dev_alloc(ctx, m, p, b); };
    // One workgroup per head serves a short cache; from RT_ATTN_SPLIT_MIN positions on, a head's positions are spread over
    // up to sixteen workgroups of 128 positions or more each (a fixed shape per model, so a captured step stays valid;
    // 64 positions per workgroup measured slower, 256 slower too).
    m->attn_splits = cfg->max_pos >= RT_ATTN_SPLIT_MIN ? std::min(16, (cfg->max_pos + RT_ATTN_SPLIT_MIN / 4 - 1) / (RT_ATTN_SPLIT_MIN / 4)) : 1;
    A((void **)&m->attn_part, (size_t)cfg->n_heads * (size_t)m->attn_splits * (size_t)(hd + 2) * sizeof(float));
    A((void **)&m->kcache, L * P * m->kv_dim * 2); A((void **)&m->vcache, L * P * m->kv_dim * 2);
    m->pf_kcache = m->kcache; m->pf_vcache = m->vcache; m->pf_layer_stride = P * m->kv_dim;
    A((void **)&m->x, H * 4); A((void **)&m->q, H * 4); A((void **)&m->k, H * 4); A((void **)&m->v, H * 4);
    A((void **)&m->g, F * 4); A((void **)&m->u, F * 4); A((void **)&m->logits, V * 4);
    A((void **)&m->xq_h, rt::xq_stride(H)); A((void **)&m->xq_a, rt::xq_stride(H)); A((void **)&m->xq_f, rt::xq_stride(F));
    A((void **)&m->inv_freq, (size_t)(hd / 2) * 4); A((void **)&m->state, 4 * sizeof(int));
    A((void **)&m->forced_dev, (P + 1) * sizeof(int)); A((void **)&m->out_tokens_dev, (P + 1) * sizeof(int));
    A((void **)&m->a, H * 4);
    if (rc != RT_HIP_OK) { free_all(m); delete m; return rc; }
    std::vector<float> inv((size_t)hd / 2);
    for (int i = 0; i < hd / 2; i++) inv[(size_t)i] = (float)std::pow((double)cfg->rope_theta, -2.0 * (double)i / (double)hd);
    hipError_t e = hipMemcpyAsync(m->inv_freq, inv.data(), inv.size() * 4, hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) e = hipMemsetAsync(m->state, 0, 4 * sizeof(int), ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) { free_all(m); delete m; return hip_fail(ctx, e, "llama_create init"); }
    *out = m;
    return RT_HIP_OK;
}

int rt_hip_llama_destroy(rt_hip_ctx *ctx, rt_hip_llama *m) {
    if (!m) return RT_HIP_OK;
    if (!ctx) return fail(nullptr, RT_HIP_ERR_INVALID_ARG, "ctx is NULL");
    Guard g(ctx);
    (void)hipStreamSynchronize(ctx->stream);
    free_all(m);
    delete m;
    return RT_HIP_OK;
}

int rt_hip_llama_upload_tensor(rt_hip_ctx *ctx, rt_hip_llama *m, int slot, int layer, int ggml_type, size_t n_rows,
                               size_t n_cols, const void *raw, size_t nbytes) {
    if (!ctx || !m || !raw) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_llama_upload_tensor: NULL argument");
    const rt_hip_llama_config &c = m->cfg;
    size_t H = (size_t)c.hidden, F = (size_t)c.ffn, V = (size_t)c.vocab;
    bool per_layer = slot >= RT_LLAMA_ATTN_Q;
    if (per_layer) RT_REQUIRE(ctx, layer >= 0 && layer < c.n_layers, RT_HIP_ERR_INVALID_ARG, "layer %d outside 0..%d", layer, c.n_layers - 1);
    bool is_norm = slot == RT_LLAMA_OUTPUT_NORM || slot == RT_LLAMA_ATTN_NORM || slot == RT_LLAMA_FFN_NORM;
    size_t er = 0, ec = 0;
    switch (slot) {
    case RT_LLAMA_TOK_EMBD: case RT_LLAMA_OUTPUT: er = V; ec = H; break;
    case RT_LLAMA_ATTN_Q: case RT_LLAMA_ATTN_OUT: er = H; ec = H; break;
    case RT_LLAMA_ATTN_K: case RT_LLAMA_ATTN_V: er = m->kv_dim; ec = H; break;
    case RT_LLAMA_FFN_GATE: case RT_LLAMA_FFN_UP: er = F; ec = H; break;
    case RT_LLAMA_FFN_DOWN: er = H; ec = F; break;
    case RT_LLAMA_OUTPUT_NORM: case RT_LLAMA_ATTN_NORM: case RT_LLAMA_FFN_NORM: er = 1; ec = H; break;
    default: return fail(ctx, RT_HIP_ERR_INVALID_ARG, "unknown tensor slot %d", slot);
    }
    if (is_norm) {
        RT_REQUIRE(ctx, ggml_type == RT_GGML_F32, RT_HIP_ERR_UNSUPPORTED_TYPE, "norm weights must be F32 (got type id %d)", ggml_type);
        RT_REQUIRE(ctx, n_rows * n_cols == H && nbytes == H * 4, RT_HIP_ERR_SHAPE, "norm weight has %zu x %zu elements / %zu bytes, expected %zu floats",
                   n_rows, n_cols, nbytes, H);
    } else {
        RT_REQUIRE(ctx, n_rows == er && n_cols == ec, RT_HIP_ERR_SHAPE, "slot %d expects %zu x %zu, got %zu x %zu", slot, er, ec, n_rows, n_cols);
        size_t be = rt::type_block_elems(ggml_type), bb = rt::type_block_bytes(ggml_type);
        RT_REQUIRE(ctx, be != 0, RT_HIP_ERR_UNSUPPORTED_TYPE, "unsupported GGML type id %d", ggml_type);
        if (slot != RT_LLAMA_TOK_EMBD) {
            RT_REQUIRE(ctx, gemv_type_ok(ggml_type), RT_HIP_ERR_UNSUPPORTED_TYPE, "GGML type id %d has no GEMV kernel", ggml_type);
            RT_REQUIRE(ctx, n_cols % 32 == 0 && rt::gemv_lds_bytes(ggml_type, n_cols) <= rt::kGemvLdsMax, RT_HIP_ERR_SHAPE,
                       "rows of %zu elements of type %d do not fit the GEMV's staging", n_cols, ggml_type);
        }
        RT_REQUIRE(ctx, n_cols % be == 0 && nbytes == n_rows * (n_cols / be) * bb, RT_HIP_ERR_SHAPE, "payload of %zu bytes does not match %zu x %zu of type %d",
                   nbytes, n_rows, n_cols, ggml_type);
    }
    Guard g(ctx);
    void *dev = nullptr;
    drop_step_graphs(m);      // a captured step names the old buffer of this slot
    int rc = dev_alloc(ctx, m, &dev, nbytes + 64);
    if (rc) return rc;
    RT_TRY_HIP(ctx, hipMemcpyAsync(dev, raw, nbytes, hipMemcpyHostToDevice, ctx->stream));
    RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));
    if (is_norm) {
        float *f = (float *)dev;
        float *&dst = slot == RT_LLAMA_OUTPUT_NORM ? m->out_norm : (slot == RT_LLAMA_ATTN_NORM ? m->attn_norm[(size_t)layer] : m->ffn_norm[(size_t)layer]);
        dev_release(ctx, m, dst);        // a slot uploaded again: the old vector goes back
        dst = f;
        return RT_HIP_OK;
    }
    rt_hip_llama::T t;
    t.type = ggml_type; t.n_rows = n_rows; t.n_cols = n_cols; t.nbytes = nbytes;
    t.row_bytes = n_cols / rt::type_block_elems(ggml_type) * rt::type_block_bytes(ggml_type);
    t.dev = (uint8_t *)dev;
    size_t l = (size_t)(layer < 0 ? 0 : layer);
    rt_hip_llama::T *dst = nullptr;
    switch (slot) {
    case RT_LLAMA_TOK_EMBD: dst = &m->tok_embd; break;
    case RT_LLAMA_OUTPUT: dst = &m->output; break;
    case RT_LLAMA_ATTN_Q: dst = &m->wq[l]; break;
    case RT_LLAMA_ATTN_K: dst = &m->wk[l]; break;
    case RT_LLAMA_ATTN_V: dst = &m->wv[l]; break;
    case RT_LLAMA_ATTN_OUT: dst = &m->wo[l]; break;
    case RT_LLAMA_FFN_GATE: dst = &m->wgate[l]; break;
    case RT_LLAMA_FFN_UP: dst = &m->wup[l]; break;
    case RT_LLAMA_FFN_DOWN: dst = &m->wdown[l]; break;
    }
    // a slot uploaded again: the old blocks and the fp16 copy the prefill may have made of them go back
    dev_release(ctx, m, dst->dev);
    dev_release(ctx, m, dst->f16);
    *dst = t;
    return RT_HIP_OK;
}

int rt_hip_llama_reset(rt_hip_ctx *ctx, rt_hip_llama *m) {
    if (!ctx || !m) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_llama_reset: NULL argument");
    Guard g(ctx);
    m->n_fed = 0;
    return RT_HIP_OK;
}

// Enqueue the step for the token in the device state.  advance: afterwards the state names the next token
// (forced_dev[step] when use_forced, else the pick) and the next position.
static int enqueue_token(rt_hip_ctx *ctx, rt_hip_llama *m, bool want_logits, bool advance, bool use_forced) {
    auto enqueue = [&]() -> int {
        int rc = enqueue_step(ctx, m, want_logits);
        if (rc) return rc;
        if (want_logits && advance)
            RT_TRY_HIP(ctx, rt::launch_argmax_advance(ctx->stream, m->logits, (size_t)m->cfg.vocab, m->state + 2, m->state + 0, m->state + 1,
                                                      use_forced ? m->forced_dev : nullptr, m->out_tokens_dev, m->state + 3));
        else if (want_logits)
            RT_TRY_HIP(ctx, rt::launch_argmax(ctx->stream, m->logits, (size_t)m->cfg.vocab, m->state + 2));
        else if (advance)
            RT_TRY_HIP(ctx, rt::launch_step_advance(ctx->stream, m->state + 0, m->state + 1, m->state + 2, use_forced ? m->forced_dev : nullptr,
                                                    m->out_tokens_dev, m->state + 3));
        return RT_HIP_OK;
    };
    if (m->mode != 2) return enqueue();
    rt_hip_llama::StepGraph &sg = m->step_graphs[(want_logits ? 1 : 0) | (advance ? 2 : 0) | (use_forced ? 4 : 0)];
    if (sg.exec) {
        RT_TRY_HIP(ctx, hipGraphLaunch(sg.exec, ctx->stream));
        return RT_HIP_OK;
    }
    if (sg.uses++ == 0) return enqueue();          // first use eagerly: whatever a launcher sets up lazily is set up outside a capture
    RT_TRY_HIP(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    int rc = enqueue();
    hipError_t e = hipStreamEndCapture(ctx->stream, &sg.graph);
    if (rc) {
        if (sg.graph) (void)hipGraphDestroy(sg.graph);
        sg.graph = nullptr;
        return rc;
    }
    RT_TRY_HIP(ctx, e);
    RT_TRY_HIP(ctx, hipGraphInstantiate(&sg.exec, sg.graph, nullptr, nullptr, 0));
    RT_TRY_HIP(ctx, hipGraphLaunch(sg.exec, ctx->stream));
    return RT_HIP_OK;
}

int rt_hip_llama_set_mode(rt_hip_ctx *ctx, rt_hip_llama *m, int mode) {
    if (!ctx || !m) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_llama_set_mode: NULL argument");
    RT_REQUIRE(ctx, mode >= 0 && mode <= 2, RT_HIP_ERR_INVALID_ARG,
               "mode %d (0 = persistent step kernel, 1 = separate launches, 2 = separate launches replayed from a graph)", mode);
    // The persistent step kernel took a GPU memory fault on its first run and the cause has not been found:
    // the path stays switched off until it is, and asking for it is an error rather than a silent fallback.
    RT_REQUIRE(ctx, mode != 0, RT_HIP_ERR_UNSUPPORTED_TYPE, "persistent step kernel is switched off in this build (unresolved GPU memory fault)");
    Guard g(ctx);
    m->mode = mode;
    if (mode != 2) drop_step_graphs(m);
    return RT_HIP_OK;
}

int rt_hip_llama_step(rt_hip_ctx *ctx, rt_hip_llama *m, int token, int pos, int *next_token) {
    if (!ctx || !m) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_llama_step: NULL argument");
    RT_REQUIRE(ctx, token >= 0 && token < m->cfg.vocab, RT_HIP_ERR_INVALID_ARG, "token %d outside the vocabulary of %d", token, m->cfg.vocab);
    RT_REQUIRE(ctx, pos == m->n_fed, RT_HIP_ERR_INVALID_ARG, "pos=%d but %d tokens have been fed", pos, m->n_fed);
    RT_REQUIRE(ctx, pos < m->cfg.max_pos, RT_HIP_ERR_SHAPE, "pos=%d reaches max_pos=%d", pos, m->cfg.max_pos);
    int rc = check_complete(ctx, m);
    if (rc) return rc;
    Guard g(ctx);
    RT_TRY_HIP(ctx, rt::launch_set_state(ctx->stream, m->state, pos, token, 0));
    rc = enqueue_token(ctx, m, true, false, false);
    if (rc) return rc;
    m->n_fed = pos + 1;
    if (next_token) {
        RT_TRY_HIP(ctx, hipMemcpyAsync(next_token, m->state + 2, sizeof(int), hipMemcpyDeviceToHost, ctx->stream));
        RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));
        return RT_HIP_OK;
    }
    return RT_HIP_OK;
}

int rt_hip_llama_prefill(rt_hip_ctx *ctx, rt_hip_llama *m, const int *tokens, int n_tok, int pos0) {
    if (!ctx || !m || !tokens) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_llama_prefill: NULL argument");
    RT_REQUIRE(ctx, n_tok > 0, RT_HIP_ERR_SHAPE, "prefill of %d tokens", n_tok);
    RT_REQUIRE(ctx, pos0 == m->n_fed, RT_HIP_ERR_INVALID_ARG, "pos0=%d but %d tokens have been fed", pos0, m->n_fed);
    RT_REQUIRE(ctx, pos0 + n_tok <= m->cfg.max_pos, RT_HIP_ERR_SHAPE, "pos0+n_tok=%d exceeds max_pos=%d", pos0 + n_tok, m->cfg.max_pos);
    for (int i = 0; i < n_tok; i++)
        RT_REQUIRE(ctx, tokens[i] >= 0 && tokens[i] < m->cfg.vocab, RT_HIP_ERR_INVALID_ARG, "token %d (index %d) outside the vocabulary", tokens[i], i);
    int rc = check_complete(ctx, m);
    if (rc) return rc;
    Guard g(ctx);
    if (n_tok >= kPrefillMinRows && prefill_batchable(m)) {
        // dense-contraction path, kPrefillChunk tokens per pass; the logits of the last token come from the head GEMV
        rc = ensure_prefill_buffers(ctx, m, std::min((size_t)n_tok, kPrefillChunk));
        if (rc) return rc;
        for (size_t t0 = 0; t0 < (size_t)n_tok; t0 += kPrefillChunk) {
            const size_t M = std::min(kPrefillChunk, (size_t)n_tok - t0);
            RT_TRY_HIP(ctx, hipMemcpyAsync(m->pf_tok, tokens + t0, M * sizeof(int), hipMemcpyHostToDevice, ctx->stream));
            if (M >= (size_t)kPrefillMinRows) {
                rc = prefill_chainable(m, M) ? enqueue_prefill_chain(ctx, m, M, pos0 + (int)t0) : enqueue_prefill_batch(ctx, m, M, pos0 + (int)t0);
                if (rc) return rc;
            } else {
                // a tail of one or two tokens goes token by token
                for (size_t i = 0; i < M; i++) {
                    RT_TRY_HIP(ctx, rt::launch_set_state(ctx->stream, m->state, pos0 + (int)(t0 + i), tokens[t0 + i], 0));
                    rc = enqueue_step(ctx, m, false);
                    if (rc) return rc;
                }
            }
            RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));       // `tokens` is the caller's buffer; pf_tok is reused by the next pass
        }
        // logits of the last token: rmsnorm + output head on its hidden state
        rt::GemvArgs a;
        memset(&a, 0, sizeof a);
        a.n = 1;
        a.p[0] = make_prob(m->output, m->x, rt::kStageRms, m->logits, nullptr);
        a.p[0].gamma = m->out_norm; a.p[0].eps = m->cfg.rms_eps;
        RT_TRY_HIP(ctx, rt::launch_qgemv(ctx->stream, a, 1));
        RT_TRY_HIP(ctx, rt::launch_argmax(ctx->stream, m->logits, (size_t)m->cfg.vocab, m->state + 2));
        RT_TRY_HIP(ctx, rt::launch_set_state(ctx->stream, m->state, pos0 + n_tok, tokens[n_tok - 1], 0));
        m->n_fed = pos0 + n_tok;
        return RT_HIP_OK;
    }
    // forced_dev[i] = token fed after step i (the last entry repeats the last token and is never used)
    std::vector<int> next((size_t)n_tok);
    for (int i = 0; i < n_tok; i++) next[(size_t)i] = tokens[i + 1 < n_tok ? i + 1 : i];
    RT_TRY_HIP(ctx, hipMemcpyAsync(m->forced_dev, next.data(), next.size() * sizeof(int), hipMemcpyHostToDevice, ctx->stream));
    RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));  // `next` is a stack-lifetime staging buffer
    RT_TRY_HIP(ctx, rt::launch_set_state(ctx->stream, m->state, pos0, tokens[0], 0));
    for (int i = 0; i < n_tok; i++) {
        rc = enqueue_token(ctx, m, i == n_tok - 1, true, true);
        if (rc) return rc;
    }
    m->n_fed = pos0 + n_tok;
    return RT_HIP_OK;
}

int rt_hip_llama_logits(rt_hip_ctx *ctx, rt_hip_llama *m, float *logits_host) {
    if (!ctx || !m || !logits_host) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_llama_logits: NULL argument");
    Guard g(ctx);
    RT_TRY_HIP(ctx, hipMemcpyAsync(logits_host, m->logits, (size_t)m->cfg.vocab * 4, hipMemcpyDeviceToHost, ctx->stream));
    RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return RT_HIP_OK;
}

int rt_hip_llama_decode(rt_hip_ctx *ctx, rt_hip_llama *m, int first_token, int pos0, int n_steps, const int *forced,
                        int *out_tokens) {
    if (!ctx || !m || !out_tokens) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_llama_decode: NULL argument");
    RT_REQUIRE(ctx, n_steps > 0, RT_HIP_ERR_SHAPE, "decode of %d steps", n_steps);
    RT_REQUIRE(ctx, first_token >= 0 && first_token < m->cfg.vocab, RT_HIP_ERR_INVALID_ARG, "token %d outside the vocabulary", first_token);
    RT_REQUIRE(ctx, pos0 == m->n_fed, RT_HIP_ERR_INVALID_ARG, "pos0=%d but %d tokens have been fed", pos0, m->n_fed);
    RT_REQUIRE(ctx, pos0 + n_steps <= m->cfg.max_pos, RT_HIP_ERR_SHAPE, "pos0+n_steps=%d exceeds max_pos=%d", pos0 + n_steps, m->cfg.max_pos);
    if (forced)
        for (int i = 0; i < n_steps; i++)
            RT_REQUIRE(ctx, forced[i] >= 0 && forced[i] < m->cfg.vocab, RT_HIP_ERR_INVALID_ARG, "forced token %d (index %d) outside the vocabulary", forced[i], i);
    int rc = check_complete(ctx, m);
    if (rc) return rc;
    Guard g(ctx);
    if (forced) {
        RT_TRY_HIP(ctx, hipMemcpyAsync(m->forced_dev, forced, (size_t)n_steps * sizeof(int), hipMemcpyHostToDevice, ctx->stream));
        RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));
    }
    RT_TRY_HIP(ctx, rt::launch_set_state(ctx->stream, m->state, pos0, first_token, 0));
    for (int i = 0; i < n_steps; i++) {
        rc = enqueue_token(ctx, m, true, true, forced != nullptr);
        if (rc) return rc;
    }
    m->n_fed = pos0 + n_steps;
    RT_TRY_HIP(ctx, hipMemcpyAsync(out_tokens, m->out_tokens_dev, (size_t)n_steps * sizeof(int), hipMemcpyDeviceToHost, ctx->stream));
    RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return RT_HIP_OK;
}

int rt_hip_llama_batch_create(rt_hip_ctx *ctx, rt_hip_llama *m, int n_seq, int max_pos, rt_hip_llama_batch **out) {
    if (!ctx || !m || !out) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_llama_batch_create: NULL argument");
    *out = nullptr;
    RT_REQUIRE(ctx, n_seq >= 1 && n_seq <= 8, RT_HIP_ERR_SHAPE, "a batch holds 1..8 sequences, got %d", n_seq);
    RT_REQUIRE(ctx, max_pos >= 1 && max_pos <= 8192, RT_HIP_ERR_SHAPE, "max_pos=%d outside 1..8192", max_pos);
    RT_REQUIRE(ctx, prefill_batchable(m), RT_HIP_ERR_SHAPE, "head_dim=%d (64 or 128 supported)", m->head_dim);
    Guard g(ctx);
    rt_hip_llama_batch *b = new (std::nothrow) rt_hip_llama_batch();
    if (!b) return fail(ctx, RT_HIP_ERR_OOM, "host allocation failed");
    b->m = m; b->n_seq = n_seq; b->max_pos = max_pos;
    b->fed.assign((size_t)n_seq, 0);
    const rt_hip_llama_config &c = m->cfg;
    const size_t L = (size_t)c.n_layers, H = (size_t)c.hidden, F = (size_t)c.ffn, V = (size_t)c.vocab, M = (size_t)n_seq, P = (size_t)max_pos;
    hipError_t e = hipSuccess;
    auto A = [&](void **p, size_t bytes) {
        if (e != hipSuccess) return;
        e = hipMalloc(p, bytes ? bytes : 1);
        if (e == hipSuccess) b->allocs.push_back(*p);
    };
    A((void **)&b->kcache, L * M * P * m->kv_dim * 2); A((void **)&b->vcache, L * M * P * m->kv_dim * 2);
    A((void **)&b->x, M * H * 4); A((void **)&b->x2, M * H * 4); A((void **)&b->n, M * H * 4); A((void **)&b->q, M * H * 4);
    A((void **)&b->k, M * m->kv_dim * 4); A((void **)&b->v, M * m->kv_dim * 4); A((void **)&b->a, M * H * 4);
    A((void **)&b->g, M * F * 4); A((void **)&b->u, M * F * 4); A((void **)&b->logits, M * V * 4);
    A((void **)&b->tok, M * sizeof(int)); A((void **)&b->pos, M * sizeof(int)); A((void **)&b->pick, M * sizeof(int));
    if (e != hipSuccess) { free_batch(b); delete b; return hip_fail(ctx, e, "llama_batch_create"); }
    *out = b;
    return RT_HIP_OK;
}

int rt_hip_llama_batch_destroy(rt_hip_ctx *ctx, rt_hip_llama_batch *b) {
    if (!b) return RT_HIP_OK;
    if (!ctx) return fail(nullptr, RT_HIP_ERR_INVALID_ARG, "ctx is NULL");
    Guard g(ctx);
    (void)hipStreamSynchronize(ctx->stream);
    free_batch(b);
    delete b;
    return RT_HIP_OK;
}

int rt_hip_llama_batch_reset(rt_hip_ctx *ctx, rt_hip_llama_batch *b, int seq) {
    if (!ctx || !b) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_llama_batch_reset: NULL argument");
    RT_REQUIRE(ctx, seq >= -1 && seq < b->n_seq, RT_HIP_ERR_INVALID_ARG, "sequence %d of %d", seq, b->n_seq);
    Guard g(ctx);
    RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));
    if (seq < 0) b->fed.assign((size_t)b->n_seq, 0);
    else b->fed[(size_t)seq] = 0;
    return RT_HIP_OK;
}

int rt_hip_llama_batch_step(rt_hip_ctx *ctx, rt_hip_llama_batch *b, const int *tokens, const int *positions, int *next_tokens) {
    if (!ctx || !b || !tokens || !positions) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_llama_batch_step: NULL argument");
    rt_hip_llama *m = b->m;
    int tok[8], pos[8], active = 0;
    for (int i = 0; i < b->n_seq; i++) {
        const int fed = b->fed[(size_t)i];
        if (tokens[i] < 0) {
            // idle this step: the row still runs (token 0 at the row the sequence would write next, which its next real token
            // overwrites); nothing is counted and its pick is reported as -1
            tok[i] = 0;
            pos[i] = std::min(fed, b->max_pos - 1);
            continue;
        }
        RT_REQUIRE(ctx, tokens[i] < m->cfg.vocab, RT_HIP_ERR_INVALID_ARG, "sequence %d: token %d outside the vocabulary of %d", i, tokens[i], m->cfg.vocab);
        RT_REQUIRE(ctx, positions[i] == fed, RT_HIP_ERR_INVALID_ARG, "sequence %d: pos=%d but %d tokens have been fed", i, positions[i], fed);
        RT_REQUIRE(ctx, positions[i] < b->max_pos, RT_HIP_ERR_SHAPE, "sequence %d: pos=%d reaches max_pos=%d", i, positions[i], b->max_pos);
        tok[i] = tokens[i];
        pos[i] = positions[i];
        active++;
    }
    RT_REQUIRE(ctx, active > 0, RT_HIP_ERR_INVALID_ARG, "batch step: every sequence is idle");
    int rc = check_complete(ctx, m);
    if (rc) return rc;
    Guard g(ctx);
    const size_t bytes = (size_t)b->n_seq * sizeof(int);
    // (pageable host memory: the copies have left tok / pos when the calls return)
    RT_TRY_HIP(ctx, hipMemcpyAsync(b->tok, tok, bytes, hipMemcpyHostToDevice, ctx->stream));
    RT_TRY_HIP(ctx, hipMemcpyAsync(b->pos, pos, bytes, hipMemcpyHostToDevice, ctx->stream));
    rc = enqueue_batch_step(ctx, b);
    if (rc) return rc;
    for (int i = 0; i < b->n_seq; i++)
        if (tokens[i] >= 0) b->fed[(size_t)i]++;
    if (next_tokens) {
        RT_TRY_HIP(ctx, hipMemcpyAsync(next_tokens, b->pick, bytes, hipMemcpyDeviceToHost, ctx->stream));
        RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));
        for (int i = 0; i < b->n_seq; i++)
            if (tokens[i] < 0) next_tokens[i] = -1;
    }
    return RT_HIP_OK;
}

int rt_hip_llama_batch_prefill(rt_hip_ctx *ctx, rt_hip_llama_batch *b, int seq, const int *tokens, int n_tok, int pos0) {
    if (!ctx || !b || !tokens) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_llama_batch_prefill: NULL argument");
    rt_hip_llama *m = b->m;
    RT_REQUIRE(ctx, seq >= 0 && seq < b->n_seq, RT_HIP_ERR_INVALID_ARG, "sequence %d of %d", seq, b->n_seq);
    RT_REQUIRE(ctx, n_tok >= kPrefillMinRows, RT_HIP_ERR_SHAPE, "batch prefill takes %d tokens or more (fewer go through rt_hip_llama_batch_step), got %d",
               kPrefillMinRows, n_tok);
    RT_REQUIRE(ctx, pos0 == b->fed[(size_t)seq], RT_HIP_ERR_INVALID_ARG, "sequence %d: pos0=%d but %d tokens have been fed", seq, pos0, b->fed[(size_t)seq]);
    RT_REQUIRE(ctx, pos0 + n_tok <= b->max_pos, RT_HIP_ERR_SHAPE, "pos0+n_tok=%d exceeds max_pos=%d", pos0 + n_tok, b->max_pos);
    for (int i = 0; i < n_tok; i++)
        RT_REQUIRE(ctx, tokens[i] >= 0 && tokens[i] < m->cfg.vocab, RT_HIP_ERR_INVALID_ARG, "token %d (index %d) outside the vocabulary", tokens[i], i);
    int rc = check_complete(ctx, m);
    if (rc) return rc;
    Guard g(ctx);
    rc = ensure_prefill_buffers(ctx, m, std::min((size_t)n_tok, kPrefillChunk));
    if (rc) return rc;
    // the model's own passes, writing and attending this sequence's cache for the length of the call
    const size_t seq_stride = (size_t)b->max_pos * m->kv_dim;
    m->pf_kcache = b->kcache + (size_t)seq * seq_stride;
    m->pf_vcache = b->vcache + (size_t)seq * seq_stride;
    m->pf_layer_stride = (size_t)b->n_seq * seq_stride;
    struct Restore {
        rt_hip_llama *m;
        ~Restore() { m->pf_kcache = m->kcache; m->pf_vcache = m->vcache; m->pf_layer_stride = (size_t)m->cfg.max_pos * m->kv_dim; }
    } restore{ m };
    for (size_t t0 = 0; t0 < (size_t)n_tok;) {
        size_t M = std::min(kPrefillChunk, (size_t)n_tok - t0);
        const size_t left = (size_t)n_tok - t0 - M;
        if (left > 0 && left < (size_t)kPrefillMinRows) M -= (size_t)kPrefillMinRows;      // no pass of one or two tokens: the last two share
        RT_TRY_HIP(ctx, hipMemcpyAsync(m->pf_tok, tokens + t0, M * sizeof(int), hipMemcpyHostToDevice, ctx->stream));
        rc = prefill_chainable(m, M) ? enqueue_prefill_chain(ctx, m, M, pos0 + (int)t0) : enqueue_prefill_batch(ctx, m, M, pos0 + (int)t0);
        if (rc) return rc;
        RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));       // `tokens` is the caller's buffer; pf_tok is reused by the next pass
        t0 += M;
    }
    // logits of the last token into this sequence's row, and its greedy pick
    float *row = b->logits + (size_t)seq * (size_t)m->cfg.vocab;
    rt::GemvArgs a;
    memset(&a, 0, sizeof a);
    a.n = 1;
    a.p[0] = make_prob(m->output, m->x, rt::kStageRms, row, nullptr);
    a.p[0].gamma = m->out_norm; a.p[0].eps = m->cfg.rms_eps;
    RT_TRY_HIP(ctx, rt::launch_qgemv(ctx->stream, a, 1));
    RT_TRY_HIP(ctx, rt::launch_argmax(ctx->stream, row, (size_t)m->cfg.vocab, b->pick + seq));
    RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));
    b->fed[(size_t)seq] = pos0 + n_tok;
    return RT_HIP_OK;
}

int rt_hip_llama_batch_logits(rt_hip_ctx *ctx, rt_hip_llama_batch *b, float *logits_host) {
    if (!ctx || !b || !logits_host) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_llama_batch_logits: NULL argument");
    Guard g(ctx);
    RT_TRY_HIP(ctx, hipMemcpyAsync(logits_host, b->logits, (size_t)b->n_seq * (size_t)b->m->cfg.vocab * sizeof(float), hipMemcpyDeviceToHost,
                                   ctx->stream));
    RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return RT_HIP_OK;
}

}  // extern "C"
