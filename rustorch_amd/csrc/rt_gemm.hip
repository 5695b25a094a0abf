// Prefill contraction Y[M,N] = X[M,K] . dequant(W)^T.
#include "rt_internal.h"

#include <cstring>

namespace rt {

size_t qgemm_scratch_bytes(size_t M, size_t K) { (void)M; (void)K; return 0; }

// Row-by-row form: the GEMV kernel with one grid slice per row of X.
hipError_t launch_qgemm(hipStream_t s, int type, const uint8_t *w, size_t N, size_t K, size_t row_bytes,
                        const float *X, size_t M, float *Y, const float *res, void *scratch, size_t scratch_bytes) {
    (void)scratch; (void)scratch_bytes;
    GemvArgs a;
    memset(&a, 0, sizeof a);
    a.n = 1;
    a.p[0].w = w; a.p[0].x = X; a.p[0].stage = kStageF32; a.p[0].y = Y; a.p[0].res = res; a.p[0].row_bytes = row_bytes;
    a.p[0].type = type; a.p[0].N = (int)N; a.p[0].K = (int)K;
    return launch_qgemv(s, a, (int)M);
}

}  // namespace rt
