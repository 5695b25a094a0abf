// Prefill contraction Y[M,N] = X[M,K] . dequant(W)^T.
#include "rt_internal.h"

#include <cstring>

namespace rt {

size_t qgemm_scratch_bytes(size_t M, size_t K) { return M * xq_stride(K); }

// Row-by-row form: quantize every row of X, then run the GEMV kernel with one grid slice per row.
hipError_t launch_qgemm(hipStream_t s, int type, const uint8_t *w, size_t N, size_t K, size_t row_bytes,
                        const float *X, size_t M, float *Y, const float *res, void *scratch, size_t scratch_bytes) {
    if (scratch_bytes < qgemm_scratch_bytes(M, K)) return hipErrorInvalidValue;
    uint8_t *xq = (uint8_t *)scratch;
    hipError_t e = launch_quantize_x(s, X, xq, K, M);
    if (e != hipSuccess) return e;
    GemvArgs a;
    memset(&a, 0, sizeof a);
    a.n = 1;
    a.p[0].w = w; a.p[0].xq = xq; a.p[0].y = Y; a.p[0].res = res; a.p[0].row_bytes = row_bytes;
    a.p[0].type = type; a.p[0].N = (int)N; a.p[0].K = (int)K;
    return launch_qgemv(s, a, (int)M);
}

}  // namespace rt
