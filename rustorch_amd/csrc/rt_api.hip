// extern "C" surface of librustorch_hip: contexts, resident buffers, quantized
// weights, GEMV / GEMM entry points and the decode-step operators.  Every entry
// point validates shapes on the host before a kernel is launched, returns a
// status code and leaves the failure text in the context.
#include "rt_internal.h"

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <new>
#include <vector>

namespace rt {

thread_local std::string g_tls_err;

int fail(rt_hip_ctx *ctx, int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    if (ctx) ctx->err = buf;
    g_tls_err = buf;
    return code;
}

int hip_fail(rt_hip_ctx *ctx, hipError_t e, const char *what) {
    int code = (e == hipErrorOutOfMemory) ? RT_HIP_ERR_OOM : RT_HIP_ERR_HIP;
    (void)hipGetLastError();
    return fail(ctx, code, "%s: %s", what, hipGetErrorString(e));
}

// Code-path switches: one atomic per option, -1 until the environment has been consulted.
namespace {
constexpr int kOptions = 3;      // option ids 1 .. kOptions - 1
std::atomic<int> g_option[kOptions] = { { 0 }, { -1 }, { -1 } };
const char *option_env(int option) {
    switch (option) {
    case RT_HIP_OPT_GEMV_LEAN: return "RUSTORCH_HIP_GEMV_LEAN";
    case RT_HIP_OPT_DENSE_MFMA: return "RUSTORCH_HIP_DENSE_MFMA";
    default: return nullptr;
    }
}
}  // namespace
static int option_max(int option) { return option == RT_HIP_OPT_GEMV_LEAN ? 2 : 1; }
int path_option(int option) {
    const char *env = option_env(option);
    if (!env) return -1;
    int v = g_option[option].load(std::memory_order_relaxed);
    if (v < 0) {
        const char *e = getenv(env);      // one digit within the option's range, anything else counts as 0
        v = (e && e[0] >= '0' && e[0] <= '0' + option_max(option) && e[1] == 0) ? e[0] - '0' : 0;
        int expected = -1;
        if (!g_option[option].compare_exchange_strong(expected, v, std::memory_order_relaxed)) v = expected;      // a set_option got there first
    }
    return v;
}
bool set_path_option(int option, int value) {
    if (!option_env(option) || value < 0 || value > option_max(option)) return false;
    g_option[option].store(value, std::memory_order_relaxed);
    return true;
}

// Grow the context scratch to at least `bytes` (contents are not preserved).
int ensure_scratch(rt_hip_ctx *ctx, size_t bytes) {
    if (ctx->scratch_bytes >= bytes) return RT_HIP_OK;
    if (ctx->scratch) {
        RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));
        RT_TRY_HIP(ctx, hipFree(ctx->scratch));
        ctx->scratch = nullptr;
        ctx->scratch_bytes = 0;
    }
    size_t want = (bytes + ((size_t)1 << 20) - 1) & ~(((size_t)1 << 20) - 1);
    RT_TRY_HIP(ctx, hipMalloc(&ctx->scratch, want));
    ctx->scratch_bytes = want;
    return RT_HIP_OK;
}

}  // namespace rt

using rt::fail;
using rt::hip_fail;
using rt::ensure_scratch;
using rt::Guard;

namespace {

bool gemv_type_ok(int t) {
    return t == RT_GGML_F32 || t == RT_GGML_F16 || t == RT_GGML_Q8_0 || t == RT_GGML_Q8_1 || t == RT_GGML_Q4_0 || t == RT_GGML_Q4_1 || t == RT_GGML_Q5_0 ||
           t == RT_GGML_Q5_1 || t == RT_GGML_Q2_K || t == RT_GGML_Q3_K || t == RT_GGML_Q4_K || t == RT_GGML_Q5_K || t == RT_GGML_Q6_K;
}

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace

extern "C" {

int rt_hip_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

int rt_hip_device_info(int device, rt_hip_devinfo *out) {
    if (!out) return fail(nullptr, RT_HIP_ERR_INVALID_ARG, "rt_hip_device_info: out is NULL");
    int n = rt_hip_device_count();
    if (device < 0 || device >= n) return fail(nullptr, RT_HIP_ERR_NO_DEVICE, "hip:%d not available (%d devices)", device, n);
    hipDeviceProp_t p;
    hipError_t e = hipGetDeviceProperties(&p, device);
    if (e != hipSuccess) return hip_fail(nullptr, e, "hipGetDeviceProperties");
    memset(out, 0, sizeof *out);
    snprintf(out->name, sizeof out->name, "%s", p.name);
    snprintf(out->arch, sizeof out->arch, "%s", p.gcnArchName);
    out->compute_units = p.multiProcessorCount;
    out->wavefront_size = p.warpSize;
    out->hbm_bytes = p.totalGlobalMem;
    out->lds_bytes_per_block = p.sharedMemPerBlock;
    return RT_HIP_OK;
}

int rt_hip_create(int device, rt_hip_ctx **out) {
    if (!out) return fail(nullptr, RT_HIP_ERR_INVALID_ARG, "rt_hip_create: out is NULL");
    *out = nullptr;
    int n = rt_hip_device_count();
    if (device < 0 || device >= n) return fail(nullptr, RT_HIP_ERR_NO_DEVICE, "hip:%d not available (%d devices)", device, n);
    hipError_t e = hipSetDevice(device);
    if (e != hipSuccess) return hip_fail(nullptr, e, "hipSetDevice");
    rt_hip_ctx *c = new (std::nothrow) rt_hip_ctx();
    if (!c) return fail(nullptr, RT_HIP_ERR_OOM, "rt_hip_create: host allocation failed");
    c->device = device;
    e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
        delete c;
        return hip_fail(nullptr, e, "hipStreamCreate");
    }
    *out = c;
    return RT_HIP_OK;
}

int rt_hip_destroy(rt_hip_ctx *ctx) {
    if (!ctx) return RT_HIP_OK;
    {
        Guard g(ctx);
        (void)hipStreamSynchronize(ctx->stream);
        if (ctx->scratch) (void)hipFree(ctx->scratch);
        (void)hipStreamDestroy(ctx->stream);
    }
    delete ctx;
    return RT_HIP_OK;
}

int rt_hip_synchronize(rt_hip_ctx *ctx) {
    if (!ctx) return fail(nullptr, RT_HIP_ERR_INVALID_ARG, "ctx is NULL");
    Guard g(ctx);
    RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return RT_HIP_OK;
}

const char *rt_hip_last_error(rt_hip_ctx *ctx) { return ctx ? ctx->err.c_str() : rt::g_tls_err.c_str(); }

size_t rt_hip_type_block_bytes(int t) { return rt::type_block_bytes(t); }
size_t rt_hip_type_block_elems(int t) { return rt::type_block_elems(t); }

// ------------------------------------------------------------------ buffers

int rt_hip_malloc(rt_hip_ctx *ctx, size_t nbytes, void **out_dev) {
    if (!ctx || !out_dev) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_malloc: NULL argument");
    Guard g(ctx);
    *out_dev = nullptr;
    RT_TRY_HIP(ctx, hipMalloc(out_dev, nbytes ? nbytes : 1));
    return RT_HIP_OK;
}

int rt_hip_free(rt_hip_ctx *ctx, void *dev) {
    if (!ctx) return fail(nullptr, RT_HIP_ERR_INVALID_ARG, "ctx is NULL");
    if (!dev) return RT_HIP_OK;
    Guard g(ctx);
    RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));
    RT_TRY_HIP(ctx, hipFree(dev));
    return RT_HIP_OK;
}

int rt_hip_memcpy_h2d(rt_hip_ctx *ctx, void *dst_dev, const void *src_host, size_t nbytes) {
    if (!ctx || (nbytes && (!dst_dev || !src_host))) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_memcpy_h2d: NULL argument");
    Guard g(ctx);
    if (!nbytes) return RT_HIP_OK;
    RT_TRY_HIP(ctx, hipMemcpyAsync(dst_dev, src_host, nbytes, hipMemcpyHostToDevice, ctx->stream));
    RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return RT_HIP_OK;
}

int rt_hip_memcpy_d2h(rt_hip_ctx *ctx, void *dst_host, const void *src_dev, size_t nbytes) {
    if (!ctx || (nbytes && (!dst_host || !src_dev))) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_memcpy_d2h: NULL argument");
    Guard g(ctx);
    if (!nbytes) return RT_HIP_OK;
    RT_TRY_HIP(ctx, hipMemcpyAsync(dst_host, src_dev, nbytes, hipMemcpyDeviceToHost, ctx->stream));
    RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return RT_HIP_OK;
}

int rt_hip_memset_dev(rt_hip_ctx *ctx, void *dst_dev, int byte, size_t nbytes) {
    if (!ctx || (nbytes && !dst_dev)) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_memset_dev: NULL argument");
    Guard g(ctx);
    if (!nbytes) return RT_HIP_OK;
    RT_TRY_HIP(ctx, hipMemsetAsync(dst_dev, byte, nbytes, ctx->stream));
    return RT_HIP_OK;
}

// ------------------------------------------------------------------- events

int rt_hip_event_create(rt_hip_ctx *ctx, rt_hip_event **out) {
    if (!ctx || !out) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_event_create: NULL argument");
    Guard g(ctx);
    rt_hip_event *e = new (std::nothrow) rt_hip_event();
    if (!e) return fail(ctx, RT_HIP_ERR_OOM, "host allocation failed");
    hipError_t r = hipEventCreate(&e->ev);
    if (r != hipSuccess) {
        delete e;
        return hip_fail(ctx, r, "hipEventCreate");
    }
    *out = e;
    return RT_HIP_OK;
}

int rt_hip_event_record(rt_hip_ctx *ctx, rt_hip_event *ev) {
    if (!ctx || !ev) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_event_record: NULL argument");
    Guard g(ctx);
    RT_TRY_HIP(ctx, hipEventRecord(ev->ev, ctx->stream));
    return RT_HIP_OK;
}

int rt_hip_event_elapsed_ms(rt_hip_ctx *ctx, rt_hip_event *start, rt_hip_event *stop, float *ms) {
    if (!ctx || !start || !stop || !ms) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_event_elapsed_ms: NULL argument");
    Guard g(ctx);
    RT_TRY_HIP(ctx, hipEventSynchronize(stop->ev));
    RT_TRY_HIP(ctx, hipEventElapsedTime(ms, start->ev, stop->ev));
    return RT_HIP_OK;
}

int rt_hip_event_destroy(rt_hip_ctx *ctx, rt_hip_event *ev) {
    if (!ev) return RT_HIP_OK;
    if (ctx) {
        Guard g(ctx);
        (void)hipEventDestroy(ev->ev);
    } else {
        (void)hipEventDestroy(ev->ev);
    }
    delete ev;
    return RT_HIP_OK;
}

// ------------------------------------------------------------- dense matmul

int rt_hip_matmul_f32(rt_hip_ctx *ctx, const float *a, const float *b, float *c, size_t m, size_t n, size_t k) {
    if (!ctx) return fail(nullptr, RT_HIP_ERR_INVALID_ARG, "ctx is NULL");
    RT_REQUIRE(ctx, a && b && c, RT_HIP_ERR_INVALID_ARG, "matmul_f32: NULL operand");
    RT_REQUIRE(ctx, m > 0 && n > 0 && k > 0, RT_HIP_ERR_SHAPE, "matmul_f32: empty dimension (m=%zu n=%zu k=%zu)", m, n, k);
    Guard g(ctx);
    size_t ab = align_up(m * k * 4, 256), bb = align_up(k * n * 4, 256), cb = m * n * 4;
    int rc = ensure_scratch(ctx, ab + bb + cb);
    if (rc) return rc;
    char *base = (char *)ctx->scratch;
    float *da = (float *)base, *db = (float *)(base + ab), *dc = (float *)(base + ab + bb);
    RT_TRY_HIP(ctx, hipMemcpyAsync(da, a, m * k * 4, hipMemcpyHostToDevice, ctx->stream));
    RT_TRY_HIP(ctx, hipMemcpyAsync(db, b, k * n * 4, hipMemcpyHostToDevice, ctx->stream));
    RT_TRY_HIP(ctx, rt::launch_matmul_f32(ctx->stream, da, db, dc, m, n, k));
    RT_TRY_HIP(ctx, hipMemcpyAsync(c, dc, cb, hipMemcpyDeviceToHost, ctx->stream));
    RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return RT_HIP_OK;
}

int rt_hip_matmul_f32_dev(rt_hip_ctx *ctx, const float *a_dev, const float *b_dev, float *c_dev, size_t m, size_t n, size_t k, size_t batch) {
    if (!ctx) return fail(nullptr, RT_HIP_ERR_INVALID_ARG, "ctx is NULL");
    RT_REQUIRE(ctx, a_dev && b_dev && c_dev, RT_HIP_ERR_INVALID_ARG, "matmul_f32_dev: NULL operand");
    RT_REQUIRE(ctx, m > 0 && n > 0 && k > 0 && batch > 0, RT_HIP_ERR_SHAPE, "matmul_f32_dev: empty dimension (m=%zu n=%zu k=%zu batch=%zu)", m, n, k,
               batch);
    RT_REQUIRE(ctx, batch <= 65535 && (m + 31) / 32 <= 65535, RT_HIP_ERR_SHAPE, "matmul_f32_dev: batch=%zu or m=%zu beyond one grid", batch, m);
    Guard g(ctx);
    RT_TRY_HIP(ctx, rt::launch_matmul_f32(ctx->stream, a_dev, b_dev, c_dev, m, n, k, batch));
    return RT_HIP_OK;
}

int rt_hip_qmatmul_i8(rt_hip_ctx *ctx, const int8_t *a, float scale_a, int zero_point_a, const int8_t *b, float scale_b,
                      int zero_point_b, size_t m, size_t n, size_t k, int8_t *out, float *out_scale, int *out_zero_point) {
    if (!ctx) return fail(nullptr, RT_HIP_ERR_INVALID_ARG, "ctx is NULL");
    RT_REQUIRE(ctx, a && b && out, RT_HIP_ERR_INVALID_ARG, "qmatmul_i8: NULL operand");
    RT_REQUIRE(ctx, m > 0 && n > 0 && k > 0, RT_HIP_ERR_SHAPE, "qmatmul_i8: empty dimension (m=%zu n=%zu k=%zu)", m, n, k);
    RT_REQUIRE(ctx, zero_point_a >= -1024 && zero_point_a <= 1024 && zero_point_b >= -1024 && zero_point_b <= 1024,
               RT_HIP_ERR_INVALID_ARG, "qmatmul_i8: zero points %d, %d outside -1024..1024", zero_point_a, zero_point_b);
    Guard g(ctx);
    size_t ab = align_up(m * k, 256), bb = align_up(k * n, 256), cb = m * n;
    int rc = ensure_scratch(ctx, ab + bb + cb);
    if (rc) return rc;
    char *base = (char *)ctx->scratch;
    int8_t *da = (int8_t *)base, *db = (int8_t *)(base + ab), *dc = (int8_t *)(base + ab + bb);
    const float scale = scale_a * scale_b;       // "output scale is product of input scales"
    RT_TRY_HIP(ctx, hipMemcpyAsync(da, a, m * k, hipMemcpyHostToDevice, ctx->stream));
    RT_TRY_HIP(ctx, hipMemcpyAsync(db, b, k * n, hipMemcpyHostToDevice, ctx->stream));
    RT_TRY_HIP(ctx, rt::launch_qmatmul_i8(ctx->stream, da, db, dc, m, n, k, zero_point_a, zero_point_b, scale));
    RT_TRY_HIP(ctx, hipMemcpyAsync(out, dc, cb, hipMemcpyDeviceToHost, ctx->stream));
    RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));
    if (out_scale) *out_scale = scale;
    if (out_zero_point) *out_zero_point = 0;
    return RT_HIP_OK;
}

// --------------------------------------------------------- quantized weights

static int qweight_check(rt_hip_ctx *ctx, int type, size_t n_rows, size_t n_cols, size_t nbytes, size_t *row_bytes) {
    size_t be = rt::type_block_elems(type), bb = rt::type_block_bytes(type);
    RT_REQUIRE(ctx, be != 0, RT_HIP_ERR_UNSUPPORTED_TYPE, "unsupported GGML type id %d", type);
    RT_REQUIRE(ctx, n_rows > 0 && n_cols > 0, RT_HIP_ERR_SHAPE, "empty tensor (%zu x %zu)", n_rows, n_cols);
    RT_REQUIRE(ctx, n_cols % be == 0, RT_HIP_ERR_SHAPE, "n_cols=%zu is not a multiple of the block size %zu", n_cols, be);
    size_t rb = n_cols / be * bb;
    RT_REQUIRE(ctx, nbytes == rb * n_rows, RT_HIP_ERR_SHAPE, "payload is %zu bytes, expected %zu (= %zu rows x %zu)", nbytes,
               rb * n_rows, n_rows, rb);
    *row_bytes = rb;
    return RT_HIP_OK;
}

int rt_hip_qweight_upload(rt_hip_ctx *ctx, int ggml_type, size_t n_rows, size_t n_cols, const void *raw_blocks,
                          size_t nbytes, rt_hip_qweight **out) {
    if (!ctx || !out) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_qweight_upload: NULL argument");
    *out = nullptr;
    RT_REQUIRE(ctx, raw_blocks, RT_HIP_ERR_INVALID_ARG, "rt_hip_qweight_upload: raw_blocks is NULL");
    size_t rb = 0;
    int rc = qweight_check(ctx, ggml_type, n_rows, n_cols, nbytes, &rb);
    if (rc) return rc;
    Guard g(ctx);
    rt_hip_qweight *w = new (std::nothrow) rt_hip_qweight();
    if (!w) return fail(ctx, RT_HIP_ERR_OOM, "host allocation failed");
    // 64 bytes of slack: the last lanes of a row may issue 16-byte loads that start inside the payload
    hipError_t e = hipMalloc((void **)&w->dev, nbytes + 64);
    if (e != hipSuccess) {
        delete w;
        return hip_fail(ctx, e, "hipMalloc(weights)");
    }
    e = hipMemcpyAsync(w->dev, raw_blocks, nbytes, hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) {
        (void)hipFree(w->dev);
        delete w;
        return hip_fail(ctx, e, "hipMemcpy(weights)");
    }
    w->type = ggml_type; w->n_rows = n_rows; w->n_cols = n_cols; w->nbytes = nbytes; w->row_bytes = rb; w->owns = true;
    *out = w;
    return RT_HIP_OK;
}

int rt_hip_qweight_wrap_dev(rt_hip_ctx *ctx, int ggml_type, size_t n_rows, size_t n_cols, const void *dev_blocks,
                            size_t nbytes, rt_hip_qweight **out) {
    if (!ctx || !out) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_qweight_wrap_dev: NULL argument");
    *out = nullptr;
    RT_REQUIRE(ctx, dev_blocks, RT_HIP_ERR_INVALID_ARG, "rt_hip_qweight_wrap_dev: dev_blocks is NULL");
    RT_REQUIRE(ctx, ((uintptr_t)dev_blocks & 15) == 0, RT_HIP_ERR_INVALID_ARG, "device blocks must be 16-byte aligned");
    size_t rb = 0;
    int rc = qweight_check(ctx, ggml_type, n_rows, n_cols, nbytes, &rb);
    if (rc) return rc;
    rt_hip_qweight *w = new (std::nothrow) rt_hip_qweight();
    if (!w) return fail(ctx, RT_HIP_ERR_OOM, "host allocation failed");
    w->type = ggml_type; w->n_rows = n_rows; w->n_cols = n_cols; w->nbytes = nbytes; w->row_bytes = rb;
    w->dev = (uint8_t *)dev_blocks; w->owns = false;
    *out = w;
    return RT_HIP_OK;
}

int rt_hip_qweight_free(rt_hip_ctx *ctx, rt_hip_qweight *w) {
    if (!w) return RT_HIP_OK;
    if (!ctx) return fail(nullptr, RT_HIP_ERR_INVALID_ARG, "ctx is NULL");
    Guard g(ctx);
    if (w->owns && w->dev) {
        (void)hipStreamSynchronize(ctx->stream);
        (void)hipFree(w->dev);
    }
    delete w;
    return RT_HIP_OK;
}

int rt_hip_dequant_dev(rt_hip_ctx *ctx, const rt_hip_qweight *w, float *out_dev) {
    if (!ctx || !w || !out_dev) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_dequant_dev: NULL argument");
    Guard g(ctx);
    RT_TRY_HIP(ctx, rt::launch_dequant(ctx->stream, w->type, w->dev, w->n_rows, w->n_cols, out_dev));
    return RT_HIP_OK;
}

int rt_hip_dequant(rt_hip_ctx *ctx, const rt_hip_qweight *w, float *out_host) {
    if (!ctx || !w || !out_host) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_dequant: NULL argument");
    Guard g(ctx);
    size_t bytes = w->n_rows * w->n_cols * sizeof(float);
    int rc = ensure_scratch(ctx, bytes);
    if (rc) return rc;
    RT_TRY_HIP(ctx, rt::launch_dequant(ctx->stream, w->type, w->dev, w->n_rows, w->n_cols, (float *)ctx->scratch));
    RT_TRY_HIP(ctx, hipMemcpyAsync(out_host, ctx->scratch, bytes, hipMemcpyDeviceToHost, ctx->stream));
    RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return RT_HIP_OK;
}

// Enqueue the GEMV for one weight; x is quantized by the kernel while it is staged into LDS.  Batches that the
// matrix-core kernel serves go there (one pass over the weights); `work` then holds its operand buffers.
static int enqueue_qgemv(rt_hip_ctx *ctx, const rt_hip_qweight *w, const float *x_dev, float *y_dev, int batch, void *work) {
    if (work && rt::qgemv_mb_serves(w->type, w->n_rows, w->n_cols, batch)) {
        RT_TRY_HIP(ctx, rt::launch_qgemv_mb(ctx->stream, w->type, w->dev, w->row_bytes, w->n_rows, w->n_cols, x_dev, batch, y_dev,
                                            nullptr, work));
        return RT_HIP_OK;
    }
    rt::GemvArgs a;
    memset(&a, 0, sizeof a);
    a.n = 1;
    a.p[0].w = w->dev; a.p[0].x = x_dev; a.p[0].stage = rt::kStageF32; a.p[0].y = y_dev; a.p[0].row_bytes = w->row_bytes;
    a.p[0].type = w->type; a.p[0].N = (int)w->n_rows; a.p[0].K = (int)w->n_cols;
    RT_TRY_HIP(ctx, rt::launch_qgemv(ctx->stream, a, batch));
    return RT_HIP_OK;
}

static int qgemv_check(rt_hip_ctx *ctx, const rt_hip_qweight *w, int batch) {
    RT_REQUIRE(ctx, gemv_type_ok(w->type), RT_HIP_ERR_UNSUPPORTED_TYPE, "qgemv: GGML type id %d has no GEMV kernel", w->type);
    RT_REQUIRE(ctx, w->n_cols % 32 == 0, RT_HIP_ERR_SHAPE, "qgemv: n_cols=%zu is not a multiple of 32", w->n_cols);
    RT_REQUIRE(ctx, batch >= 1 && batch <= 8, RT_HIP_ERR_INVALID_ARG, "qgemv: batch=%d outside 1..8 (use rt_hip_qgemm)", batch);
    RT_REQUIRE(ctx, w->n_rows < ((size_t)1 << 31) && w->n_cols < ((size_t)1 << 24), RT_HIP_ERR_SHAPE, "qgemv: tensor too large");
    RT_REQUIRE(ctx, rt::gemv_lds_bytes(w->type, w->n_cols) <= rt::kGemvLdsMax, RT_HIP_ERR_SHAPE, "qgemv: n_cols=%zu exceeds the LDS staging limit", w->n_cols);
    return RT_HIP_OK;
}

int rt_hip_qgemv_dev(rt_hip_ctx *ctx, const rt_hip_qweight *w, const float *x_dev, float *y_dev, int batch) {
    if (!ctx || !w || !x_dev || !y_dev) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_qgemv_dev: NULL argument");
    int rc = qgemv_check(ctx, w, batch);
    if (rc) return rc;
    RT_REQUIRE(ctx, ((uintptr_t)x_dev & 15) == 0, RT_HIP_ERR_INVALID_ARG, "qgemv: x must be 16-byte aligned");
    Guard g(ctx);
    void *work = nullptr;
    if (rt::qgemv_mb_serves(w->type, w->n_rows, w->n_cols, batch)) {
        rc = ensure_scratch(ctx, rt::qgemv_mb_scratch_bytes(w->n_cols));
        if (rc) return rc;
        work = ctx->scratch;
    }
    return enqueue_qgemv(ctx, w, x_dev, y_dev, batch, work);
}

int rt_hip_qgemv(rt_hip_ctx *ctx, const rt_hip_qweight *w, const float *x, float *y, int batch) {
    if (!ctx || !w || !x || !y) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_qgemv: NULL argument");
    int rc = qgemv_check(ctx, w, batch);
    if (rc) return rc;
    Guard g(ctx);
    size_t xb = align_up((size_t)batch * w->n_cols * 4, 256), yb = align_up((size_t)batch * w->n_rows * 4, 256);
    const bool mb = rt::qgemv_mb_serves(w->type, w->n_rows, w->n_cols, batch);
    rc = ensure_scratch(ctx, xb + yb + (mb ? rt::qgemv_mb_scratch_bytes(w->n_cols) : 0));
    if (rc) return rc;
    char *base = (char *)ctx->scratch;
    float *dx = (float *)base, *dy = (float *)(base + xb);
    RT_TRY_HIP(ctx, hipMemcpyAsync(dx, x, (size_t)batch * w->n_cols * 4, hipMemcpyHostToDevice, ctx->stream));
    rc = enqueue_qgemv(ctx, w, dx, dy, batch, mb ? base + xb + yb : nullptr);
    if (rc) return rc;
    RT_TRY_HIP(ctx, hipMemcpyAsync(y, dy, (size_t)batch * w->n_rows * 4, hipMemcpyDeviceToHost, ctx->stream));
    RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return RT_HIP_OK;
}

int rt_hip_qgemv_shared_x_dev(rt_hip_ctx *ctx, int n, const rt_hip_qweight *const *ws, const float *x_dev, float *const *ys_dev, int batch) {
    if (!ctx || !ws || !x_dev || !ys_dev) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_qgemv_shared_x_dev: NULL argument");
    RT_REQUIRE(ctx, n >= 1 && n <= 8, RT_HIP_ERR_INVALID_ARG, "shared-x GEMV takes 1..8 weights, got %d", n);
    RT_REQUIRE(ctx, ((uintptr_t)x_dev & 15) == 0, RT_HIP_ERR_INVALID_ARG, "shared-x GEMV: x must be 16-byte aligned");
    bool any_mb = false;
    for (int i = 0; i < n; i++) {
        if (!ws[i] || !ys_dev[i]) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "shared-x GEMV: weight or output %d is NULL", i);
        int rc = qgemv_check(ctx, ws[i], batch);
        if (rc) return rc;
        RT_REQUIRE(ctx, ws[i]->n_cols == ws[0]->n_cols, RT_HIP_ERR_SHAPE, "shared-x GEMV: weight %d has %zu columns, weight 0 has %zu", i,
                   ws[i]->n_cols, ws[0]->n_cols);
        any_mb = any_mb || rt::qgemv_mb_serves(ws[i]->type, ws[i]->n_rows, ws[i]->n_cols, batch);
    }
    Guard g(ctx);
    const size_t K = ws[0]->n_cols;
    if (any_mb) {
        // the rows are quantized once; the matrices of each format go out together, up to four per launch
        int rc = ensure_scratch(ctx, rt::qgemv_mb_scratch_bytes(K));
        if (rc) return rc;
        RT_TRY_HIP(ctx, rt::launch_qgemv_mb_prep(ctx->stream, x_dev, batch, K, ctx->scratch));
        for (int type : { (int)RT_GGML_Q4_K, (int)RT_GGML_Q6_K }) {
            rt::MbProb probs[4];
            int m = 0;
            for (int i = 0; i <= n; i++) {
                const bool take = i < n && ws[i]->type == type && rt::qgemv_mb_serves(type, ws[i]->n_rows, K, batch);
                if (take) probs[m++] = rt::MbProb{ ws[i]->dev, ws[i]->row_bytes, ws[i]->n_rows, ys_dev[i], nullptr };
                if (m == 4 || (i == n && m > 0)) {
                    RT_TRY_HIP(ctx, rt::launch_qgemv_mb_group(ctx->stream, type, probs, m, K, batch, ctx->scratch));
                    m = 0;
                }
            }
        }
    }
    // the others (another format, fewer than three rows): problems of one launch of the one-row kernel, a grid slice per row
    rt::GemvArgs a;
    memset(&a, 0, sizeof a);
    for (int i = 0; i < n; i++) {
        const rt_hip_qweight *w = ws[i];
        if (rt::qgemv_mb_serves(w->type, w->n_rows, K, batch)) continue;
        rt::GemvProb &p = a.p[a.n++];
        p.w = w->dev; p.x = x_dev; p.stage = rt::kStageF32; p.y = ys_dev[i]; p.row_bytes = w->row_bytes;
        p.type = w->type; p.N = (int)w->n_rows; p.K = (int)w->n_cols;
    }
    if (a.n > 0) RT_TRY_HIP(ctx, rt::launch_qgemv(ctx->stream, a, batch));
    return RT_HIP_OK;
}

int rt_hip_qgemv_grouped_dev(rt_hip_ctx *ctx, int n, const rt_hip_qweight *const *ws, const float *const *xs_dev,
                             float *const *ys_dev) {
    if (!ctx || !ws || !xs_dev || !ys_dev) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_qgemv_grouped_dev: NULL argument");
    RT_REQUIRE(ctx, n >= 1 && n <= rt::kMaxGemvProbs, RT_HIP_ERR_INVALID_ARG, "grouped GEMV takes 1..%d problems, got %d",
               rt::kMaxGemvProbs, n);
    rt::GemvArgs a;
    memset(&a, 0, sizeof a);
    a.n = n;
    for (int i = 0; i < n; i++) {
        if (!ws[i] || !xs_dev[i] || !ys_dev[i]) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "grouped GEMV: problem %d has a NULL member", i);
        int rc = qgemv_check(ctx, ws[i], 1);
        if (rc) return rc;
        RT_REQUIRE(ctx, ((uintptr_t)xs_dev[i] & 15) == 0, RT_HIP_ERR_INVALID_ARG, "grouped GEMV: x %d is not 16-byte aligned", i);
        const rt_hip_qweight *w = ws[i];
        a.p[i].w = w->dev; a.p[i].x = xs_dev[i]; a.p[i].stage = rt::kStageF32; a.p[i].y = ys_dev[i]; a.p[i].row_bytes = w->row_bytes;
        a.p[i].type = w->type; a.p[i].N = (int)w->n_rows; a.p[i].K = (int)w->n_cols;
    }
    Guard g(ctx);
    RT_TRY_HIP(ctx, rt::launch_qgemv(ctx->stream, a, 1));
    return RT_HIP_OK;
}

size_t rt_hip_xq_bytes(size_t n_cols) { return rt::xq_stride(n_cols); }

int rt_hip_quantize_act_dev(rt_hip_ctx *ctx, int n, const float *const *xs_dev, const size_t *n_cols, void *const *xqs_dev) {
    if (!ctx || !xs_dev || !n_cols || !xqs_dev) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_quantize_act_dev: NULL argument");
    RT_REQUIRE(ctx, n >= 1 && n <= rt::kMaxGemvProbs, RT_HIP_ERR_INVALID_ARG, "quantize_act takes 1..%d vectors, got %d", rt::kMaxGemvProbs, n);
    rt::QuantGroupArgs qa;
    memset(&qa, 0, sizeof qa);
    qa.n = n;
    for (int i = 0; i < n; i++) {
        RT_REQUIRE(ctx, xs_dev[i] && xqs_dev[i], RT_HIP_ERR_INVALID_ARG, "quantize_act: vector %d has a NULL pointer", i);
        RT_REQUIRE(ctx, n_cols[i] > 0 && n_cols[i] % 32 == 0 && n_cols[i] < ((size_t)1 << 24), RT_HIP_ERR_SHAPE,
                   "quantize_act: n_cols[%d]=%zu is not a positive multiple of 32", i, n_cols[i]);
        RT_REQUIRE(ctx, ((uintptr_t)xqs_dev[i] & 15) == 0 && ((uintptr_t)xs_dev[i] & 15) == 0, RT_HIP_ERR_INVALID_ARG,
                   "quantize_act: vector %d is not 16-byte aligned", i);
        qa.x[i] = xs_dev[i]; qa.xq[i] = (uint8_t *)xqs_dev[i]; qa.K[i] = (int)n_cols[i];
    }
    Guard g(ctx);
    RT_TRY_HIP(ctx, rt::launch_quantize_group(ctx->stream, qa));
    return RT_HIP_OK;
}

int rt_hip_qgemv_xq_grouped_dev(rt_hip_ctx *ctx, int n, const rt_hip_qweight *const *ws, const void *const *xqs_dev,
                                float *const *ys_dev) {
    if (!ctx || !ws || !xqs_dev || !ys_dev) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_qgemv_xq_grouped_dev: NULL argument");
    RT_REQUIRE(ctx, n >= 1 && n <= rt::kMaxGemvProbs, RT_HIP_ERR_INVALID_ARG, "grouped GEMV takes 1..%d problems, got %d", rt::kMaxGemvProbs, n);
    rt::GemvArgs a;
    memset(&a, 0, sizeof a);
    a.n = n;
    for (int i = 0; i < n; i++) {
        if (!ws[i] || !xqs_dev[i] || !ys_dev[i]) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "grouped GEMV: problem %d has a NULL member", i);
        int rc = qgemv_check(ctx, ws[i], 1);
        if (rc) return rc;
        RT_REQUIRE(ctx, ((uintptr_t)xqs_dev[i] & 15) == 0, RT_HIP_ERR_INVALID_ARG, "grouped GEMV: xq %d is not 16-byte aligned", i);
        const rt_hip_qweight *w = ws[i];
        a.p[i].w = w->dev; a.p[i].x = xqs_dev[i]; a.p[i].y = ys_dev[i]; a.p[i].res = nullptr;
        a.p[i].row_bytes = w->row_bytes; a.p[i].type = w->type; a.p[i].N = (int)w->n_rows; a.p[i].K = (int)w->n_cols;
    }
    Guard g(ctx);
    RT_TRY_HIP(ctx, rt::launch_qgemv(ctx->stream, a, 1));
    return RT_HIP_OK;
}

int rt_hip_qgemv_describe(rt_hip_ctx *ctx, int n, const rt_hip_qweight *const *ws, int batch, char *out, size_t out_bytes) {
    if (!ctx || !ws || !out || out_bytes == 0) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_qgemv_describe: NULL argument");
    RT_REQUIRE(ctx, n >= 1 && n <= rt::kMaxGemvProbs, RT_HIP_ERR_INVALID_ARG, "grouped GEMV takes 1..%d problems, got %d", rt::kMaxGemvProbs, n);
    rt::GemvArgs a;
    memset(&a, 0, sizeof a);
    a.n = n;
    for (int i = 0; i < n; i++) {
        if (!ws[i]) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_qgemv_describe: weight %d is NULL", i);
        int rc = qgemv_check(ctx, ws[i], batch);
        if (rc) return rc;
        a.p[i].w = ws[i]->dev; a.p[i].row_bytes = ws[i]->row_bytes; a.p[i].type = ws[i]->type; a.p[i].N = (int)ws[i]->n_rows; a.p[i].K = (int)ws[i]->n_cols;
    }
    out[0] = 0;
    if (!rt::describe_qgemv(a, batch, out, out_bytes)) return fail(ctx, RT_HIP_ERR_SHAPE, "rt_hip_qgemv_describe: no launch takes these problems");
    return RT_HIP_OK;
}

int rt_hip_qgemm_dev(rt_hip_ctx *ctx, const rt_hip_qweight *w, const float *X_dev, size_t M, float *Y_dev) {
    if (!ctx || !w || !X_dev || !Y_dev) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_qgemm_dev: NULL argument");
    RT_REQUIRE(ctx, gemv_type_ok(w->type), RT_HIP_ERR_UNSUPPORTED_TYPE, "qgemm: GGML type id %d has no kernel", w->type);
    RT_REQUIRE(ctx, w->n_cols % 32 == 0, RT_HIP_ERR_SHAPE, "qgemm: n_cols=%zu is not a multiple of 32", w->n_cols);
    RT_REQUIRE(ctx, M >= 1 && M <= 65535, RT_HIP_ERR_SHAPE, "qgemm: M=%zu outside 1..65535", M);
    RT_REQUIRE(ctx, rt::gemv_lds_bytes(w->type, w->n_cols) <= rt::kGemvLdsMax, RT_HIP_ERR_SHAPE, "qgemm: n_cols=%zu too large", w->n_cols);
    Guard g(ctx);
    size_t sb = rt::qgemm_scratch_bytes(w->type, M, w->n_rows, w->n_cols);
    int rc = ensure_scratch(ctx, sb);
    if (rc) return rc;
    RT_TRY_HIP(ctx, rt::launch_qgemm(ctx->stream, w->type, w->dev, w->n_rows, w->n_cols, w->row_bytes, X_dev, M, Y_dev,
                                     nullptr, ctx->scratch, ctx->scratch_bytes));
    return RT_HIP_OK;
}

int rt_hip_qgemm(rt_hip_ctx *ctx, const rt_hip_qweight *w, const float *X, size_t M, float *Y) {
    if (!ctx || !w || !X || !Y) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_qgemm: NULL argument");
    RT_REQUIRE(ctx, gemv_type_ok(w->type), RT_HIP_ERR_UNSUPPORTED_TYPE, "qgemm: GGML type id %d has no kernel", w->type);
    RT_REQUIRE(ctx, w->n_cols % 32 == 0, RT_HIP_ERR_SHAPE, "qgemm: n_cols=%zu is not a multiple of 32", w->n_cols);
    RT_REQUIRE(ctx, M >= 1 && M <= 65535, RT_HIP_ERR_SHAPE, "qgemm: M=%zu outside 1..65535", M);
    RT_REQUIRE(ctx, rt::gemv_lds_bytes(w->type, w->n_cols) <= rt::kGemvLdsMax, RT_HIP_ERR_SHAPE, "qgemm: n_cols=%zu too large", w->n_cols);
    Guard g(ctx);
    size_t xb = align_up(M * w->n_cols * 4, 256), yb = align_up(M * w->n_rows * 4, 256);
    size_t sb = rt::qgemm_scratch_bytes(w->type, M, w->n_rows, w->n_cols);
    int rc = ensure_scratch(ctx, xb + yb + sb);
    if (rc) return rc;
    char *base = (char *)ctx->scratch;
    float *dx = (float *)base, *dy = (float *)(base + xb);
    RT_TRY_HIP(ctx, hipMemcpyAsync(dx, X, M * w->n_cols * 4, hipMemcpyHostToDevice, ctx->stream));
    RT_TRY_HIP(ctx, rt::launch_qgemm(ctx->stream, w->type, w->dev, w->n_rows, w->n_cols, w->row_bytes, dx, M, dy, nullptr,
                                     base + xb + yb, sb));
    RT_TRY_HIP(ctx, hipMemcpyAsync(Y, dy, M * w->n_rows * 4, hipMemcpyDeviceToHost, ctx->stream));
    RT_TRY_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return RT_HIP_OK;
}

// ------------------------------------------------------------ decode steps

int rt_hip_rmsnorm_dev(rt_hip_ctx *ctx, const float *x, const float *gamma, float *y, size_t rows, size_t n, float eps) {
    if (!ctx || !x || !gamma || !y) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_rmsnorm_dev: NULL argument");
    RT_REQUIRE(ctx, n > 0, RT_HIP_ERR_SHAPE, "rmsnorm: n is 0");
    RT_REQUIRE(ctx, rows < ((size_t)1 << 31), RT_HIP_ERR_SHAPE, "rmsnorm: too many rows");
    Guard g(ctx);
    RT_TRY_HIP(ctx, rt::launch_rmsnorm(ctx->stream, x, gamma, y, nullptr, rows, n, eps));
    return RT_HIP_OK;
}

int rt_hip_swiglu_dev(rt_hip_ctx *ctx, const float *gate, const float *up, float *out, size_t n) {
    if (!ctx || !gate || !up || !out) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_swiglu_dev: NULL argument");
    Guard g(ctx);
    RT_TRY_HIP(ctx, rt::launch_swiglu(ctx->stream, gate, up, out, nullptr, n));
    return RT_HIP_OK;
}

int rt_hip_rope_dev(rt_hip_ctx *ctx, float *x, int n_heads, int head_dim, int pos, float theta) {
    if (!ctx || !x) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_rope_dev: NULL argument");
    RT_REQUIRE(ctx, n_heads > 0 && head_dim > 0 && head_dim % 2 == 0, RT_HIP_ERR_SHAPE, "rope: n_heads=%d head_dim=%d", n_heads, head_dim);
    RT_REQUIRE(ctx, pos >= 0 && theta > 0.f, RT_HIP_ERR_INVALID_ARG, "rope: pos=%d theta=%g", pos, (double)theta);
    Guard g(ctx);
    RT_TRY_HIP(ctx, rt::launch_rope(ctx->stream, x, n_heads, head_dim, nullptr, pos, nullptr, theta));
    return RT_HIP_OK;
}

int rt_hip_kv_append_dev(rt_hip_ctx *ctx, uint16_t *cache, const float *v, size_t pos, size_t row_elems) {
    if (!ctx || !cache || !v) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_kv_append_dev: NULL argument");
    Guard g(ctx);
    RT_TRY_HIP(ctx, rt::launch_kv_append(ctx->stream, cache, v, nullptr, pos, row_elems));
    return RT_HIP_OK;
}

int rt_hip_attn_decode_dev(rt_hip_ctx *ctx, const float *q, const uint16_t *kcache, const uint16_t *vcache, int n_pos,
                           int n_heads, int head_dim, float *out) {
    if (!ctx || !q || !kcache || !vcache || !out) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_attn_decode_dev: NULL argument");
    RT_REQUIRE(ctx, head_dim == 64 || head_dim == 128, RT_HIP_ERR_SHAPE, "attn_decode: head_dim=%d (64 or 128 supported)", head_dim);
    RT_REQUIRE(ctx, n_heads > 0 && n_pos > 0 && n_pos <= 16000, RT_HIP_ERR_SHAPE, "attn_decode: n_heads=%d n_pos=%d", n_heads, n_pos);
    Guard g(ctx);
    RT_TRY_HIP(ctx, rt::launch_attn_decode(ctx->stream, const_cast<float *>(q), nullptr, nullptr, const_cast<uint16_t *>(kcache),
                                           const_cast<uint16_t *>(vcache), nullptr, n_pos, n_heads, n_heads, head_dim, nullptr, out, nullptr, false));
    return RT_HIP_OK;
}

int rt_hip_attn_causal_dev(rt_hip_ctx *ctx, const float *q, const uint16_t *kcache, const uint16_t *vcache, int pos0, int n_queries,
                           int n_heads, int n_kv_heads, int head_dim, float *out) {
    if (!ctx || !q || !kcache || !vcache || !out) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_attn_causal_dev: NULL argument");
    if (n_kv_heads == 0) n_kv_heads = n_heads;
    RT_REQUIRE(ctx, head_dim == 64 || head_dim == 128, RT_HIP_ERR_SHAPE, "attn_causal: head_dim=%d (64 or 128 supported)", head_dim);
    RT_REQUIRE(ctx, n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0, RT_HIP_ERR_SHAPE, "attn_causal: n_heads=%d n_kv_heads=%d",
               n_heads, n_kv_heads);
    RT_REQUIRE(ctx, pos0 >= 0 && n_queries > 0 && (long long)pos0 + n_queries <= (1 << 24), RT_HIP_ERR_SHAPE, "attn_causal: pos0=%d n_queries=%d",
               pos0, n_queries);
    RT_REQUIRE(ctx, (((uintptr_t)q | (uintptr_t)kcache | (uintptr_t)vcache | (uintptr_t)out) & 15) == 0, RT_HIP_ERR_INVALID_ARG,
               "attn_causal: operands must be 16-byte aligned");
    Guard g(ctx);
    RT_TRY_HIP(ctx, rt::launch_attn_causal(ctx->stream, q, kcache, vcache, pos0, (size_t)n_queries, n_heads, n_kv_heads, head_dim, out));
    return RT_HIP_OK;
}

int rt_hip_add_dev(rt_hip_ctx *ctx, float *x, const float *y, size_t n) {
    if (!ctx || !x || !y) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_add_dev: NULL argument");
    Guard g(ctx);
    RT_TRY_HIP(ctx, rt::launch_add(ctx->stream, x, y, n));
    return RT_HIP_OK;
}

int rt_hip_set_option(rt_hip_ctx *ctx, int option, int value) {
    if (!rt::set_path_option(option, value)) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_set_option: option %d, value %d", option, value);
    return RT_HIP_OK;
}

int rt_hip_get_option(rt_hip_ctx *ctx, int option, int *value) {
    if (!value) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_get_option: NULL argument");
    const int v = rt::path_option(option);
    if (v < 0) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_get_option: option %d", option);
    *value = v;
    return RT_HIP_OK;
}

int rt_hip_stream_read_dev(rt_hip_ctx *ctx, const void *dev, size_t nbytes) {
    if (!ctx || !dev) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_stream_read_dev: NULL argument");
    RT_REQUIRE(ctx, ((uintptr_t)dev & 15) == 0, RT_HIP_ERR_INVALID_ARG, "stream_read: the buffer must be 16-byte aligned");
    Guard g(ctx);
    int rc = ensure_scratch(ctx, 256);
    if (rc) return rc;
    RT_TRY_HIP(ctx, rt::launch_stream_read(ctx->stream, dev, nbytes, (unsigned *)ctx->scratch));
    return RT_HIP_OK;
}

int rt_hip_argmax_dev(rt_hip_ctx *ctx, const float *v, size_t n, int *out_index_dev) {
    if (!ctx || !v || !out_index_dev) return fail(ctx, RT_HIP_ERR_INVALID_ARG, "rt_hip_argmax_dev: NULL argument");
    RT_REQUIRE(ctx, n > 0 && n < ((size_t)1 << 31), RT_HIP_ERR_SHAPE, "argmax: n=%zu", n);
    Guard g(ctx);
    RT_TRY_HIP(ctx, rt::launch_argmax(ctx->stream, v, n, out_index_dev));
    return RT_HIP_OK;
}

}  // extern "C"
