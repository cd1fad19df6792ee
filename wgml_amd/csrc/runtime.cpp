// Context, buffers, timers and error reporting of the C ABI.
#include "common.h"

namespace wgml {

static thread_local std::string g_last_error;

int set_error(int code, const char *fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

int check_view(const wgml_view &v, const char *what) {
    WGML_REQUIRE(v.buf != nullptr && v.buf->ptr != nullptr, "%s: null buffer", what);
    WGML_REQUIRE((v.offset + (uint64_t)v.len) * 4 <= v.buf->bytes,
                 "%s: view [%llu, +%u) exceeds buffer of %llu bytes", what,
                 (unsigned long long)v.offset, v.len, (unsigned long long)v.buf->bytes);
    return WGML_OK;
}

bool graphs_disabled() {
    const char *v = getenv("WGML_DISABLE_GRAPHS");
    return v && *v && strcmp(v, "0") != 0;
}

void ctx_retain(wgml_ctx *ctx) {
    if (ctx) ++ctx->refs;
}

void ctx_release(wgml_ctx *ctx) {
    if (!ctx || --ctx->refs > 0) return;
    (void)hipSetDevice(ctx->device);
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    if (ctx->attn_ws) (void)hipFree(ctx->attn_ws);
    if (ctx->prefill_xh) (void)hipFree(ctx->prefill_xh);
    if (ctx->prefill_xscale) (void)hipFree(ctx->prefill_xscale);
    if (ctx->gemm_part) (void)hipFree(ctx->gemm_part);
    for (void *p : ctx->retired) (void)hipFree(p);
    if (ctx->d_scalar) (void)hipFree(ctx->d_scalar);
    if (ctx->h_scalar) (void)hipHostFree(ctx->h_scalar);
    if (ctx->ev_start) (void)hipEventDestroy(ctx->ev_start);
    if (ctx->ev_stop) (void)hipEventDestroy(ctx->ev_stop);
    if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

}  // namespace wgml

using namespace wgml;

extern "C" {

const char *wgml_last_error(void) { return g_last_error.c_str(); }

const char *wgml_version(void) { return "wgml_hip 0.1 (gfx950)"; }

int wgml_ctx_create(int device, wgml_ctx **out) {
    WGML_REQUIRE(out != nullptr, "wgml_ctx_create: out is null");
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0)
        return set_error(WGML_E_NO_DEVICE, "wgml_ctx_create: no HIP device (%s)",
                         e == hipSuccess ? "count is 0" : hipGetErrorString(e));
    WGML_REQUIRE(device >= 0 && device < count, "wgml_ctx_create: device %d of %d", device, count);
    WGML_CHECK_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    WGML_CHECK_HIP(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return set_error(WGML_E_NO_DEVICE,
                         "wgml_ctx_create: device %d is %s; the kernels are built for gfx950 only",
                         device, prop.gcnArchName);
    wgml_ctx *ctx = new wgml_ctx();
    ctx->device = device;
    ctx->n_cu = prop.multiProcessorCount;
    snprintf(ctx->name, sizeof(ctx->name), "%s (%s)", prop.name, prop.gcnArchName);
    hipError_t err = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
    if (err == hipSuccess) err = hipEventCreate(&ctx->ev_start);
    if (err == hipSuccess) err = hipEventCreate(&ctx->ev_stop);
    if (err == hipSuccess) err = hipMalloc((void **)&ctx->d_scalar, 256);
    if (err == hipSuccess) err = hipHostMalloc((void **)&ctx->h_scalar, 256, hipHostMallocDefault);
    if (err != hipSuccess) {
        wgml_ctx_destroy(ctx);
        return set_error(WGML_E_HIP, "wgml_ctx_create: %s", hipGetErrorString(err));
    }
    const int rc = resolve_noalloc_scratch(ctx);  // the device is current (hipSetDevice above)
    if (rc != WGML_OK) {
        wgml_ctx_destroy(ctx);
        return rc;
    }
    *out = ctx;
    return WGML_OK;
}

int wgml_ctx_destroy(wgml_ctx *ctx) {
    if (!ctx) return WGML_OK;
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    ctx_release(ctx);
    return WGML_OK;
}

// Launch-shape overrides of one context, for kernel sweeps and for tests that must reach
// every kernel variant.  0 restores the heuristic.
int wgml_ctx_set_tuning(wgml_ctx *ctx, int key, int value) {
    WGML_REQUIRE(ctx != nullptr, "wgml_ctx_set_tuning: null context");
    WGML_REQUIRE(key >= 0 && key < WGML_TUNE_COUNT, "wgml_ctx_set_tuning: unknown key %d", key);
    bool ok = value >= 0;
    switch (key) {
    case WGML_TUNE_GEMV_ROWS_PER_WAVE: ok = value >= 0 && value <= 2; break;
    case WGML_TUNE_GEMV_WAVES_PER_WG: ok = value == 0 || value == 4 || value == 8 || value == 12 || value == 16; break;
    case WGML_TUNE_GEMV_WG_PER_CU: ok = value >= 0 && value <= 8; break;
    case WGML_TUNE_ATTN_WIDE_POSITIONS: ok = value >= 0 && value <= (1 << 20); break;
    case WGML_TUNE_GEMV_DEPTH: ok = value >= 0 && value <= 4; break;
    case WGML_TUNE_GEMV_F32_ACTIVATIONS:
    case WGML_TUNE_PREFILL_ATTENTION_PER_TOKEN: ok = value == 0 || value == 1; break;
    case WGML_TUNE_GEMM_K_SPLIT: ok = value >= 0 && value <= 8; break;
    case WGML_TUNE_ATTN_SPLITS: ok = value == 0 || (value >= 2 && value <= 64); break;
    case WGML_TUNE_ATTN_MERGE: ok = value == 0 || value == 1; break;
    default: break;
    }
    WGML_REQUIRE(ok, "wgml_ctx_set_tuning: value %d is not valid for key %d", value, key);
    // models drop the launch sequences they recorded under other settings (build_graph)
    if (ctx->tuning[key] != value) ++ctx->tuning_generation;
    ctx->tuning[key] = value;
    return WGML_OK;
}

int wgml_ctx_synchronize(wgml_ctx *ctx) {
    WGML_REQUIRE(ctx != nullptr, "wgml_ctx_synchronize: null context");
    WGML_CHECK_HIP(hipStreamSynchronize(ctx->stream));
    return WGML_OK;
}

int wgml_ctx_stream(wgml_ctx *ctx, void **stream) {
    WGML_REQUIRE(ctx && stream, "wgml_ctx_stream: null argument");
    *stream = ctx->stream;
    return WGML_OK;
}

int wgml_ctx_info(wgml_ctx *ctx, char *name, size_t name_len, int *n_cu) {
    WGML_REQUIRE(ctx != nullptr, "wgml_ctx_info: null context");
    if (name && name_len) snprintf(name, name_len, "%s", ctx->name);
    if (n_cu) *n_cu = ctx->n_cu;
    return WGML_OK;
}

int wgml_timer_start(wgml_ctx *ctx) {
    WGML_REQUIRE(ctx != nullptr, "wgml_timer_start: null context");
    WGML_CHECK_HIP(hipEventRecord(ctx->ev_start, ctx->stream));
    return WGML_OK;
}

int wgml_timer_stop(wgml_ctx *ctx, float *ms) {
    WGML_REQUIRE(ctx != nullptr && ms != nullptr, "wgml_timer_stop: null argument");
    WGML_CHECK_HIP(hipEventRecord(ctx->ev_stop, ctx->stream));
    WGML_CHECK_HIP(hipEventSynchronize(ctx->ev_stop));
    WGML_CHECK_HIP(hipEventElapsedTime(ms, ctx->ev_start, ctx->ev_stop));
    return WGML_OK;
}

int wgml_buf_create(wgml_ctx *ctx, uint64_t bytes, wgml_buf **out) {
    WGML_REQUIRE(ctx != nullptr && out != nullptr, "wgml_buf_create: null argument");
    *out = nullptr;
    WGML_REQUIRE(bytes > 0, "wgml_buf_create: zero-sized buffer");
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess)
        return set_error(WGML_E_OOM, "wgml_buf_create: hipMalloc(%llu) failed: %s",
                         (unsigned long long)bytes, hipGetErrorString(e));
    wgml_buf *b = new wgml_buf();
    b->ctx = ctx;
    ctx_retain(ctx);
    b->ptr = p;
    b->bytes = bytes;
    *out = b;
    return WGML_OK;
}

int wgml_buf_destroy(wgml_buf *buf) {
    if (!buf) return WGML_OK;
    if (buf->ctx && buf->ctx->stream) (void)hipStreamSynchronize(buf->ctx->stream);
    if (buf->ptr) (void)hipFree(buf->ptr);
    ctx_release(buf->ctx);
    delete buf;
    return WGML_OK;
}

uint64_t wgml_buf_size(const wgml_buf *buf) { return buf ? buf->bytes : 0; }

int wgml_buf_upload(wgml_buf *buf, uint64_t off, const void *src, uint64_t bytes) {
    WGML_REQUIRE(buf != nullptr && src != nullptr, "wgml_buf_upload: null argument");
    WGML_REQUIRE(off + bytes <= buf->bytes, "wgml_buf_upload: range exceeds buffer");
    if (bytes == 0) return WGML_OK;
    // Ordered after earlier work on the stream; the source may be reused on return.
    WGML_CHECK_HIP(hipMemcpyAsync((char *)buf->ptr + off, src, bytes, hipMemcpyHostToDevice,
                                  buf->ctx->stream));
    WGML_CHECK_HIP(hipStreamSynchronize(buf->ctx->stream));
    return WGML_OK;
}

int wgml_buf_download(wgml_buf *buf, uint64_t off, void *dst, uint64_t bytes) {
    WGML_REQUIRE(buf != nullptr && dst != nullptr, "wgml_buf_download: null argument");
    WGML_REQUIRE(off + bytes <= buf->bytes, "wgml_buf_download: range exceeds buffer");
    if (bytes == 0) return WGML_OK;
    WGML_CHECK_HIP(hipMemcpyAsync(dst, (const char *)buf->ptr + off, bytes, hipMemcpyDeviceToHost,
                                  buf->ctx->stream));
    WGML_CHECK_HIP(hipStreamSynchronize(buf->ctx->stream));
    return WGML_OK;
}

int wgml_buf_copy(wgml_buf *dst, uint64_t doff, const wgml_buf *src, uint64_t soff,
                  uint64_t bytes) {
    WGML_REQUIRE(dst != nullptr && src != nullptr, "wgml_buf_copy: null argument");
    WGML_REQUIRE(doff + bytes <= dst->bytes && soff + bytes <= src->bytes,
                 "wgml_buf_copy: range exceeds buffer");
    if (bytes == 0) return WGML_OK;
    WGML_CHECK_HIP(hipMemcpyAsync((char *)dst->ptr + doff, (const char *)src->ptr + soff, bytes,
                                  hipMemcpyDeviceToDevice, dst->ctx->stream));
    return WGML_OK;
}

int wgml_buf_zero(wgml_buf *buf) {
    WGML_REQUIRE(buf != nullptr, "wgml_buf_zero: null buffer");
    WGML_CHECK_HIP(hipMemsetAsync(buf->ptr, 0, buf->bytes, buf->ctx->stream));
    return WGML_OK;
}

}  // extern "C"
