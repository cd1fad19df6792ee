// GPU-timed back-to-back GEMV launches: the measuring loop of wgml-bench's
// bench_gemv (crates/wgml-bench/src/main.rs:187-250 of the reference: N
// dispatches between two GPU timestamps), with the launches recorded into a HIP
// graph so that host launch overhead does not sit between the kernels.
#include "common.h"

using namespace wgml;

namespace {

// A kernel that only reads: rows of 2304 bytes (4096 columns of Q4_K: sixteen 144-byte
// super-blocks), one wave per row and step, each lane requesting the three 16-byte words of
// its 64-element tile (header + two words of nibbles) with one tile in flight, rows dealt out
// to the waves of the machine the way the GEMV kernels deal them out.  Nothing is computed and
// nothing is stored: what it takes is what the memory system takes to deliver the bytes to
// the compute units with this access pattern.
__global__ __launch_bounds__(1024) void read_chain_kernel(const uint8_t *__restrict__ base,
                                                          uint32_t nrows, uint32_t *sink) {
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const uint32_t gw = blockIdx.x * nw + wave, GW = gridDim.x * nw;
    constexpr size_t kRowBytes = 16 * 144;
    uint4 buf[3];
    auto load = [&](uint32_t row) {
        const uint8_t *blk = base + (size_t)row * kRowBytes + (lane >> 2) * 144;
        buf[0] = *reinterpret_cast<const uint4 *>(blk);
        buf[1] = *reinterpret_cast<const uint4 *>(blk + 16 + (lane & 3) * 32);
        buf[2] = *reinterpret_cast<const uint4 *>(blk + 32 + (lane & 3) * 32);
    };
    uint32_t next = gw, acc = 0;
    if (next < nrows) load(next);
    next += GW;
    for (uint32_t r = gw; r < nrows; r += GW) {
        acc ^= buf[0].x ^ buf[1].y ^ buf[2].z ^ buf[1].w ^ buf[2].x;
        if (next < nrows) load(next);
        next += GW;
    }
    if (acc == 0x12345678u) sink[0] = acc;  // keeps the loads alive; the pool holds no such word
}

}  // namespace

extern "C" {

int wgml_bench_read_chain(wgml_ctx *ctx, uint32_t nrows, uint32_t iters, int use_graph,
                          float *total_ms) {
    WGML_REQUIRE(ctx && total_ms && nrows > 0 && iters > 0, "wgml_bench_read_chain: bad argument");
    constexpr size_t kRowBytes = 16 * 144;
    const size_t bytes = (size_t)nrows * kRowBytes;
    const size_t pool_bytes = (size_t)1536 << 20;  // six times the 256 MB memory-side cache
    WGML_REQUIRE(bytes * 2 <= pool_bytes, "wgml_bench_read_chain: %u rows exceed half the pool", nrows);
    const uint32_t ncopies = (uint32_t)(pool_bytes / bytes);
    uint8_t *pool = nullptr;
    hipError_t e = hipMalloc((void **)&pool, pool_bytes + 4096);
    if (e != hipSuccess)
        return set_error(WGML_E_OOM, "wgml_bench_read_chain: hipMalloc: %s", hipGetErrorString(e));
    uint32_t *sink = ctx->d_scalar + 16;
    const uint32_t cu = ctx->n_cu > 0 ? (uint32_t)ctx->n_cu : 256u;
    auto launch = [&](uint32_t i) {
        read_chain_kernel<<<dim3(cu), dim3(1024), 0, ctx->stream>>>(
            pool + (size_t)(i % ncopies) * bytes, nrows, sink);
    };
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    e = hipMemsetAsync(pool, 1, pool_bytes, ctx->stream);
    if (e == hipSuccess) {
        launch(0);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    const bool graphed = use_graph && !graphs_disabled();
    if (e == hipSuccess && graphed) {
        e = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal);
        if (e == hipSuccess) {
            for (uint32_t i = 0; i < iters; ++i) launch(i);
            e = hipStreamEndCapture(ctx->stream, &graph);
        }
        if (e == hipSuccess) e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
        if (e == hipSuccess) e = hipGraphLaunch(exec, ctx->stream);  // warm replay, untimed
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    }
    if (e == hipSuccess) e = hipEventRecord(ctx->ev_start, ctx->stream);
    if (e == hipSuccess) {
        if (graphed) {
            e = hipGraphLaunch(exec, ctx->stream);
        } else {
            for (uint32_t i = 0; i < iters; ++i) launch(i);
            e = hipGetLastError();
        }
    }
    if (e == hipSuccess) e = hipEventRecord(ctx->ev_stop, ctx->stream);
    if (e == hipSuccess) e = hipEventSynchronize(ctx->ev_stop);
    if (e == hipSuccess) e = hipEventElapsedTime(total_ms, ctx->ev_start, ctx->ev_stop);
    (void)hipStreamSynchronize(ctx->stream);
    if (exec) (void)hipGraphExecDestroy(exec);
    if (graph) (void)hipGraphDestroy(graph);
    (void)hipFree(pool);
    ctx->launches += iters;
    if (e != hipSuccess) return set_error(WGML_E_HIP, "wgml_bench_read_chain: %s", hipGetErrorString(e));
    return WGML_OK;
}

int wgml_bench_gemv_quant(wgml_ctx *ctx, const wgml_qmat *const *mats, uint32_t n_mats,
                          wgml_view out, wgml_view v, uint32_t iters, int use_graph,
                          float *total_ms) {
    WGML_REQUIRE(ctx && mats && total_ms && n_mats > 0 && iters > 0,
                 "wgml_bench_gemv_quant: bad argument");
    WGML_TRY(check_view(out, "wgml_bench_gemv_quant: out"));
    WGML_TRY(check_view(v, "wgml_bench_gemv_quant: v"));
    for (uint32_t i = 0; i < n_mats; ++i) {
        WGML_REQUIRE(mats[i] != nullptr, "wgml_bench_gemv_quant: null matrix %u", i);
        WGML_REQUIRE(mats[i]->ncols == v.len && mats[i]->nrows == out.len,
                     "wgml_bench_gemv_quant: matrix %u does not match the vectors", i);
    }
    float *po = view_ptr(out);
    const float *pv = view_ptr(v);
    if (!use_graph || graphs_disabled()) {
        WGML_CHECK_HIP(hipEventRecord(ctx->ev_start, ctx->stream));
        for (uint32_t i = 0; i < iters; ++i)
            WGML_TRY(launch_gemv_quant(ctx, po, mats[i % n_mats], pv, GemvEpilogue{}));
        WGML_CHECK_HIP(hipEventRecord(ctx->ev_stop, ctx->stream));
        WGML_CHECK_HIP(hipEventSynchronize(ctx->ev_stop));
        WGML_CHECK_HIP(hipEventElapsedTime(total_ms, ctx->ev_start, ctx->ev_stop));
        return WGML_OK;
    }
    // one untimed launch per matrix first: opt-in attributes and lazy module
    // loading must not happen during capture
    for (uint32_t i = 0; i < n_mats && i < iters; ++i)
        WGML_TRY(launch_gemv_quant(ctx, po, mats[i], pv, GemvEpilogue{}));
    WGML_CHECK_HIP(hipStreamSynchronize(ctx->stream));
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    WGML_CHECK_HIP(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    int rc = WGML_OK;
    for (uint32_t i = 0; i < iters && rc == WGML_OK; ++i)
        rc = launch_gemv_quant(ctx, po, mats[i % n_mats], pv, GemvEpilogue{});
    hipError_t e = hipStreamEndCapture(ctx->stream, &graph);
    if (rc != WGML_OK) {
        if (graph) (void)hipGraphDestroy(graph);
        return rc;
    }
    if (e != hipSuccess)
        return set_error(WGML_E_HIP, "wgml_bench_gemv_quant: end capture: %s", hipGetErrorString(e));
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    if (e == hipSuccess) e = hipGraphLaunch(exec, ctx->stream);  // warm replay, untimed
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e == hipSuccess) e = hipEventRecord(ctx->ev_start, ctx->stream);
    if (e == hipSuccess) e = hipGraphLaunch(exec, ctx->stream);
    if (e == hipSuccess) e = hipEventRecord(ctx->ev_stop, ctx->stream);
    if (e == hipSuccess) e = hipEventSynchronize(ctx->ev_stop);
    if (e == hipSuccess) e = hipEventElapsedTime(total_ms, ctx->ev_start, ctx->ev_stop);
    if (exec) (void)hipGraphExecDestroy(exec);
    if (graph) (void)hipGraphDestroy(graph);
    if (e != hipSuccess)
        return set_error(WGML_E_HIP, "wgml_bench_gemv_quant: %s", hipGetErrorString(e));
    return WGML_OK;
}

int wgml_bench_gemv_fused(wgml_ctx *ctx, const wgml_qmat *const *a,
                          const wgml_qmat *const *b, const int *modes, uint32_t njobs,
                          uint32_t nsets, wgml_view out, uint32_t stride, wgml_view v,
                          const wgml_view *norm_w, uint32_t iters, float *total_ms) {
    WGML_REQUIRE(ctx && a && modes && total_ms && njobs >= 1 && njobs <= 3 && nsets > 0 && iters > 0,
                 "wgml_bench_gemv_fused: bad argument");
    WGML_TRY(check_view(out, "wgml_bench_gemv_fused: out"));
    WGML_TRY(check_view(v, "wgml_bench_gemv_fused: v"));
    WGML_REQUIRE((uint64_t)stride * njobs <= out.len, "wgml_bench_gemv_fused: out too small");
    std::vector<FusedGemv> sets(nsets);
    for (uint32_t s = 0; s < nsets; ++s) {
        FusedGemv &f = sets[s];
        f.njobs = (int)njobs;
        f.x = view_ptr(v);
        if (norm_w && norm_w->buf) {
            WGML_TRY(check_view(*norm_w, "wgml_bench_gemv_fused: norm_w"));
            f.norm_w = view_ptr(*norm_w);
            f.norm_eps = 1e-5f;
        }
        f.head_size = 128;
        for (uint32_t j = 0; j < njobs; ++j) {
            const wgml_qmat *m = a[s * njobs + j];
            WGML_REQUIRE(m && m->ncols == v.len && m->nrows <= stride,
                         "wgml_bench_gemv_fused: matrix %u/%u does not fit", s, j);
            f.jobs[j].a = m;
            f.jobs[j].b = b ? b[s * njobs + j] : nullptr;
            f.jobs[j].mode = modes[j];
            f.jobs[j].out = view_ptr(out) + (size_t)j * stride;
        }
    }
    for (uint32_t s = 0; s < nsets && s < iters; ++s) WGML_TRY(launch_gemv_fused(ctx, sets[s]));
    WGML_CHECK_HIP(hipStreamSynchronize(ctx->stream));
    if (graphs_disabled()) {
        WGML_CHECK_HIP(hipEventRecord(ctx->ev_start, ctx->stream));
        for (uint32_t i = 0; i < iters; ++i) WGML_TRY(launch_gemv_fused(ctx, sets[i % nsets]));
        WGML_CHECK_HIP(hipEventRecord(ctx->ev_stop, ctx->stream));
        WGML_CHECK_HIP(hipEventSynchronize(ctx->ev_stop));
        WGML_CHECK_HIP(hipEventElapsedTime(total_ms, ctx->ev_start, ctx->ev_stop));
        return WGML_OK;
    }
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    WGML_CHECK_HIP(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    int rc = WGML_OK;
    for (uint32_t i = 0; i < iters && rc == WGML_OK; ++i) rc = launch_gemv_fused(ctx, sets[i % nsets]);
    hipError_t e = hipStreamEndCapture(ctx->stream, &graph);
    if (rc != WGML_OK) {
        if (graph) (void)hipGraphDestroy(graph);
        return rc;
    }
    if (e == hipSuccess) e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    if (e == hipSuccess) e = hipGraphLaunch(exec, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
    if (e == hipSuccess) e = hipEventRecord(ctx->ev_start, ctx->stream);
    if (e == hipSuccess) e = hipGraphLaunch(exec, ctx->stream);
    if (e == hipSuccess) e = hipEventRecord(ctx->ev_stop, ctx->stream);
    if (e == hipSuccess) e = hipEventSynchronize(ctx->ev_stop);
    if (e == hipSuccess) e = hipEventElapsedTime(total_ms, ctx->ev_start, ctx->ev_stop);
    if (exec) (void)hipGraphExecDestroy(exec);
    if (graph) (void)hipGraphDestroy(graph);
    if (e != hipSuccess)
        return set_error(WGML_E_HIP, "wgml_bench_gemv_fused: %s", hipGetErrorString(e));
    return WGML_OK;
}

int wgml_bench_attention(wgml_ctx *ctx, const wgml_attn_params *p, uint32_t plan_positions,
                         wgml_view q, const wgml_view *key_caches, const wgml_view *value_caches,
                         uint32_t n_sets, wgml_view xb, uint32_t iters, float *total_ms) {
    WGML_REQUIRE(ctx && p && key_caches && value_caches && total_ms && n_sets > 0 && iters > 0,
                 "wgml_bench_attention: bad argument");
    WGML_REQUIRE(p->n_heads > 0 && p->kv_mul > 0 && p->head_size > 0 && p->pos < p->seq_len &&
                     plan_positions > p->pos && plan_positions <= p->seq_len &&
                     p->kv_dim == p->n_heads / p->kv_mul * p->head_size,
                 "wgml_bench_attention: inconsistent parameters");
    WGML_TRY(check_view(q, "wgml_bench_attention: q"));
    WGML_TRY(check_view(xb, "wgml_bench_attention: xb"));
    const uint64_t dim = (uint64_t)p->n_heads * p->head_size;
    WGML_REQUIRE(q.len >= dim && xb.len >= dim, "wgml_bench_attention: q / xb too short");
    for (uint32_t s = 0; s < n_sets; ++s) {
        WGML_TRY(check_view(key_caches[s], "wgml_bench_attention: key cache"));
        WGML_TRY(check_view(value_caches[s], "wgml_bench_attention: value cache"));
        WGML_REQUIRE(key_caches[s].len >= (uint64_t)p->seq_len * p->kv_dim &&
                         value_caches[s].len >= (uint64_t)p->seq_len * p->kv_dim,
                     "wgml_bench_attention: cache %u shorter than seq_len x kv_dim", s);
    }
    // the position comes from device memory, as in a recorded decode step
    DynState *dyn = nullptr;
    WGML_CHECK_HIP(hipMalloc(&dyn, sizeof(DynState)));
    const DynState init{p->pos, 0, 0, 0};
    hipError_t e = hipMemcpy(dyn, &init, sizeof(init), hipMemcpyHostToDevice);
    DynPos dpos{};
    dpos.ptr = &dyn->pos;
    auto launch = [&](uint32_t i) {
        return launch_attention_planned(ctx, *p, dpos, plan_positions, p->seq_len, view_ptr(q),
                                        view_ptr(key_caches[i % n_sets]),
                                        view_ptr(value_caches[i % n_sets]), nullptr, view_ptr(xb));
    };
    int rc = e == hipSuccess ? reserve_attention_workspace(ctx, *p, plan_positions) : WGML_E_HIP;
    for (uint32_t s = 0; s < n_sets && s < iters && rc == WGML_OK; ++s) rc = launch(s);
    if (rc == WGML_OK && hipStreamSynchronize(ctx->stream) != hipSuccess) rc = WGML_E_HIP;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    if (rc == WGML_OK) {
        const bool eager = graphs_disabled();
        if (!eager) {
            e = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal);
            for (uint32_t i = 0; i < iters && rc == WGML_OK && e == hipSuccess; ++i) rc = launch(i);
            if (e == hipSuccess) e = hipStreamEndCapture(ctx->stream, &graph);
            if (e == hipSuccess && rc == WGML_OK) e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
            if (e == hipSuccess && rc == WGML_OK) e = hipGraphLaunch(exec, ctx->stream);
            if (e == hipSuccess && rc == WGML_OK) e = hipStreamSynchronize(ctx->stream);
        }
        if (e == hipSuccess && rc == WGML_OK) e = hipEventRecord(ctx->ev_start, ctx->stream);
        if (e == hipSuccess && rc == WGML_OK) {
            if (eager)
                for (uint32_t i = 0; i < iters && rc == WGML_OK; ++i) rc = launch(i);
            else
                e = hipGraphLaunch(exec, ctx->stream);
        }
        if (e == hipSuccess && rc == WGML_OK) e = hipEventRecord(ctx->ev_stop, ctx->stream);
        if (e == hipSuccess && rc == WGML_OK) e = hipEventSynchronize(ctx->ev_stop);
        if (e == hipSuccess && rc == WGML_OK) e = hipEventElapsedTime(total_ms, ctx->ev_start, ctx->ev_stop);
    }
    (void)hipStreamSynchronize(ctx->stream);
    if (exec) (void)hipGraphExecDestroy(exec);
    if (graph) (void)hipGraphDestroy(graph);
    (void)hipFree(dyn);
    if (rc != WGML_OK) return rc;
    if (e != hipSuccess) return set_error(WGML_E_HIP, "wgml_bench_attention: %s", hipGetErrorString(e));
    return WGML_OK;
}

}  // extern "C"
