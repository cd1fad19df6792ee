// GPU-timed back-to-back GEMV launches: the measuring loop of wgml-bench's
// bench_gemv (crates/wgml-bench/src/main.rs:187-250 of the reference: N
// dispatches between two GPU timestamps), with the launches recorded into a HIP
// graph so that host launch overhead does not sit between the kernels.
#include "common.h"

using namespace wgml;

extern "C" {

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
