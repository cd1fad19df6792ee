// Llama-family decoder: state, weights and the per-token launch sequence.
// Mirrors Llama2State / Llama2Weights / Llama2::dispatch
// (models/llama2/transformer.rs:17-476 of the reference) and the token loop of
// ChatLlama2 (wgml-chat/src/chat_llama2.rs:51-228).
//
// One decode step is a fixed sequence of launches.  It exists in two forms:
//   * eager: token and position are host values (wgml_llama2_forward);
//   * recorded: token and position live in a small device struct that the
//     kernels read, the arg-max kernel writes the next token and advances the
//     position, and the whole step is a HIP graph replayed once per token with
//     no host round trip in between (the greedy loops).
#include "common.h"

using namespace wgml;

namespace wgml {
int reserve_attention_workspace(wgml_ctx *ctx, const wgml_attn_params &p, uint32_t plan_positions);
}  // namespace wgml

struct LlamaLayer {
    const wgml_qmat *attn_q = nullptr, *attn_k = nullptr, *attn_v = nullptr, *attn_output = nullptr,
                    *ffn_gate = nullptr, *ffn_up = nullptr, *ffn_down = nullptr;
    float *attn_norm = nullptr, *ffn_norm = nullptr;
    float *bq = nullptr, *bk = nullptr, *bv = nullptr;
    float *key_cache = nullptr, *value_cache = nullptr;
};

struct wgml_llama2 {
    wgml_ctx *ctx = nullptr;
    wgml_llama2_config cfg{};
    int model_type = WGML_MODEL_LLAMA;
    int fusion = 3;
    uint32_t kv_dim = 0, head_size = 0, kv_mul = 0;
    std::vector<LlamaLayer> layers;
    const wgml_qmat *output = nullptr;
    float *output_norm = nullptr;
    float *token_embd = nullptr;
    // Llama2State (models/llama2/transformer.rs:17-45)
    float *x = nullptr, *xb = nullptr, *xb2 = nullptr, *hb = nullptr, *hb2 = nullptr, *q = nullptr,
          *logits = nullptr;
    float *rope_cs = nullptr;  // (cos, sin) of the current position, head_size/2 pairs
    // token-loop state on the device
    DynState *dyn = nullptr;
    uint32_t *d_prompt = nullptr, *d_tokens = nullptr;  // seq_len entries each
    // the recorded step, one capture per bucket of positions (plan_bucket)
    hipGraph_t graph[kMaxPlanBuckets] = {};
    hipGraphExec_t graph_exec[kMaxPlanBuckets] = {};
    uint64_t graph_launches[kMaxPlanBuckets] = {};  // launches of the recorded step
    // kStepsPerGraph consecutive steps as one graph (the token loop replays it where that many
    // steps stay inside a bucket): a replay costs the host a call and the GPU a few microseconds
    // between two graphs, whatever the graph holds
    hipGraph_t graph_multi[kMaxPlanBuckets] = {};
    hipGraphExec_t graph_exec_multi[kMaxPlanBuckets] = {};
    int graph_fusion = -1;
    uint64_t graph_tuning = 0;  // the context's tuning generation the captures were made under
    // state of the batched prompt pass, allocated at its first use: one row per token
    // of a run (up to kPrefillMaxTokens)
    float *pf_x = nullptr, *pf_xb = nullptr, *pf_q = nullptr, *pf_hb = nullptr, *pf_hb2 = nullptr;
    uint32_t *pf_tokens = nullptr;
    std::vector<void *> allocs;
    uint64_t launches_last = 0;   // launches of the last step that ran
};

namespace {

int dev_alloc_bytes(wgml_llama2 *m, void **p, uint64_t bytes, bool zero) {
    void *d = nullptr;
    hipError_t e = hipMalloc(&d, bytes);
    if (e != hipSuccess)
        return set_error(WGML_E_OOM, "wgml_llama2: hipMalloc(%llu) failed: %s",
                         (unsigned long long)bytes, hipGetErrorString(e));
    m->allocs.push_back(d);
    if (zero) WGML_CHECK_HIP(hipMemsetAsync(d, 0, bytes, m->ctx->stream));
    *p = d;
    return WGML_OK;
}

int dev_alloc(wgml_llama2 *m, float **p, uint64_t n_floats, bool zero) {
    return dev_alloc_bytes(m, (void **)p, n_floats * 4, zero);
}

int check_ready(const wgml_llama2 *m) {
    for (size_t l = 0; l < m->layers.size(); ++l) {
        const LlamaLayer &w = m->layers[l];
        WGML_REQUIRE(w.attn_q && w.attn_k && w.attn_v && w.attn_output && w.ffn_gate && w.ffn_up &&
                         w.ffn_down && w.attn_norm && w.ffn_norm,
                     "wgml_llama2: layer %zu has unset weights", l);
    }
    WGML_REQUIRE(m->output && m->output_norm && m->token_embd,
                 "wgml_llama2: output / output_norm / token_embd not set");
    return WGML_OK;
}

void drop_graph(wgml_llama2 *m) {
    for (int b = 0; b < kMaxPlanBuckets; ++b) {
        if (m->graph_exec[b]) (void)hipGraphExecDestroy(m->graph_exec[b]);
        if (m->graph[b]) (void)hipGraphDestroy(m->graph[b]);
        m->graph_exec[b] = nullptr;
        m->graph[b] = nullptr;
        if (m->graph_exec_multi[b]) (void)hipGraphExecDestroy(m->graph_exec_multi[b]);
        if (m->graph_multi[b]) (void)hipGraphDestroy(m->graph_multi[b]);
        m->graph_exec_multi[b] = nullptr;
        m->graph_multi[b] = nullptr;
    }
    m->graph_fusion = -1;
}

// Enqueues one decode step (Llama2::dispatch, models/llama2/transformer.rs:298-431,
// preceded by the embedding copy of chat_llama2.rs:185-187).
//   dynamic == false: token/pos are the given host values;
//   dynamic == true : they are read from m->dyn on the device, the attention
//                     grid is planned for `plan_positions` positions (0: seq_len).
// fusion 0: one launch per reference op.  1: bias and residual adds folded into
// the GEMV epilogues.  2: additionally every RMSNorm folded into the staging of
// the GEMVs that consume it.
//   embed == false : m->x and the RoPE table already hold the token's embedding and the
//                     position's angles (the sampling launch of the step before wrote them).
int enqueue_step(wgml_llama2 *m, bool dynamic, uint32_t token, uint32_t pos,
                 uint32_t plan_positions = 0, bool embed = true) {
    const wgml_llama2_config &c = m->cfg;
    wgml_ctx *ctx = m->ctx;
    const uint32_t dim = c.dim, kv_dim = m->kv_dim;
    const DynPos dpos{dynamic ? &m->dyn->pos : nullptr, pos};
    const DynPos dtok{dynamic ? &m->dyn->token : nullptr, token};
    const int variant = m->model_type == WGML_MODEL_QWEN2 ? WGML_ROPE_NEOX : WGML_ROPE_ORIGINAL;
    const wgml_attn_params ap{c.seq_len, kv_dim, m->kv_mul, c.n_q_heads, m->head_size, pos};
    const int fusion = m->fusion;
    const uint32_t plan = dynamic ? (plan_positions ? plan_positions : c.seq_len) : pos + 1;

    // dim >= head_size / 2, so the embedding launch also covers the RoPE table
    if (embed)
        WGML_TRY(launch_embed(ctx, m->x, m->token_embd, dim, dtok, m->rope_cs, m->head_size,
                              c.rope_base_freq, dpos));

    for (uint32_t l = 0; l < c.n_layers; ++l) {
        const LlamaLayer &w = m->layers[l];
        const wgml_qmat *const qkv[3] = {w.attn_q, w.attn_k, w.attn_v};
        const wgml_qmat *const gate_up[2] = {w.ffn_gate, w.ffn_up};
        if (fusion >= 3 && gemv_fused_set_supported(ctx, qkv, 3) &&
            gemv_fused_set_supported(ctx, gate_up, 2) && w.ffn_gate->type == w.ffn_up->type) {
            // 5 launches per layer: [norm + Q,K,V + bias + RoPE + KV-cache write],
            // attention (+ merge), [Wo + residual], [norm + gate,up + SiLU], [down + residual]
            const bool rope_fused = variant == WGML_ROPE_ORIGINAL;
            FusedGemv f;
            f.njobs = 3;
            f.x = m->x;
            f.norm_w = w.attn_norm;
            f.norm_eps = c.rms_norm_eps;
            f.pos = dpos;
            f.head_size = m->head_size;
            f.rope_base = c.rope_base_freq;
            f.rope_cs = m->rope_cs;
            f.jobs[0].a = w.attn_q;
            f.jobs[0].out = m->q;
            f.jobs[0].bias = w.bq;
            f.jobs[0].mode = rope_fused ? FUSED_ROPE : FUSED_PLAIN;
            f.jobs[1].a = w.attn_k;
            f.jobs[1].out = w.key_cache;
            f.jobs[1].bias = w.bk;
            f.jobs[1].mode = rope_fused ? FUSED_ROPE : FUSED_PLAIN;
            f.jobs[1].out_pos_stride = kv_dim;
            f.jobs[2].a = w.attn_v;
            f.jobs[2].out = w.value_cache;
            f.jobs[2].bias = w.bv;
            f.jobs[2].out_pos_stride = kv_dim;
            WGML_TRY(launch_gemv_fused(ctx, f));
            if (!rope_fused)
                WGML_TRY(launch_rope(ctx, variant, m->head_size, kv_dim, dpos, c.rope_base_freq,
                                     m->q, dim, w.key_cache, kv_dim));
            // attention leaves its output as per-workgroup partial results where it can, and
            // the output projection merges them while it stages its input: no merge launch,
            // and no reason to hold short contexts to one workgroup per head
            AttnPartials parts;
            WGML_TRY(launch_attention_planned(ctx, ap, dpos, plan, ap.seq_len, m->q, w.key_cache,
                                              w.value_cache, nullptr, m->xb, nullptr, 0,
                                              gemv_partials_supported(ctx, w.attn_output) ? &parts
                                                                                          : nullptr));
            GemvEpilogue eacc;
            eacc.accumulate = 1;
            GemvEpilogue ewo = eacc;
            ewo.partials = parts;
            WGML_TRY(launch_gemv_quant(ctx, m->x, w.attn_output, m->xb, ewo));
            FusedGemv g;
            g.njobs = 1;
            g.x = m->x;
            g.norm_w = w.ffn_norm;
            g.norm_eps = c.rms_norm_eps;
            g.jobs[0].a = w.ffn_gate;
            g.jobs[0].b = w.ffn_up;
            g.jobs[0].out = m->hb;
            g.jobs[0].mode = FUSED_SILU;
            WGML_TRY(launch_gemv_fused(ctx, g));
            WGML_TRY(launch_gemv_quant(ctx, m->x, w.ffn_down, m->hb, eacc));
            continue;
        }
        // the KV-cache column of this position
        float *k_cache = w.key_cache, *v_cache = w.value_cache;
        GemvEpilogue eq, ek, ev;
        if (dynamic) {
            ek.dyn_pos = ev.dyn_pos = &m->dyn->pos;
            ek.out_pos_stride = ev.out_pos_stride = kv_dim;
        } else {
            k_cache += (size_t)pos * kv_dim;
            v_cache += (size_t)pos * kv_dim;
        }
        const float *qkv_in = m->xb;
        if (fusion >= 2) {
            qkv_in = m->x;
            eq.norm_w = ek.norm_w = ev.norm_w = w.attn_norm;
            eq.norm_eps = ek.norm_eps = ev.norm_eps = c.rms_norm_eps;
        } else {
            WGML_TRY(launch_rms_norm(ctx, c.rms_norm_eps, m->xb, m->x, w.attn_norm, dim));
        }
        // recorded steps always add the biases in the epilogue: a separate add would
        // need the position-dependent cache column as its destination
        const bool bias_in_epilogue = fusion >= 1 || dynamic;
        if (bias_in_epilogue) {
            eq.bias = w.bq;
            ek.bias = w.bk;
            ev.bias = w.bv;
        }
        WGML_TRY(launch_gemv_quant(ctx, m->q, w.attn_q, qkv_in, eq));
        WGML_TRY(launch_gemv_quant(ctx, k_cache, w.attn_k, qkv_in, ek));
        WGML_TRY(launch_gemv_quant(ctx, v_cache, w.attn_v, qkv_in, ev));
        if (!bias_in_epilogue) {
            if (w.bq) WGML_TRY(launch_op_assign(ctx, WGML_ASSIGN_ADD, m->q, w.bq, dim));
            if (w.bk) WGML_TRY(launch_op_assign(ctx, WGML_ASSIGN_ADD, k_cache, w.bk, kv_dim));
            if (w.bv) WGML_TRY(launch_op_assign(ctx, WGML_ASSIGN_ADD, v_cache, w.bv, kv_dim));
        }
        WGML_TRY(launch_rope(ctx, variant, m->head_size, kv_dim, dpos, c.rope_base_freq, m->q, dim,
                             dynamic ? w.key_cache : k_cache, dynamic ? kv_dim : 0));
        WGML_TRY(launch_attention_planned(ctx, ap, dpos, plan, ap.seq_len, m->q, w.key_cache, w.value_cache,
                                          nullptr, m->xb));
        if (fusion >= 1) {
            // x += Wo * xb in the GEMV epilogue
            GemvEpilogue e;
            e.accumulate = 1;
            WGML_TRY(launch_gemv_quant(ctx, m->x, w.attn_output, m->xb, e));
        } else {
            WGML_TRY(launch_gemv_quant(ctx, m->xb2, w.attn_output, m->xb, GemvEpilogue{}));
            WGML_TRY(launch_op_assign(ctx, WGML_ASSIGN_ADD, m->x, m->xb2, dim));
        }
        GemvEpilogue eg;
        const float *ffn_in = m->xb;
        if (fusion >= 2) {
            ffn_in = m->x;
            eg.norm_w = w.ffn_norm;
            eg.norm_eps = c.rms_norm_eps;
        } else {
            WGML_TRY(launch_rms_norm(ctx, c.rms_norm_eps, m->xb, m->x, w.ffn_norm, dim));
        }
        WGML_TRY(launch_gemv_quant(ctx, m->hb, w.ffn_gate, ffn_in, eg));
        WGML_TRY(launch_gemv_quant(ctx, m->hb2, w.ffn_up, ffn_in, eg));
        WGML_TRY(launch_silu(ctx, m->hb, m->hb2, c.hidden_dim));
        if (fusion >= 1) {
            GemvEpilogue e;
            e.accumulate = 1;
            WGML_TRY(launch_gemv_quant(ctx, m->x, w.ffn_down, m->hb, e));
        } else {
            WGML_TRY(launch_gemv_quant(ctx, m->xb2, w.ffn_down, m->hb, GemvEpilogue{}));
            WGML_TRY(launch_op_assign(ctx, WGML_ASSIGN_ADD, m->x, m->xb2, dim));
        }
    }
    GemvEpilogue eo;
    const float *out_in = m->xb;
    if (fusion >= 2) {
        out_in = m->x;
        eo.norm_w = m->output_norm;
        eo.norm_eps = c.rms_norm_eps;
    } else {
        WGML_TRY(launch_rms_norm(ctx, c.rms_norm_eps, m->xb, m->x, m->output_norm, dim));
    }
    WGML_TRY(launch_gemv_quant(ctx, m->logits, m->output, out_in, eo));
    return WGML_OK;
}

// The attention workspace for the largest plan of any bucket (recorded launches hold its
// address, so it must not grow between captures).
int reserve_all_plans(wgml_llama2 *m) {
    const wgml_llama2_config &c = m->cfg;
    const wgml_attn_params ap{c.seq_len, m->kv_dim, m->kv_mul, c.n_q_heads, m->head_size, 0};
    for (uint32_t pos = 0;;) {
        const uint32_t limit = plan_bucket(pos, c.seq_len, nullptr);
        WGML_TRY(reserve_attention_workspace(m->ctx, ap, limit));
        if (limit >= c.seq_len) break;
        pos = limit;
    }
    return WGML_OK;
}

constexpr uint32_t kStepsPerGraph = 8;

// A step of the token loops that keep their state on the device: the layers and the output
// projection, then the launch that samples (arg-max), does the loop's bookkeeping and writes the
// embedding and the RoPE table of the token and position it has chosen, for the step that follows.
// The loop's first step finds them written by loop_first_embed.
int enqueue_loop_step(wgml_llama2 *m, uint32_t plan) {
    const wgml_llama2_config &c = m->cfg;
    WGML_TRY(enqueue_step(m, true, 0, 0, plan, false));
    const NextEmbed ne{m->x, m->token_embd, c.dim, m->rope_cs, m->head_size, c.rope_base_freq, nullptr, 0};
    return launch_argmax_next(m->ctx, m->logits, c.vocab_size, m->dyn, m->d_prompt, m->d_tokens, &ne);
}
int loop_first_embed(wgml_llama2 *m) {
    const wgml_llama2_config &c = m->cfg;
    return launch_embed(m->ctx, m->x, m->token_embd, c.dim, DynPos{&m->dyn->token, 0}, m->rope_cs,
                        m->head_size, c.rope_base_freq, DynPos{&m->dyn->pos, 0});
}

// Records `steps` consecutive steps (each followed by greedy sampling and the loop's
// bookkeeping, all on the device) into one HIP graph.
int capture_steps(wgml_llama2 *m, uint32_t plan, uint32_t steps, hipGraph_t *graph,
                  hipGraphExec_t *exec, uint64_t *launches_per_step) {
    wgml_ctx *ctx = m->ctx;
    const wgml_llama2_config &c = m->cfg;
    WGML_CHECK_HIP(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    const uint64_t launches0 = ctx->launches;
    int rc = WGML_OK;
    for (uint32_t k = 0; k < steps && rc == WGML_OK; ++k) rc = enqueue_loop_step(m, plan);
    if (launches_per_step) *launches_per_step = (ctx->launches - launches0) / steps;
    hipError_t e = hipStreamEndCapture(ctx->stream, graph);
    if (rc != WGML_OK) return rc;
    if (e != hipSuccess)
        return set_error(WGML_E_HIP, "wgml_llama2: graph capture failed: %s", hipGetErrorString(e));
    e = hipGraphInstantiate(exec, *graph, nullptr, nullptr, 0);
    if (e != hipSuccess)
        return set_error(WGML_E_HIP, "wgml_llama2: graph instantiate failed: %s",
                         hipGetErrorString(e));
    if (steps > 1) {
        // A graph's first replay costs milliseconds (2.2 ms for the eight steps of the 7B
        // shape; uploading the graph ahead of time does not remove it): do it here, from
        // position 0, with the cache rows it writes saved and put back.
        const size_t bytes = (size_t)steps * m->kv_dim * 4;
        void *saved = nullptr;
        WGML_CHECK_HIP(hipMalloc(&saved, bytes * 2 * c.n_layers));
        for (uint32_t l = 0; l < c.n_layers; ++l) {
            (void)hipMemcpyAsync((char *)saved + bytes * (2 * l), m->layers[l].key_cache, bytes,
                                 hipMemcpyDeviceToDevice, ctx->stream);
            (void)hipMemcpyAsync((char *)saved + bytes * (2 * l + 1), m->layers[l].value_cache, bytes,
                                 hipMemcpyDeviceToDevice, ctx->stream);
        }
        const DynState init{0, 0, 0, 0};
        e = hipMemcpyAsync(m->dyn, &init, sizeof(init), hipMemcpyHostToDevice, ctx->stream);
        if (e == hipSuccess && loop_first_embed(m) != WGML_OK) e = hipErrorUnknown;
        if (e == hipSuccess) e = hipGraphLaunch(*exec, ctx->stream);
        for (uint32_t l = 0; l < c.n_layers; ++l) {
            (void)hipMemcpyAsync(m->layers[l].key_cache, (char *)saved + bytes * (2 * l), bytes,
                                 hipMemcpyDeviceToDevice, ctx->stream);
            (void)hipMemcpyAsync(m->layers[l].value_cache, (char *)saved + bytes * (2 * l + 1), bytes,
                                 hipMemcpyDeviceToDevice, ctx->stream);
        }
        const hipError_t es = hipStreamSynchronize(ctx->stream);  // `init` is a stack object
        (void)hipFree(saved);
        if (e == hipSuccess) e = es;
        if (e != hipSuccess)
            return set_error(WGML_E_HIP, "wgml_llama2: first replay failed: %s", hipGetErrorString(e));
    }
    return WGML_OK;
}

// Records one step (+ greedy sampling and bookkeeping) into a HIP graph, for the bucket of
// positions that `pos` lies in, and the graph of kStepsPerGraph such steps where the bucket
// holds that many positions (both at once, so that a short first run leaves nothing to build
// for a longer one).
int build_graph(wgml_llama2 *m, uint32_t pos) {
    wgml_ctx *ctx = m->ctx;
    const wgml_llama2_config &c = m->cfg;
    // captures made at another fusion level or under other launch-shape overrides are stale
    if (m->graph_fusion != m->fusion || m->graph_tuning != ctx->tuning_generation) drop_graph(m);
    int b = 0;
    const uint32_t plan = plan_bucket(pos, c.seq_len, &b);
    // the bucket's positions are [256 << (b - 1), plan), from 0 for the first bucket
    const bool multi = plan - (b == 0 ? 0u : 256u << (b - 1)) >= kStepsPerGraph;
    if (m->graph_exec[b]) {
        if (multi && !m->graph_exec_multi[b]) {
            const int rc = capture_steps(m, plan, kStepsPerGraph, &m->graph_multi[b],
                                         &m->graph_exec_multi[b], nullptr);
            if (rc != WGML_OK) drop_graph(m);
            return rc;
        }
        return WGML_OK;
    }
    // Everything that allocates or sets function attributes happens before capture:
    // the attention workspace for the largest plan, and one eager step.
    WGML_TRY(reserve_all_plans(m));
    // The eager step runs at position 0 and would overwrite that column of every KV
    // cache (the caller may have filled it): keep a copy and put it back.
    const size_t col = (size_t)m->kv_dim * 4;
    void *saved = nullptr;
    WGML_CHECK_HIP(hipMalloc(&saved, col * 2 * c.n_layers));
    for (uint32_t l = 0; l < c.n_layers; ++l) {
        (void)hipMemcpyAsync((char *)saved + col * (2 * l), m->layers[l].key_cache, col,
                             hipMemcpyDeviceToDevice, ctx->stream);
        (void)hipMemcpyAsync((char *)saved + col * (2 * l + 1), m->layers[l].value_cache, col,
                             hipMemcpyDeviceToDevice, ctx->stream);
    }
    const DynState init{0, 0, 0, 0};
    hipError_t ew = hipMemcpyAsync(m->dyn, &init, sizeof(init), hipMemcpyHostToDevice, ctx->stream);
    int rcw = ew == hipSuccess ? loop_first_embed(m) : WGML_E_HIP;
    if (rcw == WGML_OK) rcw = enqueue_loop_step(m, plan);
    for (uint32_t l = 0; l < c.n_layers; ++l) {
        (void)hipMemcpyAsync(m->layers[l].key_cache, (char *)saved + col * (2 * l), col,
                             hipMemcpyDeviceToDevice, ctx->stream);
        (void)hipMemcpyAsync(m->layers[l].value_cache, (char *)saved + col * (2 * l + 1), col,
                             hipMemcpyDeviceToDevice, ctx->stream);
    }
    ew = hipStreamSynchronize(ctx->stream);
    (void)hipFree(saved);
    if (rcw != WGML_OK) return rcw;
    if (ew != hipSuccess)
        return set_error(WGML_E_HIP, "wgml_llama2: warm-up step failed: %s", hipGetErrorString(ew));

    int rc = capture_steps(m, plan, 1, &m->graph[b], &m->graph_exec[b], &m->graph_launches[b]);
    if (rc == WGML_OK && multi)
        rc = capture_steps(m, plan, kStepsPerGraph, &m->graph_multi[b], &m->graph_exec_multi[b], nullptr);
    if (rc != WGML_OK) {
        drop_graph(m);
        return rc;
    }
    m->graph_fusion = m->fusion;
    m->graph_tuning = ctx->tuning_generation;
    return WGML_OK;
}

// The recorded steps of every bucket that a run of n_steps from start_pos passes through,
// before its first launch.
int record_steps(wgml_llama2 *m, uint32_t start_pos, uint32_t n_steps) {
    if (graphs_disabled()) return reserve_all_plans(m);
    for (uint32_t pos = start_pos; n_steps > 0;) {
        const uint32_t limit = plan_bucket(pos, m->cfg.seq_len, nullptr);
        WGML_TRY(build_graph(m, pos));
        if (limit >= start_pos + n_steps || limit >= m->cfg.seq_len) break;
        pos = limit;
    }
    return WGML_OK;
}

// Runs n_steps recorded steps from (first_token, start_pos); prompt tokens (if
// any) are forced.  One synchronisation at the end.
int run_recorded(wgml_llama2 *m, uint32_t first_token, uint32_t start_pos, uint32_t n_steps,
                 const uint32_t *prompt, uint32_t n_prompt, uint32_t *out_tokens) {
    wgml_ctx *ctx = m->ctx;
    WGML_TRY(check_ready(m));
    const bool use_graph = !graphs_disabled();
    WGML_TRY(record_steps(m, start_pos, n_steps));
    if (n_prompt)
        WGML_CHECK_HIP(hipMemcpyAsync(m->d_prompt, prompt, (size_t)n_prompt * 4,
                                      hipMemcpyHostToDevice, ctx->stream));
    const DynState init{start_pos, first_token, 0, n_prompt};
    WGML_CHECK_HIP(hipMemcpyAsync(m->dyn, &init, sizeof(init), hipMemcpyHostToDevice, ctx->stream));
    WGML_CHECK_HIP(hipStreamSynchronize(ctx->stream));  // `init` is a stack object
    uint64_t launches0 = ctx->launches;
    WGML_TRY(loop_first_embed(m));
    for (uint32_t i = 0; i < n_steps; ++i) {
        int b = 0;
        const uint32_t plan = plan_bucket(start_pos + i, m->cfg.seq_len, &b);
        if (use_graph) {
            // steps left in this run that stay inside the bucket (positions below `plan`;
            // the last bucket also takes what lies beyond, as single steps do)
            const uint32_t in_bucket = plan > start_pos + i ? plan - (start_pos + i) : 1;
            if (m->graph_exec_multi[b] && n_steps - i >= kStepsPerGraph && in_bucket >= kStepsPerGraph) {
                WGML_CHECK_HIP(hipGraphLaunch(m->graph_exec_multi[b], ctx->stream));
                i += kStepsPerGraph - 1;
            } else {
                WGML_CHECK_HIP(hipGraphLaunch(m->graph_exec[b], ctx->stream));
            }
            m->launches_last = m->graph_launches[b];
        } else {
            // the same launches, enqueued one by one (no host synchronisation either)
            launches0 = ctx->launches;
            WGML_TRY(enqueue_loop_step(m, plan));
            m->launches_last = ctx->launches - launches0;
        }
    }
    WGML_CHECK_HIP(hipMemcpyAsync(out_tokens, m->d_tokens, (size_t)n_steps * 4,
                                  hipMemcpyDeviceToHost, ctx->stream));
    WGML_CHECK_HIP(hipStreamSynchronize(ctx->stream));
    return WGML_OK;
}

// The batched products take these formats, and weights that fit their f16 operands.
bool gemm_supported(const wgml_qmat *q) {
    return gemv_fused_supported(q) && q->max_abs <= kGemmMaxWeight;  // the nine quantized formats
}

// One run of T <= kPrefillMaxTokens prompt tokens at positions pos0 .. pos0 + T - 1: the
// launches of enqueue_step with every matrix-vector product replaced by a product
// with the T vectors at once.  Leaves the last token's residual stream in m->x.
int enqueue_prefill_run(wgml_llama2 *m, const uint32_t *tokens, uint32_t T, uint32_t pos0) {
    const wgml_llama2_config &c = m->cfg;
    wgml_ctx *ctx = m->ctx;
    const uint32_t dim = c.dim, kv_dim = m->kv_dim, hidden = c.hidden_dim;
    const int variant = m->model_type == WGML_MODEL_QWEN2 ? WGML_ROPE_NEOX : WGML_ROPE_ORIGINAL;
    const wgml_attn_params ap{c.seq_len, kv_dim, m->kv_mul, c.n_q_heads, m->head_size, pos0};
    void *xh = ctx->prefill_xh;
    float *xs = ctx->prefill_xscale;

    // the caller's token array may be reused as soon as this returns
    WGML_CHECK_HIP(hipMemcpyAsync(m->pf_tokens, tokens, (size_t)T * 4, hipMemcpyHostToDevice,
                                  ctx->stream));
    WGML_CHECK_HIP(hipStreamSynchronize(ctx->stream));
    WGML_TRY(launch_embed_rows(ctx, m->pf_x, m->token_embd, m->pf_tokens, dim, T));
    for (uint32_t l = 0; l < c.n_layers; ++l) {
        const LlamaLayer &w = m->layers[l];
        float *kc = w.key_cache + (size_t)pos0 * kv_dim, *vc = w.value_cache + (size_t)pos0 * kv_dim;
        WGML_TRY(launch_prefill_prep(ctx, m->pf_x, dim, nullptr, w.attn_norm, c.rms_norm_eps, xh, xs,
                                     dim, T));
        // Q, K and V in as few launches as their formats allow (one launch takes matrices
        // of one format); K and V go straight to their cache rows.  Q and K are rotated by the
        // kernel that adds up the partial sums of their launch where there is one, by a launch
        // of their own otherwise.
        bool roped[3] = {false, false, true};
        {
            GemmTarget tq{w.attn_q, m->pf_q, dim, w.bq}, tk{w.attn_k, kc, kv_dim, w.bk},
                tv{w.attn_v, vc, kv_dim, w.bv};
            tq.rope = tk.rope = true;
            GemmTarget group[3] = {tq, tk, tv};
            bool done[3] = {false, false, false};
            for (int i = 0; i < 3; ++i) {
                if (done[i]) continue;
                GemmTarget launch[3];
                int n = 0, members[3];
                for (int k = i; k < 3; ++k) {
                    if (!done[k] && group[k].m->type == group[i].m->type) {
                        members[n] = k;
                        launch[n++] = group[k];
                        done[k] = true;
                    }
                }
                GemmRope rope{variant, m->head_size, pos0, c.rope_base_freq, false};
                WGML_TRY(launch_gemm_quant_multi(ctx, launch, n, xh, xs, T, 0, false, &rope));
                for (int k = 0; k < n; ++k) roped[members[k]] = roped[members[k]] || rope.applied;
            }
        }
        if (!roped[0] || !roped[1])
            WGML_TRY(launch_rope_rows(ctx, variant, m->head_size, kv_dim, pos0, c.rope_base_freq,
                                      roped[0] ? nullptr : m->pf_q, dim, dim, roped[1] ? nullptr : kc, kv_dim, T));
        WGML_TRY(launch_attention_rows(ctx, ap, pos0, T, m->pf_q, dim, w.key_cache, w.value_cache,
                                       m->pf_xb, dim));
        WGML_TRY(launch_prefill_prep(ctx, m->pf_xb, dim, nullptr, nullptr, 0.f, xh, xs, dim, T));
        WGML_TRY(launch_gemm_quant(ctx, m->pf_x, dim, w.attn_output, xh, xs, T, nullptr, 1, true));
        WGML_TRY(launch_prefill_prep(ctx, m->pf_x, dim, nullptr, w.ffn_norm, c.rms_norm_eps, xh, xs,
                                     dim, T));
        if (w.ffn_gate->type == w.ffn_up->type) {
            const GemmTarget gu[2] = {{w.ffn_gate, m->pf_hb, hidden, nullptr},
                                      {w.ffn_up, m->pf_hb2, hidden, nullptr}};
            WGML_TRY(launch_gemm_quant_multi(ctx, gu, 2, xh, xs, T, 0, true));
        } else {
            WGML_TRY(launch_gemm_quant(ctx, m->pf_hb, hidden, w.ffn_gate, xh, xs, T, nullptr, 0));
            WGML_TRY(launch_gemm_quant(ctx, m->pf_hb2, hidden, w.ffn_up, xh, xs, T, nullptr, 0));
        }
        WGML_TRY(launch_prefill_prep(ctx, m->pf_hb, hidden, m->pf_hb2, nullptr, 0.f, xh, xs, hidden,
                                     T));
        WGML_TRY(launch_gemm_quant(ctx, m->pf_x, dim, w.ffn_down, xh, xs, T, nullptr, 1, true));
    }
    WGML_TRY(launch_gemm_flush(ctx, m->pf_x, dim, xs, dim, T));  // the last layer's down projection
    WGML_CHECK_HIP(hipMemcpyAsync(m->x, m->pf_x + (size_t)(T - 1) * dim, (size_t)dim * 4,
                                  hipMemcpyDeviceToDevice, ctx->stream));
    return WGML_OK;
}

}  // namespace

extern "C" {

int wgml_llama2_create(wgml_ctx *ctx, const wgml_llama2_config *cfg, int model_type,
                       wgml_llama2 **out) {
    WGML_REQUIRE(ctx && cfg && out, "wgml_llama2_create: null argument");
    *out = nullptr;
    WGML_REQUIRE(model_type == WGML_MODEL_LLAMA || model_type == WGML_MODEL_QWEN2,
                 "wgml_llama2_create: unknown model type %d", model_type);
    WGML_REQUIRE(cfg->dim && cfg->hidden_dim && cfg->n_layers && cfg->n_q_heads &&
                     cfg->n_kv_heads && cfg->vocab_size && cfg->seq_len,
                 "wgml_llama2_create: zero field in config");
    WGML_REQUIRE(cfg->dim % cfg->n_q_heads == 0 && cfg->n_q_heads % cfg->n_kv_heads == 0,
                 "wgml_llama2_create: dim %u / heads %u / kv heads %u do not divide", cfg->dim,
                 cfg->n_q_heads, cfg->n_kv_heads);
    WGML_REQUIRE(cfg->dim % 4 == 0 && cfg->hidden_dim % 4 == 0,
                 "wgml_llama2_create: dim and hidden_dim must be multiples of 4");
    const uint32_t head_size = cfg->dim / cfg->n_q_heads;
    if (head_size % 2 != 0 || head_size > 256)
        return set_error(WGML_E_UNSUPPORTED, "wgml_llama2_create: head_size %u unsupported",
                         head_size);
    wgml_llama2 *m = new wgml_llama2();
    m->ctx = ctx;
    ctx_retain(ctx);
    m->cfg = *cfg;
    m->model_type = model_type;
    // Llama2Config::derived_configs (models/llama2/cpu.rs:111-141)
    m->kv_dim = cfg->dim * cfg->n_kv_heads / cfg->n_q_heads;
    m->head_size = head_size;
    m->kv_mul = cfg->n_q_heads / cfg->n_kv_heads;
    m->layers.resize(cfg->n_layers);
    int rc = WGML_OK;
    auto A = [&](float **p, uint64_t n, bool z) {
        if (rc == WGML_OK) rc = dev_alloc(m, p, n, z);
    };
    A(&m->x, cfg->dim, true);
    A(&m->xb, cfg->dim, true);
    A(&m->xb2, cfg->dim, true);
    A(&m->hb, cfg->hidden_dim, true);
    A(&m->hb2, cfg->hidden_dim, true);
    A(&m->q, cfg->dim, true);
    A(&m->logits, cfg->vocab_size, true);
    A(&m->rope_cs, head_size, true);
    for (auto &l : m->layers) {
        A(&l.key_cache, (uint64_t)m->kv_dim * cfg->seq_len, true);
        A(&l.value_cache, (uint64_t)m->kv_dim * cfg->seq_len, true);
    }
    if (rc == WGML_OK) rc = dev_alloc_bytes(m, (void **)&m->dyn, 256, true);
    if (rc == WGML_OK) rc = dev_alloc_bytes(m, (void **)&m->d_prompt, (uint64_t)cfg->seq_len * 4, true);
    if (rc == WGML_OK) rc = dev_alloc_bytes(m, (void **)&m->d_tokens, (uint64_t)cfg->seq_len * 4, true);
    if (rc == WGML_OK && hipStreamSynchronize(ctx->stream) != hipSuccess)
        rc = set_error(WGML_E_HIP, "wgml_llama2_create: synchronize failed");
    if (rc != WGML_OK) {
        wgml_llama2_destroy(m);
        return rc;
    }
    *out = m;
    return WGML_OK;
}

int wgml_llama2_destroy(wgml_llama2 *m) {
    if (!m) return WGML_OK;
    if (m->ctx && m->ctx->stream) (void)hipStreamSynchronize(m->ctx->stream);
    drop_graph(m);
    for (void *p : m->allocs) (void)hipFree(p);
    ctx_release(m->ctx);
    delete m;
    return WGML_OK;
}

int wgml_llama2_set_matrix(wgml_llama2 *m, int which, uint32_t layer, const wgml_qmat *mat) {
    WGML_REQUIRE(m && mat, "wgml_llama2_set_matrix: null argument");
    const wgml_llama2_config &c = m->cfg;
    uint32_t er = 0, ec = 0;
    switch (which) {  // shapes: models/llama2/transformer.rs:174-213,244-257
    case WGML_LLAMA2_ATTN_Q:
    case WGML_LLAMA2_ATTN_OUTPUT: er = c.dim; ec = c.dim; break;
    case WGML_LLAMA2_ATTN_K:
    case WGML_LLAMA2_ATTN_V: er = m->kv_dim; ec = c.dim; break;
    case WGML_LLAMA2_FFN_GATE:
    case WGML_LLAMA2_FFN_UP: er = c.hidden_dim; ec = c.dim; break;
    case WGML_LLAMA2_FFN_DOWN: er = c.dim; ec = c.hidden_dim; break;
    case WGML_LLAMA2_OUTPUT: er = c.vocab_size; ec = c.dim; break;
    default: return set_error(WGML_E_INVALID, "wgml_llama2_set_matrix: unknown matrix %d", which);
    }
    WGML_REQUIRE(mat->nrows == er && mat->ncols == ec,
                 "wgml_llama2_set_matrix: matrix %d is %ux%u, expected %ux%u", which, mat->nrows,
                 mat->ncols, er, ec);
    drop_graph(m);  // recorded launches hold the old pointers
    if (which == WGML_LLAMA2_OUTPUT) {
        m->output = mat;
        return WGML_OK;
    }
    WGML_REQUIRE(layer < c.n_layers, "wgml_llama2_set_matrix: layer %u of %u", layer, c.n_layers);
    LlamaLayer &l = m->layers[layer];
    switch (which) {
    case WGML_LLAMA2_ATTN_Q: l.attn_q = mat; break;
    case WGML_LLAMA2_ATTN_K: l.attn_k = mat; break;
    case WGML_LLAMA2_ATTN_V: l.attn_v = mat; break;
    case WGML_LLAMA2_ATTN_OUTPUT: l.attn_output = mat; break;
    case WGML_LLAMA2_FFN_GATE: l.ffn_gate = mat; break;
    case WGML_LLAMA2_FFN_UP: l.ffn_up = mat; break;
    case WGML_LLAMA2_FFN_DOWN: l.ffn_down = mat; break;
    }
    return WGML_OK;
}

int wgml_llama2_set_vector(wgml_llama2 *m, int which, uint32_t layer, const float *host,
                           uint32_t len) {
    WGML_REQUIRE(m && host, "wgml_llama2_set_vector: null argument");
    const wgml_llama2_config &c = m->cfg;
    uint32_t expect = 0;
    float **slot = nullptr;
    if (which == WGML_LLAMA2_OUTPUT_NORM) {
        expect = c.dim;
        slot = &m->output_norm;
    } else {
        WGML_REQUIRE(layer < c.n_layers, "wgml_llama2_set_vector: layer %u of %u", layer,
                     c.n_layers);
        LlamaLayer &l = m->layers[layer];
        switch (which) {
        case WGML_LLAMA2_ATTN_NORM: expect = c.dim; slot = &l.attn_norm; break;
        case WGML_LLAMA2_FFN_NORM: expect = c.dim; slot = &l.ffn_norm; break;
        case WGML_LLAMA2_ATTN_Q_BIAS: expect = c.dim; slot = &l.bq; break;
        case WGML_LLAMA2_ATTN_K_BIAS: expect = m->kv_dim; slot = &l.bk; break;
        case WGML_LLAMA2_ATTN_V_BIAS: expect = m->kv_dim; slot = &l.bv; break;
        default:
            return set_error(WGML_E_INVALID, "wgml_llama2_set_vector: unknown vector %d", which);
        }
    }
    WGML_REQUIRE(len == expect, "wgml_llama2_set_vector: vector %d has %u elements, expected %u",
                 which, len, expect);
    if (!*slot) {
        WGML_TRY(dev_alloc(m, slot, len, false));
        drop_graph(m);
    }
    WGML_CHECK_HIP(hipMemcpyAsync(*slot, host, (size_t)len * 4, hipMemcpyHostToDevice,
                                  m->ctx->stream));
    WGML_CHECK_HIP(hipStreamSynchronize(m->ctx->stream));
    return WGML_OK;
}

int wgml_llama2_set_token_embd(wgml_llama2 *m, const float *host) {
    WGML_REQUIRE(m && host, "wgml_llama2_set_token_embd: null argument");
    const uint64_t n = (uint64_t)m->cfg.dim * m->cfg.vocab_size;
    if (!m->token_embd) {
        WGML_TRY(dev_alloc(m, &m->token_embd, n, false));
        drop_graph(m);
    }
    WGML_CHECK_HIP(hipMemcpyAsync(m->token_embd, host, n * 4, hipMemcpyHostToDevice,
                                  m->ctx->stream));
    WGML_CHECK_HIP(hipStreamSynchronize(m->ctx->stream));
    return WGML_OK;
}

int wgml_llama2_set_fusion(wgml_llama2 *m, int level) {
    WGML_REQUIRE(m != nullptr, "wgml_llama2_set_fusion: null model");
    WGML_REQUIRE(level >= 0 && level <= 3, "wgml_llama2_set_fusion: level %d not in 0..3", level);
    m->fusion = level;
    return WGML_OK;
}

int wgml_llama2_launches_per_token(const wgml_llama2 *m) {
    return m ? (int)m->launches_last : 0;
}

int wgml_llama2_forward(wgml_llama2 *m, uint32_t token, uint32_t pos) {
    WGML_REQUIRE(m != nullptr, "wgml_llama2_forward: null model");
    WGML_TRY(check_ready(m));
    const wgml_llama2_config &c = m->cfg;
    WGML_REQUIRE(token < c.vocab_size, "wgml_llama2_forward: token %u outside vocabulary %u", token,
                 c.vocab_size);
    WGML_REQUIRE(pos < c.seq_len, "wgml_llama2_forward: pos %u outside seq_len %u", pos, c.seq_len);
    const uint64_t launches0 = m->ctx->launches;
    WGML_TRY(enqueue_step(m, false, token, pos));
    m->launches_last = m->ctx->launches - launches0;
    return WGML_OK;
}

int wgml_llama2_prefill(wgml_llama2 *m, const uint32_t *tokens, uint32_t n_tokens,
                        uint32_t start_pos) {
    WGML_REQUIRE(m && tokens, "wgml_llama2_prefill: null argument");
    WGML_TRY(check_ready(m));
    const wgml_llama2_config &c = m->cfg;
    WGML_REQUIRE(n_tokens >= 1, "wgml_llama2_prefill: empty prompt");
    WGML_REQUIRE((uint64_t)start_pos + n_tokens <= c.seq_len,
                 "wgml_llama2_prefill: %u tokens from position %u exceed seq_len %u", n_tokens,
                 start_pos, c.seq_len);
    for (uint32_t i = 0; i < n_tokens; ++i)
        WGML_REQUIRE(tokens[i] < c.vocab_size,
                     "wgml_llama2_prefill: token %u outside vocabulary %u", tokens[i], c.vocab_size);
    wgml_ctx *ctx = m->ctx;
    bool batched = true;
    for (const LlamaLayer &w : m->layers)
        for (const wgml_qmat *q : {w.attn_q, w.attn_k, w.attn_v, w.attn_output, w.ffn_gate, w.ffn_up,
                                   w.ffn_down})
            if (!gemm_supported(q)) batched = false;
    if (!batched) {
        // The batched products exist for the quantized formats, with weights of at most
        // 255.875 in magnitude.  A model with any other matrix takes the prompt the way the reference does: one step per token
        // (chat_llama2.rs:155-228), which leaves the same state.
        const uint64_t launches0 = ctx->launches;
        for (uint32_t i = 0; i < n_tokens; ++i) WGML_TRY(enqueue_step(m, false, tokens[i], start_pos + i));
        m->launches_last = ctx->launches - launches0;
        return WGML_OK;
    }
    if (!m->pf_x) {
        int rc = WGML_OK;
        auto A = [&](float **p, uint64_t n) {
            if (rc == WGML_OK) rc = dev_alloc(m, p, n, false);
        };
        A(&m->pf_xb, (uint64_t)kPrefillMaxTokens * c.dim);
        A(&m->pf_q, (uint64_t)kPrefillMaxTokens * c.dim);
        A(&m->pf_hb, (uint64_t)kPrefillMaxTokens * c.hidden_dim);
        A(&m->pf_hb2, (uint64_t)kPrefillMaxTokens * c.hidden_dim);
        if (rc == WGML_OK) rc = dev_alloc_bytes(m, (void **)&m->pf_tokens, kPrefillMaxTokens * 4, false);
        A(&m->pf_x, (uint64_t)kPrefillMaxTokens * c.dim);  // last: marks the set as complete
        WGML_TRY(rc);
    }
    const uint32_t kmax = c.dim > c.hidden_dim ? c.dim : c.hidden_dim;
    WGML_TRY(ensure_prefill_scratch(ctx, (size_t)kPrefillMaxTokens * prefill_kpad(kmax) * 2));
    const uint64_t launches0 = ctx->launches;
    ctx->gemm_pending_ks = 0;  // nothing is owed from an earlier call that failed half way
    ctx->gemm_pending_pair = 0;
    for (uint32_t done = 0; done < n_tokens; done += kPrefillMaxTokens) {
        const uint32_t T = n_tokens - done < kPrefillMaxTokens ? n_tokens - done : kPrefillMaxTokens;
        WGML_TRY(enqueue_prefill_run(m, tokens + done, T, start_pos + done));
    }
    // logits of the last token, as a decode step ends (final norm folded into the product)
    GemvEpilogue eo;
    eo.norm_w = m->output_norm;
    eo.norm_eps = c.rms_norm_eps;
    WGML_TRY(launch_gemv_quant(ctx, m->logits, m->output, m->x, eo));
    m->launches_last = ctx->launches - launches0;
    return WGML_OK;
}

int wgml_llama2_prefill_decode_greedy(wgml_llama2 *m, const uint32_t *prompt, uint32_t n_prompt,
                                      uint32_t n_new, uint32_t *out_tokens) {
    WGML_REQUIRE(m && prompt && out_tokens, "wgml_llama2_prefill_decode_greedy: null argument");
    WGML_REQUIRE((uint64_t)n_prompt + n_new <= (uint64_t)m->cfg.seq_len + 1,
                 "wgml_llama2_prefill_decode_greedy: %u + %u positions exceed seq_len %u", n_prompt,
                 n_new, m->cfg.seq_len);
    WGML_TRY(wgml_llama2_prefill(m, prompt, n_prompt, 0));
    if (n_new == 0) return WGML_OK;
    wgml_ctx *ctx = m->ctx;
    WGML_TRY(launch_argmax(ctx, m->logits, m->cfg.vocab_size, ctx->d_scalar));
    WGML_CHECK_HIP(hipMemcpyAsync(ctx->h_scalar, ctx->d_scalar, 4, hipMemcpyDeviceToHost, ctx->stream));
    WGML_CHECK_HIP(hipStreamSynchronize(ctx->stream));
    out_tokens[0] = ctx->h_scalar[0];
    if (n_new == 1) return WGML_OK;
    return run_recorded(m, out_tokens[0], n_prompt, n_new - 1, nullptr, 0, out_tokens + 1);
}

int wgml_llama2_read_logits(wgml_llama2 *m, float *host_out) {
    WGML_REQUIRE(m && host_out, "wgml_llama2_read_logits: null argument");
    WGML_CHECK_HIP(hipMemcpyAsync(host_out, m->logits, (size_t)m->cfg.vocab_size * 4,
                                  hipMemcpyDeviceToHost, m->ctx->stream));
    WGML_CHECK_HIP(hipStreamSynchronize(m->ctx->stream));
    return WGML_OK;
}

int wgml_llama2_decode_greedy(wgml_llama2 *m, uint32_t first_token, uint32_t start_pos,
                              uint32_t n_steps, uint32_t *out_tokens) {
    WGML_REQUIRE(m && out_tokens, "wgml_llama2_decode_greedy: null argument");
    WGML_REQUIRE((uint64_t)start_pos + n_steps <= m->cfg.seq_len,
                 "wgml_llama2_decode_greedy: %u steps from %u exceed seq_len %u", n_steps, start_pos,
                 m->cfg.seq_len);
    WGML_REQUIRE(first_token < m->cfg.vocab_size, "wgml_llama2_decode_greedy: token outside vocabulary");
    if (n_steps == 0) return WGML_OK;
    return run_recorded(m, first_token, start_pos, n_steps, nullptr, 0, out_tokens);
}

int wgml_llama2_record_steps(wgml_llama2 *m, uint32_t start_pos, uint32_t n_steps) {
    WGML_REQUIRE(m, "wgml_llama2_record_steps: null argument");
    WGML_REQUIRE((uint64_t)start_pos + n_steps <= m->cfg.seq_len,
                 "wgml_llama2_record_steps: %u steps from %u exceed seq_len %u", n_steps, start_pos,
                 m->cfg.seq_len);
    WGML_TRY(check_ready(m));
    // recording runs steps of its own (from position 0, cache rows saved and put back): the
    // logits the caller may still want to read are kept aside as well
    const size_t bytes = (size_t)m->cfg.vocab_size * 4;
    void *saved = nullptr;
    WGML_CHECK_HIP(hipMalloc(&saved, bytes));
    (void)hipMemcpyAsync(saved, m->logits, bytes, hipMemcpyDeviceToDevice, m->ctx->stream);
    const int rc = record_steps(m, start_pos, n_steps);
    (void)hipMemcpyAsync(m->logits, saved, bytes, hipMemcpyDeviceToDevice, m->ctx->stream);
    const hipError_t e = hipStreamSynchronize(m->ctx->stream);
    (void)hipFree(saved);
    if (rc != WGML_OK) return rc;
    WGML_CHECK_HIP(e);
    return WGML_OK;
}

int wgml_llama2_generate_greedy(wgml_llama2 *m, const uint32_t *prompt, uint32_t n_prompt,
                                uint32_t n_total, uint32_t *out_tokens) {
    WGML_REQUIRE(m && prompt && out_tokens, "wgml_llama2_generate_greedy: null argument");
    WGML_REQUIRE(n_prompt >= 1, "wgml_llama2_generate_greedy: empty prompt");
    WGML_REQUIRE(n_total <= m->cfg.seq_len && n_prompt <= m->cfg.seq_len,
                 "wgml_llama2_generate_greedy: %u positions exceed seq_len %u", n_total,
                 m->cfg.seq_len);
    for (uint32_t i = 0; i < n_prompt; ++i)
        WGML_REQUIRE(prompt[i] < m->cfg.vocab_size,
                     "wgml_llama2_generate_greedy: prompt token %u outside vocabulary", prompt[i]);
    if (n_total == 0) return WGML_OK;
    return run_recorded(m, prompt[0], 0, n_total, prompt, n_prompt, out_tokens);
}

// The same loop with a host round trip per token, as the reference's chat loop
// does it (read back after every step): for comparison and for callers that
// stream tokens out as they appear.
int wgml_llama2_decode_greedy_sync(wgml_llama2 *m, uint32_t first_token, uint32_t start_pos,
                                   uint32_t n_steps, uint32_t *out_tokens) {
    WGML_REQUIRE(m && out_tokens, "wgml_llama2_decode_greedy_sync: null argument");
    WGML_REQUIRE((uint64_t)start_pos + n_steps <= m->cfg.seq_len,
                 "wgml_llama2_decode_greedy_sync: steps exceed seq_len");
    wgml_ctx *ctx = m->ctx;
    uint32_t token = first_token;
    for (uint32_t i = 0; i < n_steps; ++i) {
        WGML_TRY(wgml_llama2_forward(m, token, start_pos + i));
        WGML_TRY(launch_argmax(ctx, m->logits, m->cfg.vocab_size, ctx->d_scalar));
        WGML_CHECK_HIP(hipMemcpyAsync(ctx->h_scalar, ctx->d_scalar, 4, hipMemcpyDeviceToHost,
                                      ctx->stream));
        WGML_CHECK_HIP(hipStreamSynchronize(ctx->stream));
        token = ctx->h_scalar[0];
        out_tokens[i] = token;
    }
    return WGML_OK;
}

// ChatLlama2::forward with the CPU sampler (chat_llama2.rs:51-153): logits come
// back to the host after every step, as in the reference.
int wgml_llama2_generate_sampled(wgml_llama2 *m, const uint32_t *prompt, uint32_t n_prompt,
                                 uint32_t n_total, float temperature, float topp, uint64_t seed,
                                 uint32_t *out_tokens) {
    WGML_REQUIRE(m && prompt && out_tokens, "wgml_llama2_generate_sampled: null argument");
    WGML_REQUIRE(n_prompt >= 1, "wgml_llama2_generate_sampled: empty prompt");
    WGML_REQUIRE(n_total <= m->cfg.seq_len,
                 "wgml_llama2_generate_sampled: %u positions exceed seq_len %u", n_total,
                 m->cfg.seq_len);
    if (n_total == 0) return WGML_OK;
    std::vector<float> logits(m->cfg.vocab_size), coins(n_total);
    WGML_TRY(wgml_rng_uniform_f32(seed, coins.data(), n_total));
    uint32_t token = prompt[0];
    for (uint32_t pos = 0; pos < n_total; ++pos) {
        WGML_TRY(wgml_llama2_forward(m, token, pos));
        WGML_TRY(wgml_llama2_read_logits(m, logits.data()));
        uint32_t next = 0;
        WGML_TRY(wgml_sample(logits.data(), m->cfg.vocab_size, temperature, topp, coins[pos],
                             &next));
        out_tokens[pos] = next;
        token = (pos + 1 < n_prompt) ? prompt[pos + 1] : next;
    }
    return WGML_OK;
}

static int kv_range(wgml_llama2 *m, uint32_t layer, int which, uint32_t first_pos, uint32_t n_pos,
                    float **p) {
    WGML_REQUIRE(layer < m->cfg.n_layers, "kv: layer %u of %u", layer, m->cfg.n_layers);
    WGML_REQUIRE(which == 0 || which == 1, "kv: which must be 0 (key) or 1 (value)");
    WGML_REQUIRE((uint64_t)first_pos + n_pos <= m->cfg.seq_len, "kv: positions exceed seq_len");
    float *base = which == 0 ? m->layers[layer].key_cache : m->layers[layer].value_cache;
    *p = base + (size_t)first_pos * m->kv_dim;
    return WGML_OK;
}

int wgml_llama2_kv_upload(wgml_llama2 *m, uint32_t layer, int which, uint32_t first_pos,
                          uint32_t n_pos, const float *host) {
    WGML_REQUIRE(m && host, "wgml_llama2_kv_upload: null argument");
    float *p = nullptr;
    WGML_TRY(kv_range(m, layer, which, first_pos, n_pos, &p));
    WGML_CHECK_HIP(hipMemcpyAsync(p, host, (size_t)n_pos * m->kv_dim * 4, hipMemcpyHostToDevice,
                                  m->ctx->stream));
    WGML_CHECK_HIP(hipStreamSynchronize(m->ctx->stream));
    return WGML_OK;
}

int wgml_llama2_kv_download(wgml_llama2 *m, uint32_t layer, int which, uint32_t first_pos,
                            uint32_t n_pos, float *host) {
    WGML_REQUIRE(m && host, "wgml_llama2_kv_download: null argument");
    float *p = nullptr;
    WGML_TRY(kv_range(m, layer, which, first_pos, n_pos, &p));
    WGML_CHECK_HIP(hipMemcpyAsync(host, p, (size_t)n_pos * m->kv_dim * 4, hipMemcpyDeviceToHost,
                                  m->ctx->stream));
    WGML_CHECK_HIP(hipStreamSynchronize(m->ctx->stream));
    return WGML_OK;
}

}  // extern "C"
