// GPT-2 decoder: state, weights and the per-token launch sequence.  Mirrors
// Gpt2State / Gpt2Weights / Gpt2::dispatch (models/gpt2/transformer.rs:14-477 of
// the reference) and ChatGpt2's token loop (wgml-chat/src/chat_gpt2.rs:43-151).
// Unlike the reference, which expands every weight to f32 at load
// (models/gpt2/transformer.rs:133-141), the matrices stay in their GGUF
// quantization and go through the quantized GEMV.
#include "common.h"

using namespace wgml;

namespace wgml {
int reserve_attention_workspace(wgml_ctx *ctx, const wgml_attn_params &p, uint32_t plan_positions);
}

struct Gpt2Layer {
    const wgml_qmat *attn_w = nullptr, *proj_w = nullptr, *fc_w = nullptr, *mlp_proj_w = nullptr;
    float *ln_1_g = nullptr, *ln_1_b = nullptr, *ln_2_g = nullptr, *ln_2_b = nullptr;
    float *attn_b = nullptr, *proj_b = nullptr, *fc_b = nullptr, *mlp_proj_b = nullptr;
    float *key_cache = nullptr, *value_cache = nullptr;
};

struct wgml_gpt2 {
    wgml_ctx *ctx = nullptr;
    wgml_gpt2_params p{};
    std::vector<Gpt2Layer> layers;
    const wgml_qmat *lm_head = nullptr;
    float *ln_f_g = nullptr, *ln_f_b = nullptr, *wte = nullptr, *wpe = nullptr;
    // Gpt2State (models/gpt2/transformer.rs:14-25)
    float *layer_input = nullptr, *curr_768 = nullptr, *curr_768_b = nullptr, *curr_2304 = nullptr,
          *curr_3072 = nullptr, *curr_vocab = nullptr;
    std::vector<void *> allocs;
    // recorded token loop: position / token / output cursor on the device
    DynState *dyn = nullptr;
    uint32_t *d_prompt = nullptr, *d_tokens = nullptr;
    // the recorded step, one capture per bucket of positions (plan_bucket)
    hipGraph_t graph[kMaxPlanBuckets] = {};
    hipGraphExec_t graph_exec[kMaxPlanBuckets] = {};
    // kStepsPerGraph consecutive steps as one graph, replayed where that many steps stay inside
    // a bucket (a replay costs the same between two graphs whatever the graph holds)
    hipGraph_t graph_multi[kMaxPlanBuckets] = {};
    hipGraphExec_t graph_exec_multi[kMaxPlanBuckets] = {};
    uint64_t graph_launches[kMaxPlanBuckets] = {};  // launches of the recorded step
    int fusion = 1;  // 0: one launch per op group as before; 1: folded launches
    int graph_fusion = -1;
    uint64_t graph_tuning = 0;  // the context's tuning generation the captures were made under
    uint64_t launches_last = 0;   // launches of the last step that ran
};

namespace {

int dev_alloc(wgml_gpt2 *m, float **p, uint64_t n_floats, bool zero) {
    void *d = nullptr;
    hipError_t e = hipMalloc(&d, n_floats * 4);
    if (e != hipSuccess)
        return set_error(WGML_E_OOM, "wgml_gpt2: hipMalloc(%llu) failed: %s",
                         (unsigned long long)(n_floats * 4), hipGetErrorString(e));
    m->allocs.push_back(d);
    if (zero) WGML_CHECK_HIP(hipMemsetAsync(d, 0, n_floats * 4, m->ctx->stream));
    *p = (float *)d;
    return WGML_OK;
}

int check_ready(const wgml_gpt2 *m) {
    for (size_t l = 0; l < m->layers.size(); ++l) {
        const Gpt2Layer &w = m->layers[l];
        WGML_REQUIRE(w.attn_w && w.proj_w && w.fc_w && w.mlp_proj_w && w.ln_1_g && w.ln_1_b &&
                         w.ln_2_g && w.ln_2_b && w.attn_b && w.proj_b && w.fc_b && w.mlp_proj_b,
                     "wgml_gpt2: layer %zu has unset weights", l);
    }
    WGML_REQUIRE(m->lm_head && m->ln_f_g && m->ln_f_b && m->wte && m->wpe,
                 "wgml_gpt2: lm_head / ln_f / embeddings not set");
    return WGML_OK;
}

}  // namespace

namespace {
void drop_graph(wgml_gpt2 *m);  // recorded launches hold device pointers
}

extern "C" {

int wgml_gpt2_create(wgml_ctx *ctx, const wgml_gpt2_params *p, wgml_gpt2 **out) {
    WGML_REQUIRE(ctx && p && out, "wgml_gpt2_create: null argument");
    *out = nullptr;
    WGML_REQUIRE(p->n_vocab && p->n_seq && p->n_embd && p->n_head && p->n_layer && p->ff_len,
                 "wgml_gpt2_create: zero field in params");
    WGML_REQUIRE(p->n_embd % p->n_head == 0 && p->attn_b == 3 * p->n_embd,
                 "wgml_gpt2_create: n_embd %u, n_head %u, attn_b %u are inconsistent", p->n_embd,
                 p->n_head, p->attn_b);
    WGML_REQUIRE(p->n_embd % 4 == 0 && p->ff_len % 4 == 0,
                 "wgml_gpt2_create: n_embd and ff_len must be multiples of 4");
    WGML_REQUIRE(p->n_embd / p->n_head <= 256, "wgml_gpt2_create: head size above 256");
    wgml_gpt2 *m = new wgml_gpt2();
    m->ctx = ctx;
    ctx_retain(ctx);
    m->p = *p;
    m->layers.resize(p->n_layer);
    int rc = WGML_OK;
    auto A = [&](float **q, uint64_t n, bool z) {
        if (rc == WGML_OK) rc = dev_alloc(m, q, n, z);
    };
    A(&m->layer_input, p->n_embd, true);
    A(&m->curr_768, p->n_embd, true);
    A(&m->curr_768_b, p->n_embd, true);
    A(&m->curr_2304, p->attn_b, true);
    A(&m->curr_3072, p->ff_len, true);
    A(&m->curr_vocab, p->n_vocab, true);
    {
        float *tmp = nullptr;
        A(&tmp, 4, true);
        m->dyn = reinterpret_cast<DynState *>(tmp);
        A(&tmp, p->n_seq, true);
        m->d_prompt = reinterpret_cast<uint32_t *>(tmp);
        A(&tmp, p->n_seq, true);
        m->d_tokens = reinterpret_cast<uint32_t *>(tmp);
    }
    for (auto &l : m->layers) {
        A(&l.key_cache, (uint64_t)p->n_embd * p->n_seq, true);
        A(&l.value_cache, (uint64_t)p->n_embd * p->n_seq, true);
    }
    if (rc == WGML_OK && hipStreamSynchronize(ctx->stream) != hipSuccess)
        rc = set_error(WGML_E_HIP, "wgml_gpt2_create: synchronize failed");
    if (rc != WGML_OK) {
        wgml_gpt2_destroy(m);
        return rc;
    }
    *out = m;
    return WGML_OK;
}

int wgml_gpt2_destroy(wgml_gpt2 *m) {
    if (!m) return WGML_OK;
    if (m->ctx && m->ctx->stream) (void)hipStreamSynchronize(m->ctx->stream);
    drop_graph(m);
    for (void *p : m->allocs) (void)hipFree(p);
    ctx_release(m->ctx);
    delete m;
    return WGML_OK;
}

int wgml_gpt2_set_matrix(wgml_gpt2 *m, int which, uint32_t layer, const wgml_qmat *mat) {
    WGML_REQUIRE(m && mat, "wgml_gpt2_set_matrix: null argument");
    const wgml_gpt2_params &p = m->p;
    uint32_t er = 0, ec = 0;
    switch (which) {  // models/gpt2/cpu.rs:150-158,193-196
    case WGML_GPT2_ATTN_W: er = p.attn_b; ec = p.n_embd; break;
    case WGML_GPT2_ATTN_PROJ_W: er = p.n_embd; ec = p.n_embd; break;
    case WGML_GPT2_MLP_FC_W: er = p.ff_len; ec = p.n_embd; break;
    case WGML_GPT2_MLP_PROJ_W: er = p.n_embd; ec = p.ff_len; break;
    case WGML_GPT2_LM_HEAD: er = p.n_vocab; ec = p.n_embd; break;
    default: return set_error(WGML_E_INVALID, "wgml_gpt2_set_matrix: unknown matrix %d", which);
    }
    WGML_REQUIRE(mat->nrows == er && mat->ncols == ec,
                 "wgml_gpt2_set_matrix: matrix %d is %ux%u, expected %ux%u", which, mat->nrows,
                 mat->ncols, er, ec);
    drop_graph(m);  // a recorded step holds the plane pointers of the matrix it replaces
    if (which == WGML_GPT2_LM_HEAD) {
        m->lm_head = mat;
        return WGML_OK;
    }
    WGML_REQUIRE(layer < p.n_layer, "wgml_gpt2_set_matrix: layer %u of %u", layer, p.n_layer);
    Gpt2Layer &l = m->layers[layer];
    switch (which) {
    case WGML_GPT2_ATTN_W: l.attn_w = mat; break;
    case WGML_GPT2_ATTN_PROJ_W: l.proj_w = mat; break;
    case WGML_GPT2_MLP_FC_W: l.fc_w = mat; break;
    case WGML_GPT2_MLP_PROJ_W: l.mlp_proj_w = mat; break;
    }
    return WGML_OK;
}

int wgml_gpt2_set_vector(wgml_gpt2 *m, int which, uint32_t layer, const float *host,
                         uint32_t len) {
    WGML_REQUIRE(m && host, "wgml_gpt2_set_vector: null argument");
    const wgml_gpt2_params &p = m->p;
    uint32_t expect = p.n_embd;
    float **slot = nullptr;
    if (which == WGML_GPT2_LN_F_G) slot = &m->ln_f_g;
    else if (which == WGML_GPT2_LN_F_B) slot = &m->ln_f_b;
    else {
        WGML_REQUIRE(layer < p.n_layer, "wgml_gpt2_set_vector: layer %u of %u", layer, p.n_layer);
        Gpt2Layer &l = m->layers[layer];
        switch (which) {
        case WGML_GPT2_LN_1_G: slot = &l.ln_1_g; break;
        case WGML_GPT2_LN_1_B: slot = &l.ln_1_b; break;
        case WGML_GPT2_LN_2_G: slot = &l.ln_2_g; break;
        case WGML_GPT2_LN_2_B: slot = &l.ln_2_b; break;
        case WGML_GPT2_ATTN_B: slot = &l.attn_b; expect = p.attn_b; break;
        case WGML_GPT2_ATTN_PROJ_B: slot = &l.proj_b; break;
        case WGML_GPT2_MLP_FC_B: slot = &l.fc_b; expect = p.ff_len; break;
        case WGML_GPT2_MLP_PROJ_B: slot = &l.mlp_proj_b; break;
        default: return set_error(WGML_E_INVALID, "wgml_gpt2_set_vector: unknown vector %d", which);
        }
    }
    WGML_REQUIRE(len == expect, "wgml_gpt2_set_vector: vector %d has %u elements, expected %u",
                 which, len, expect);
    if (!*slot) {
        WGML_TRY(dev_alloc(m, slot, len, false));
        drop_graph(m);  // a step recorded without this vector (optional biases) is stale
    }
    WGML_CHECK_HIP(hipMemcpyAsync(*slot, host, (size_t)len * 4, hipMemcpyHostToDevice,
                                  m->ctx->stream));
    WGML_CHECK_HIP(hipStreamSynchronize(m->ctx->stream));
    return WGML_OK;
}

int wgml_gpt2_set_embeddings(wgml_gpt2 *m, const float *wte, const float *wpe) {
    WGML_REQUIRE(m && wte && wpe, "wgml_gpt2_set_embeddings: null argument");
    const uint64_t nt = (uint64_t)m->p.n_embd * m->p.n_vocab, np = (uint64_t)m->p.n_embd * m->p.n_seq;
    if (!m->wte || !m->wpe) drop_graph(m);
    if (!m->wte) WGML_TRY(dev_alloc(m, &m->wte, nt, false));
    if (!m->wpe) WGML_TRY(dev_alloc(m, &m->wpe, np, false));
    WGML_CHECK_HIP(hipMemcpyAsync(m->wte, wte, nt * 4, hipMemcpyHostToDevice, m->ctx->stream));
    WGML_CHECK_HIP(hipMemcpyAsync(m->wpe, wpe, np * 4, hipMemcpyHostToDevice, m->ctx->stream));
    WGML_CHECK_HIP(hipStreamSynchronize(m->ctx->stream));
    return WGML_OK;
}

}  // extern "C"

namespace {

// Gpt2::dispatch (models/gpt2/transformer.rs:265-477) for one token.  `dynamic`:
// token and position are read from m->dyn on the device (a recorded step), else
// they are the given values.
// Folded launches (fusion 1): the reference's mul_assign/add_assign after each
// layernorm and the add_assign after each matmul disappear into the GEMVs
// (LayerNorm in the staging of x, bias / residual / GELU in the epilogue); q, k and
// v are row slices of the one attn_w matrix, k and v written straight into their
// cache columns (:329-353 copies them).  fusion 0 keeps layernorm, GELU and the
// cache copies as launches of their own.
// The folded launches exist for the quantized formats only.
bool can_fold(const wgml_gpt2 *m) {
    if (!gemv_fused_supported(m->lm_head)) return false;
    for (const Gpt2Layer &w : m->layers)
        if (!gemv_fused_supported(w.attn_w) || !gemv_fused_supported(w.proj_w) ||
            !gemv_fused_supported(w.fc_w) || !gemv_fused_supported(w.mlp_proj_w))
            return false;
    return true;
}

// embed == false: m->layer_input already holds wte[:, token] + wpe[:, pos] (the sampling launch
// of the step before wrote it).
int enqueue_step(wgml_gpt2 *m, bool dynamic, uint32_t token, uint32_t pos,
                 uint32_t plan_positions = 0, bool embed = true) {
    const wgml_gpt2_params &p = m->p;
    wgml_ctx *ctx = m->ctx;
    const uint32_t n = p.n_embd;
    const DynPos dpos = dynamic ? DynPos{&m->dyn->pos, 0} : DynPos{nullptr, pos};
    const DynPos dtok = dynamic ? DynPos{&m->dyn->token, 0} : DynPos{nullptr, token};
    const wgml_attn_params ap{p.n_seq, n, 1u, p.n_head, n / p.n_head, pos};
    const uint32_t plan = dynamic ? (plan_positions ? plan_positions : p.n_seq) : pos + 1;
    const bool fold = m->fusion >= 1 && can_fold(m);
    if (dynamic && !fold)
        return set_error(WGML_E_UNSUPPORTED, "wgml_gpt2: the recorded step needs fusion 1");

    // layer_input = wte[:, token] + wpe[:, pos]   (:277-290)
    if (embed) WGML_TRY(launch_embed(ctx, m->layer_input, m->wte, n, dtok, nullptr, 2, 0.f, dpos, m->wpe));

    for (uint32_t l = 0; l < p.n_layer; ++l) {
        const Gpt2Layer &w = m->layers[l];
        if (fold) {
            FusedGemv f;
            f.njobs = 3;
            f.x = m->layer_input;
            f.ln_gamma = w.ln_1_g;
            f.ln_beta = w.ln_1_b;
            f.pos = dpos;
            float *outs[3] = {m->curr_2304, w.key_cache, w.value_cache};
            for (int j = 0; j < 3; ++j) {
                f.jobs[j].a = w.attn_w;
                f.jobs[j].row0 = (uint32_t)j * n;
                f.jobs[j].nrows = n;
                f.jobs[j].bias = w.attn_b + (size_t)j * n;
                f.jobs[j].out = outs[j];
                f.jobs[j].out_pos_stride = j ? n : 0;
            }
            WGML_TRY(launch_gemv_fused(ctx, f));
        } else {
            WGML_TRY(launch_layernorm(ctx, m->curr_768, m->layer_input, w.ln_1_g, w.ln_1_b, n));
            GemvEpilogue e;
            e.bias = w.attn_b;
            WGML_TRY(launch_gemv_quant(ctx, m->curr_2304, w.attn_w, m->curr_768, e));
            // k -> key_cache[:, pos], v -> value_cache[:, pos]; contiguous so one copy each
            WGML_CHECK_HIP(hipMemcpyAsync(w.key_cache + (size_t)pos * n, m->curr_2304 + n,
                                          (size_t)n * 4, hipMemcpyDeviceToDevice, ctx->stream));
            WGML_CHECK_HIP(hipMemcpyAsync(w.value_cache + (size_t)pos * n, m->curr_2304 + 2 * n,
                                          (size_t)n * 4, hipMemcpyDeviceToDevice, ctx->stream));
        }
        // with the fused launches, attention may leave per-workgroup partial results that the
        // projection merges while it stages its input (no merge launch)
        AttnPartials parts;
        WGML_TRY(launch_attention_planned(ctx, ap, dpos, plan, ap.seq_len, m->curr_2304,
                                          w.key_cache, w.value_cache, nullptr, m->curr_768, nullptr, 0,
                                          fold && gemv_partials_supported(ctx, w.proj_w) ? &parts
                                                                                         : nullptr));
        // layer_input += proj_w * attn + proj_b   (:372-395)
        {
            GemvEpilogue e;
            e.bias = w.proj_b;
            e.accumulate = 1;
            e.partials = parts;
            WGML_TRY(launch_gemv_quant(ctx, m->layer_input, w.proj_w, m->curr_768, e));
        }
        if (fold) {
            GemvEpilogue e;  // h = gelu(fc_w * ln_2(layer_input) + fc_b)   (:397-431)
            e.bias = w.fc_b;
            e.ln_gamma = w.ln_2_g;
            e.ln_beta = w.ln_2_b;
            e.act = 1;
            WGML_TRY(launch_gemv_quant(ctx, m->curr_3072, w.fc_w, m->layer_input, e));
        } else {
            WGML_TRY(launch_layernorm(ctx, m->curr_768, m->layer_input, w.ln_2_g, w.ln_2_b, n));
            GemvEpilogue e;
            e.bias = w.fc_b;
            WGML_TRY(launch_gemv_quant(ctx, m->curr_3072, w.fc_w, m->curr_768, e));
            WGML_TRY(launch_unary(ctx, WGML_UNARY_GELU, m->curr_3072, p.ff_len, nullptr));
        }
        // layer_input += mlp_proj_w * h + mlp_proj_b   (:433-452)
        {
            GemvEpilogue e;
            e.bias = w.mlp_proj_b;
            e.accumulate = 1;
            WGML_TRY(launch_gemv_quant(ctx, m->layer_input, w.mlp_proj_w, m->curr_3072, e));
        }
    }
    if (fold) {
        GemvEpilogue e;
        e.ln_gamma = m->ln_f_g;
        e.ln_beta = m->ln_f_b;
        WGML_TRY(launch_gemv_quant(ctx, m->curr_vocab, m->lm_head, m->layer_input, e));
    } else {
        WGML_TRY(launch_layernorm(ctx, m->curr_768, m->layer_input, m->ln_f_g, m->ln_f_b, n));
        WGML_TRY(launch_gemv_quant(ctx, m->curr_vocab, m->lm_head, m->curr_768, GemvEpilogue{}));
    }
    return WGML_OK;
}

void drop_graph(wgml_gpt2 *m) {
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

// The attention workspace for the largest plan of any bucket (recorded launches hold its
// address, so it must not grow between captures).
int reserve_all_plans(wgml_gpt2 *m) {
    const wgml_gpt2_params &p = m->p;
    const wgml_attn_params ap{p.n_seq, p.n_embd, 1u, p.n_head, p.n_embd / p.n_head, 0};
    for (uint32_t pos = 0;;) {
        const uint32_t limit = plan_bucket(pos, p.n_seq, nullptr);
        WGML_TRY(reserve_attention_workspace(m->ctx, ap, limit));
        if (limit >= p.n_seq) break;
        pos = limit;
    }
    return WGML_OK;
}

constexpr uint32_t kStepsPerGraph = 8;

// A step of the token loop that keeps its state on the device: the layers and the output
// projection, then the launch that samples (arg-max), does the loop's bookkeeping and writes
// wte[:, token] + wpe[:, pos] of the token and position it has chosen, for the step that
// follows.  The loop's first step finds it written by loop_first_embed.
int enqueue_loop_step(wgml_gpt2 *m, uint32_t plan) {
    const wgml_gpt2_params &p = m->p;
    WGML_TRY(enqueue_step(m, true, 0, 0, plan, false));
    const NextEmbed ne{m->layer_input, m->wte, p.n_embd, nullptr, 2, 0.f, m->wpe, p.n_seq};
    return launch_argmax_next(m->ctx, m->curr_vocab, p.n_vocab, m->dyn, m->d_prompt, m->d_tokens, &ne);
}
int loop_first_embed(wgml_gpt2 *m) {
    return launch_embed(m->ctx, m->layer_input, m->wte, m->p.n_embd, DynPos{&m->dyn->token, 0}, nullptr, 2,
                        0.f, DynPos{&m->dyn->pos, 0}, m->wpe);
}

// Records `steps` consecutive steps (each followed by greedy sampling and the loop's
// bookkeeping, all on the device) into one HIP graph.
int capture_steps(wgml_gpt2 *m, uint32_t plan, uint32_t steps, hipGraph_t *graph,
                  hipGraphExec_t *exec, uint64_t *launches_per_step) {
    wgml_ctx *ctx = m->ctx;
    WGML_CHECK_HIP(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    const uint64_t launches0 = ctx->launches;
    int rc = WGML_OK;
    for (uint32_t k = 0; k < steps && rc == WGML_OK; ++k) rc = enqueue_loop_step(m, plan);
    if (launches_per_step) *launches_per_step = (ctx->launches - launches0) / steps;
    hipError_t e = hipStreamEndCapture(ctx->stream, graph);
    if (rc != WGML_OK) return rc;
    if (e != hipSuccess)
        return set_error(WGML_E_HIP, "wgml_gpt2: graph capture failed: %s", hipGetErrorString(e));
    e = hipGraphInstantiate(exec, *graph, nullptr, nullptr, 0);
    if (e != hipSuccess)
        return set_error(WGML_E_HIP, "wgml_gpt2: graph instantiate failed: %s", hipGetErrorString(e));
    if (steps > 1) {
        // A graph's first replay costs milliseconds (uploading the graph ahead of time does
        // not remove it): do it here, from position 0, with the cache rows it writes saved
        // and put back.
        const size_t bytes = (size_t)steps * m->p.n_embd * 4;
        void *saved = nullptr;
        WGML_CHECK_HIP(hipMalloc(&saved, bytes * 2 * m->p.n_layer));
        for (uint32_t l = 0; l < m->p.n_layer; ++l) {
            (void)hipMemcpyAsync((char *)saved + bytes * (2 * l), m->layers[l].key_cache, bytes,
                                 hipMemcpyDeviceToDevice, ctx->stream);
            (void)hipMemcpyAsync((char *)saved + bytes * (2 * l + 1), m->layers[l].value_cache, bytes,
                                 hipMemcpyDeviceToDevice, ctx->stream);
        }
        const DynState init{0, 0, 0, 0};
        e = hipMemcpyAsync(m->dyn, &init, sizeof(init), hipMemcpyHostToDevice, ctx->stream);
        if (e == hipSuccess && loop_first_embed(m) != WGML_OK) e = hipErrorUnknown;
        if (e == hipSuccess) e = hipGraphLaunch(*exec, ctx->stream);
        for (uint32_t l = 0; l < m->p.n_layer; ++l) {
            (void)hipMemcpyAsync(m->layers[l].key_cache, (char *)saved + bytes * (2 * l), bytes,
                                 hipMemcpyDeviceToDevice, ctx->stream);
            (void)hipMemcpyAsync(m->layers[l].value_cache, (char *)saved + bytes * (2 * l + 1), bytes,
                                 hipMemcpyDeviceToDevice, ctx->stream);
        }
        const hipError_t es = hipStreamSynchronize(ctx->stream);  // `init` is a stack object
        (void)hipFree(saved);
        if (e == hipSuccess) e = es;
        if (e != hipSuccess)
            return set_error(WGML_E_HIP, "wgml_gpt2: first replay failed: %s", hipGetErrorString(e));
    }
    return WGML_OK;
}

// Records one step (+ greedy sampling and bookkeeping) into a HIP graph, for the bucket of
// positions that `pos` lies in, and the graph of kStepsPerGraph such steps where the bucket
// holds that many positions (both at once, so that a short first run leaves nothing to build
// for a longer one).
int build_graph(wgml_gpt2 *m, uint32_t pos) {
    wgml_ctx *ctx = m->ctx;
    const wgml_gpt2_params &p = m->p;
    const uint32_t n = p.n_embd;
    // captures made at another fusion level or under other launch-shape overrides are stale
    if (m->graph_fusion != m->fusion || m->graph_tuning != ctx->tuning_generation) drop_graph(m);
    int b = 0;
    const uint32_t plan = plan_bucket(pos, p.n_seq, &b);
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
    WGML_TRY(reserve_all_plans(m));
    // An eager step first (function attributes, lazy loading); it runs at position 0
    // and would overwrite that column of every cache: keep a copy and put it back.
    const size_t col = (size_t)n * 4;
    void *saved = nullptr;
    WGML_CHECK_HIP(hipMalloc(&saved, col * 2 * p.n_layer));
    for (uint32_t l = 0; l < p.n_layer; ++l) {
        (void)hipMemcpyAsync((char *)saved + col * (2 * l), m->layers[l].key_cache, col,
                             hipMemcpyDeviceToDevice, ctx->stream);
        (void)hipMemcpyAsync((char *)saved + col * (2 * l + 1), m->layers[l].value_cache, col,
                             hipMemcpyDeviceToDevice, ctx->stream);
    }
    const DynState init{0, 0, 0, 0};
    hipError_t ew = hipMemcpyAsync(m->dyn, &init, sizeof(init), hipMemcpyHostToDevice, ctx->stream);
    int rcw = ew == hipSuccess ? loop_first_embed(m) : WGML_E_HIP;
    if (rcw == WGML_OK) rcw = enqueue_loop_step(m, plan);
    for (uint32_t l = 0; l < p.n_layer; ++l) {
        (void)hipMemcpyAsync(m->layers[l].key_cache, (char *)saved + col * (2 * l), col,
                             hipMemcpyDeviceToDevice, ctx->stream);
        (void)hipMemcpyAsync(m->layers[l].value_cache, (char *)saved + col * (2 * l + 1), col,
                             hipMemcpyDeviceToDevice, ctx->stream);
    }
    ew = hipStreamSynchronize(ctx->stream);
    (void)hipFree(saved);
    if (rcw != WGML_OK) return rcw;
    if (ew != hipSuccess)
        return set_error(WGML_E_HIP, "wgml_gpt2: warm-up step failed: %s", hipGetErrorString(ew));

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

// The recorded steps of every bucket that a run over positions 0 .. n_total - 1 passes through.
int record_steps(wgml_gpt2 *m, uint32_t n_total) {
    if (graphs_disabled()) return reserve_all_plans(m);
    for (uint32_t pos = 0; n_total > 0;) {
        const uint32_t limit = plan_bucket(pos, m->p.n_seq, nullptr);
        WGML_TRY(build_graph(m, pos));
        if (limit >= n_total || limit >= m->p.n_seq) break;
        pos = limit;
    }
    return WGML_OK;
}

}  // namespace

extern "C" {

int wgml_gpt2_forward(wgml_gpt2 *m, uint32_t token, uint32_t pos) {
    WGML_REQUIRE(m != nullptr, "wgml_gpt2_forward: null model");
    WGML_TRY(check_ready(m));
    WGML_REQUIRE(token < m->p.n_vocab, "wgml_gpt2_forward: token %u outside vocabulary %u", token,
                 m->p.n_vocab);
    WGML_REQUIRE(pos < m->p.n_seq, "wgml_gpt2_forward: pos %u outside n_seq %u", pos, m->p.n_seq);
    return enqueue_step(m, false, token, pos);
}

// 0: layernorm, GELU and the cache copies are launches of their own; 1 (default):
// folded into the GEMVs.  Same results to fp32 rounding.
int wgml_gpt2_set_fusion(wgml_gpt2 *m, int level) {
    WGML_REQUIRE(m != nullptr, "wgml_gpt2_set_fusion: null model");
    WGML_REQUIRE(level == 0 || level == 1, "wgml_gpt2_set_fusion: level %d not in {0,1}", level);
    m->fusion = level;
    return WGML_OK;
}

int wgml_gpt2_launches_per_token(const wgml_gpt2 *m) { return m ? (int)m->launches_last : 0; }

int wgml_gpt2_read_logits(wgml_gpt2 *m, float *host_out) {
    WGML_REQUIRE(m && host_out, "wgml_gpt2_read_logits: null argument");
    WGML_CHECK_HIP(hipMemcpyAsync(host_out, m->curr_vocab, (size_t)m->p.n_vocab * 4,
                                  hipMemcpyDeviceToHost, m->ctx->stream));
    WGML_CHECK_HIP(hipStreamSynchronize(m->ctx->stream));
    return WGML_OK;
}

int wgml_gpt2_record_steps(wgml_gpt2 *m, uint32_t n_total) {
    WGML_REQUIRE(m, "wgml_gpt2_record_steps: null argument");
    WGML_REQUIRE(n_total <= m->p.n_seq, "wgml_gpt2_record_steps: %u positions exceed n_seq %u", n_total,
                 m->p.n_seq);
    WGML_TRY(check_ready(m));
    if (m->fusion < 1 || !can_fold(m)) return WGML_OK;  // the unfused loop records nothing
    // recording runs steps of its own: the logits the caller may still want are kept aside
    const size_t bytes = (size_t)m->p.n_vocab * 4;
    void *saved = nullptr;
    WGML_CHECK_HIP(hipMalloc(&saved, bytes));
    (void)hipMemcpyAsync(saved, m->curr_vocab, bytes, hipMemcpyDeviceToDevice, m->ctx->stream);
    const int rc = record_steps(m, n_total);
    (void)hipMemcpyAsync(m->curr_vocab, saved, bytes, hipMemcpyDeviceToDevice, m->ctx->stream);
    const hipError_t e = hipStreamSynchronize(m->ctx->stream);
    (void)hipFree(saved);
    if (rc != WGML_OK) return rc;
    WGML_CHECK_HIP(e);
    return WGML_OK;
}

int wgml_gpt2_generate_greedy(wgml_gpt2 *m, const uint32_t *prompt, uint32_t n_prompt,
                              uint32_t n_total, uint32_t *out_tokens) {
    WGML_REQUIRE(m && prompt && out_tokens, "wgml_gpt2_generate_greedy: null argument");
    WGML_REQUIRE(n_prompt >= 1, "wgml_gpt2_generate_greedy: empty prompt");
    WGML_REQUIRE(n_total <= m->p.n_seq, "wgml_gpt2_generate_greedy: %u positions exceed n_seq %u",
                 n_total, m->p.n_seq);
    WGML_TRY(check_ready(m));
    for (uint32_t i = 0; i < n_prompt && i < n_total; ++i)
        WGML_REQUIRE(prompt[i] < m->p.n_vocab, "wgml_gpt2_generate_greedy: prompt token %u outside "
                                                "the vocabulary", prompt[i]);
    wgml_ctx *ctx = m->ctx;
    if (n_total == 0) return WGML_OK;
    if (m->fusion < 1 || !can_fold(m)) {
        // one launch per op group and a host round trip per token, as the reference's
        // chat loop does (chat_gpt2.rs:61-110)
        uint32_t token = prompt[0];
        for (uint32_t pos = 0; pos < n_total; ++pos) {
            const uint64_t l0 = ctx->launches;
            WGML_TRY(enqueue_step(m, false, token, pos));
            WGML_TRY(launch_argmax(ctx, m->curr_vocab, m->p.n_vocab, ctx->d_scalar));
            m->launches_last = ctx->launches - l0;
            WGML_CHECK_HIP(hipMemcpyAsync(ctx->h_scalar, ctx->d_scalar, 4, hipMemcpyDeviceToHost,
                                          ctx->stream));
            WGML_CHECK_HIP(hipStreamSynchronize(ctx->stream));
            const uint32_t best = ctx->h_scalar[0];
            out_tokens[pos] = best;
            token = (pos + 1 < n_prompt) ? prompt[pos + 1] : best;
        }
        return WGML_OK;
    }
    // Recorded step replayed per token: sampling and bookkeeping stay on the device,
    // one synchronisation at the end.
    const bool use_graph = !graphs_disabled();
    WGML_TRY(record_steps(m, n_total));
    const uint32_t np = n_prompt < n_total ? n_prompt : n_total;
    WGML_CHECK_HIP(hipMemcpyAsync(m->d_prompt, prompt, (size_t)np * 4, hipMemcpyHostToDevice,
                                  ctx->stream));
    const DynState init{0, prompt[0], 0, np};
    WGML_CHECK_HIP(hipMemcpyAsync(m->dyn, &init, sizeof(init), hipMemcpyHostToDevice, ctx->stream));
    WGML_TRY(loop_first_embed(m));
    for (uint32_t i = 0; i < n_total; ++i) {
        int b = 0;
        const uint32_t plan = plan_bucket(i, m->p.n_seq, &b);
        if (use_graph) {
            // steps left in this run that stay inside the bucket (positions below `plan`)
            const uint32_t in_bucket = plan > i ? plan - i : 1;
            if (m->graph_exec_multi[b] && n_total - i >= kStepsPerGraph && in_bucket >= kStepsPerGraph) {
                WGML_CHECK_HIP(hipGraphLaunch(m->graph_exec_multi[b], ctx->stream));
                i += kStepsPerGraph - 1;
            } else {
                WGML_CHECK_HIP(hipGraphLaunch(m->graph_exec[b], ctx->stream));
            }
            m->launches_last = m->graph_launches[b];
        } else {
            const uint64_t l0 = ctx->launches;
            WGML_TRY(enqueue_loop_step(m, plan));
            m->launches_last = ctx->launches - l0;
        }
    }
    WGML_CHECK_HIP(hipMemcpyAsync(out_tokens, m->d_tokens, (size_t)n_total * 4,
                                  hipMemcpyDeviceToHost, ctx->stream));
    WGML_CHECK_HIP(hipStreamSynchronize(ctx->stream));
    return WGML_OK;
}

}  // extern "C"
