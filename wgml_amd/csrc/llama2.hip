// Llama-family decoder: state, weights and the per-token launch sequence.
// Mirrors Llama2State / Llama2Weights / Llama2::dispatch
// (models/llama2/transformer.rs:17-476 of the reference) and the token loop of
// ChatLlama2 (wgml-chat/src/chat_llama2.rs:51-228).
#include "common.h"

using namespace wgml;

namespace wgml {
int launch_attention_planned(wgml_ctx *ctx, const wgml_attn_params &p, DynPos pos,
                             uint32_t plan_positions, const float *q, const float *kc,
                             const float *vc, float *att, float *xb);
}

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
    int fusion = 1;
    uint32_t kv_dim = 0, head_size = 0, kv_mul = 0;
    std::vector<LlamaLayer> layers;
    const wgml_qmat *output = nullptr;
    float *output_norm = nullptr;
    float *token_embd = nullptr;
    // Llama2State (models/llama2/transformer.rs:17-45)
    float *x = nullptr, *xb = nullptr, *xb2 = nullptr, *hb = nullptr, *hb2 = nullptr, *q = nullptr,
          *logits = nullptr;
    std::vector<void *> allocs;
    uint64_t launches_last = 0;
};

namespace {

int dev_alloc(wgml_llama2 *m, float **p, uint64_t n_floats, bool zero) {
    void *d = nullptr;
    hipError_t e = hipMalloc(&d, n_floats * 4);
    if (e != hipSuccess)
        return set_error(WGML_E_OOM, "wgml_llama2: hipMalloc(%llu) failed: %s",
                         (unsigned long long)(n_floats * 4), hipGetErrorString(e));
    m->allocs.push_back(d);
    if (zero) WGML_CHECK_HIP(hipMemsetAsync(d, 0, n_floats * 4, m->ctx->stream));
    *p = (float *)d;
    return WGML_OK;
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
    wgml_llama2 *m = new wgml_llama2();
    m->ctx = ctx;
    ctx_retain(ctx);
    m->cfg = *cfg;
    m->model_type = model_type;
    // Llama2Config::derived_configs (models/llama2/cpu.rs:111-141)
    m->kv_dim = cfg->dim * cfg->n_kv_heads / cfg->n_q_heads;
    m->head_size = cfg->dim / cfg->n_q_heads;
    m->kv_mul = cfg->n_q_heads / cfg->n_kv_heads;
    if (m->head_size % 2 != 0 || m->head_size > 256) {
        ctx_release(ctx);
        delete m;
        return set_error(WGML_E_UNSUPPORTED, "wgml_llama2_create: head_size %u unsupported",
                         cfg->dim / cfg->n_q_heads);
    }
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
    for (auto &l : m->layers) {
        A(&l.key_cache, (uint64_t)m->kv_dim * cfg->seq_len, true);
        A(&l.value_cache, (uint64_t)m->kv_dim * cfg->seq_len, true);
    }
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
    if (!*slot) WGML_TRY(dev_alloc(m, slot, len, false));
    WGML_CHECK_HIP(hipMemcpyAsync(*slot, host, (size_t)len * 4, hipMemcpyHostToDevice,
                                  m->ctx->stream));
    WGML_CHECK_HIP(hipStreamSynchronize(m->ctx->stream));
    return WGML_OK;
}

int wgml_llama2_set_token_embd(wgml_llama2 *m, const float *host) {
    WGML_REQUIRE(m && host, "wgml_llama2_set_token_embd: null argument");
    const uint64_t n = (uint64_t)m->cfg.dim * m->cfg.vocab_size;
    if (!m->token_embd) WGML_TRY(dev_alloc(m, &m->token_embd, n, false));
    WGML_CHECK_HIP(hipMemcpyAsync(m->token_embd, host, n * 4, hipMemcpyHostToDevice,
                                  m->ctx->stream));
    WGML_CHECK_HIP(hipStreamSynchronize(m->ctx->stream));
    return WGML_OK;
}

int wgml_llama2_set_fusion(wgml_llama2 *m, int level) {
    WGML_REQUIRE(m != nullptr, "wgml_llama2_set_fusion: null model");
    WGML_REQUIRE(level == 0 || level == 1, "wgml_llama2_set_fusion: level %d not in {0,1}", level);
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
    wgml_ctx *ctx = m->ctx;
    const uint64_t launches0 = ctx->launches;
    const uint32_t dim = c.dim, kv_dim = m->kv_dim;
    const DynPos dpos{nullptr, pos};
    const int variant = m->model_type == WGML_MODEL_QWEN2 ? WGML_ROPE_NEOX : WGML_ROPE_ORIGINAL;
    const wgml_attn_params ap{c.seq_len, kv_dim, m->kv_mul, c.n_q_heads, m->head_size, pos};
    const bool fused = m->fusion >= 1;

    // state.x.copy_from_view(token_embd.column(token))  (chat_llama2.rs:185-187)
    WGML_CHECK_HIP(hipMemcpyAsync(m->x, m->token_embd + (size_t)token * dim, (size_t)dim * 4,
                                  hipMemcpyDeviceToDevice, ctx->stream));

    for (uint32_t l = 0; l < c.n_layers; ++l) {
        const LlamaLayer &w = m->layers[l];
        float *k_cache = w.key_cache + (size_t)pos * kv_dim;
        float *v_cache = w.value_cache + (size_t)pos * kv_dim;

        WGML_TRY(launch_rms_norm(ctx, c.rms_norm_eps, m->xb, m->x, w.attn_norm, dim));
        if (fused) {
            WGML_TRY(launch_gemv_quant(ctx, m->q, w.attn_q, m->xb, GemvEpilogue{w.bq, 0}));
            WGML_TRY(launch_gemv_quant(ctx, k_cache, w.attn_k, m->xb, GemvEpilogue{w.bk, 0}));
            WGML_TRY(launch_gemv_quant(ctx, v_cache, w.attn_v, m->xb, GemvEpilogue{w.bv, 0}));
        } else {
            WGML_TRY(launch_gemv_quant(ctx, m->q, w.attn_q, m->xb, GemvEpilogue{}));
            WGML_TRY(launch_gemv_quant(ctx, k_cache, w.attn_k, m->xb, GemvEpilogue{}));
            WGML_TRY(launch_gemv_quant(ctx, v_cache, w.attn_v, m->xb, GemvEpilogue{}));
            if (w.bq) WGML_TRY(launch_op_assign(ctx, WGML_ASSIGN_ADD, m->q, w.bq, dim));
            if (w.bk) WGML_TRY(launch_op_assign(ctx, WGML_ASSIGN_ADD, k_cache, w.bk, kv_dim));
            if (w.bv) WGML_TRY(launch_op_assign(ctx, WGML_ASSIGN_ADD, v_cache, w.bv, kv_dim));
        }
        WGML_TRY(launch_rope(ctx, variant, m->head_size, kv_dim, dpos, c.rope_base_freq, m->q, dim,
                             k_cache, 0));
        WGML_TRY(launch_attention_planned(ctx, ap, dpos, pos + 1, m->q, w.key_cache,
                                          w.value_cache, nullptr, m->xb));
        if (fused) {
            // x += Wo * xb in the GEMV epilogue
            WGML_TRY(launch_gemv_quant(ctx, m->x, w.attn_output, m->xb, GemvEpilogue{nullptr, 1}));
        } else {
            WGML_TRY(launch_gemv_quant(ctx, m->xb2, w.attn_output, m->xb, GemvEpilogue{}));
            WGML_TRY(launch_op_assign(ctx, WGML_ASSIGN_ADD, m->x, m->xb2, dim));
        }
        WGML_TRY(launch_rms_norm(ctx, c.rms_norm_eps, m->xb, m->x, w.ffn_norm, dim));
        WGML_TRY(launch_gemv_quant(ctx, m->hb, w.ffn_gate, m->xb, GemvEpilogue{}));
        WGML_TRY(launch_gemv_quant(ctx, m->hb2, w.ffn_up, m->xb, GemvEpilogue{}));
        WGML_TRY(launch_silu(ctx, m->hb, m->hb2, c.hidden_dim));
        if (fused) {
            WGML_TRY(launch_gemv_quant(ctx, m->x, w.ffn_down, m->hb, GemvEpilogue{nullptr, 1}));
        } else {
            WGML_TRY(launch_gemv_quant(ctx, m->xb2, w.ffn_down, m->hb, GemvEpilogue{}));
            WGML_TRY(launch_op_assign(ctx, WGML_ASSIGN_ADD, m->x, m->xb2, dim));
        }
    }
    WGML_TRY(launch_rms_norm(ctx, c.rms_norm_eps, m->xb, m->x, m->output_norm, dim));
    WGML_TRY(launch_gemv_quant(ctx, m->logits, m->output, m->xb, GemvEpilogue{}));
    m->launches_last = ctx->launches - launches0;
    return WGML_OK;
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

int wgml_llama2_generate_greedy(wgml_llama2 *m, const uint32_t *prompt, uint32_t n_prompt,
                                uint32_t n_total, uint32_t *out_tokens) {
    WGML_REQUIRE(m && prompt && out_tokens, "wgml_llama2_generate_greedy: null argument");
    WGML_REQUIRE(n_prompt >= 1, "wgml_llama2_generate_greedy: empty prompt");
    WGML_REQUIRE(n_total <= m->cfg.seq_len,
                 "wgml_llama2_generate_greedy: %u positions exceed seq_len %u", n_total,
                 m->cfg.seq_len);
    wgml_ctx *ctx = m->ctx;
    uint32_t token = prompt[0];
    for (uint32_t pos = 0; pos < n_total; ++pos) {
        WGML_TRY(wgml_llama2_forward(m, token, pos));
        WGML_TRY(launch_argmax(ctx, m->logits, m->cfg.vocab_size, ctx->d_scalar));
        WGML_CHECK_HIP(hipMemcpyAsync(ctx->h_scalar, ctx->d_scalar, 4, hipMemcpyDeviceToHost,
                                      ctx->stream));
        WGML_CHECK_HIP(hipStreamSynchronize(ctx->stream));
        const uint32_t best = ctx->h_scalar[0];
        out_tokens[pos] = best;
        // forced prompt tokens win over the sample (wgml-chat/src/sampler.rs:102-107)
        token = (pos + 1 < n_prompt) ? prompt[pos + 1] : best;
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
