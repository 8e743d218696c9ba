// Llama-architecture decoder built from the C-ABI operators of this library.
// Reference: models/kalosm-llama/src/raw/mod.rs:851-865, :925-1049 (Model::forward),
// raw/attention_layer.rs:130-237 (feed-forward), :281-426 / :514-694 (attention),
// raw/rope.rs:87-112 (interleaved RoPE for the llama architecture), model/inference.rs:11-396
// (decode loop, here greedy).
#include "fh_internal.h"

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <string>

struct fh_llama_layer {
    fh_qmatrix *wq = nullptr, *wk = nullptr, *wv = nullptr, *wo = nullptr;
    fh_qmatrix *gate = nullptr, *up = nullptr, *down = nullptr;
    fh_qmatrix *qkv = nullptr, *gate_up = nullptr;
    float *attn_norm = nullptr, *ffn_norm = nullptr;
};

struct fh_llama {
    fh_device *dev = nullptr;
    fh_llama_config c{};
    std::vector<fh_llama_layer> layers;
    fh_qmatrix *embd = nullptr, *output = nullptr;
    bool output_is_embd = false;
    float *out_norm = nullptr;
    float *cos_t = nullptr, *sin_t = nullptr;
    std::vector<float> rope_freq_weight; // rope_freqs.weight when the file has one
    bool has_rope_scaling = false;
    fh_rope_scaling rope_scaling = {};
    fh_kvcache *cache = nullptr;
    bool finalized = false;
    int pos = 0;
    // the token ids whose keys and values the cache holds (KvCache::tokens of the reference, raw/cache.rs): what a
    // forward pass re-runs the tail of when the context is full
    std::vector<uint32_t> history;
    // step buffers (sized for `cap_s` tokens)
    int cap_s = 0;
    uint32_t *ids = nullptr;
    float *x = nullptr, *xn = nullptr, *qkv = nullptr, *qrot = nullptr, *krot = nullptr, *att = nullptr, *att_t = nullptr,
          *attn_out = nullptr, *gu = nullptr, *act = nullptr, *ff = nullptr, *logits = nullptr;
    // greedy decode state
    uint32_t *tok_dev = nullptr, *out_tok_dev = nullptr;
    int *step_dev = nullptr;
    hipGraphExec_t graph_exec = nullptr;
    hipGraph_t graph = nullptr;
    int captured_capacity = -1;
    uint64_t captured_gen = 0, samp_gen = 0; // dev->scratch_gen at the captures
    uint64_t captured_opt = 0, samp_opt = 0; // dev->opt_gen at the captures (options pick the kernels of a step)
    // sampled decode state: [0..63] previous ids, [64] their count, [65] next slot, [66] Mirostat mu (f32),
    // [68..69] status and token of the last step, [128..] one random number per step
    uint32_t *samp_dev = nullptr;
    hipGraphExec_t samp_exec = nullptr;
    hipGraph_t samp_graph = nullptr;
    int samp_capacity = -1;
    uint32_t samp_range = 0;
    fh_sampler_params samp_params = {};
    // trace of the last fh_llama_forward (options trace_nan / trace_timing): the lines, and the stage marks
    std::string trace_text;
    std::vector<hipEvent_t> trace_ev;      // pool, reused from call to call
    std::vector<std::string> trace_label;  // label of the stage that ends at mark i (marks used: trace_label.size())
    int trace_first = -1, trace_last = -1; // the marks before the first and after the last layer
};

// Tracing of the eager forward pass, off unless an option (or the reference's environment variable, read when the
// device is created) switches it on.  Non-finite probes: KALOSM_TRACE_LAYER_NAN, raw/mod.rs:955-1041 - the reference
// looks at the embedding and layer 0 only (raw/mod.rs:20-22), this looks at every layer.  Timing:
// KALOSM_TRACE_FORWARD_TIMING ("[timing] text layer loop", raw/mod.rs:943-1043) and, per stage of a layer, the
// timestamp queries of FUSOR_TRACE_GPU_KERNELS (fusor-ml/core/src/compute_graph/resolve/run.rs:141, :483-497).
static void trace_line(fh_llama *m, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    m->trace_text += buf;
    m->trace_text += '\n';
    if (m->dev->opt_trace_stderr) fprintf(stderr, "%s\n", buf);
}
static fh_status trace_probe(fh_llama *m, const float *t, int rows, int cols, int layer, const char *label) {
    if (!m->dev->opt_trace_nan) return FH_OK;
    fh_finite_stats st;
    FH_TRY(fh_check_finite(m->dev, t, (int64_t)rows * cols, &st));
    if (!st.nan && !st.pos_inf && !st.neg_inf) return FH_OK;
    char idx[128];
    int o = 0;
    idx[0] = 0;
    for (uint32_t i = 0; i < st.first_nan_count; i++)
        o += snprintf(idx + o, sizeof idx - o, "%s%llu", i ? ", " : "", (unsigned long long)st.first_nan[i]);
    trace_line(m, "trace_nan layer=%d label=%s index_pos=%d shape=[1, %d, %d] nan=%llu (first_nan_indices=[%s]) +inf=%llu "
                  "-inf=%llu max_abs=%g",
               layer, label, m->pos, rows, cols, (unsigned long long)st.nan, idx, (unsigned long long)st.pos_inf,
               (unsigned long long)st.neg_inf, (double)st.max_abs);
    return FH_OK;
}
// Ends a stage: an event on the stream, labelled with what ran since the previous mark.  level: 1 marks belong to the
// layer-loop total, 2 to the per-stage trace.
static fh_status trace_mark(fh_llama *m, int level, int layer, const char *label) {
    if (m->dev->opt_trace_timing < level) return FH_OK;
    const size_t i = m->trace_label.size();
    if (i == m->trace_ev.size()) {
        hipEvent_t e;
        FH_HIP(hipEventCreate(&e));
        m->trace_ev.push_back(e);
    }
    FH_HIP(hipEventRecord(m->trace_ev[i], m->dev->stream));
    char buf[96];
    if (layer >= 0) snprintf(buf, sizeof buf, "layer %d %s", layer, label);
    else snprintf(buf, sizeof buf, "%s", label);
    m->trace_label.push_back(buf);
    return FH_OK;
}
// After the stream has been synchronised: one line per stage, then the total of the layer loop.
static fh_status trace_report(fh_llama *m, int s) {
    const int n = (int)m->trace_label.size();
    if (m->dev->opt_trace_timing >= 2)
        for (int i = 1; i < n; i++) {
            float ms = 0;
            FH_HIP(hipEventElapsedTime(&ms, m->trace_ev[i - 1], m->trace_ev[i]));
            trace_line(m, "[timing] %s: %.1f us", m->trace_label[i].c_str(), ms * 1e3);
        }
    if (m->trace_first >= 0 && m->trace_last > m->trace_first) {
        float ms = 0;
        FH_HIP(hipEventElapsedTime(&ms, m->trace_ev[m->trace_first], m->trace_ev[m->trace_last]));
        trace_line(m, "[timing] text layer loop: %.2f ms seq_len=%d", ms, s);
    }
    return FH_OK;
}

static void free_dev(void *p) {
    if (p) (void)hipFree(p);
}

extern "C" fh_status fh_llama_create(fh_device *dev, const fh_llama_config *cfg, fh_llama **out) {
    FH_REQUIRE(dev && cfg && out, "NULL argument");
    *out = nullptr;
    FH_REQUIRE(cfg->n_layers > 0 && cfg->d_model > 0 && cfg->n_heads > 0 && cfg->n_kv_heads > 0 && cfg->head_dim > 0 &&
                   cfg->ffn > 0 && cfg->vocab > 0 && cfg->ctx > 0,
               "bad decoder configuration");
    FH_REQUIRE(cfg->n_heads % cfg->n_kv_heads == 0, "n_heads %d not divisible by n_kv_heads %d", cfg->n_heads, cfg->n_kv_heads);
    FH_REQUIRE(cfg->head_dim == 64 || cfg->head_dim == 128, "head_dim %d unsupported (64 or 128)", cfg->head_dim);
    if (cfg->n_heads / cfg->n_kv_heads > 8)
        FH_FAIL(FH_ERR_UNSUPPORTED, "%d query heads per KV head: the decode-step attention handles groups of at most 8",
                cfg->n_heads / cfg->n_kv_heads);
    fh_llama *m = new fh_llama();
    m->dev = dev;
    m->c = *cfg;
    m->layers.resize(cfg->n_layers);
    *out = m;
    return FH_OK;
}

extern "C" fh_status fh_llama_set_rope_scaling(fh_llama *m, const fh_rope_scaling *scaling) {
    FH_REQUIRE(m, "NULL decoder");
    FH_REQUIRE(!m->finalized, "the RoPE tables are built by fh_llama_finalize: set the scaling before it");
    if (scaling) {
        FH_REQUIRE(scaling->factor != 0.0f && scaling->low_freq_factor != 0.0f && scaling->high_freq_factor != 0.0f,
                   "rope scaling factors must not be zero");
        m->rope_scaling = *scaling;
    }
    m->has_rope_scaling = scaling != nullptr;
    return FH_OK;
}

static void free_steps(fh_llama *m) {
    free_dev(m->ids); free_dev(m->x); free_dev(m->xn); free_dev(m->qkv); free_dev(m->qrot); free_dev(m->krot);
    free_dev(m->att); free_dev(m->att_t); free_dev(m->attn_out); free_dev(m->gu); free_dev(m->act); free_dev(m->ff);
    m->ids = nullptr;
    m->x = m->xn = m->qkv = m->qrot = m->krot = m->att = m->att_t = m->attn_out = m->gu = m->act = m->ff = nullptr;
    m->cap_s = 0;
    m->captured_capacity = -1; // a captured decode step holds these pointers
    m->samp_capacity = -1;
}

extern "C" fh_status fh_llama_destroy(fh_llama *m) {
    if (!m) return FH_OK;
    (void)hipStreamSynchronize(m->dev->stream);
    if (m->graph_exec) (void)hipGraphExecDestroy(m->graph_exec);
    if (m->graph) (void)hipGraphDestroy(m->graph);
    for (auto &l : m->layers) {
        fh_qmatrix_free(l.wq); fh_qmatrix_free(l.wk); fh_qmatrix_free(l.wv); fh_qmatrix_free(l.wo);
        fh_qmatrix_free(l.gate); fh_qmatrix_free(l.up); fh_qmatrix_free(l.down);
        fh_qmatrix_free(l.qkv); fh_qmatrix_free(l.gate_up);
        free_dev(l.attn_norm); free_dev(l.ffn_norm);
    }
    fh_qmatrix_free(m->embd);
    if (!m->output_is_embd) fh_qmatrix_free(m->output);
    free_dev(m->out_norm); free_dev(m->cos_t); free_dev(m->sin_t);
    free_dev(m->logits); free_dev(m->tok_dev); free_dev(m->out_tok_dev); free_dev(m->step_dev); free_dev(m->samp_dev);
    if (m->samp_exec) (void)hipGraphExecDestroy(m->samp_exec);
    if (m->samp_graph) (void)hipGraphDestroy(m->samp_graph);
    free_steps(m);
    fh_kvcache_destroy(m->cache);
    for (hipEvent_t e : m->trace_ev) (void)hipEventDestroy(e);
    delete m;
    return FH_OK;
}

static fh_status load_f32(fh_llama *m, float **dst, int64_t want, int64_t n, int64_t k, const void *bytes, size_t len,
                          const char *name) {
    int64_t count = n * (k > 0 ? k : 1);
    FH_REQUIRE(count == want && len == (size_t)want * 4, "%s: expected %lld f32 values, got [%lld, %lld] / %zu bytes", name,
               (long long)want, (long long)n, (long long)k, len);
    free_dev(*dst);
    *dst = nullptr;
    FH_TRY(fh_malloc(m->dev, len, (void **)dst));
    return fh_upload(m->dev, *dst, bytes, len);
}

extern "C" fh_status fh_llama_load_tensor(fh_llama *m, const char *name, uint32_t ggml_type, int64_t n, int64_t k,
                                          const void *bytes, size_t len) {
    FH_REQUIRE(m && name && bytes, "NULL argument");
    FH_REQUIRE(!m->finalized, "decoder already finalized");
    const fh_llama_config &c = m->c;
    const int64_t D = c.d_model, QD = (int64_t)c.n_heads * c.head_dim, KD = (int64_t)c.n_kv_heads * c.head_dim;
    auto loadq = [&](fh_qmatrix **dst, int64_t wn, int64_t wk) -> fh_status {
        FH_REQUIRE(n == wn && k == wk, "%s: expected [%lld, %lld], got [%lld, %lld]", name, (long long)wn, (long long)wk,
                   (long long)n, (long long)k);
        fh_qmatrix_free(*dst);
        *dst = nullptr;
        return fh_qmatrix_from_gguf_bytes(m->dev, ggml_type, n, k, bytes, len, dst);
    };
    if (!strcmp(name, "token_embd.weight")) return loadq(&m->embd, c.vocab, D);
    if (!strcmp(name, "output.weight")) return loadq(&m->output, c.vocab, D);
    if (!strcmp(name, "output_norm.weight")) return load_f32(m, &m->out_norm, D, n, k, bytes, len, name);
    if (!strcmp(name, "rope_freqs.weight")) {
        const int64_t half = c.head_dim / 2, count = n * (k > 0 ? k : 1);
        FH_REQUIRE(ggml_type == 0 && count == half && len == (size_t)half * 4,
                   "%s: expected %lld f32 values, got type %u [%lld, %lld] / %zu bytes", name, (long long)half, ggml_type,
                   (long long)n, (long long)k, len);
        m->rope_freq_weight.resize((size_t)half);
        memcpy(m->rope_freq_weight.data(), bytes, len);
        return FH_OK;
    }
    int li = -1;
    char field[64] = "";
    if (sscanf(name, "blk.%d.%63s", &li, field) == 2 && li >= 0 && li < c.n_layers) {
        fh_llama_layer &l = m->layers[li];
        if (!strcmp(field, "attn_q.weight")) return loadq(&l.wq, QD, D);
        if (!strcmp(field, "attn_k.weight")) return loadq(&l.wk, KD, D);
        if (!strcmp(field, "attn_v.weight")) return loadq(&l.wv, KD, D);
        if (!strcmp(field, "attn_output.weight")) return loadq(&l.wo, D, QD);
        if (!strcmp(field, "ffn_gate.weight")) return loadq(&l.gate, c.ffn, D);
        if (!strcmp(field, "ffn_up.weight")) return loadq(&l.up, c.ffn, D);
        if (!strcmp(field, "ffn_down.weight")) return loadq(&l.down, D, c.ffn);
        if (!strcmp(field, "attn_norm.weight")) return load_f32(m, &l.attn_norm, D, n, k, bytes, len, name);
        if (!strcmp(field, "ffn_norm.weight")) return load_f32(m, &l.ffn_norm, D, n, k, bytes, len, name);
    }
    FH_FAIL(FH_ERR_INVALID, "unknown tensor name '%s'", name);
}

static fh_status ensure_steps(fh_llama *m, int s) {
    if (s <= m->cap_s) return FH_OK;
    (void)hipStreamSynchronize(m->dev->stream);
    free_steps(m);
    const fh_llama_config &c = m->c;
    const size_t D = c.d_model, QD = (size_t)c.n_heads * c.head_dim, KD = (size_t)c.n_kv_heads * c.head_dim, F = c.ffn;
    size_t S = (size_t)s;
    FH_TRY(fh_malloc(m->dev, S * 4, (void **)&m->ids));
    FH_TRY(fh_malloc(m->dev, S * D * 4, (void **)&m->x));
    FH_TRY(fh_malloc(m->dev, S * D * 4, (void **)&m->xn));
    FH_TRY(fh_malloc(m->dev, S * (QD + 2 * KD) * 4, (void **)&m->qkv));
    FH_TRY(fh_malloc(m->dev, S * QD * 4, (void **)&m->qrot));
    FH_TRY(fh_malloc(m->dev, S * KD * 4, (void **)&m->krot));
    FH_TRY(fh_malloc(m->dev, S * QD * 4, (void **)&m->att));
    FH_TRY(fh_malloc(m->dev, S * QD * 4, (void **)&m->att_t));
    FH_TRY(fh_malloc(m->dev, S * D * 4, (void **)&m->attn_out));
    FH_TRY(fh_malloc(m->dev, S * 2 * F * 4, (void **)&m->gu));
    FH_TRY(fh_malloc(m->dev, S * F * 4, (void **)&m->act));
    FH_TRY(fh_malloc(m->dev, S * D * 4, (void **)&m->ff));
    m->cap_s = s;
    return FH_OK;
}

extern "C" fh_status fh_llama_finalize(fh_llama *m) {
    FH_REQUIRE(m, "NULL argument");
    FH_REQUIRE(!m->finalized, "decoder already finalized");
    const fh_llama_config &c = m->c;
    FH_REQUIRE(m->embd && m->out_norm, "token_embd.weight / output_norm.weight missing");
    if (!m->output) { // falls back to the embedding table, raw/mod.rs:480-486
        m->output = m->embd;
        m->output_is_embd = true;
    }
    for (int i = 0; i < c.n_layers; i++) {
        fh_llama_layer &l = m->layers[i];
        FH_REQUIRE(l.wq && l.wk && l.wv && l.wo && l.gate && l.up && l.down && l.attn_norm && l.ffn_norm,
                   "layer %d is missing tensors", i);
        if (c.fuse_qkv) {
            const fh_qmatrix *parts[3] = {l.wq, l.wk, l.wv};
            fh_status st = fh_qmatrix_concat_rows(m->dev, parts, 3, &l.qkv);
            if (st == FH_OK) {
                FH_HIP(hipStreamSynchronize(m->dev->stream));
                fh_qmatrix_free(l.wq); fh_qmatrix_free(l.wk); fh_qmatrix_free(l.wv);
                l.wq = l.wk = l.wv = nullptr;
            } else if (st != FH_ERR_UNSUPPORTED) return st;
        }
        if (c.fuse_gate_up) {
            const fh_qmatrix *parts[2] = {l.gate, l.up};
            fh_status st = fh_qmatrix_concat_rows(m->dev, parts, 2, &l.gate_up);
            if (st == FH_OK) {
                FH_HIP(hipStreamSynchronize(m->dev->stream));
                fh_qmatrix_free(l.gate); fh_qmatrix_free(l.up);
                l.gate = l.up = nullptr;
            } else if (st != FH_ERR_UNSUPPORTED) return st;
        }
    }
    size_t tbl = (size_t)c.ctx * (c.head_dim / 2) * 4;
    FH_TRY(fh_malloc(m->dev, tbl, (void **)&m->cos_t));
    FH_TRY(fh_malloc(m->dev, tbl, (void **)&m->sin_t));
    FH_TRY(fh_rope_tables_scaled(m->dev, c.head_dim, c.ctx, c.theta, m->has_rope_scaling ? &m->rope_scaling : nullptr,
                                 m->rope_freq_weight.empty() ? nullptr : m->rope_freq_weight.data(), m->cos_t, m->sin_t));
    FH_TRY(fh_kvcache_create(m->dev, c.n_layers, c.n_kv_heads, c.head_dim, c.ctx, c.kv_dtype, &m->cache));
    FH_TRY(fh_malloc(m->dev, (size_t)c.vocab * 4, (void **)&m->logits));
    FH_TRY(fh_malloc(m->dev, 256, (void **)&m->tok_dev));
    FH_TRY(fh_malloc(m->dev, (size_t)c.ctx * 4 + 256, (void **)&m->out_tok_dev));
    FH_TRY(fh_malloc(m->dev, 256, (void **)&m->step_dev));
    FH_TRY(fh_malloc(m->dev, (size_t)(128 + c.ctx) * 4, (void **)&m->samp_dev));
    FH_TRY(ensure_steps(m, 1));
    m->finalized = true;
    return FH_OK;
}

extern "C" fh_status fh_llama_reset(fh_llama *m) {
    FH_REQUIRE(m && m->finalized, "decoder not finalized");
    m->pos = 0;
    m->history.clear();
    return fh_kvcache_reset(m->cache);
}

extern "C" fh_status fh_llama_weight_bytes(const fh_llama *m, uint64_t *bytes) {
    FH_REQUIRE(m && bytes, "NULL argument");
    uint64_t t = 0;
    auto add = [&](const fh_qmatrix *q) {
        if (q) t += (uint64_t)q->n * q->kb * fh_block_bytes(q->type);
    };
    for (auto &l : m->layers) {
        add(l.wq); add(l.wk); add(l.wv); add(l.wo); add(l.gate); add(l.up); add(l.down); add(l.qkv); add(l.gate_up);
    }
    add(m->output); // the lm-head; the embedding table contributes one row per token
    *bytes = t;
    return FH_OK;
}

// One decoder pass over `s` tokens whose ids are already in m->ids.  dev_pos: read the position
// from the cache's device-side length (graph replay, s == 1) instead of m->pos.
static fh_status run_layers(fh_llama *m, int s, bool dev_pos) {
    const fh_llama_config &c = m->c;
    fh_device *dev = m->dev;
    const int D = c.d_model, H = c.n_heads, HK = c.n_kv_heads, hd = c.head_dim, F = c.ffn;
    const int QD = H * hd, KD = HK * hd;
    const int pos = m->pos;
    const float scale = (float)(1.0 / sqrt((double)hd)); // attention_layer.rs:674
    FH_TRY(fh_embed_rows(m->embd, m->ids, nullptr, s, m->x));
    const bool trace = !dev_pos && (dev->opt_trace_nan || dev->opt_trace_timing); // never inside a captured step
    if (trace) {
        FH_TRY(trace_probe(m, m->x, s, D, -1, "embed"));
        FH_TRY(trace_mark(m, 1, -1, "embed"));
        m->trace_first = (int)m->trace_label.size() - 1;
    }
    for (int li = 0; li < c.n_layers; li++) {
        fh_llama_layer &l = m->layers[li];
        // Decode steps fold each rms_norm into the matvec that consumes it (one launch instead of two).
        const bool fuse = dev_pos && s == 1 && dev->opt_fuse_norm == 0 && dev->opt_matvec_kernel == 0;
        bool qkv_done = false, wo_done = false, xacc = false;
        bool rope_done = false;
        if (fuse && l.qkv && l.qkv->type == FH_Q4_K) {
            // norm + projection + rope + cache append in one launch; without the rope epilogue as second choice
            fh_status st = fh_launch_q4k_m1_ropekv(l.qkv, m->x, l.attn_norm, c.eps, m->cache, li, H, m->cos_t, m->sin_t, c.ctx,
                                                   m->qrot);
            rope_done = st == FH_OK;
            if (st == FH_ERR_UNSUPPORTED)
                st = fh_launch_q4k_m1_norm(l.qkv, m->x, nullptr, l.attn_norm, c.eps, m->qkv, FH_EPI_NONE, nullptr, nullptr);
            if (st != FH_ERR_UNSUPPORTED) FH_TRY(st);
            qkv_done = st == FH_OK;
        }
        if (!qkv_done) FH_TRY(fh_rms_norm(dev, m->x, nullptr, l.attn_norm, nullptr, c.eps, s, D, m->xn));
        const float *qp, *kp, *vp;
        int64_t row;
        if (l.qkv) {
            if (!qkv_done) FH_TRY(fh_qmatmul(l.qkv, m->xn, s, m->qkv));
            row = QD + 2 * KD;
            qp = m->qkv;
            kp = m->qkv + QD;
            vp = m->qkv + QD + KD;
        } else {
            float *qb = m->qkv, *kb2 = m->qkv + (size_t)s * QD, *vb = kb2 + (size_t)s * KD;
            FH_TRY(fh_qmatmul(l.wq, m->xn, s, qb));
            FH_TRY(fh_qmatmul(l.wk, m->xn, s, kb2));
            FH_TRY(fh_qmatmul(l.wv, m->xn, s, vb));
            row = 0; // per-tensor strides below
            qp = qb; kp = kb2; vp = vb;
        }
        const int64_t q_st = row ? row : QD, k_st = row ? row : KD;
        if (trace) {
            FH_TRY(trace_probe(m, m->xn, s, D, li, "post_attn_norm"));
            FH_TRY(trace_mark(m, 2, li, "attn_norm+qkv"));
        }
        if (dev_pos) {
            if (!rope_done) FH_TRY(fh_rope_kv_decode(m->cache, li, qp, kp, vp, H, m->cos_t, m->sin_t, c.ctx, m->qrot));
            size_t plane = (size_t)HK * m->cache->capacity * hd * fh_dtype_size(c.kv_dtype);
            const uint8_t *kc = (const uint8_t *)m->cache->k + li * plane, *vc = (const uint8_t *)m->cache->v + li * plane;
            // The partial results of the attention splits are merged by the output projection itself when it is a
            // Q4_K matrix (no launch for the merge); otherwise by a small kernel.
            const bool merge_in_wo = fuse && l.wo->type == FH_Q4_K && hd == 128;
            int nsplit = 0;
            fh_status ast = dev->opt_attn_kernel == 1
                                ? FH_ERR_UNSUPPORTED
                                : fh_attention_decode_devlen(dev, c.kv_dtype, m->qrot, kc, vc, (int64_t)m->cache->capacity * hd,
                                                             hd, H, HK, hd, scale, m->cache->len_dev, m->cache->capacity,
                                                             merge_in_wo ? nullptr : m->att, &nsplit);
            const bool parts = ast != FH_ERR_UNSUPPORTED; // the attention left partial results per key split
            if (!parts)
                ast = fh_attention_decode_devlen_v1(dev, c.kv_dtype, m->qrot, kc, vc, (int64_t)m->cache->capacity * hd, hd, H,
                                                    HK, hd, scale, m->cache->len_dev, m->cache->capacity, m->att);
            if (parts && ast == FH_OK && merge_in_wo) {
                // first choice: x += Wo . att with k split over small workgroups; the residual stream then already
                // holds x + attn for the FFN norm and the final sum ((ffn + attn) + residual, raw/mod.rs:1036)
                fh_status st = (dev->opt_wo_acc == 1 || dev->opt_deterministic) ? FH_ERR_UNSUPPORTED
                                                    : fh_launch_q4k_m1_attn_acc(l.wo, dev->part_buf, nsplit, m->x);
                xacc = st == FH_OK;
                if (st == FH_ERR_UNSUPPORTED) st = fh_launch_q4k_m1_attn(l.wo, dev->part_buf, nsplit, m->attn_out);
                if (st == FH_ERR_UNSUPPORTED) st = fh_attention_combine_dl(dev, H, nsplit, m->att);
                else wo_done = st == FH_OK;
                ast = st;
            }
            FH_TRY(ast);
        } else {
            FH_TRY(fh_rope_pair(dev, qp, 0, hd, q_st, kp, 0, hd, k_st, 1, H, HK, s, hd, m->cos_t, m->sin_t, c.ctx, pos, 1,
                                m->qrot, m->krot));
            FH_TRY(fh_kvcache_reserve(m->cache, pos + s));
            // K (rotated) is [HK, s, hd] contiguous; V is a view of the projection output
            FH_TRY(fh_kvcache_append_kv(m->cache, li, m->krot, (int64_t)s * hd, hd, vp, hd, k_st, s, pos));
            size_t plane = (size_t)HK * m->cache->capacity * hd * fh_dtype_size(c.kv_dtype);
            const uint8_t *kc = (const uint8_t *)m->cache->k + li * plane, *vc = (const uint8_t *)m->cache->v + li * plane;
            FH_TRY(fh_flash_attention_ex(dev, FH_F32, c.kv_dtype, m->qrot, 0, (int64_t)s * hd, hd, kc, vc, 0,
                                         (int64_t)m->cache->capacity * hd, hd, 1, H, HK, s, pos + s, hd, scale,
                                         s > 1 ? FH_MASK_CAUSAL : FH_MASK_NONE, nullptr, m->att));
        }
        if (trace) FH_TRY(trace_mark(m, 2, li, "rope+cache+attention"));
        const float *att_in = m->att; // [H, s, hd]; for s == 1 this already is [s, H*hd]
        if (s > 1) {
            FH_TRY(fh_transpose_shd(dev, m->att, H, s, hd, m->att_t));
            att_in = m->att_t;
        }
        if (!wo_done) FH_TRY(fh_qmatmul(l.wo, att_in, s, m->attn_out));
        if (trace) {
            FH_TRY(trace_probe(m, m->attn_out, s, D, li, "attn_out"));
            FH_TRY(trace_mark(m, 2, li, "wo"));
        }
        // input of the FFN norm: attn + residual, or the residual stream alone when it already holds the sum
        const float *hin = xacc ? m->x : m->attn_out, *hres = xacc ? nullptr : m->x, *hadd = xacc ? nullptr : m->attn_out;
        bool ffn_done = false, late_swiglu = false;
        if (fuse && l.gate_up && l.gate_up->type == FH_Q4_K) {
            // On request (down_splitk = 3; measured slower on MI355X) SwiGLU moves into the staging of a split-k Q6_K down
            // projection: the gate | up
            // projection then runs in its plain (fastest) form and writes both halves.
            late_swiglu = l.down->type == FH_Q6_K && dev->opt_down_splitk == 3 && !dev->opt_deterministic &&
                          l.down->kb % 4 == 0 && l.down->kb >= 8;
            fh_status st = late_swiglu ? fh_launch_q4k_m1_norm(l.gate_up, hin, hres, l.ffn_norm, c.eps, m->gu, FH_EPI_NONE,
                                                               nullptr, nullptr)
                                       : fh_launch_q4k_m1_norm(l.gate_up, hin, hres, l.ffn_norm, c.eps, m->act,
                                                               FH_EPI_SWIGLU, nullptr, nullptr);
            if (st != FH_ERR_UNSUPPORTED) FH_TRY(st);
            ffn_done = st == FH_OK;
            late_swiglu = late_swiglu && ffn_done;
        }
        if (!ffn_done) FH_TRY(fh_rms_norm(dev, hin, hres, l.ffn_norm, nullptr, c.eps, s, D, m->xn));
        if (ffn_done) {
        } else if (l.gate_up && s <= 2) {
            FH_TRY(fh_qmatmul_swiglu(l.gate_up, m->xn, s, m->act));
        } else if (l.gate_up) {
            FH_TRY(fh_qmatmul(l.gate_up, m->xn, s, m->gu)); // [s, 2F]: gate | up per row
            // split the halves: silu(gate) * up with row stride 2F
            FH_TRY(fh_swiglu_rows(dev, m->gu, s, F, m->act));
        } else {
            FH_TRY(fh_qmatmul(l.gate, m->xn, s, m->gu));
            FH_TRY(fh_qmatmul(l.up, m->xn, s, m->gu + (size_t)s * F));
            FH_TRY(fh_swiglu(dev, m->gu, m->gu + (size_t)s * F, m->act, (int64_t)s * F));
        }
        if (trace) FH_TRY(trace_mark(m, 2, li, "ffn_norm+gate_up+swiglu"));
        if (s == 1) { // forward_add_residuals, attention_layer.rs:147-174: (down(act) + attn) + residual
            fh_status st = FH_ERR_UNSUPPORTED;
            if (late_swiglu) { // x += down(silu(gate) * up) + attn
                st = fh_launch_q6k_m1_acc(l.down, m->gu, m->gu + F, m->x, hadd);
                if (st == FH_ERR_UNSUPPORTED) FH_TRY(fh_swiglu(dev, m->gu, m->gu + F, m->act, F));
            } else if (fuse && l.down->type == FH_Q6_K && dev->opt_down_splitk != 1 && !dev->opt_deterministic) {
                st = fh_launch_q6k_m1_acc(l.down, m->act, nullptr, m->x, hadd); // x += down(act) [+ attn]
            }
            if (st == FH_ERR_UNSUPPORTED && xacc) { // x already holds x + attn
                FH_TRY(fh_qmatmul(l.down, m->act, 1, m->ff));
                st = fh_add3(dev, m->ff, m->x, nullptr, m->x, D);
            } else if (st == FH_ERR_UNSUPPORTED) {
                st = fh_qmatmul_add2(l.down, m->act, 1, m->attn_out, m->x, m->x);
            }
            FH_TRY(st);
        } else {      // raw/mod.rs:1036
            FH_TRY(fh_qmatmul(l.down, m->act, s, m->ff));
            FH_TRY(fh_add3(dev, m->ff, m->attn_out, m->x, m->x, (int64_t)s * D));
        }
        if (trace) {
            FH_TRY(trace_probe(m, m->x, s, D, li, s == 1 ? "ffn_fused" : "ffn_unfused"));
            FH_TRY(trace_mark(m, 2, li, "down+residuals"));
        }
    }
    if (trace) {
        if (dev->opt_trace_timing == 1) FH_TRY(trace_mark(m, 1, -1, "layers"));
        m->trace_last = (int)m->trace_label.size() - 1;
    }
    FH_TRY(fh_rms_norm(dev, m->x + (size_t)(s - 1) * D, nullptr, m->out_norm, nullptr, c.eps, 1, D, m->xn));
    FH_TRY(fh_qmatmul(m->output, m->xn, 1, m->logits));
    if (trace) FH_TRY(trace_mark(m, 2, -1, "out_norm+lm_head"));
    return FH_OK;
}

extern "C" fh_status fh_llama_forward(fh_llama *m, const uint32_t *tokens_host, int32_t count, float *logits_host,
                                      float *hidden_host) {
    FH_REQUIRE(m && m->finalized && tokens_host, "decoder not finalized or NULL tokens");
    FH_REQUIRE(count > 0 && count <= 65535, "count %d out of range", count);
    for (int i = 0; i < count; i++)
        FH_REQUIRE(tokens_host[i] < (uint32_t)m->c.vocab, "token id %u at %d outside the vocabulary of %d", tokens_host[i], i,
                   m->c.vocab);
    // Model::forward, raw/mod.rs:769-801: when the new tokens do not fit the context, the cache is cleared and the last
    // context_length - 32 (at least 8) of all tokens, cached and new, are run again from position 0.
    std::vector<uint32_t> trimmed;
    if (m->pos + count > m->c.ctx) {
        const int cutoff = std::max(m->c.ctx - 32, 8);
        FH_REQUIRE(cutoff <= m->c.ctx && cutoff <= 65535, "context of %d positions is too short to trim to %d", m->c.ctx, cutoff);
        FH_REQUIRE((int)m->history.size() == m->pos, "the cache holds %d positions but %zu token ids are on record", m->pos,
                   m->history.size());
        trimmed = m->history;
        trimmed.insert(trimmed.end(), tokens_host, tokens_host + count);
        trimmed.erase(trimmed.begin(), trimmed.end() - cutoff);
        FH_TRY(fh_llama_reset(m));
        tokens_host = trimmed.data();
        count = cutoff;
    }
    FH_TRY(ensure_steps(m, count));
    FH_TRY(fh_upload(m->dev, m->ids, tokens_host, (size_t)count * 4));
    m->trace_text.clear();
    m->trace_label.clear();
    m->trace_first = m->trace_last = -1;
    FH_TRY(run_layers(m, count, false));
    // all layers appended: advance the cache
    m->history.insert(m->history.end(), tokens_host, tokens_host + count);
    m->pos += count;
    m->cache->len = m->pos;
    FH_TRY(fh_kvcache_set_len_dev(m->cache, m->pos));
    if (hidden_host) FH_TRY(fh_download(m->dev, hidden_host, m->xn, (size_t)m->c.d_model * 4));
    if (logits_host) FH_TRY(fh_download(m->dev, logits_host, m->logits, (size_t)m->c.vocab * 4));
    FH_TRY(fh_device_sync(m->dev));
    if (m->dev->opt_trace_timing) FH_TRY(trace_report(m, count));
    return FH_OK;
}

extern "C" fh_status fh_llama_trace_text(const fh_llama *m, char *buf, size_t capacity, size_t *length) {
    FH_REQUIRE(m && (buf || capacity == 0), "NULL argument");
    if (length) *length = m->trace_text.size();
    if (capacity) {
        const size_t n = std::min(capacity - 1, m->trace_text.size());
        memcpy(buf, m->trace_text.data(), n);
        buf[n] = 0;
    }
    return FH_OK;
}

__global__ void k_set_u32(uint32_t *p, uint32_t v) { *p = v; }

static fh_status decode_step_enqueue(fh_llama *m) {
    FH_TRY(run_layers(m, 1, true));
    // the last stage of the pick also stores the token, feeds it to the next step and advances the cache length
    return fh_argmax_step(m->dev, m->logits, m->c.vocab, m->tok_dev,
                          FhStepTail{m->ids, m->out_tok_dev, m->step_dev, m->cache->len_dev});
}

extern "C" fh_status fh_llama_decode_greedy(fh_llama *m, uint32_t first_token, int32_t steps, uint32_t *out_tokens_host,
                                            float *elapsed_ms) {
    FH_REQUIRE(m && m->finalized && out_tokens_host, "decoder not finalized or NULL output");
    FH_REQUIRE(steps > 0 && m->pos + steps <= m->c.ctx,
               "context overflow: %d + %d > %d (the device-side loops stop at the context length; fh_llama_forward trims)", m->pos,
               steps, m->c.ctx);
    FH_REQUIRE(first_token < (uint32_t)m->c.vocab, "token id %u outside the vocabulary", first_token);
    fh_device *dev = m->dev;
    hipStream_t s = dev->stream;
    // capacity is fixed for the whole run so that no reallocation happens between steps
    FH_TRY(fh_kvcache_reserve(m->cache, m->pos + steps));
    k_set_u32<<<1, 1, 0, s>>>(m->ids, first_token);
    k_set_u32<<<1, 1, 0, s>>>((uint32_t *)m->step_dev, 0u);
    FH_HIP(hipGetLastError());
    int done = 0;
    if (m->c.use_graph) {
        // One eager step sizes every scratch buffer and sets kernel attributes; the capture then
        // records launches only.  The graph depends on the cache capacity (strides), so it is
        // rebuilt when the capacity changed since the last capture.
        if (!m->graph_exec || m->captured_capacity != m->cache->capacity || m->captured_gen != dev->scratch_gen ||
            m->captured_opt != dev->opt_gen) {
            FH_TRY(fh_timer_start(dev));
            FH_TRY(decode_step_enqueue(m));
            done = 1;
            FH_HIP(hipStreamSynchronize(s));
            if (m->graph_exec) { (void)hipGraphExecDestroy(m->graph_exec); m->graph_exec = nullptr; }
            if (m->graph) { (void)hipGraphDestroy(m->graph); m->graph = nullptr; }
            FH_HIP(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
            fh_status st = decode_step_enqueue(m);
            hipError_t e = hipStreamEndCapture(s, &m->graph);
            if (st != FH_OK) return st;
            FH_HIP(e);
            FH_HIP(hipGraphInstantiate(&m->graph_exec, m->graph, nullptr, nullptr, 0));
            m->captured_capacity = m->cache->capacity;
            m->captured_gen = dev->scratch_gen;
            m->captured_opt = dev->opt_gen;
        } else {
            FH_TRY(fh_timer_start(dev));
        }
        for (; done < steps; done++) FH_HIP(hipGraphLaunch(m->graph_exec, s));
    } else {
        FH_TRY(fh_timer_start(dev));
        for (; done < steps; done++) FH_TRY(decode_step_enqueue(m));
    }
    float ms = 0.f;
    FH_TRY(fh_timer_stop(dev, &ms));
    if (elapsed_ms) *elapsed_ms = ms;
    m->pos += steps;
    m->cache->len = m->pos;
    FH_TRY(fh_download(dev, out_tokens_host, m->out_tok_dev, (size_t)steps * 4));
    m->history.push_back(first_token); // the cache now holds the step inputs: the first token and all outputs but the last
    m->history.insert(m->history.end(), out_tokens_host, out_tokens_host + steps - 1);
    return FH_OK;
}

// Sampled decode (models/kalosm-llama/src/model/inference.rs:38-173, forward.rs:346-404): the sampled id stays in
// device memory and feeds the next step; it also joins the window of previous ids that the repetition penalty
// looks at (membership only, so the window is a ring).
__global__ void k_store_sampled(const uint32_t *result, uint32_t *ids, uint32_t *out, int *step, uint32_t *prev,
                                uint32_t range, int *kv_len) {
    *kv_len = *kv_len + 1;
    const uint32_t t = result[0] == FH_SAMPLE_STATUS_SAMPLED ? result[1] : 0xFFFFFFFFu;
    const uint32_t next = t == 0xFFFFFFFFu ? 0u : t;
    ids[0] = next;
    out[*step] = t;
    *step = *step + 1;
    if (range) {
        const uint32_t slot = prev[65];
        prev[slot] = next;
        prev[65] = slot + 1 == range ? 0u : slot + 1;
        if (prev[64] < range) prev[64] = prev[64] + 1;
    }
}

static fh_status sampled_step_enqueue(fh_llama *m) {
    FH_TRY(run_layers(m, 1, true));
    uint32_t *sd = m->samp_dev;
    FH_TRY(fh_sample_token_dev(m->dev, m->logits, m->c.vocab, &m->samp_params, sd, sd + 64, 0, (const float *)(sd + 128),
                               m->step_dev, (float *)(sd + 66), sd + 68, nullptr, nullptr));
    k_store_sampled<<<1, 1, 0, m->dev->stream>>>(sd + 68, m->ids, m->out_tok_dev, m->step_dev, sd, m->samp_range,
                                                m->cache->len_dev);
    FH_HIP(hipGetLastError());
    return FH_OK;
}

extern "C" fh_status fh_llama_decode_sampled(fh_llama *m, uint32_t first_token, int32_t steps,
                                             const fh_sampler_params *params, const float *randoms_host,
                                             const uint32_t *previous_host, uint32_t n_previous, uint32_t repetition_range,
                                             float *mu, uint32_t *out_tokens_host, float *elapsed_ms) {
    FH_REQUIRE(m && m->finalized && out_tokens_host && params && randoms_host, "decoder not finalized or NULL argument");
    FH_REQUIRE(steps > 0 && m->pos + steps <= m->c.ctx,
               "context overflow: %d + %d > %d (the device-side loops stop at the context length; fh_llama_forward trims)", m->pos,
               steps, m->c.ctx);
    FH_REQUIRE(first_token < (uint32_t)m->c.vocab, "token id %u outside the vocabulary", first_token);
    FH_REQUIRE(n_previous == 0 || previous_host, "previous tokens missing");
    FH_REQUIRE(params->kind != FH_SAMPLER_MIROSTAT2 || mu, "Mirostat 2 needs its state");
    fh_device *dev = m->dev;
    hipStream_t s = dev->stream;
    const uint32_t range = repetition_range < FH_SAMPLER_PREVIOUS_TOKENS ? repetition_range : FH_SAMPLER_PREVIOUS_TOKENS;
    // window = the last `range` ids of (history, first_token)
    uint32_t head[128] = {0};
    uint32_t len = 0;
    if (range) {
        const uint32_t keep = n_previous < range - 1 ? n_previous : range - 1;
        for (uint32_t i = 0; i < keep; i++) head[len++] = previous_host[n_previous - keep + i];
        head[len++] = first_token;
    }
    head[64] = len;
    head[65] = range ? len % range : 0u;
    const float mu0 = mu ? *mu : 0.f;
    memcpy(&head[66], &mu0, 4);
    FH_TRY(fh_upload(dev, m->samp_dev, head, sizeof(head)));
    FH_TRY(fh_upload(dev, m->samp_dev + 128, randoms_host, (size_t)steps * 4));
    FH_TRY(fh_kvcache_reserve(m->cache, m->pos + steps));
    k_set_u32<<<1, 1, 0, s>>>(m->ids, first_token);
    k_set_u32<<<1, 1, 0, s>>>((uint32_t *)m->step_dev, 0u);
    FH_HIP(hipGetLastError());
    int done = 0;
    if (m->c.use_graph) {
        // the captured step holds the sampler's parameters and the window size as kernel arguments
        fh_sampler_params want = *params;
        want.random = 0.f; // every step takes its number from randoms_host
        const bool same = m->samp_exec && m->samp_capacity == m->cache->capacity && m->samp_range == range &&
                          m->samp_gen == dev->scratch_gen && m->samp_opt == dev->opt_gen &&
                          memcmp(&m->samp_params, &want, sizeof(want)) == 0;
        m->samp_params = want;
        m->samp_range = range;
        if (!same) {
            FH_TRY(fh_timer_start(dev));
            FH_TRY(sampled_step_enqueue(m));
            done = 1;
            FH_HIP(hipStreamSynchronize(s));
            if (m->samp_exec) { (void)hipGraphExecDestroy(m->samp_exec); m->samp_exec = nullptr; }
            if (m->samp_graph) { (void)hipGraphDestroy(m->samp_graph); m->samp_graph = nullptr; }
            m->samp_capacity = -1;
            FH_HIP(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
            fh_status st = sampled_step_enqueue(m);
            hipError_t e = hipStreamEndCapture(s, &m->samp_graph);
            if (st != FH_OK) return st;
            FH_HIP(e);
            FH_HIP(hipGraphInstantiate(&m->samp_exec, m->samp_graph, nullptr, nullptr, 0));
            m->samp_capacity = m->cache->capacity;
            m->samp_gen = dev->scratch_gen;
            m->samp_opt = dev->opt_gen;
        } else {
            FH_TRY(fh_timer_start(dev));
        }
        for (; done < steps; done++) FH_HIP(hipGraphLaunch(m->samp_exec, s));
    } else {
        m->samp_params = *params;
        m->samp_range = range;
        FH_TRY(fh_timer_start(dev));
        for (; done < steps; done++) FH_TRY(sampled_step_enqueue(m));
    }
    float ms = 0.f;
    FH_TRY(fh_timer_stop(dev, &ms));
    if (elapsed_ms) *elapsed_ms = ms;
    m->pos += steps;
    m->cache->len = m->pos;
    FH_TRY(fh_download(dev, out_tokens_host, m->out_tok_dev, (size_t)steps * 4));
    if (mu) FH_TRY(fh_download(dev, mu, m->samp_dev + 66, 4));
    m->history.push_back(first_token);
    m->history.insert(m->history.end(), out_tokens_host, out_tokens_host + steps - 1);
    return FH_OK;
}
