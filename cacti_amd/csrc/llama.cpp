// The LLaMA training cycle staged on the spine, and the runtime's C ABI.
// Llama::apply, src/librarium/llama.rs:420-548; step recipe,
// examples/open_llama_3b_train.rs:350-389.
#include <math.h>
#include <string.h>

#include <string>

#include "../../include/cacti_hip_runtime.h"
#include "common.h"
#include "thunks.h"

using namespace cacti;

struct cacti_ctx {
    Ctx c;
};

struct LayerCells {
    CellPtr pre_norm, q, k, v, o, post_norm, gate, up, down;
};

struct cacti_llama {
    cacti_ctx *ctx;
    cacti_llama_cfg cfg;
    std::vector<CellPtr> params, grads;
    std::vector<CellPtr> master, grad_avg, grad2_avg;           // f32 optimiser state (adamw_init)
    std::vector<std::string> names;
    CellPtr embed, head_norm, lm_head;
    std::vector<LayerCells> layers;
    CellPtr cos, sin;
    CellPtr in_tok, in_lm_tok, in_loss_scale;
    CellPtr out_logit = 0, out_loss = 0, out_amax = 0, out_prob = 0;
};

namespace {

CellPtr new_param(cacti_llama *m, const std::string &name, std::vector<int64_t> shape)
{
    Ctx &c = m->ctx->c;
    CellPtr p = c.cell_new(CellType(shape, F16), true, name.c_str());
    CellPtr g = c.cell_new(CellType(shape, F16), true, ("grad:" + name).c_str());
    m->params.push_back(p);
    m->grads.push_back(g);
    m->names.push_back(name);
    return p;
}

// one staged thunk with a single output
int ap(Ctx &c, std::unique_ptr<ThunkSpec> spec, const std::vector<CellPtr> &args, CellPtr *out)
{
    std::vector<CellPtr> outs;
    int rc = c.stage_apply(c.add_thunk(std::move(spec)), args, &outs);
    if (rc) return rc;
    *out = outs[0];
    return 0;
}

#define TRY(x)             \
    do {                   \
        int rc_ = (x);     \
        if (rc_) return rc_; \
    } while (0)

}  // namespace

// ===========================================================================
// context + spine

CACTI_API int cacti_ctx_create(cacti_ctx **ctx, int dev, size_t pool_bytes, int host_pagelocked)
{
    CACTI_REQUIRE(ctx, CACTI_E_INVALID, "ctx_create: null out pointer");
    cacti_ctx *x = new cacti_ctx();
    int rc = x->c.init(dev, pool_bytes, host_pagelocked);
    if (rc) {
        delete x;
        return rc;
    }
    *ctx = x;
    return 0;
}

CACTI_API int cacti_ctx_destroy(cacti_ctx *ctx)
{
    delete ctx;
    return 0;
}

CACTI_API int cacti_ctx_stats(cacti_ctx *ctx, cacti_stats *out)
{
    CACTI_REQUIRE(ctx && out, CACTI_E_INVALID, "ctx_stats: null pointer");
    static_assert(sizeof(cacti_stats) == sizeof(Stats), "stats layouts must agree");
    ctx->c.stats(reinterpret_cast<Stats *>(out));
    return 0;
}

CACTI_API int cacti_ctx_sync(cacti_ctx *ctx) { return ctx->c.check_status(); }
CACTI_API void *cacti_ctx_stream(cacti_ctx *ctx) { return (void *)ctx->c.stream(); }

CACTI_API int cacti_ctx_set_timing(cacti_ctx *ctx, int on)
{
    ctx->c.set_timing(on);
    if (!on) ctx->c.clear_timings();
    return 0;
}

CACTI_API int cacti_ctx_set_timing_filter(cacti_ctx *ctx, const char *label_prefix, int every)
{
    CACTI_REQUIRE(ctx && every >= 1, CACTI_E_INVALID, "set_timing_filter: null context or every < 1");
    ctx->c.set_timing_filter(label_prefix ? label_prefix : "", every);
    return 0;
}

CACTI_API int cacti_ctx_timing_report(cacti_ctx *ctx, char *buf, size_t cap)
{
    CACTI_REQUIRE(ctx && buf && cap > 0, CACTI_E_INVALID, "timing_report: null pointer");
    size_t n = 0;
    buf[0] = 0;
    int rc = ctx->c.collect_timings();
    if (rc) return rc;
    for (auto &kv : ctx->c.timings()) {
        int w = snprintf(buf + n, cap - n, "%s %llu %.4f\n", kv.first.c_str(),
                         (unsigned long long)kv.second.second, kv.second.first);
        if (w < 0 || (size_t)w >= cap - n) break;
        n += (size_t)w;
    }
    return 0;
}

CACTI_API int cacti_reset(cacti_ctx *ctx)
{
    ctx->c.reset();
    return 0;
}
CACTI_API int cacti_compile(cacti_ctx *ctx) { return ctx->c.compile(); }
CACTI_API int cacti_resume(cacti_ctx *ctx, int *yield_cell)
{
    CellPtr y = 0;
    int rc = ctx->c.resume(&y);
    if (yield_cell) *yield_cell = y;
    return rc;
}
CACTI_API int cacti_resume_put(cacti_ctx *ctx, int cell, const void *host, size_t bytes)
{
    return ctx->c.resume_put(cell, host, bytes);
}
CACTI_API int cacti_cell_bytes(cacti_ctx *ctx, int cell, size_t *bytes)
{
    CACTI_REQUIRE(ctx && bytes && cell > 0, CACTI_E_INVALID, "cell_bytes: bad arguments");
    *bytes = ctx->c.cell(cell).ty.bytes();
    return 0;
}
CACTI_API int cacti_cell_get(cacti_ctx *ctx, int cell, void *host, size_t bytes)
{
    return ctx->c.cell_get(cell, host, bytes);
}
CACTI_API int cacti_log_len(cacti_ctx *ctx) { return (int)ctx->c.log().size(); }
CACTI_API const char *cacti_log_name(cacti_ctx *ctx, int i)
{
    if (i < 0 || (size_t)i >= ctx->c.log().size()) return "";
    return ctx->c.entry_name((size_t)i);
}

// ===========================================================================
// pool policy over a plain offset range

struct cacti_mempool {
    MemPool p;
};

CACTI_API int cacti_mempool_create(cacti_mempool **pool, uint64_t cap)
{
    CACTI_REQUIRE(pool, CACTI_E_INVALID, "mempool_create: null out pointer");
    *pool = new cacti_mempool();
    (*pool)->p.reset((size_t)cap);
    return 0;
}
CACTI_API int cacti_mempool_destroy(cacti_mempool *pool)
{
    delete pool;
    return 0;
}
CACTI_API uint64_t cacti_mempool_alloc(cacti_mempool *pool, uint64_t bytes)
{
    size_t o = pool->p.alloc((size_t)bytes);
    return o == kNoOffset ? UINT64_MAX : (uint64_t)o;
}
CACTI_API int cacti_mempool_free(cacti_mempool *pool, uint64_t offset)
{
    CACTI_REQUIRE(pool->p.size_of((size_t)offset) != 0, CACTI_E_INVALID,
                  "mempool_free: offset %llu is not an allocation", (unsigned long long)offset);
    pool->p.free((size_t)offset);
    return 0;
}
CACTI_API int cacti_mempool_stats(cacti_mempool *pool, uint64_t out[5])
{
    out[0] = pool->p.cap();
    out[1] = pool->p.used();
    out[2] = pool->p.peak();
    out[3] = pool->p.front();
    out[4] = pool->p.largest_free();
    return 0;
}

// ===========================================================================
// model

CACTI_API int cacti_llama_create(cacti_ctx *ctx, const cacti_llama_cfg *cfg, cacti_llama **model)
{
    CACTI_REQUIRE(ctx && cfg && model, CACTI_E_INVALID, "llama_create: null pointer");
    CACTI_REQUIRE(cfg->S > 0 && cfg->L >= 0 && cfg->H > 0 && cfg->H * cfg->Dh == cfg->D &&
                      cfg->F > 0 && cfg->V > 0 && cfg->V <= 65536 && cfg->Dh % 2 == 0,
                  CACTI_E_INVALID, "llama_create: inconsistent configuration");
    cacti_llama *m = new cacti_llama();
    m->ctx = ctx;
    m->cfg = *cfg;
    Ctx &c = ctx->c;
    const int64_t D = cfg->D, F = cfg->F, V = cfg->V, S = cfg->S;
    m->embed = new_param(m, "embed", {V, D});
    for (int64_t l = 0; l < cfg->L; l++) {
        LayerCells lc;
        const std::string p = "l" + std::to_string(l) + ".";
        lc.pre_norm = new_param(m, p + "pre_norm", {D});
        lc.q = new_param(m, p + "q", {D, D});
        lc.k = new_param(m, p + "k", {D, D});
        lc.v = new_param(m, p + "v", {D, D});
        lc.o = new_param(m, p + "o", {D, D});
        lc.post_norm = new_param(m, p + "post_norm", {D});
        lc.gate = new_param(m, p + "gate", {F, D});
        lc.up = new_param(m, p + "up", {F, D});
        lc.down = new_param(m, p + "down", {D, F});
        m->layers.push_back(lc);
    }
    m->head_norm = new_param(m, "head_norm", {D});
    m->lm_head = new_param(m, "lm_head", {V, D});
    // init_constants, src/librarium/llama.rs:389-411: computed once, kept on the device
    m->cos = c.cell_new(CellType({S, cfg->Dh}, F16), true, "cos");
    m->sin = c.cell_new(CellType({S, cfg->Dh}, F16), true, "sin");
    c.set_const(m->cos);
    c.set_const(m->sin);
    int rc = c.ensure_vmem(m->cos, false);
    if (!rc) rc = c.ensure_vmem(m->sin, false);
    if (!rc)
        rc = cacti_hip_rope_tables(S, cfg->Dh, c.dev_ptr(c.cell(m->cos).voff),
                                   c.dev_ptr(c.cell(m->sin).voff), (void *)c.stream());
    if (rc) {
        delete m;
        return rc;
    }
    c.cell(m->cos).v_valid = c.cell(m->sin).v_valid = true;
    // fresh_input, src/librarium/llama.rs:380-387
    m->in_tok = c.cell_new(CellType({S}, U16), true, "in_tok");
    m->in_lm_tok = c.cell_new(CellType({S}, U16), true, "in_lm_tok");
    m->in_loss_scale = c.cell_new(CellType({S}, F32), true, "in_lm_loss_scale");
    c.set_const(m->in_tok);
    c.set_const(m->in_lm_tok);
    c.set_const(m->in_loss_scale);
    *model = m;
    return 0;
}

CACTI_API int cacti_llama_destroy(cacti_llama *model)
{
    delete model;
    return 0;
}

CACTI_API int cacti_llama_num_params(cacti_llama *m) { return (int)m->params.size(); }

CACTI_API int cacti_llama_param_info(cacti_llama *m, int i, char *name, size_t name_cap,
                                     int64_t *rows, int64_t *cols, int *param_cell, int *grad_cell)
{
    CACTI_REQUIRE(m && i >= 0 && (size_t)i < m->params.size(), CACTI_E_INVALID,
                  "param_info: index out of range");
    const CellType &t = m->ctx->c.cell(m->params[i]).ty;
    if (name && name_cap) snprintf(name, name_cap, "%s", m->names[i].c_str());
    if (rows) *rows = t.shape[0];
    if (cols) *cols = t.shape.size() > 1 ? t.shape[1] : 1;
    if (param_cell) *param_cell = m->params[i];
    if (grad_cell) *grad_cell = m->grads[i];
    return 0;
}

CACTI_API int cacti_llama_param_put(cacti_llama *m, int i, const void *host, size_t bytes)
{
    CACTI_REQUIRE(m && i >= 0 && (size_t)i < m->params.size(), CACTI_E_INVALID,
                  "param_put: index out of range");
    return m->ctx->c.cell_put(m->params[i], host, bytes);
}

CACTI_API int cacti_llama_grad_get(cacti_llama *m, int i, void *host, size_t bytes)
{
    CACTI_REQUIRE(m && i >= 0 && (size_t)i < m->grads.size(), CACTI_E_INVALID,
                  "grad_get: index out of range");
    return m->ctx->c.cell_get(m->grads[i], host, bytes);
}

CACTI_API int cacti_llama_digests(cacti_llama *m, int of_grads, int64_t *hist, int64_t *nan)
{
    CACTI_REQUIRE(m && hist && nan, CACTI_E_INVALID, "digests: null argument");
    const std::vector<CellPtr> &cells = of_grads ? m->grads : m->params;
    return m->ctx->c.cells_digest(cells.data(), (int)cells.size(), hist, nan);
}

CACTI_API int cacti_llama_adamw_init(cacti_llama *m)
{
    CACTI_REQUIRE(m, CACTI_E_INVALID, "adamw_init: null model");
    Ctx &c = m->ctx->c;
    if (m->master.empty()) {
        for (size_t i = 0; i < m->params.size(); i++) {
            const CellType ty(c.cell(m->params[i]).ty.shape, F32);
            m->master.push_back(c.cell_new(ty, true, ("master:" + m->names[i]).c_str()));
            m->grad_avg.push_back(c.cell_new(ty, true, ("grad_avg:" + m->names[i]).c_str()));
            m->grad2_avg.push_back(c.cell_new(ty, true, ("grad2_avg:" + m->names[i]).c_str()));
        }
        for (CellPtr x : m->master) c.set_const(x);
        for (CellPtr x : m->grad_avg) c.set_const(x);
        for (CellPtr x : m->grad2_avg) c.set_const(x);
    }
    for (size_t i = 0; i < m->params.size(); i++) {
        int rc = c.cell_cast_f16_f32(m->params[i], m->master[i]);
        if (!rc) rc = c.cell_zero(m->grad_avg[i]);
        if (!rc) rc = c.cell_zero(m->grad2_avg[i]);
        if (rc) return rc;
    }
    return 0;
}

CACTI_API int cacti_llama_adamw_step(cacti_llama *m, int iter_nr, const cacti_adamw32 *opt, int skip_embed)
{
    CACTI_REQUIRE(m && opt, CACTI_E_INVALID, "adamw_step: null argument");
    CACTI_REQUIRE(!m->master.empty(), CACTI_E_STATE, "adamw_step before adamw_init");
    float sc[7];
    int rc = cacti_adamw32_scalars(iter_nr, opt->grad_scale, opt->lr, opt->wd, opt->a1, opt->a2, opt->eps, sc);
    if (rc) return rc;
    const size_t first = skip_embed ? 1 : 0;                     // the embedding is parameter 0
    return m->ctx->c.cells_adamw32((int)(m->params.size() - first), m->grads.data() + first,
                                   m->grad_avg.data() + first, m->grad2_avg.data() + first,
                                   m->master.data() + first, m->params.data() + first, sc);
}

CACTI_API int cacti_llama_adamw_state_get(cacti_llama *m, int i, int which, void *host, size_t bytes)
{
    CACTI_REQUIRE(m && i >= 0 && (size_t)i < m->params.size() && which >= 0 && which <= 2, CACTI_E_INVALID,
                  "adamw_state_get: index out of range");
    CACTI_REQUIRE(!m->master.empty(), CACTI_E_STATE, "adamw_state_get before adamw_init");
    const std::vector<CellPtr> &v = which == 0 ? m->master : which == 1 ? m->grad_avg : m->grad2_avg;
    return m->ctx->c.cell_get(v[(size_t)i], host, bytes);
}

namespace cacti {

int tensors_dir_keys(cacti_tensors_dir *dir, std::vector<const char *> *keys);
int tensors_dir_lookup(cacti_tensors_dir *dir, int i, const char **dtype, const std::vector<int64_t> **shape,
                       int *fd, uint64_t *off, size_t *bytes);

int llama_load_tensors(cacti_llama *m, cacti_tensors_dir *dir, int *n_matched)
{
    Ctx &c = m->ctx->c;
    // Llama::match_pickle_dir, src/librarium/llama.rs:284-302: one rule per parameter, in parameter order
    std::vector<std::string> rules;
    rules.push_back("embed");
    static const char *const per_layer[9] = {"input_layernorm", "attn/q_proj", "attn/k_proj", "attn/v_proj", "attn/o_proj",
                                             "post_attention_layernorm", "mlp/gate", "mlp/up", "mlp/down"};
    for (size_t l = 0; l < m->layers.size(); l++)
        for (const char *r : per_layer) rules.push_back("#" + std::to_string(l) + "/" + r);
    rules.push_back("norm");
    rules.push_back("lm_head");
    CACTI_REQUIRE(rules.size() == m->params.size(), CACTI_E_STATE, "load_tensors: rule table out of step");
    std::vector<const char *> keys, rp;
    tensors_dir_keys(dir, &keys);
    for (const std::string &r : rules) rp.push_back(r.c_str());
    std::vector<int> match(rules.size(), -1);
    int rc = cacti_cell_matcher_match(keys.data(), (int)keys.size(), rp.data(), (int)rp.size(), match.data());
    if (rc) return rc;
    int matched = 0;
    for (size_t i = 0; i < m->params.size(); i++) {
        if (match[i] < 0) continue;
        const char *dtype;
        const std::vector<int64_t> *shape;
        int fd;
        uint64_t off;
        size_t bytes;
        tensors_dir_lookup(dir, match[i], &dtype, &shape, &fd, &off, &bytes);
        const CellPtr p = m->params[i];
        CACTI_REQUIRE(*shape == c.cell(p).ty.shape, CACTI_E_INVALID,
                      "load_tensors: %s matched %s, whose shape differs from the parameter's", m->names[i].c_str(),
                      keys[(size_t)match[i]]);
        // F16 as it is (resume_put); BF16 and F32 through the cast set_lossy_cast stages
        const int cast = !strcmp(dtype, "F16") ? 0 : !strcmp(dtype, "BF16") ? 1 : !strcmp(dtype, "F32") ? 2 : -1;
        CACTI_REQUIRE(cast >= 0, CACTI_E_NOTIMPL, "load_tensors: %s: dtype %s cannot be stored into an f16 parameter",
                      keys[(size_t)match[i]], dtype);
        rc = c.cell_ingest(p, fd, off, bytes, cast);
        if (rc) return rc;
        matched++;
    }
    if (n_matched) *n_matched = matched;
    return c.sync();
}

}  // namespace cacti

CACTI_API int cacti_llama_io_cells(cacti_llama *m, int *tok, int *lm_tok, int *loss_scale,
                                   int *logit, int *loss, int *amax, int *prob)
{
    if (tok) *tok = m->in_tok;
    if (lm_tok) *lm_tok = m->in_lm_tok;
    if (loss_scale) *loss_scale = m->in_loss_scale;
    if (logit) *logit = m->out_logit;
    if (loss) *loss = m->out_loss;
    if (amax) *amax = m->out_amax;
    if (prob) *prob = m->out_prob;
    return 0;
}

CACTI_API int cacti_llama_stage(cacti_llama *m, int want_prob, int want_grad)
{
    Ctx &c = m->ctx->c;
    const cacti_llama_cfg &g = m->cfg;
    const float alpha = 1.0f / sqrtf((float)g.Dh);
    // in_.in_tok.mem_set_yield_() ..., examples/open_llama_3b_train.rs:350-358
    c.stage_yield_set(m->in_tok);
    c.stage_yield_set(m->in_lm_tok);
    c.stage_yield_set(m->in_loss_scale);

    // The residual stream enters every norm as the sum of two cells (x1 = stream + o,
    // x2 = x1 + down, llama.rs:512-532); sum and norm are staged as one fused thunk with both
    // outputs.  `add_a`, `add_b`: the pending sum's operands (0: `stream` is a plain cell).
    CellPtr stream, add_a = 0, add_b = 0;
    auto norm_of_stream = [&](CellPtr w, CellPtr *y) -> int {
        if (!add_a) return ap(c, make_rms_norm(g.eps), {stream, w}, y);
        std::vector<CellPtr> outs;
        int rc = c.stage_apply(c.add_thunk(make_add_rms_norm(g.eps)), {add_a, add_b, w}, &outs);
        if (rc) return rc;
        stream = outs[0];
        *y = outs[1];
        add_a = add_b = 0;
        return 0;
    };
    TRY(ap(c, make_embed(), {m->embed, m->in_tok}, &stream));
    for (size_t l = 0; l < m->layers.size(); l++) {
        const LayerCells &w = m->layers[l];
        CellPtr pre, q, k, v, qr, kr, s16, p16, attn, o, post, up, gate, h, down;
        TRY(norm_of_stream(w.pre_norm, &pre));
        TRY(ap(c, make_matmul(false, true, 1.f), {pre, w.q}, &q));
        TRY(ap(c, make_rope(g.H), {q, m->cos, m->sin}, &qr));
        TRY(ap(c, make_matmul(false, true, 1.f), {pre, w.k}, &k));
        TRY(ap(c, make_rope(g.H), {k, m->cos, m->sin}, &kr));
        TRY(ap(c, make_matmul(false, true, 1.f), {pre, w.v}, &v));
        TRY(ap(c, make_causal_scores(alpha, g.H), {qr, kr}, &s16));
        TRY(ap(c, make_causal_softmax(g.H), {s16}, &p16));
        TRY(ap(c, make_causal_pv(g.H), {p16, v}, &attn));
        TRY(ap(c, make_matmul(false, true, 1.f), {attn, w.o}, &o));
        add_a = stream;                                       // x1 = stream + o
        add_b = o;
        TRY(norm_of_stream(w.post_norm, &post));
        TRY(ap(c, make_matmul(false, true, 1.f), {post, w.up}, &up));
        TRY(ap(c, make_matmul(false, true, 1.f), {post, w.gate}, &gate));
        TRY(ap(c, make_silu_gate(), {gate, up}, &h));
        TRY(ap(c, make_matmul(false, true, 1.f), {h, w.down}, &down));
        add_a = stream;                                       // x2 = x1 + down
        add_b = down;
    }
    CellPtr hn, logit;
    TRY(norm_of_stream(m->head_norm, &hn));
    TRY(ap(c, make_matmul(false, true, 1.f), {hn, m->lm_head}, &logit));
    std::vector<CellPtr> outs;
    TRY(c.stage_apply(c.add_thunk(make_softmax_ce(want_prob != 0)), {logit, m->in_lm_tok}, &outs));
    m->out_logit = logit;
    m->out_loss = outs[0];
    m->out_amax = outs[1];
    m->out_prob = want_prob ? outs[2] : 0;
    c.keep(m->out_logit);                                  // .keep(), llama.rs:541-546
    c.keep(m->out_loss);
    c.keep(m->out_amax);
    if (m->out_prob) c.keep(m->out_prob);

    if (want_grad) {
        // sink.add(out_lm_loss, in_lm_loss_scale); grad_map.add(p, g); vadd_vjp(src, sink)
        c.adj_seed(m->out_loss, m->in_loss_scale);
        for (size_t i = 0; i < m->params.size(); i++) c.adj_bind(m->params[i], m->grads[i]);
        TRY(c.vadd_vjp());
    }
    return 0;
}

CACTI_API int cacti_llama_step(cacti_llama *m, const uint16_t *tok, const uint16_t *lm_tok,
                               const float *loss_scale, int want_prob, int want_grad,
                               float *loss_out)
{
    CACTI_REQUIRE(m && tok && lm_tok && loss_scale, CACTI_E_INVALID, "llama_step: null input");
    Ctx &c = m->ctx->c;
    const size_t S = (size_t)m->cfg.S;
    c.reset();
    TRY(cacti_llama_stage(m, want_prob, want_grad));
    TRY(c.compile());
    for (;;) {
        CellPtr y = 0;
        int rc = c.resume(&y);
        if (rc == R_DONE) break;
        if (rc != R_YIELD) return rc;
        if (y == m->in_tok) TRY(c.resume_put(y, tok, S * 2));
        else if (y == m->in_lm_tok) TRY(c.resume_put(y, lm_tok, S * 2));
        else if (y == m->in_loss_scale) TRY(c.resume_put(y, loss_scale, S * 4));
        else CACTI_REQUIRE(false, CACTI_E_STATE, "llama_step: unexpected yield of cell %d", y);
    }
    // Without a loss read-back the call returns with the cycle still running on the stream
    // (the next cycle's staging then overlaps it); an out-of-range token id is reported by
    // the next synchronizing call (cacti_ctx_sync, or a step that reads the loss).
    if (!loss_out) return 0;
    TRY(c.check_status());
    return c.cell_get(m->out_loss, loss_out, S * 4);
}
