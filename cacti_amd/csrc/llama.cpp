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
    bool grads_written = false;                                 // a gradient cycle has been staged
    int attention_mode = 0;                                     // 0 fused thunk, 1 the chain of separate thunks
    int group_products = 1;                                     // 0 none, 1 up + gate forward, 2 also q, k, v and the weight gradients
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

CACTI_API int cacti_ctx_usage_report(cacti_ctx *ctx, char *buf, size_t cap)
{
    CACTI_REQUIRE(ctx && buf && cap > 0, CACTI_E_INVALID, "ctx_usage_report: null pointer");
    const std::string s = ctx->c.usage_report();
    CACTI_REQUIRE(s.size() < cap, CACTI_E_INVALID, "ctx_usage_report: the report needs %zu bytes", s.size() + 1);
    memcpy(buf, s.c_str(), s.size() + 1);
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
        int w = snprintf(buf + n, cap - n, "%s %llu %.4f %llu\n", kv.first.c_str(),
                         (unsigned long long)kv.second.second, kv.second.first,
                         (unsigned long long)ctx->c.operand_bytes(kv.first));
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
    CACTI_REQUIRE(ctx && bytes, CACTI_E_INVALID, "cell_bytes: null argument");
    CACTI_REQUIRE(ctx->c.is_live(cell), CACTI_E_STATE, "cell_bytes: dead cell %d", cell);
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
CACTI_API uint64_t cacti_mempool_alloc_high(cacti_mempool *pool, uint64_t bytes)
{
    size_t o = pool->p.alloc((size_t)bytes, true);
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

CACTI_API int cacti_llama_set_attention(cacti_llama *m, int mode)
{
    CACTI_REQUIRE(m && (mode == 0 || mode == 1), CACTI_E_INVALID, "llama_set_attention: mode must be 0 or 1");
    m->attention_mode = mode;
    return 0;
}

CACTI_API int cacti_llama_set_product_groups(cacti_llama *m, int on)
{
    CACTI_REQUIRE(m && on >= 0 && on <= 2, CACTI_E_INVALID, "llama_set_product_groups: 0, 1 or 2");
    m->group_products = on;
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
        if (m->group_products >= 2) {
            // the three projections of the normed input (llama.rs:478-497) as one thunk and one launch;
            // values, and the order of the adjoint's accumulations, as with three matmul thunks
            std::vector<CellPtr> po;
            TRY(c.stage_apply(c.add_thunk(make_projections(3, true)), {pre, w.q, w.k, w.v}, &po));
            q = po[0];
            k = po[1];
            v = po[2];
        } else {
            TRY(ap(c, make_matmul(false, true, 1.f), {pre, w.q}, &q));
            TRY(ap(c, make_matmul(false, true, 1.f), {pre, w.k}, &k));
        }
        {
            // symplectic_embed on the query and on the key (llama.rs:483, 490) as one two-output thunk:
            // one launch, the values and the order of the adjoint's accumulations as with two thunks
            std::vector<CellPtr> ro;
            TRY(c.stage_apply(c.add_thunk(make_rope2(g.H)), {q, k, m->cos, m->sin}, &ro));
            qr = ro[0];
            kr = ro[1];
        }
        if (m->group_products < 2) TRY(ap(c, make_matmul(false, true, 1.f), {pre, w.v}, &v));
        if (m->attention_mode == 0) {
            // scores, mask, softmax and the product with v as one thunk: the [S, H, S] cells of
            // llama.rs:501-505 exist only tile by tile in registers
            std::vector<CellPtr> ao;
            TRY(c.stage_apply(c.add_thunk(make_attention(alpha, g.H)), {qr, kr, v}, &ao));
            attn = ao[0];
        } else {
            TRY(ap(c, make_causal_scores(alpha, g.H), {qr, kr}, &s16));
            TRY(ap(c, make_causal_softmax(g.H), {s16}, &p16));
            TRY(ap(c, make_causal_pv(g.H), {p16, v}, &attn));
        }
        TRY(ap(c, make_matmul(false, true, 1.f), {attn, w.o}, &o));
        add_a = stream;                                       // x1 = stream + o
        add_b = o;
        TRY(norm_of_stream(w.post_norm, &post));
        if (m->group_products >= 1) {
            std::vector<CellPtr> po;
            TRY(c.stage_apply(c.add_thunk(make_projections(2, m->group_products >= 2)), {post, w.up, w.gate}, &po));
            up = po[0];
            gate = po[1];
        } else {
            TRY(ap(c, make_matmul(false, true, 1.f), {post, w.up}, &up));
            TRY(ap(c, make_matmul(false, true, 1.f), {post, w.gate}, &gate));
        }
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
        // want_grad = 2: g.cache() on every gradient before the cycle, the micro-batch accumulation of
        // examples/open_llama_3b_train.rs:334-345 -- this cycle's gradients add to the held ones
        CACTI_REQUIRE(want_grad != 2 || m->grads_written, CACTI_E_STATE,
                      "llama_stage: gradients cached before any cycle has written them");
        c.adj_seed(m->out_loss, m->in_loss_scale);
        for (size_t i = 0; i < m->params.size(); i++) c.adj_bind(m->params[i], m->grads[i], want_grad == 2);
        TRY(c.vadd_vjp());
        m->grads_written = true;
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

// ---------------------------------------------------------------------------
// KV-cached forward pass: LlamaCached, src/librarium/llama.rs:561-963 (batch 1, q_group 1).
// The pass runs eagerly on the context's stream: temporaries come from the pool and go back at
// the end of the call (reuse is ordered on the stream), parameters and caches are stable cells.
struct cacti_llama_cached {
    cacti_llama *base;                       // shares the parameter cells (LlamaCached::from(Llama))
    int64_t cap;
    std::vector<CellPtr> k_cache, v_cache;   // per layer [cap, H, Dh] f16
    CellPtr in_tok;                          // [cap] u16
    // outputs of the last apply (pool regions kept until the next apply or destroy)
    size_t out_logit = kNoOffset, out_prob = kNoOffset, out_tok = kNoOffset;
    int64_t out_rows = 0;
};

namespace {

void cached_drop_outputs(cacti_llama_cached *k)
{
    Ctx &c = k->base->ctx->c;
    for (size_t *o : {&k->out_logit, &k->out_prob, &k->out_tok})
        if (*o != kNoOffset) {
            c.pool_free(*o);
            *o = kNoOffset;
        }
    k->out_rows = 0;
}

}  // namespace

CACTI_API int cacti_llama_cached_create(cacti_llama *model, int64_t seq_cap, cacti_llama_cached **out)
{
    CACTI_REQUIRE(model && out, CACTI_E_INVALID, "llama_cached_create: null argument");
    // the position tables are the model's (from_train keeps model.cos / model.sin, llama.rs:657-686)
    CACTI_REQUIRE(seq_cap > 0 && seq_cap % 8 == 0 && seq_cap <= model->cfg.S, CACTI_E_INVALID,
                  "llama_cached_create: seq_cap must be a multiple of 8 and at most the model's %lld",
                  (long long)model->cfg.S);
    Ctx &c = model->ctx->c;
    cacti_llama_cached *k = new cacti_llama_cached();
    k->base = model;
    k->cap = seq_cap;
    for (int64_t l = 0; l < model->cfg.L; l++) {
        const std::string p = "l" + std::to_string(l) + ".";
        k->k_cache.push_back(c.cell_new(CellType({seq_cap, model->cfg.H, model->cfg.Dh}, F16), true, (p + "k_cache").c_str()));
        k->v_cache.push_back(c.cell_new(CellType({seq_cap, model->cfg.H, model->cfg.Dh}, F16), true, (p + "v_cache").c_str()));
        c.set_const(k->k_cache.back());
        c.set_const(k->v_cache.back());
    }
    k->in_tok = c.cell_new(CellType({seq_cap}, U16), true, "cached_in_tok");
    c.set_const(k->in_tok);
    int rc = cacti_llama_cached_reset_state(k);
    if (!rc) rc = c.cell_zero(k->in_tok);

    if (rc) {
        delete k;
        return rc;
    }
    *out = k;
    return 0;
}

CACTI_API int cacti_llama_cached_destroy(cacti_llama_cached *k)
{
    if (!k) return 0;
    Ctx &c = k->base->ctx->c;
    cached_drop_outputs(k);
    for (CellPtr x : k->k_cache) { c.cell_free_all(x); c.cell(x).alive = false; }
    for (CellPtr x : k->v_cache) { c.cell_free_all(x); c.cell(x).alive = false; }
    c.cell_free_all(k->in_tok);
    c.cell(k->in_tok).alive = false;
    delete k;
    return 0;
}

// LlamaCached::reset_state, src/librarium/llama.rs:784-789
CACTI_API int cacti_llama_cached_reset_state(cacti_llama_cached *k)
{
    CACTI_REQUIRE(k, CACTI_E_INVALID, "llama_cached_reset_state: null model");
    Ctx &c = k->base->ctx->c;
    for (size_t l = 0; l < k->k_cache.size(); l++) {
        int rc = c.cell_zero(k->k_cache[l]);
        if (!rc) rc = c.cell_zero(k->v_cache[l]);
        if (rc) return rc;
    }
    return 0;
}

CACTI_API int cacti_llama_cached_set_tokens(cacti_llama_cached *k, const uint16_t *tok, int64_t n)
{
    CACTI_REQUIRE(k && (tok || n == 0) && n >= 0 && n <= k->cap, CACTI_E_INVALID,
                  "llama_cached_set_tokens: %lld tokens do not fit the capacity", (long long)n);
    std::vector<uint16_t> buf((size_t)k->cap, 0);                 // the rest of the input is the pad token 0
    for (int64_t i = 0; i < n; i++) buf[(size_t)i] = tok[i];
    return k->base->ctx->c.cell_put(k->in_tok, buf.data(), buf.size() * 2);
}

CACTI_API int cacti_llama_cached_get_tokens(cacti_llama_cached *k, uint16_t *tok)
{
    CACTI_REQUIRE(k && tok, CACTI_E_INVALID, "llama_cached_get_tokens: null argument");
    return k->base->ctx->c.cell_get(k->in_tok, tok, (size_t)k->cap * 2);
}

CACTI_API int cacti_llama_cached_apply(cacti_llama_cached *k, int64_t prev, int64_t next, int want_prob)
{
    CACTI_REQUIRE(k, CACTI_E_INVALID, "llama_cached_apply: null model");
    cacti_llama *m = k->base;
    Ctx &c = m->ctx->c;
    const cacti_llama_cfg &g = m->cfg;
    const int64_t T = next - prev, D = g.D, H = g.H, Dh = g.Dh, F = g.F, V = g.V, cap = k->cap;
    CACTI_REQUIRE(prev >= 0 && T > 0 && next <= cap, CACTI_E_INVALID,
                  "llama_cached_apply: positions [%lld, %lld) outside the capacity %lld", (long long)prev,
                  (long long)next, (long long)cap);
    const int64_t Cw = (next + 7) / 8 * 8;                        // cached columns, rounded up to the vector width
    const float alpha = 1.0f / sqrtf((float)Dh);
    hipStream_t st = c.stream();
    cached_drop_outputs(k);

    // every cell the pass touches is made resident and pinned for the duration of the call
    std::vector<CellPtr> used = m->params;
    used.insert(used.end(), k->k_cache.begin(), k->k_cache.end());
    used.insert(used.end(), k->v_cache.begin(), k->v_cache.end());
    used.push_back(k->in_tok);
    used.push_back(m->cos);
    used.push_back(m->sin);
    int rc = 0;
    size_t npinned = 0;
    for (; npinned < used.size() && !rc; npinned++) {
        c.cell(used[npinned]).pin++;
        rc = c.ensure_vmem(used[npinned], true);
    }
    std::vector<size_t> temps;
    auto tmp = [&](int64_t elems, size_t esz) -> char * {
        size_t off;
        if (rc) return nullptr;
        rc = c.pool_alloc((size_t)elems * esz, &off);
        if (rc) return nullptr;
        temps.push_back(off);
        return static_cast<char *>(c.dev_ptr(off));
    };
    auto P = [&](CellPtr x) { return c.dev_ptr(c.cell(x).voff); };
    char *x = tmp(T * D, 2), *pre = tmp(T * D, 2), *q = tmp(T * D, 2), *qr = tmp(T * D, 2), *kk = tmp(T * D, 2),
         *kr = tmp(T * D, 2), *v = tmp(T * D, 2), *attn = tmp(T * D, 2), *o = tmp(T * D, 2), *x1 = tmp(T * D, 2),
         *post = tmp(T * D, 2), *up = tmp(T * F, 2), *gate = tmp(T * F, 2), *h = tmp(T * F, 2), *down = tmp(T * D, 2),
         *s16 = nullptr, *aws = nullptr;
    // one to four rows: the fused decoding attention; more: scores, softmax and P V as three products
    const bool fused_attn = T <= 4 && Dh % 4 == 0 && Dh <= 100 && next <= 8192;
    const size_t aws_bytes = fused_attn ? cacti_hip_attn_decode_workspace(T, H, Dh, next) : 0;
    if (fused_attn) aws = tmp((int64_t)aws_bytes, 1);
    else s16 = tmp(T * H * Cw, 2);
    // outputs
    if (!rc) rc = c.pool_alloc((size_t)(T * V) * 2, &k->out_logit);
    if (!rc) rc = c.pool_alloc((size_t)T * 2, &k->out_tok);
    if (!rc && want_prob) rc = c.pool_alloc((size_t)(T * V) * 4, &k->out_prob);
#define STEP(call)          \
    do {                    \
        if (!rc) rc = (call); \
    } while (0)
    if (!rc) {
        const char *cosr = static_cast<const char *>(P(m->cos)) + prev * Dh * 2;
        const char *sinr = static_cast<const char *>(P(m->sin)) + prev * Dh * 2;
        char *tok = static_cast<char *>(P(k->in_tok));
        // stream = embed.outer_select(in_tok[prev .. next])
        STEP(cacti_hip_embed_fwd(V, D, P(m->embed), T, tok + prev * 2, x, c.status_ptr(), st));
        void *logit = c.dev_ptr(k->out_logit);
        if (fused_attn && D <= 8192) {
            // One to four rows: the norms, the residual adds and the SiLU gate ride in the product
            // kernels (cacti_hip_rows_norm_matmul_f16), which stream each weight matrix once.
            // The residual stream is (xa) or the pending sum f16(xa + xb).
            const char *xa = x, *xb = nullptr;
            for (size_t l = 0; l < m->layers.size() && !rc; l++) {
                const LayerCells &w = m->layers[l];
                char *kc = static_cast<char *>(P(k->k_cache[l])), *vc = static_cast<char *>(P(k->v_cache[l]));
                // q, k, v projections of the normed stream, rotation, k_cache[prev ..] += k, v_cache[prev ..] += v
                STEP(cacti_hip_rows_qkv_rope_cache_f16(T, H, Dh, xa, xb, P(w.pre_norm), g.eps, xb ? x : nullptr, P(w.q), P(w.k),
                                                       P(w.v), cosr, sinr, qr, kc + prev * D * 2, vc + prev * D * 2, st));
                STEP(cacti_hip_attn_decode_f16(T, H, Dh, next, prev, alpha, qr, D, kc, vc, D, Dh, attn, D, aws, aws_bytes, st));
                STEP(cacti_hip_gemm_f16(0, 1, T, D, D, 1.f, attn, D, P(w.o), D, 0.f, o, D, st));
                // x1 = stream + o; post = rms_norm(x1); h = silu(post gate^T) * (post up^T)
                STEP(cacti_hip_rows_norm_matmul_f16(T, F, D, x, o, P(w.post_norm), g.eps, x1, P(w.gate), P(w.up), h, st));
                STEP(cacti_hip_gemm_f16(0, 1, T, D, F, 1.f, h, F, P(w.down), F, 0.f, down, D, st));
                xa = x1;                                          // stream = x1 + down, formed by the next consumer
                xb = down;
            }
            STEP(cacti_hip_rows_norm_matmul_f16(T, V, D, xa, xb, P(m->head_norm), g.eps, nullptr, P(m->lm_head), nullptr, logit, st));
        } else {
            STEP(cacti_hip_rms_norm_fwd(T, D, x, P(m->layers.empty() ? m->head_norm : m->layers[0].pre_norm), g.eps, pre, st));
            for (size_t l = 0; l < m->layers.size() && !rc; l++) {
                const LayerCells &w = m->layers[l];
                char *kc = static_cast<char *>(P(k->k_cache[l])), *vc = static_cast<char *>(P(k->v_cache[l]));
                STEP(cacti_hip_gemm_f16(0, 1, T, D, D, 1.f, pre, D, P(w.q), D, 0.f, q, D, st));
                STEP(cacti_hip_rope_fwd(T, H, Dh, q, cosr, sinr, qr, st));
                STEP(cacti_hip_gemm_f16(0, 1, T, D, D, 1.f, pre, D, P(w.k), D, 0.f, kk, D, st));
                STEP(cacti_hip_rope_fwd(T, H, Dh, kk, cosr, sinr, kr, st));
                // k_cache[prev .. next] += k, v_cache[prev .. next] += v
                STEP(cacti_hip_add_f16(T * D, kc + prev * D * 2, kr, kc + prev * D * 2, st));
                STEP(cacti_hip_gemm_f16(0, 1, T, D, D, 1.f, pre, D, P(w.v), D, 0.f, v, D, st));
                STEP(cacti_hip_add_f16(T * D, vc + prev * D * 2, v, vc + prev * D * 2, st));
                // scores against the cache, row-causal mask + softmax (in place), P V.  Columns from
                // `next` on are masked for every row, so only the first Cw of the cap columns are formed.
                if (fused_attn) {
                    STEP(cacti_hip_attn_decode_f16(T, H, Dh, next, prev, alpha, qr, D, kc, vc, D, Dh, attn, D, aws, aws_bytes, st));
                } else {
                    STEP(cacti_hip_gemm_f16_strided_batched(0, 1, H, T, Cw, Dh, alpha, qr, D, Dh, kc, D, Dh, 0.f, s16, H * Cw, Cw, st));
                    STEP(cacti_hip_row_causal_softmax_fwd(T, H, Cw, Cw, prev, s16, s16, st));
                    STEP(cacti_hip_gemm_f16_strided_batched(0, 0, H, T, Dh, Cw, 1.f, s16, H * Cw, Cw, vc, D, Dh, 0.f, attn, D, Dh, st));
                }
                STEP(cacti_hip_gemm_f16(0, 1, T, D, D, 1.f, attn, D, P(w.o), D, 0.f, o, D, st));
                STEP(cacti_hip_add_rms_norm_fwd(T, D, x, o, P(w.post_norm), g.eps, x1, post, st));
                STEP(cacti_hip_gemm_f16(0, 1, T, F, D, 1.f, post, D, P(w.up), D, 0.f, up, F, st));
                STEP(cacti_hip_gemm_f16(0, 1, T, F, D, 1.f, post, D, P(w.gate), D, 0.f, gate, F, st));
                STEP(cacti_hip_silu_gate_fwd(T * F, gate, up, h, st));
                STEP(cacti_hip_gemm_f16(0, 1, T, D, F, 1.f, h, F, P(w.down), F, 0.f, down, D, st));
                const CellPtr wn = l + 1 < m->layers.size() ? m->layers[l + 1].pre_norm : m->head_norm;
                STEP(cacti_hip_add_rms_norm_fwd(T, D, x1, down, P(wn), g.eps, x, pre, st));
            }
            STEP(cacti_hip_gemm_f16(0, 1, T, V, D, 1.f, pre, D, P(m->lm_head), D, 0.f, logit, V, st));
        }
        void *otok = c.dev_ptr(k->out_tok);
        STEP(cacti_hip_softmax_ce_fwd(T, V, logit, nullptr, want_prob ? c.dev_ptr(k->out_prob) : nullptr, nullptr,
                                      otok, nullptr, st));
        // in_tok[next] += out_lm_tok[T - 1]
        if (next < cap) STEP(cacti_hip_append_token_u16(tok, next, otok, T - 1, st));
        if (!rc) {
            c.cell(k->in_tok).h_valid = false;
            for (size_t l = 0; l < m->layers.size(); l++)
                c.cell(k->k_cache[l]).h_valid = c.cell(k->v_cache[l]).h_valid = false;
            k->out_rows = T;
        }
    }
#undef STEP
    for (size_t off : temps) c.pool_free(off);                   // reuse is ordered on the stream
    for (size_t i = 0; i < npinned; i++) c.cell(used[i]).pin--;
    if (rc) cached_drop_outputs(k);
    return rc;
}

CACTI_API int cacti_llama_cached_outputs(cacti_llama_cached *k, void *logit_f16, float *prob, uint16_t *tok)
{
    CACTI_REQUIRE(k && k->out_rows > 0, CACTI_E_STATE, "llama_cached_outputs: no apply has run");
    CACTI_REQUIRE(!prob || k->out_prob != kNoOffset, CACTI_E_STATE, "llama_cached_outputs: the last apply kept no probabilities");
    Ctx &c = k->base->ctx->c;
    hipStream_t st = c.stream();
    const int64_t T = k->out_rows, V = k->base->cfg.V;
    if (logit_f16) CACTI_HIP(hipMemcpyAsync(logit_f16, c.dev_ptr(k->out_logit), (size_t)(T * V) * 2, hipMemcpyDeviceToHost, st));
    if (prob) CACTI_HIP(hipMemcpyAsync(prob, c.dev_ptr(k->out_prob), (size_t)(T * V) * 4, hipMemcpyDeviceToHost, st));
    if (tok) CACTI_HIP(hipMemcpyAsync(tok, c.dev_ptr(k->out_tok), (size_t)T * 2, hipMemcpyDeviceToHost, st));
    return c.check_status();                                     // syncs; raises a token id out of range
}

