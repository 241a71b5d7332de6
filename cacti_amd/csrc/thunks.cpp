#include "thunks.h"

#include "common.h"

namespace cacti {
namespace {

inline void *S(Ctx &c) { return (void *)c.stream(); }

#define TY_REQUIRE(cond, ...) CACTI_REQUIRE(cond, CACTI_E_INVALID, __VA_ARGS__)

// ---------------------------------------------------------------------------
// copy (the memcpy adjoint of Add / Identity, src/thunk/op.rs:1529-1534, 5474-5729)
struct CopySpec : ThunkSpec {
    const char *name() const override { return "copy"; }
    int arity() const override { return 1; }
    bool is_copy() const override { return true; }
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        o = {a[0]};
        return 0;
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t acc, void *, size_t) const override
    {
        if (acc & 1) {
            TY_REQUIRE(aty[0].dtype == F16, "copy: accumulate is f16 only");
            return cacti_hip_add_f16(aty[0].numel(), o[0], a[0], o[0], S(c));
        }
        return cacti_hip_memcpy_async(o[0], a[0], aty[0].bytes(), S(c));
    }
    int pop_adj(Ctx &c, const Entry &e, const std::vector<CellPtr> &dy) const override
    {
        return c.adj_add({e.args[0]}, make_copy(), {dy[0]});
    }
};

// ---------------------------------------------------------------------------
// y = a + b (AddFutThunkSpec src/thunk/op.rs:1480-1535); both adjoints are copies of dy
struct AddSpec : ThunkSpec {
    const char *name() const override { return "add"; }
    int arity() const override { return 2; }
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        TY_REQUIRE(a[0] == a[1] && a[0].dtype == F16, "add: operands must be equal f16 shapes");
        o = {a[0]};
        return 0;
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t acc, void *, size_t) const override
    {
        TY_REQUIRE(!(acc & 1), "add: accumulate mode not staged on this path");
        return cacti_hip_add_f16(aty[0].numel(), a[0], a[1], o[0], S(c));
    }
    int pop_adj(Ctx &c, const Entry &e, const std::vector<CellPtr> &dy) const override
    {
        int rc = c.adj_add({e.args[0]}, make_copy(), {dy[0]});
        if (rc) return rc;
        return c.adj_add({e.args[1]}, make_copy(), {dy[0]});
    }
};

// ---------------------------------------------------------------------------
// Embedding (OuterSelectFutThunkSpec src/thunk/op.rs:1229-1314) and its scatter-add adjoint
struct EmbedBwdSpec : ThunkSpec {
    int64_t V;
    explicit EmbedBwdSpec(int64_t v) : V(v) {}
    const char *name() const override { return "embed_bwd"; }
    int arity() const override { return 2; }                       // (tok, dy) -> dW
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        TY_REQUIRE(a[0].dtype == U16 && a[1].dtype == F16 && a[1].shape.size() == 2,
                   "embed_bwd: (tok u16, dy f16 [S,D]) expected");
        o = {CellType({V, a[1].shape[1]}, F16)};
        return 0;
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t acc, void *, size_t) const override
    {
        return cacti_hip_embed_bwd(V, aty[1].shape[1], aty[1].shape[0], a[0], a[1], o[0], acc & 1,
                                   S(c));
    }
};

struct EmbedSpec : ThunkSpec {
    const char *name() const override { return "embed"; }
    int arity() const override { return 2; }                       // (W, tok) -> y
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        TY_REQUIRE(a[0].dtype == F16 && a[0].shape.size() == 2 && a[1].dtype == U16,
                   "embed: (W f16 [V,D], tok u16) expected");
        o = {CellType({a[1].numel(), a[0].shape[1]}, F16)};
        return 0;
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t, void *, size_t) const override
    {
        return cacti_hip_embed_fwd(aty[0].shape[0], aty[0].shape[1], a[0], aty[1].numel(), a[1],
                                   o[0], c.status_ptr(), S(c));
    }
    int pop_adj(Ctx &c, const Entry &e, const std::vector<CellPtr> &dy) const override
    {
        const int64_t V = c.cell(e.args[0]).ty.shape[0];
        return c.adj_add({e.args[0]}, std::unique_ptr<ThunkSpec>(new EmbedBwdSpec(V)),
                         {e.args[1], dy[0]});
    }
};

// ---------------------------------------------------------------------------
// RMSNorm (rms_norm closure src/librarium/llama.rs:442-451) and its fused adjoint
struct RmsNormBwdSpec : ThunkSpec {
    float eps;
    explicit RmsNormBwdSpec(float e) : eps(e) {}
    const char *name() const override { return "rms_norm_bwd"; }
    int arity() const override { return 3; }                       // (x, w, dy) -> dx, dw
    int nout() const override { return 2; }
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        TY_REQUIRE(a[0] == a[2] && a[0].shape.size() == 2 && a[1].numel() == a[0].shape[1],
                   "rms_norm_bwd: shape mismatch");
        o = {a[0], a[1]};
        return 0;
    }
    size_t workspace(const std::vector<CellType> &a) const override
    {
        return cacti_hip_rms_norm_bwd_workspace(a[0].shape[0], a[0].shape[1]);
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t acc, void *ws, size_t wsb) const override
    {
        return cacti_hip_rms_norm_bwd(aty[0].shape[0], aty[0].shape[1], a[0], a[1], eps, a[2], o[0],
                                      acc & 1, o[1], (acc >> 1) & 1, ws, wsb, S(c));
    }
};

struct RmsNormSpec : ThunkSpec {
    float eps;
    explicit RmsNormSpec(float e) : eps(e) {}
    const char *name() const override { return "rms_norm"; }
    int arity() const override { return 2; }
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        TY_REQUIRE(a[0].dtype == F16 && a[1].dtype == F16 && a[0].shape.size() == 2 &&
                       a[1].numel() == a[0].shape[1],
                   "rms_norm: (x f16 [N,D], w f16 [D]) expected");
        o = {a[0]};
        return 0;
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t, void *, size_t) const override
    {
        return cacti_hip_rms_norm_fwd(aty[0].shape[0], aty[0].shape[1], a[0], a[1], eps, o[0], S(c));
    }
    int pop_adj(Ctx &c, const Entry &e, const std::vector<CellPtr> &dy) const override
    {
        return c.adj_add({e.args[0], e.args[1]}, std::unique_ptr<ThunkSpec>(new RmsNormBwdSpec(eps)),
                         {e.args[0], e.args[1], dy[0]});
    }
};

// x = a + b followed by y = rms_norm(x, w) as one launch with both outputs (the residual add
// always feeds a norm: llama.rs:512-516 and :532 -> the next layer's :474 / the head's :536).
// The adjoint is the two thunks' rules in their reverse order: the norm's adjoint accumulates
// into the adjoint of x, which the add's two memcpy adjoints then hand on.
struct AddRmsNormSpec : ThunkSpec {
    float eps;
    explicit AddRmsNormSpec(float e) : eps(e) {}
    const char *name() const override { return "add_rms_norm"; }
    int arity() const override { return 3; }                       // (a, b, w) -> x, y
    int nout() const override { return 2; }
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        TY_REQUIRE(a[0] == a[1] && a[0].dtype == F16 && a[2].dtype == F16 && a[0].shape.size() == 2 &&
                       a[2].numel() == a[0].shape[1],
                   "add_rms_norm: (a, b f16 [N,D], w f16 [D]) expected");
        o = {a[0], a[0]};
        return 0;
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t acc, void *, size_t) const override
    {
        TY_REQUIRE(acc == 0, "add_rms_norm: accumulate mode not staged on this path");
        return cacti_hip_add_rms_norm_fwd(aty[0].shape[0], aty[0].shape[1], a[0], a[1], a[2], eps, o[0],
                                          o[1], S(c));
    }
    int pop_adj(Ctx &c, const Entry &e, const std::vector<CellPtr> &dy) const override
    {
        if (dy[1]) {
            int rc = c.adj_add({e.outs[0], e.args[2]}, std::unique_ptr<ThunkSpec>(new RmsNormBwdSpec(eps)),
                               {e.outs[0], e.args[2], dy[1]});
            if (rc) return rc;
        }
        if (!c.adj_written(e.outs[0])) return 0;
        const CellPtr dx = c.adj_of(e.outs[0]);
        int rc = c.adj_add({e.args[0]}, make_copy(), {dx});
        if (rc) return rc;
        return c.adj_add({e.args[1]}, make_copy(), {dx});
    }
};

// ---------------------------------------------------------------------------
// MatrixMulThunkSpec src/thunk/op.rs:4284-4368 (2-d) and BlockMatrixMulThunkSpec :4719-4918
// on [R, H*C] tensors (the reference's [B,S,H,C] with B = 1, flattened) whose H per-head
// blocks are addressed by stride; H = 0 means one plain matrix.
//
// `causal` marks the two products of causal attention (scores = a Q K^T whose upper
// triangle the mask discards: CAUSAL_OUT; P V with P lower triangular: CAUSAL_A) so that
// the discarded half is not computed; the adjoint rules carry the structure along
// (dP = dO V^T is only needed below the diagonal; dV = P^T dO, dQ = a dS K, dK = a dS^T Q
// have a triangular first operand).
enum { CAUSAL_NONE = 0, CAUSAL_OUT = 1, CAUSAL_A = 2 };
struct MatMulSpec : ThunkSpec {
    bool ta, tb;
    int64_t nblk;
    bool blocked;
    float alpha;
    int causal;
    MatMulSpec(bool a, bool b, float al, int64_t h, int cz = CAUSAL_NONE)
        : ta(a), tb(b), nblk(h), blocked(h > 0), alpha(al), causal(cz) {}
    const char *name() const override { return blocked ? "block_matmul" : "matmul"; }
    int arity() const override { return 2; }
    struct Dims { int64_t H, M, N, K, lda, sa, ldb, sb, ldc, sc; };
    int dims(const std::vector<CellType> &a, Dims &d) const
    {
        TY_REQUIRE(a[0].dtype == F16 && a[1].dtype == F16 && a[0].shape.size() == 2 &&
                       a[1].shape.size() == 2,
                   "%s: f16 operands of rank 2 expected", name());
        d.H = blocked ? nblk : 1;
        TY_REQUIRE(a[0].shape[1] % d.H == 0 && a[1].shape[1] % d.H == 0,
                   "block_matmul: row length not divisible by the block count");
        const int64_t ra = a[0].shape[0], ca = a[0].shape[1] / d.H;
        const int64_t rb = a[1].shape[0], cb = a[1].shape[1] / d.H;
        d.M = ta ? ca : ra;
        d.K = ta ? ra : ca;
        const int64_t kb = tb ? cb : rb;
        d.N = tb ? rb : cb;
        TY_REQUIRE(kb == d.K, "%s: inner dimensions %lld and %lld differ", name(), (long long)d.K,
                   (long long)kb);
        d.lda = d.H * ca; d.sa = ca;
        d.ldb = d.H * cb; d.sb = cb;
        d.ldc = d.H * d.N; d.sc = d.N;
        return 0;
    }
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        Dims d;
        int rc = dims(a, d);
        if (rc) return rc;
        o = {CellType({d.M, d.H * d.N}, F16)};
        return 0;
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t acc, void *, size_t) const override
    {
        Dims d;
        int rc = dims(aty, d);
        if (rc) return rc;
        const int tri = causal == CAUSAL_OUT ? 1 : causal == CAUSAL_A ? (ta ? 3 : 2) : 0;
        return cacti_hip_gemm_f16_strided_batched_tri(ta, tb, d.H, d.M, d.N, d.K, alpha, a[0],
                                                      d.lda, d.sa, a[1], d.ldb, d.sb,
                                                      (acc & 1) ? 1.f : 0.f, o[0], d.ldc, d.sc, tri,
                                                      S(c));
    }
    std::string key(const std::vector<CellType> &aty, uint32_t acc) const override
    {
        Dims d;
        if (dims(aty, d)) return name();
        char buf[128];
        snprintf(buf, sizeof(buf), "%s[%c%c,%lldx%lldx%lldx%lld%s]", name(), ta ? 'T' : 'N',
                 tb ? 'T' : 'N', (long long)d.H, (long long)d.M, (long long)d.N, (long long)d.K,
                 (acc & 1) ? ",acc" : "");
        return buf;
    }
    std::unique_ptr<ThunkSpec> mm(bool x, bool y, int cz = CAUSAL_NONE) const
    {
        return std::unique_ptr<ThunkSpec>(new MatMulSpec(x, y, alpha, nblk, cz));
    }
    // the four transposition cases of pop_adj, src/thunk/op.rs:4335-4367 / :4882-4912:
    // arg_adj[1] first, then arg_adj[0], both carrying o_scale
    int pop_adj(Ctx &c, const Entry &e, const std::vector<CellPtr> &dy) const override
    {
        const CellPtr A = e.args[0], B = e.args[1], G = dy[0];
        int rc;
        if (causal == CAUSAL_OUT) {              // C = a A B^T, only tril(C) is used: G = tril
            TY_REQUIRE(!ta && tb, "causal scores product must be A B^T");
            if ((rc = c.adj_add({B}, mm(true, false, CAUSAL_A), {G, A}))) return rc;   // G^T A
            return c.adj_add({A}, mm(false, false, CAUSAL_A), {G, B});                  // G B
        }
        if (causal == CAUSAL_A) {                // C = A B with A = tril
            TY_REQUIRE(!ta && !tb, "causal probability product must be A B");
            if ((rc = c.adj_add({B}, mm(true, false, CAUSAL_A), {A, G}))) return rc;   // A^T G
            return c.adj_add({A}, mm(false, true, CAUSAL_OUT), {G, B});                 // tril(G B^T)
        }
        if (!ta && !tb) {
            if ((rc = c.adj_add({B}, mm(true, false), {A, G}))) return rc;      // A^T G
            return c.adj_add({A}, mm(false, true), {G, B});                      // G B^T
        }
        if (!ta && tb) {
            if ((rc = c.adj_add({B}, mm(true, false), {G, A}))) return rc;      // G^T A
            return c.adj_add({A}, mm(false, false), {G, B});                     // G B
        }
        if (ta && !tb) {
            if ((rc = c.adj_add({B}, mm(false, false), {A, G}))) return rc;     // A G
            return c.adj_add({A}, mm(false, true), {B, G});                      // B G^T
        }
        if ((rc = c.adj_add({B}, mm(true, true), {G, A}))) return rc;           // G^T A^T
        return c.adj_add({A}, mm(true, true), {B, G});                           // B^T G^T
    }
};

// ---------------------------------------------------------------------------
// Several products of one shape that share an operand, as one thunk and one launch (a pointer-array batch,
// cacti_hip_gemm_f16_batched: the shape of the reference's cublasGemmBatchedEx call,
// cacti_gpu_cu_ffi/src/lib.rs:793-885).  The reference stages the query, key and value projections of a layer
// (and the gate and up projections) as separate matmul thunks on the same input (src/librarium/llama.rs:
// 478-497); each product here is computed by the same tiles in the same order as its own launch would, so the
// results are those of the separate thunks bit for bit, and the adjoint stages what their adjoints would have
// staged, in their order: the weight gradients (one grouped thunk), then the input gradients one after the other
// (they accumulate into one cell: last product first, as the reverse sweep over separate thunks meets them).
constexpr int kMaxGroup = 4;

// dW_i = dy_i^T x: (dy_1 .. dy_n, x) -> (dW_1 .. dW_n)
struct WgradNSpec : ThunkSpec {
    int n;
    explicit WgradNSpec(int n_) : n(n_) {}
    const char *name() const override { return "matmul"; }
    int arity() const override { return n + 1; }
    int nout() const override { return n; }
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        TY_REQUIRE(n >= 2 && n <= kMaxGroup, "grouped weight gradients: 2 .. %d products", kMaxGroup);
        for (int i = 0; i <= n; i++)
            TY_REQUIRE(a[i].dtype == F16 && a[i].shape.size() == 2 && a[i].shape[0] == a[n].shape[0] &&
                           (i == n || a[i] == a[0]),
                       "grouped weight gradients: (dy f16 [S,N] x n, x f16 [S,K]) expected");
        o.assign(n, CellType({a[0].shape[1], a[n].shape[1]}, F16));
        return 0;
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t acc, void *, size_t) const override
    {
        const int64_t Sq = aty[0].shape[0], N = aty[0].shape[1], K = aty[n].shape[1];
        const uint32_t all = (1u << n) - 1;
        if ((acc & all) != 0 && (acc & all) != all) {          // mixed modes: one after the other
            for (int i = 0; i < n; i++) {
                const int rc = cacti_hip_gemm_f16(1, 0, N, K, Sq, 1.f, a[i], N, a[n], K, ((acc >> i) & 1) ? 1.f : 0.f,
                                                  o[i], K, S(c));
                if (rc) return rc;
            }
            return 0;
        }
        const void *A[kMaxGroup], *B[kMaxGroup];
        void *C[kMaxGroup];
        for (int i = 0; i < n; i++) {
            A[i] = a[i];
            B[i] = a[n];
            C[i] = o[i];
        }
        return cacti_hip_gemm_f16_batched(1, 0, n, N, K, Sq, 1.f, A, N, B, K, (acc & 1) ? 1.f : 0.f, C, K, S(c));
    }
    std::string key(const std::vector<CellType> &aty, uint32_t acc) const override
    {
        char buf[128];
        snprintf(buf, sizeof(buf), "matmul[TN,1x%lldx%lldx%lld%s]x%d", (long long)aty[0].shape[1],
                 (long long)aty[n].shape[1], (long long)aty[0].shape[0], (acc & 1) ? ",acc" : "", n);
        return buf;
    }
};

// y_i = x W_i^T: (x, W_1 .. W_n) -> (y_1 .. y_n)
struct ProjNSpec : ThunkSpec {
    int n;
    bool group_adj;                  // the weight gradients as one grouped thunk as well
    explicit ProjNSpec(int n_, bool ga = true) : n(n_), group_adj(ga) {}
    const char *name() const override { return "matmul"; }
    int arity() const override { return n + 1; }
    int nout() const override { return n; }
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        TY_REQUIRE(n >= 2 && n <= kMaxGroup, "grouped projections: 2 .. %d products", kMaxGroup);
        for (int i = 0; i <= n; i++)
            TY_REQUIRE(a[i].dtype == F16 && a[i].shape.size() == 2 && a[i].shape[1] == a[0].shape[1] &&
                           (i == 0 || a[i] == a[1]),
                       "grouped projections: (x f16 [S,K], W f16 [N,K] x n) expected");
        o.assign(n, CellType({a[0].shape[0], a[1].shape[0]}, F16));
        return 0;
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t acc, void *, size_t) const override
    {
        TY_REQUIRE(acc == 0, "grouped projections: accumulate mode not staged on this path");
        const int64_t Sq = aty[0].shape[0], K = aty[0].shape[1], N = aty[1].shape[0];
        const void *A[kMaxGroup], *B[kMaxGroup];
        void *C[kMaxGroup];
        for (int i = 0; i < n; i++) {
            A[i] = a[0];
            B[i] = a[1 + i];
            C[i] = o[i];
        }
        return cacti_hip_gemm_f16_batched(0, 1, n, Sq, N, K, 1.f, A, K, B, K, 0.f, C, N, S(c));
    }
    std::string key(const std::vector<CellType> &aty, uint32_t) const override
    {
        char buf[128];
        snprintf(buf, sizeof(buf), "matmul[NT,1x%lldx%lldx%lld]x%d", (long long)aty[0].shape[0],
                 (long long)aty[1].shape[0], (long long)aty[0].shape[1], n);
        return buf;
    }
    int pop_adj(Ctx &c, const Entry &e, const std::vector<CellPtr> &dy) const override
    {
        const CellPtr x = e.args[0];
        bool all = group_adj;
        for (int i = 0; i < n; i++) all = all && dy[i];
        int rc;
        if (all) {
            std::vector<CellPtr> ws(e.args.begin() + 1, e.args.end()), in(dy.begin(), dy.begin() + n);
            in.push_back(x);
            if ((rc = c.adj_add(ws, std::unique_ptr<ThunkSpec>(new WgradNSpec(n)), in))) return rc;
        }
        for (int i = n - 1; i >= 0; i--) {
            if (!dy[i]) continue;
            const CellPtr W = e.args[1 + i];
            if (!all && (rc = c.adj_add({W}, std::unique_ptr<ThunkSpec>(new MatMulSpec(true, false, 1.f, 0)), {dy[i], x})))
                return rc;                                                     // G^T A
            if ((rc = c.adj_add({x}, std::unique_ptr<ThunkSpec>(new MatMulSpec(false, false, 1.f, 0)), {dy[i], W})))
                return rc;                                                     // G B
        }
        return 0;
    }
};

// ---------------------------------------------------------------------------
// RoPE (symplectic_embed src/librarium/llama.rs:463-465); cos/sin are const_ cells
// x is [S, H*Dh] (the reference's [1,S,H,Dh] flattened); the head count rides in the spec.
struct RopeBwdSpec : ThunkSpec {
    int64_t H;
    explicit RopeBwdSpec(int64_t h) : H(h) {}
    const char *name() const override { return "rope_bwd"; }
    int arity() const override { return 3; }                       // (dy, cos, sin) -> dx
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        TY_REQUIRE(a[0].dtype == F16 && a[0].shape.size() == 2 && a[0].shape[1] % H == 0,
                   "rope_bwd: dy f16 [S,H*Dh] expected");
        o = {a[0]};
        return 0;
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t acc, void *, size_t) const override
    {
        const auto &s = aty[0].shape;
        return cacti_hip_rope_bwd(s[0], H, s[1] / H, a[0], a[1], a[2], o[0], acc & 1, S(c));
    }
};

// The map on the query and the key of a layer in one launch: (q, k, cos, sin) -> (qr, kr), adjoint
// (dqr, dkr, cos, sin) -> (dq, dk); values as from two RopeSpec thunks.
struct Rope2BwdSpec : ThunkSpec {
    int64_t H;
    explicit Rope2BwdSpec(int64_t h) : H(h) {}
    const char *name() const override { return "rope2_bwd"; }
    int arity() const override { return 4; }
    int nout() const override { return 2; }
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        TY_REQUIRE(a[0].dtype == F16 && a[0].shape.size() == 2 && a[0].shape[1] % H == 0 && a[1] == a[0],
                   "rope2_bwd: two dy f16 [S,H*Dh] expected");
        o = {a[0], a[1]};
        return 0;
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t acc, void *, size_t) const override
    {
        const auto &s = aty[0].shape;
        return cacti_hip_rope_bwd_pair(s[0], H, s[1] / H, a[0], a[1], a[2], a[3], o[0], acc & 1, o[1], (acc >> 1) & 1, S(c));
    }
};

struct Rope2Spec : ThunkSpec {
    int64_t H;
    explicit Rope2Spec(int64_t h) : H(h) {}
    const char *name() const override { return "rope2"; }
    int arity() const override { return 4; }
    int nout() const override { return 2; }
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        TY_REQUIRE(a[0].dtype == F16 && a[0].shape.size() == 2 && a[0].shape[1] % H == 0 && a[1] == a[0] &&
                       a[2].shape.size() == 2 && a[2].shape[0] >= a[0].shape[0] &&
                       a[2].shape[1] == a[0].shape[1] / H && a[2] == a[3],
                   "rope2: (q, k f16 [S,H*Dh], cos [S,Dh], sin [S,Dh]) expected");
        o = {a[0], a[1]};
        return 0;
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t, void *, size_t) const override
    {
        const auto &s = aty[0].shape;
        return cacti_hip_rope_fwd_pair(s[0], H, s[1] / H, a[0], a[1], a[2], a[3], o[0], o[1], S(c));
    }
    int pop_adj(Ctx &c, const Entry &e, const std::vector<CellPtr> &dy) const override
    {
        // one of the two without an adjoint: the single-tensor thunk for the other
        if (!dy[0] && !dy[1]) return 0;
        if (!dy[0] || !dy[1]) {
            const int k = dy[0] ? 0 : 1;
            return c.adj_add({e.args[k]}, std::unique_ptr<ThunkSpec>(new RopeBwdSpec(H)), {dy[k], e.args[2], e.args[3]});
        }
        return c.adj_add({e.args[0], e.args[1]}, std::unique_ptr<ThunkSpec>(new Rope2BwdSpec(H)),
                         {dy[0], dy[1], e.args[2], e.args[3]});
    }
};

struct RopeSpec : ThunkSpec {
    int64_t H;
    explicit RopeSpec(int64_t h) : H(h) {}
    const char *name() const override { return "rope"; }
    int arity() const override { return 3; }
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        TY_REQUIRE(a[0].dtype == F16 && a[0].shape.size() == 2 && a[0].shape[1] % H == 0 &&
                       a[1].shape.size() == 2 && a[1].shape[0] >= a[0].shape[0] &&
                       a[1].shape[1] == a[0].shape[1] / H && a[1] == a[2],
                   "rope: (x f16 [S,H*Dh], cos [S,Dh], sin [S,Dh]) expected");
        o = {a[0]};
        return 0;
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t, void *, size_t) const override
    {
        const auto &s = aty[0].shape;
        return cacti_hip_rope_fwd(s[0], H, s[1] / H, a[0], a[1], a[2], o[0], S(c));
    }
    int pop_adj(Ctx &c, const Entry &e, const std::vector<CellPtr> &dy) const override
    {
        return c.adj_add({e.args[0]}, std::unique_ptr<ThunkSpec>(new RopeBwdSpec(H)),
                         {dy[0], e.args[1], e.args[2]});
    }
};

// ---------------------------------------------------------------------------
// causal softmax over scores (src/librarium/llama.rs:501-505)
struct CausalSoftmaxBwdSpec : ThunkSpec {
    int64_t H;
    explicit CausalSoftmaxBwdSpec(int64_t h) : H(h) {}
    const char *name() const override { return "causal_softmax_bwd"; }
    int arity() const override { return 2; }                       // (s16, dp16) -> ds16
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        TY_REQUIRE(a[0] == a[1], "causal_softmax_bwd: shape mismatch");
        o = {a[0]};
        return 0;
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t acc, void *, size_t) const override
    {
        TY_REQUIRE(!(acc & 1), "causal_softmax_bwd: accumulate mode not staged on this path");
        return cacti_hip_causal_softmax_bwd(aty[0].shape[0], H, a[0], a[1], o[0], S(c));
    }
};

struct CausalSoftmaxSpec : ThunkSpec {
    int64_t H;
    explicit CausalSoftmaxSpec(int64_t h) : H(h) {}
    const char *name() const override { return "causal_softmax"; }
    int arity() const override { return 1; }
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        TY_REQUIRE(a[0].dtype == F16 && a[0].shape.size() == 2 && a[0].shape[1] == H * a[0].shape[0],
                   "causal_softmax: s16 f16 [S,H*S] expected");
        o = {a[0]};
        return 0;
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t, void *, size_t) const override
    {
        return cacti_hip_causal_softmax_fwd(aty[0].shape[0], H, a[0], o[0], S(c));
    }
    int pop_adj(Ctx &c, const Entry &e, const std::vector<CellPtr> &dy) const override
    {
        return c.adj_add({e.args[0]}, std::unique_ptr<ThunkSpec>(new CausalSoftmaxBwdSpec(H)),
                         {e.args[0], dy[0]});
    }
};

// ---------------------------------------------------------------------------
// The attention block of a layer as one thunk: scores, cast, mask, softmax, cast and the product with
// v (src/librarium/llama.rs:501-507) with the rounding points of the separate thunks; the adjoint thunk
// stands for the adjoints of all of them.  q, k, v, o: [S, H*Dh]; stats: f32 [2*H*S].
struct AttentionBwdSpec : ThunkSpec {
    int64_t H;
    float alpha;
    AttentionBwdSpec(int64_t h, float a) : H(h), alpha(a) {}
    const char *name() const override { return "attention_bwd"; }
    int arity() const override { return 6; }                       // (q, k, v, dO, stats, o) -> dq, dk, dv
    int nout() const override { return 3; }
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        TY_REQUIRE(a[0] == a[1] && a[0] == a[2] && a[0] == a[3] && a[0] == a[5] && a[0].shape.size() == 2 &&
                       a[4].dtype == F32,
                   "attention_bwd: (q, k, v, dO f16 [S,H*Dh], stats f32, o) expected");
        o = {a[0], a[0], a[0]};
        return 0;
    }
    size_t workspace(const std::vector<CellType> &a) const override
    {
        return cacti_hip_attention_bwd_workspace(a[0].shape[0], H);
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t acc, void *ws, size_t wsb) const override
    {
        const auto &s = aty[0].shape;
        return cacti_hip_attention_bwd(s[0], H, s[1] / H, alpha, a[0], a[1], a[2], a[5], a[3], s[1], a[4], o[0],
                                       acc & 1, o[1], (acc >> 1) & 1, o[2], (acc >> 2) & 1, ws, wsb, S(c));
    }
};

struct AttentionSpec : ThunkSpec {
    int64_t H;
    float alpha;
    AttentionSpec(int64_t h, float a) : H(h), alpha(a) {}
    const char *name() const override { return "attention"; }
    int arity() const override { return 3; }                       // (q, k, v) -> o, stats
    int nout() const override { return 2; }
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        TY_REQUIRE(a[0].dtype == F16 && a[0] == a[1] && a[0] == a[2] && a[0].shape.size() == 2 &&
                       a[0].shape[1] % H == 0,
                   "attention: (q, k, v f16 [S,H*Dh]) expected");
        o = {a[0], CellType({(int64_t)(cacti_hip_attention_stats_bytes(a[0].shape[0], H) / sizeof(float))}, F32)};
        return 0;
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t acc, void *, size_t) const override
    {
        TY_REQUIRE(acc == 0, "attention: accumulate mode not staged on this path");
        const auto &s = aty[0].shape;
        return cacti_hip_attention_fwd(s[0], H, s[1] / H, alpha, a[0], a[1], a[2], s[1], o[0], o[1], S(c));
    }
    int pop_adj(Ctx &c, const Entry &e, const std::vector<CellPtr> &dy) const override
    {
        if (!dy[0]) return 0;
        return c.adj_add({e.args[0], e.args[1], e.args[2]},
                         std::unique_ptr<ThunkSpec>(new AttentionBwdSpec(H, alpha)),
                         {e.args[0], e.args[1], e.args[2], dy[0], e.outs[1], e.outs[0]});
    }
};

// ---------------------------------------------------------------------------
// SiLU gate (src/librarium/llama.rs:526-527)
struct SiluGateBwdSpec : ThunkSpec {
    const char *name() const override { return "silu_gate_bwd"; }
    int arity() const override { return 3; }                       // (g, u, dh) -> dg, du
    int nout() const override { return 2; }
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        TY_REQUIRE(a[0] == a[1] && a[0] == a[2], "silu_gate_bwd: shape mismatch");
        o = {a[0], a[0]};
        return 0;
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t acc, void *, size_t) const override
    {
        return cacti_hip_silu_gate_bwd(aty[0].numel(), a[0], a[1], a[2], o[0], acc & 1, o[1],
                                       (acc >> 1) & 1, S(c));
    }
};

struct SiluGateSpec : ThunkSpec {
    const char *name() const override { return "silu_gate"; }
    int arity() const override { return 2; }
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        TY_REQUIRE(a[0] == a[1] && a[0].dtype == F16, "silu_gate: equal f16 shapes expected");
        o = {a[0]};
        return 0;
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t, void *, size_t) const override
    {
        return cacti_hip_silu_gate_fwd(aty[0].numel(), a[0], a[1], o[0], S(c));
    }
    int pop_adj(Ctx &c, const Entry &e, const std::vector<CellPtr> &dy) const override
    {
        return c.adj_add({e.args[0], e.args[1]}, std::unique_ptr<ThunkSpec>(new SiluGateBwdSpec()),
                         {e.args[0], e.args[1], dy[0]});
    }
};

// ---------------------------------------------------------------------------
// LM loss (src/librarium/llama.rs:541-546)
struct SoftmaxCeBwdSpec : ThunkSpec {
    const char *name() const override { return "softmax_ce_bwd"; }
    int arity() const override { return 3; }                       // (logit, tok, dloss) -> dlogit
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        TY_REQUIRE(a[0].shape.size() == 2 && a[2].dtype == F32 && a[2].numel() == a[0].shape[0],
                   "softmax_ce_bwd: (logit [N,V], tok, dloss f32 [N]) expected");
        o = {a[0]};
        return 0;
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t acc, void *, size_t) const override
    {
        return cacti_hip_softmax_ce_bwd(aty[0].shape[0], aty[0].shape[1], a[0], a[1], a[2], o[0],
                                        acc & 1, S(c));
    }
};

struct SoftmaxCeSpec : ThunkSpec {
    bool want_prob;
    explicit SoftmaxCeSpec(bool p) : want_prob(p) {}
    const char *name() const override { return "softmax_ce"; }
    int arity() const override { return 2; }
    int nout() const override { return want_prob ? 3 : 2; }
    int out_ty(const std::vector<CellType> &a, std::vector<CellType> &o) const override
    {
        TY_REQUIRE(a[0].dtype == F16 && a[0].shape.size() == 2 && a[1].dtype == U16 &&
                       a[1].numel() == a[0].shape[0],
                   "softmax_ce: (logit f16 [N,V], tok u16 [N]) expected");
        o = {CellType({a[0].shape[0]}, F32), CellType({a[0].shape[0]}, U16)};
        if (want_prob) o.push_back(CellType(a[0].shape, F32));
        return 0;
    }
    int run(Ctx &c, const std::vector<CellType> &aty, void *const *a, const std::vector<CellType> &,
            void *const *o, uint32_t, void *, size_t) const override
    {
        return cacti_hip_softmax_ce_fwd(aty[0].shape[0], aty[0].shape[1], a[0], a[1],
                                        want_prob ? o[2] : nullptr, o[0], o[1], c.status_ptr(), S(c));
    }
    int pop_adj(Ctx &c, const Entry &e, const std::vector<CellPtr> &dy) const override
    {
        if (!dy[0]) return 0;                    // only the loss output carries a gradient
        return c.adj_add({e.args[0]}, std::unique_ptr<ThunkSpec>(new SoftmaxCeBwdSpec()),
                         {e.args[0], e.args[1], dy[0]});
    }
};

}  // namespace

std::unique_ptr<ThunkSpec> make_embed() { return std::unique_ptr<ThunkSpec>(new EmbedSpec()); }
std::unique_ptr<ThunkSpec> make_rms_norm(float eps)
{
    return std::unique_ptr<ThunkSpec>(new RmsNormSpec(eps));
}
std::unique_ptr<ThunkSpec> make_matmul(bool ta, bool tb, float alpha)
{
    return std::unique_ptr<ThunkSpec>(new MatMulSpec(ta, tb, alpha, 0));
}
std::unique_ptr<ThunkSpec> make_projections(int n, bool group_adjoints)
{
    return std::unique_ptr<ThunkSpec>(new ProjNSpec(n, group_adjoints));
}
std::unique_ptr<ThunkSpec> make_block_matmul(bool ta, bool tb, float alpha, int64_t H)
{
    return std::unique_ptr<ThunkSpec>(new MatMulSpec(ta, tb, alpha, H));
}
std::unique_ptr<ThunkSpec> make_causal_scores(float alpha, int64_t H)
{
    return std::unique_ptr<ThunkSpec>(new MatMulSpec(false, true, alpha, H, CAUSAL_OUT));
}
std::unique_ptr<ThunkSpec> make_causal_pv(int64_t H)
{
    return std::unique_ptr<ThunkSpec>(new MatMulSpec(false, false, 1.f, H, CAUSAL_A));
}
std::unique_ptr<ThunkSpec> make_rope(int64_t H) { return std::unique_ptr<ThunkSpec>(new RopeSpec(H)); }
std::unique_ptr<ThunkSpec> make_rope2(int64_t H) { return std::unique_ptr<ThunkSpec>(new Rope2Spec(H)); }
std::unique_ptr<ThunkSpec> make_causal_softmax(int64_t H)
{
    return std::unique_ptr<ThunkSpec>(new CausalSoftmaxSpec(H));
}
std::unique_ptr<ThunkSpec> make_attention(float alpha, int64_t H)
{
    return std::unique_ptr<ThunkSpec>(new AttentionSpec(H, alpha));
}
std::unique_ptr<ThunkSpec> make_add() { return std::unique_ptr<ThunkSpec>(new AddSpec()); }
std::unique_ptr<ThunkSpec> make_add_rms_norm(float eps)
{
    return std::unique_ptr<ThunkSpec>(new AddRmsNormSpec(eps));
}
std::unique_ptr<ThunkSpec> make_copy() { return std::unique_ptr<ThunkSpec>(new CopySpec()); }
std::unique_ptr<ThunkSpec> make_silu_gate()
{
    return std::unique_ptr<ThunkSpec>(new SiluGateSpec());
}
std::unique_ptr<ThunkSpec> make_softmax_ce(bool want_prob)
{
    return std::unique_ptr<ThunkSpec>(new SoftmaxCeSpec(want_prob));
}

}  // namespace cacti
