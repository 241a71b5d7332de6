// Host runtime behind the C ABI: device context with a pooled allocator and host spill,
// cells with VMem / Mem replicas, the thunk interface, and the spine (staged instruction
// log, reverse-mode AD, liveness, interpreter).
//
// It mirrors the reference's structure for this path -- PCtx / NvGpuMemPool / PCell
// (src/pctx/nvgpu.rs, src/cell/mod.rs:2245-2669), ThunkSpec / ThunkImpl
// (src/thunk/mod.rs:257-351), Spine (src/spine.rs) -- at the granularity of the fused
// thunks, with one in-order HIP stream and no per-thunk stream syncs.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <deque>
#include <map>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

namespace cacti {

enum Dtype : int { F16 = 0, F32 = 1, U16 = 2, I32 = 3 };
inline size_t dtype_size(Dtype d) { return d == F16 || d == U16 ? 2 : 4; }

struct CellType {
    std::vector<int64_t> shape;
    Dtype dtype = F16;
    CellType() {}
    CellType(std::vector<int64_t> s, Dtype d) : shape(std::move(s)), dtype(d) {}
    int64_t numel() const
    {
        int64_t n = 1;
        for (int64_t v : shape) n *= v;
        return n;
    }
    size_t bytes() const { return (size_t)numel() * dtype_size(dtype); }
    bool operator==(const CellType &o) const { return dtype == o.dtype && shape == o.shape; }
};

typedef int32_t CellPtr;                 // 0 = nil
constexpr size_t kNoOffset = ~(size_t)0;
constexpr size_t kAllocAlign = 256;      // src/pctx/nvgpu.rs:30

// ---------------------------------------------------------------------------
// MemPool: offset arithmetic over one reserved region (no HIP calls, so the policy is
// testable on a CPU).  First fit over the coalesced free-region set, else bump the
// front cursor (src/pctx/nvgpu.rs:1633-1655); freeing the last region retracts it.
class MemPool {
   public:
    explicit MemPool(size_t cap = 0) : cap_(cap) {}
    void reset(size_t cap);
    // offset, or kNoOffset when it does not fit.  `high` allocations (cells that live across cycles:
    // parameters, gradients) are packed downwards from the top of the pool, the others upwards from
    // the bottom, so that the short-lived regions of a cycle do not end up scattered between the
    // long-lived ones; each kind falls back to the other's holes before it gives up.
    size_t alloc(size_t bytes, bool high = false);
    void free(size_t off);
    size_t size_of(size_t off) const;
    size_t cap() const { return cap_; }
    size_t used() const { return used_; }
    size_t peak() const { return peak_; }
    size_t front() const { return front_; }
    size_t largest_free() const;         // largest request that would succeed now
    size_t num_allocs() const { return alloc_.size(); }

   private:
    size_t cap_ = 0, front_ = 0, back_ = 0, used_ = 0, peak_ = 0;
    std::map<size_t, size_t> free_;                  // holes below front_: offset -> size, coalesced
    std::map<size_t, size_t> free_hi_;               // holes from back_ up
    size_t take_low(size_t req, std::map<size_t, size_t> &holes);
    size_t take_high(size_t req, std::map<size_t, size_t> &holes);
    std::unordered_map<size_t, size_t> alloc_;       // offset -> size
};

// ---------------------------------------------------------------------------
struct Cell {
    CellType ty;
    std::string name;
    bool stable = false;     // survives reset() (parameters, gradients, constants)
    bool konst = false;      // no adjoint is generated for it (src/spine.rs:495-498)
    bool alive = true;
    size_t voff = kNoOffset; // VMem replica: offset into the pool
    void *hptr = nullptr;    // Mem replica (host)
    bool v_valid = false, h_valid = false;
    int pin = 0;
    hipEvent_t h_busy = nullptr;   // recorded after the last copy that touches hptr
    hipEvent_t v_ready = nullptr;  // a prefetching upload into the VMem replica is in flight on the copy stream
};

struct Stats {
    uint64_t pool_cap, pool_used, pool_peak, pool_front;
    uint64_t n_alloc, n_evict, n_upload, bytes_d2h, bytes_h2d, n_soft_oom;
    uint64_t n_entries, n_thunks_run, host_bytes;
};

class Ctx;
struct Entry;

// ThunkSpec + ThunkImpl in one object: type inference, execution (`run` covers both
// apply and accumulate: bit k of acc_mask says output k already holds a value), and the
// adjoint rule (pop_adj stages further thunks).  src/thunk/mod.rs:257-351.
struct ThunkSpec {
    virtual ~ThunkSpec() {}
    virtual const char *name() const = 0;
    virtual int arity() const = 0;
    virtual int nout() const { return 1; }
    // a plain copy of argument 0 into output 0 (lets the runtime hand over the storage of a
    // source that dies at this entry instead of copying it)
    virtual bool is_copy() const { return false; }
    virtual int out_ty(const std::vector<CellType> &arg, std::vector<CellType> &out) const = 0;
    virtual size_t workspace(const std::vector<CellType> &) const { return 0; }
    // label under which launches are grouped in the timing report (name + shape for GEMMs)
    virtual std::string key(const std::vector<CellType> &, uint32_t) const { return name(); }
    virtual int run(Ctx &ctx, const std::vector<CellType> &aty, void *const *a,
                    const std::vector<CellType> &oty, void *const *o, uint32_t acc_mask,
                    void *ws, size_t ws_bytes) const = 0;
    // out_adj[k] = adjoint cell of output k or 0; stage contributions through ctx.adj_*
    virtual int pop_adj(Ctx &, const Entry &, const std::vector<CellPtr> &) const { return 0; }
};

enum EntryKind : int { E_APPLY = 0, E_YIELD_SET = 1, E_UNLIVE = 2 };

struct Entry {
    EntryKind kind = E_APPLY;
    int thunk = -1;
    std::vector<CellPtr> args, outs;
    uint32_t acc_mask = 0;
    bool move = false;       // copy whose source dies here: the output takes over its storage
    CellPtr cell = 0;        // E_YIELD_SET / E_UNLIVE
};

enum ResumeStatus : int { R_DONE = 0, R_YIELD = 1 };

class Ctx {
   public:
    Ctx();
    ~Ctx();
    int init(int dev, size_t pool_bytes, int host_pagelocked);

    // ---- cells
    CellPtr cell_new(const CellType &ty, bool stable, const char *name = "");
    Cell &cell(CellPtr c) { return cells_[c]; }
    // a handle from outside: in range and not freed
    bool is_live(CellPtr c) const { return c > 0 && (size_t)c < cells_.size() && cells_[c].alive; }
    void set_const(CellPtr c) { cells_[c].konst = true; }
    int cell_put(CellPtr c, const void *host, size_t bytes);     // host -> cell (Mem, then VMem)
    int cell_get(CellPtr c, void *host, size_t bytes);           // cell -> host (syncs)
    // NaN count and abs-log2 histogram (int64 [256]) of n f16 cells, one stream sync for all;
    // x.nan_count(), x.abs_log2_hist8() of the reference's example (open_llama_3b_train.rs:409-424)
    int cells_digest(const CellPtr *cells, int n, int64_t *hist, int64_t *nan);
    // one AdamW32 step of n tensors in one launch: grads f16 (read), avgs / avg2s / masters f32
    // (updated), params f16 (written); sc = the seven scalars of cacti_adamw32_scalars.  Returns
    // without synchronising.
    int cells_adamw32(int n, const CellPtr *grads, const CellPtr *avgs, const CellPtr *avg2s,
                      const CellPtr *masters, const CellPtr *params, const float *sc);
    // Streams `bytes` of a file (at `off` of `fd`) into the device replica of cell c: the range is
    // read by a few threads into two page-locked buffers in turn, uploaded, and (cast != 0)
    // converted on the device: 0 = bytes as they are, 1 = bf16 bit patterns -> f16, 2 = f32 -> f16.
    // The cell ends with a device value and no host replica.  Returns with the work queued.
    int cell_ingest(CellPtr c, int fd, uint64_t off, size_t bytes, int cast);
    int cell_cast_f16_f32(CellPtr src, CellPtr dst);              // set_cast, src/op.rs:1085-1096
    int cell_zero(CellPtr c);                                    // set_zeros, src/op.rs:1137-1146
    int cell_free_all(CellPtr c);
    void *dev_ptr(size_t off) { return base_ + off; }
    // make the VMem replica exist (evicting others if needed) and, if `need_value`, hold
    // the current version (uploading from the host replica)
    int ensure_vmem(CellPtr c, bool need_value);
    int pool_alloc(size_t bytes, size_t *off, bool high = false);                   // with soft-OOM eviction
    void pool_free(size_t off) { pool_.free(off); }              // later reuse is ordered on the stream
    int try_soft_oom(size_t need);
    int evict(CellPtr c);                                        // VMem -> Mem, drop VMem
    // Overlapped spilling (page-locked host memory only).  Downloads and uploads run on two further
    // streams of the same priority (PCIe carries both directions at once), ordered with events: an
    // evicted region returns to the pool when its download is done (or the streams that may reuse it
    // are made to wait for it).  Victims are resident cells whose next use in the compiled log lies
    // farthest ahead, taken in turn from those that can be dropped without a copy (a valid host
    // replica: parameters after their use in the forward pass) and those that need a download but no
    // later upload (their next use overwrites them: the gradients of the cycle before), so that
    // both directions carry about the same; then any other cell.  Before every thunk a reserve of
    // free memory is kept by evicting ahead of need, and cells the next thunks read are uploaded
    // ahead of them.
    size_t next_use(CellPtr c, bool *overwrite = nullptr) const;  // entry index, beyond the log = next cycle
    enum VictimClass : int { V_ANY = 0, V_DROP = 1, V_DOWN_ONLY = 2 };
    int pick_victim(size_t min_bytes, bool allow_prefetched = false, int cls = V_ANY) const;   // 0: none
    void reclaim(size_t need);                                   // return finished downloads' regions to the pool (need > 0: wait for more until it fits)
    int keep_reserve();
    int prefetch_ahead();

    // ---- staging (control thread side of the spine)
    void reset();                                                // src/ctx.rs:150-235
    int add_thunk(std::unique_ptr<ThunkSpec> spec);
    int stage_apply(int thunk, const std::vector<CellPtr> &args, std::vector<CellPtr> *outs);
    int stage_into(int thunk, const std::vector<CellPtr> &args, const std::vector<CellPtr> &outs,
                   uint32_t acc_mask);
    void stage_yield_set(CellPtr c);
    void keep(CellPtr c) { kept_.push_back(c); }
    // reverse-mode AD: src/spine.rs:447-690 (CellMap::vadd_vjp, src/op.rs:2386-2393)
    void adj_seed(CellPtr primal, CellPtr adj);                  // sink.add(y, dy)
    void adj_bind(CellPtr primal, CellPtr adj, bool cached = false);   // grad_map.add(p, g) [+ g.cache()]
    CellPtr adj_of(CellPtr primal);                              // 0 for const cells
    bool adj_written(CellPtr primal);
    // arg_adj[..] += thunk(args): Apply on first write, Accumulate afterwards (src/op.rs:20-188)
    int adj_add(const std::vector<CellPtr> &primals, std::unique_ptr<ThunkSpec> spec,
                const std::vector<CellPtr> &args);
    int vadd_vjp();
    int compile();                                               // liveness, src/spine.rs:1435-1478
    int resume(CellPtr *yield_cell);                             // src/spine.rs:1484-1991
    int resume_put(CellPtr c, const void *host, size_t bytes);

    hipStream_t stream() const { return stream_; }
    int sync();
    // device word that kernels raise when a token / key id is out of range (the
    // reference asserts inside the kernel, src/thunk/op.rs:3538); checked at sync points
    void *status_ptr() { return base_ + status_off_; }
    int check_status();
    void stats(Stats *s) const;
    // the pool's usage by class of cell, as text (NvGpuPCtx::_dump_usage / _dump_sizes / _dump_free,
    // src/pctx/nvgpu.rs:690-742): what an exhausted pool prints, and the per-cycle report
    std::string usage_report() const;
    const std::vector<Entry> &log() const { return log_; }
    const ThunkSpec &thunk(int i) const { return *thunks_[i]; }
    const char *entry_name(size_t i) const;
    // 0 = off; 1 = sync after every thunk; 2 = event pairs recorded without syncing and read
    // back by collect_timings() (measures each launch inside an undisturbed run)
    void set_timing(int mode) { timing_ = mode; }
    void set_timing_filter(const std::string &prefix, int every)
    {
        timing_filter_ = prefix;
        timing_every_ = every;
        timing_seen_ = 0;
    }
    int collect_timings();
    void clear_timings() { times_.clear(); }
    uint64_t operand_bytes(const std::string &key) const
    {
        auto it = op_bytes_.find(key);
        return it == op_bytes_.end() ? 0 : it->second;
    }
    const std::map<std::string, std::pair<double, uint64_t>> &timings() const { return times_; }

   private:
    int run_entry(const Entry &e);
    int host_alloc(Cell &c);
    void host_free(Cell &c);
    hipEvent_t ev_get();
    void ev_put(hipEvent_t e) { if (e) ev_spare_.push_back(e); }
    int order_after_compute(hipStream_t st);                     // st waits for the compute work queued so far

    struct PendingFree { size_t off, bytes; hipEvent_t done; };
    struct HostBuf { void *ptr; hipEvent_t busy; };
    hipStream_t down_stream_ = nullptr, up_stream_ = nullptr;
    size_t sum_dropped_ = 0, sum_downloaded_ = 0;               // bytes evicted per class so far
    // Downloads that a cycle had to wait for are started early in the next one: as soon as a thunk
    // has written a cell that this cycle does not touch again and the next one overwrites (a
    // gradient), the cell is evicted, until as many bytes have gone as the cycle before downloaded
    // in all.  The first such cells are written early in the backward pass, so their downloads
    // overlap the rest of it instead of the forward pass that needs the memory.  The budget is half
    // of what the cycle before evicted in any way: the other half is left to cells that are dropped
    // without a copy and come back on the upload stream, so that both directions of the link work.
    size_t eager_left_ = 0, cyc_eager_ = 0, prev_eager_ = 0, cyc_demand_down_ = 0, cyc_dropped_ = 0;
    bool in_eager_ = false;
    size_t stable_end_ = 0;                                      // one past the largest id a stable cell has had
    size_t pf_cursor_ = 0;                                       // entries before it have had their far prefetch
    int spill_eagerly(const Entry &e);
    int upload_ahead(Cell &c, bool *ordered);                    // one cell, on the upload stream
    size_t reserve_bytes() const { return std::min<size_t>(pool_.cap() / 24, (size_t)640 << 20); }
    bool async_spill_ = false;
    std::vector<PendingFree> pending_;                           // regions of evicted cells, oldest first
    size_t pending_bytes_ = 0;
    std::deque<hipEvent_t> ev_spare_;                            // recycled oldest first, and only when plenty
    std::unordered_map<CellPtr, std::vector<uint32_t>> uses_;    // compiled log: entries that touch a cell
    std::multimap<size_t, HostBuf> host_pool_;                   // page-locked buffers of dead cells, by size
    int dev_ = 0;
    bool counted_ = false;                      // this context is in the device's live-context count
    hipStream_t stream_ = nullptr;
    bool own_stream_ = false;
    char *base_ = nullptr;
    size_t status_off_ = 0;
    MemPool pool_;
    int host_pagelocked_ = 1;
    std::vector<Cell> cells_;
    std::vector<std::unique_ptr<ThunkSpec>> thunks_;
    std::vector<Entry> log_;
    std::vector<CellPtr> kept_;
    size_t pc_ = 0;
    bool compiled_ = false;
    size_t fwd_end_ = 0;
    std::unordered_map<CellPtr, CellPtr> adj_;       // primal -> adjoint cell
    std::unordered_map<CellPtr, bool> adj_wr_;       // adjoint already written in the log
    std::vector<CellPtr> pending_yield_;
    // statistics
    uint64_t n_alloc_ = 0, n_evict_ = 0, n_upload_ = 0, bytes_d2h_ = 0, bytes_h2d_ = 0,
             n_soft_oom_ = 0, n_run_ = 0, host_bytes_ = 0;
    uint64_t n_moved_ = 0;
    int timing_ = 0;
    std::string timing_filter_;
    int timing_every_ = 1;
    uint64_t timing_seen_ = 0;
    std::vector<std::pair<hipEvent_t, hipEvent_t>> ev_pool_;
    std::vector<std::string> ev_keys_;
    std::map<std::string, std::pair<double, uint64_t>> times_;
    std::map<std::string, uint64_t> op_bytes_;                   // label -> operand bytes of one launch
    hipEvent_t ev0_ = nullptr, ev1_ = nullptr;
    // cell_ingest: two page-locked staging buffers and the event after the last upload from each
    void *ingest_host_[2] = {nullptr, nullptr};
    hipEvent_t ingest_ev_[2] = {nullptr, nullptr};
};

}  // namespace cacti
