// Device context, pooled allocator with host spill, cells and the spine interpreter.
#include "runtime.h"

#include <stdlib.h>
#include <string.h>

#include <unistd.h>

#include <algorithm>
#include <thread>

#include "../../include/cacti_hip_runtime.h"
#include "common.h"

namespace cacti {

// ===========================================================================
// MemPool

void MemPool::reset(size_t cap)
{
    cap_ = back_ = cap;
    front_ = used_ = peak_ = 0;
    free_.clear();
    free_hi_.clear();
    alloc_.clear();
}

// first fit from the lowest offset, the low end of the hole
size_t MemPool::take_low(size_t req, std::map<size_t, size_t> &holes)
{
    for (auto it = holes.begin(); it != holes.end(); ++it) {
        if (it->second < req) continue;
        const size_t off = it->first, rest = it->second - req;
        holes.erase(it);
        if (rest) holes[off + req] = rest;
        return off;
    }
    return kNoOffset;
}

// first fit from the highest offset, the high end of the hole
size_t MemPool::take_high(size_t req, std::map<size_t, size_t> &holes)
{
    for (auto it = holes.rbegin(); it != holes.rend(); ++it) {
        if (it->second < req) continue;
        it->second -= req;
        const size_t off = it->first + it->second;
        if (it->second == 0) holes.erase(it->first);
        return off;
    }
    return kNoOffset;
}

size_t MemPool::alloc(size_t bytes, bool high)
{
    if (bytes == 0) bytes = 1;
    const size_t req = (bytes + kAllocAlign - 1) / kAllocAlign * kAllocAlign;
    size_t off = high ? take_high(req, free_hi_) : take_low(req, free_);
    if (off == kNoOffset && req <= back_ - front_) {              // move the cursor of that end
        if (high) {
            back_ -= req;
            off = back_;
        } else {
            off = front_;
            front_ += req;
        }
    }
    if (off == kNoOffset) off = high ? take_high(req, free_) : take_low(req, free_hi_);
    if (off == kNoOffset) return kNoOffset;
    alloc_[off] = req;
    used_ += req;
    if (used_ > peak_) peak_ = used_;
    return off;
}

void MemPool::free(size_t off)
{
    auto it = alloc_.find(off);
    if (it == alloc_.end()) return;
    size_t sz = it->second;
    alloc_.erase(it);
    used_ -= sz;
    const bool hi = off >= back_;
    std::map<size_t, size_t> &holes = hi ? free_hi_ : free_;
    auto next = holes.lower_bound(off);
    if (next != holes.end() && off + sz == next->first) {         // merge with the next region
        sz += next->second;
        next = holes.erase(next);
    }
    if (next != holes.begin()) {                                  // merge with the previous one
        auto prev = std::prev(next);
        if (prev->first + prev->second == off) {
            off = prev->first;
            sz += prev->second;
            holes.erase(prev);
        }
    }
    if (!hi && off + sz == front_)
        front_ = off;                                             // retract the cursor of that end
    else if (hi && off == back_)
        back_ = off + sz;
    else
        holes[off] = sz;
}

size_t MemPool::size_of(size_t off) const
{
    auto it = alloc_.find(off);
    return it == alloc_.end() ? 0 : it->second;
}

size_t MemPool::largest_free() const
{
    size_t best = back_ - front_;
    for (auto &kv : free_) best = std::max(best, kv.second);
    for (auto &kv : free_hi_) best = std::max(best, kv.second);
    return best;
}

// ===========================================================================
// Ctx

Ctx::Ctx() { cells_.emplace_back(); cells_[0].alive = false; }   // cell 0 = nil

Ctx::~Ctx()
{
    if (stream_) hipStreamSynchronize(stream_);
    if (down_stream_) hipStreamSynchronize(down_stream_);
    if (up_stream_) hipStreamSynchronize(up_stream_);
    for (auto &c : cells_) {
        host_free(c);
        if (c.v_ready) hipEventDestroy(c.v_ready);
    }
    for (auto &kv : host_pool_) {
        if (kv.second.busy) hipEventDestroy(kv.second.busy);
        hipHostFree(kv.second.ptr);
    }
    for (auto &pf : pending_) hipEventDestroy(pf.done);
    for (hipEvent_t e : ev_spare_) hipEventDestroy(e);
    if (down_stream_) hipStreamDestroy(down_stream_);
    if (up_stream_) hipStreamDestroy(up_stream_);
    for (auto &e : ev_pool_) {
        hipEventDestroy(e.first);
        hipEventDestroy(e.second);
    }
    if (ev0_) hipEventDestroy(ev0_);
    if (ev1_) hipEventDestroy(ev1_);
    for (int k = 0; k < 2; k++) {
        if (ingest_host_[k]) hipHostFree(ingest_host_[k]);
        if (ingest_ev_[k]) hipEventDestroy(ingest_ev_[k]);
    }
    if (base_) hipFree(base_);
    if (own_stream_ && stream_) hipStreamDestroy(stream_);
    if (counted_) live_contexts_add(dev_, -1);
}

int Ctx::init(int dev, size_t pool_bytes, int host_pagelocked)
{
    dev_ = dev;
    host_pagelocked_ = host_pagelocked;
    CACTI_HIP(hipSetDevice(dev));
    size_t avail = 0, total = 0;
    CACTI_HIP(hipMemGetInfo(&avail, &total));
    if (host_pagelocked < 0) host_pagelocked_ = cacti_env_host_pagelocked();
    if (pool_bytes == 0) {
        // CACTI_VMEM_SOFT_LIMIT (a byte size with a unit, or a fraction of the device), else the
        // default reserve of 90.01 % of the device: src/ctx.rs:43, src/pctx/nvgpu.rs:1434-1463
        const char *lim = getenv("CACTI_VMEM_SOFT_LIMIT");
        size_t want = 0;
        int rc = cacti_vmem_soft_limit(lim, avail, total, &want);
        if (rc) return rc;
        if (!lim || !lim[0]) {                                    // the default gives way to other users of the device
            const size_t room = avail > (512u << 20) ? avail - (512u << 20) : avail / 2;
            want = std::min(want, room);
        }
        pool_bytes = want;
    }
    pool_bytes = (pool_bytes >> 16) << 16;                        // 64 KiB granules
    CACTI_REQUIRE(pool_bytes > 0 && pool_bytes <= avail, CACTI_E_OOM,
                  "ctx: cannot reserve %zu bytes (%zu available of %zu); lower the pool cap "
                  "(the pool_bytes argument, or CACTI_VMEM_SOFT_LIMIT when that is 0)",
                  pool_bytes, avail, total);
    CACTI_HIP(hipMalloc((void **)&base_, pool_bytes));
    live_contexts_add(dev_, 1);
    counted_ = true;
    CACTI_REQUIRE(((uintptr_t)base_ % kAllocAlign) == 0, CACTI_E_STATE, "ctx: misaligned reserve");
    pool_.reset(pool_bytes);
    status_off_ = pool_.alloc(kAllocAlign);
    CACTI_HIP(hipMemset(base_ + status_off_, 0, kAllocAlign));
    CACTI_HIP(hipStreamCreateWithFlags(&stream_, hipStreamNonBlocking));
    own_stream_ = true;
    // spill copies overlap compute only from page-locked memory (a copy from pageable memory is staged
    // synchronously by the runtime); default priority, like the compute stream
    async_spill_ = host_pagelocked_ != 0;
    if (async_spill_) {
        CACTI_HIP(hipStreamCreateWithFlags(&down_stream_, hipStreamNonBlocking));
        CACTI_HIP(hipStreamCreateWithFlags(&up_stream_, hipStreamNonBlocking));
    }
    CACTI_HIP(hipEventCreate(&ev0_));
    CACTI_HIP(hipEventCreate(&ev1_));
    return 0;
}

int Ctx::sync()
{
    CACTI_HIP(hipStreamSynchronize(stream_));
    if (down_stream_) CACTI_HIP(hipStreamSynchronize(down_stream_));
    if (up_stream_) CACTI_HIP(hipStreamSynchronize(up_stream_));
    return 0;
}

hipEvent_t Ctx::ev_get()
{
    // an event goes back into use long after the waits that name it were queued
    if (ev_spare_.size() > 256) {
        hipEvent_t e = ev_spare_.front();
        ev_spare_.pop_front();
        return e;
    }
    hipEvent_t e = nullptr;
    if (hipEventCreateWithFlags(&e, hipEventDisableTiming) != hipSuccess) return nullptr;
    return e;
}

int Ctx::order_after_compute(hipStream_t st)
{
    hipEvent_t e = ev_get();
    CACTI_REQUIRE(e, CACTI_E_STATE, "ctx: cannot create an event");
    CACTI_HIP(hipEventRecord(e, stream_));
    CACTI_HIP(hipStreamWaitEvent(st, e, 0));
    ev_put(e);                         // the wait is queued; the event may be recorded again
    return 0;
}

int Ctx::check_status()
{
    int v = 0;
    CACTI_HIP(hipMemcpyAsync(&v, status_ptr(), sizeof(int), hipMemcpyDeviceToHost, stream_));
    CACTI_HIP(hipStreamSynchronize(stream_));
    if (v) {
        CACTI_HIP(hipMemsetAsync(status_ptr(), 0, sizeof(int), stream_));
        set_error("token id out of range at position %d", v - 1);
        return CACTI_E_INDEX;
    }
    return 0;
}

CellPtr Ctx::cell_new(const CellType &ty, bool stable, const char *name)
{
    Cell c;
    c.ty = ty;
    c.stable = stable;
    c.name = name ? name : "";
    cells_.push_back(std::move(c));
    if (stable) stable_end_ = cells_.size();
    return (CellPtr)(cells_.size() - 1);
}

int Ctx::host_alloc(Cell &c)
{
    if (c.hptr) return 0;
    const size_t n = std::max<size_t>(c.ty.bytes(), 1);
    if (host_pagelocked_) {
        // a buffer of a dead cell of the same size, if there is one (page-locking memory costs
        // milliseconds; the cells of a cycle have the sizes of the cycle before)
        auto it = host_pool_.find(n);
        if (it != host_pool_.end()) {
            c.hptr = it->second.ptr;
            c.h_busy = it->second.busy;        // copies of the previous owner may still be in flight
            host_pool_.erase(it);
            return 0;
        }
        CACTI_HIP(hipHostMalloc(&c.hptr, n, hipHostMallocDefault));
    } else {
        c.hptr = malloc(n);
        CACTI_REQUIRE(c.hptr, CACTI_E_OOM, "host malloc of %zu bytes failed", n);
    }
    host_bytes_ += n;
    return 0;
}

// wait until no in-flight copy reads or writes the cell's host buffer
static void host_quiesce(Cell &c)
{
    if (c.h_busy) hipEventSynchronize(c.h_busy);
}
static void host_mark_busy(Cell &c, hipStream_t st)
{
    // without an event to wait on later, wait now: the host buffer must never be handed out mid-copy
    if (!c.h_busy && hipEventCreateWithFlags(&c.h_busy, hipEventDisableTiming) != hipSuccess) c.h_busy = nullptr;
    if (!c.h_busy || hipEventRecord(c.h_busy, st) != hipSuccess) (void)hipStreamSynchronize(st);
}

void Ctx::host_free(Cell &c)
{
    if (c.hptr && host_pagelocked_) {
        // back to the pool together with the event of its last copy
        host_pool_.emplace(std::max<size_t>(c.ty.bytes(), 1), HostBuf{c.hptr, c.h_busy});
        c.hptr = nullptr;
        c.h_busy = nullptr;
        c.h_valid = false;
        return;
    }
    if (c.h_busy) {
        hipEventSynchronize(c.h_busy);
        hipEventDestroy(c.h_busy);
        c.h_busy = nullptr;
    }
    if (!c.hptr) return;
    free(c.hptr);
    host_bytes_ -= std::max<size_t>(c.ty.bytes(), 1);
    c.hptr = nullptr;
    c.h_valid = false;
}

int Ctx::cell_free_all(CellPtr ci)
{
    Cell &c = cells_[ci];
    if (c.voff != kNoOffset) {
        pool_.free(c.voff);
        c.voff = kNoOffset;
    }
    c.v_valid = false;
    if (c.v_ready) {                          // a prefetch nobody consumed: the region is free once it has landed
        hipStreamWaitEvent(stream_, c.v_ready, 0);
        ev_put(c.v_ready);
        c.v_ready = nullptr;
    }
    if (c.hptr || c.h_busy) host_free(c);     // waits for in-flight copies of this cell only
    return 0;
}

int Ctx::cell_put(CellPtr ci, const void *host, size_t bytes)
{
    CACTI_REQUIRE(is_live(ci), CACTI_E_STATE, "cell_put: dead cell %d", ci);
    Cell &c = cells_[ci];
    CACTI_REQUIRE(bytes == c.ty.bytes(), CACTI_E_INVALID, "cell_put: %zu bytes given, cell %s has %zu",
                  bytes, c.name.c_str(), c.ty.bytes());
    // an earlier upload from this host buffer may still be in flight
    host_quiesce(c);
    int rc = host_alloc(c);
    if (rc) return rc;
    memcpy(c.hptr, host, bytes);
    c.h_valid = true;
    c.v_valid = false;
    return 0;
}

int Ctx::cell_get(CellPtr ci, void *host, size_t bytes)
{
    CACTI_REQUIRE(is_live(ci), CACTI_E_STATE, "cell_get: dead cell %d", ci);
    Cell &c = cells_[ci];
    CACTI_REQUIRE(bytes == c.ty.bytes(), CACTI_E_INVALID, "cell_get: %zu bytes asked, cell %s has %zu",
                  bytes, c.name.c_str(), c.ty.bytes());
    if (c.v_valid) {
        if (c.v_ready) {                       // uploaded ahead of its use: the upload may still be under way
            CACTI_HIP(hipStreamWaitEvent(stream_, c.v_ready, 0));
            ev_put(c.v_ready);
            c.v_ready = nullptr;
        }
        CACTI_HIP(hipMemcpyAsync(host, dev_ptr(c.voff), bytes, hipMemcpyDeviceToHost, stream_));
        CACTI_HIP(hipStreamSynchronize(stream_));
        bytes_d2h_ += bytes;
        return 0;
    }
    CACTI_REQUIRE(c.h_valid, CACTI_E_STATE, "cell_get: cell %s holds no value", c.name.c_str());
    host_quiesce(c);
    memcpy(host, c.hptr, bytes);
    return 0;
}

// csrc/digest.hip
size_t digest_batch_scratch_bytes(int count);
int digest_batch_f16(int count, const void *const *xs, const int64_t *ns, void *out, void *segs_dev,
                     hipStream_t st);

// One launch digests every cell: all of them are made resident first (a cell that cannot be
// held beside the others fails the call with the pool's error).
int Ctx::cells_digest(const CellPtr *cells, int n, int64_t *hist, int64_t *nan)
{
    CACTI_REQUIRE(n >= 0 && (n == 0 || (cells && hist && nan)), CACTI_E_INVALID, "cells_digest: null argument");
    if (n == 0) return 0;
    // device scratch: per cell 256 histogram bins + the NaN count, then the launch's descriptors
    const size_t out_bytes = (size_t)n * 257 * sizeof(int64_t);
    size_t off;
    int rc = pool_alloc(out_bytes + digest_batch_scratch_bytes(n), &off);
    if (rc) return rc;
    char *scratch = static_cast<char *>(dev_ptr(off));
    std::vector<const void *> xs((size_t)n);
    std::vector<int64_t> ns((size_t)n);
    std::vector<int64_t> host((size_t)n * 257);
    int done = 0;
    while (done < n && rc == 0) {
        // as many cells as stay resident together
        int m = 0;
        for (int i = done; i < n; i++) {
            const CellPtr ci = cells[i];
            if (ci <= 0 || (size_t)ci >= cells_.size() || !cells_[ci].alive || cells_[ci].ty.dtype != F16) {
                set_error("cells_digest: cell %d is not a live f16 cell", ci);
                rc = CACTI_E_INVALID;
                break;
            }
            cells_[ci].pin++;
            rc = ensure_vmem(ci, true);
            if (rc) {
                cells_[ci].pin--;
                if (m > 0 && rc == CACTI_E_OOM) rc = 0;   // digest what fits, then go on
                break;
            }
            xs[(size_t)m] = dev_ptr(cells_[ci].voff);
            ns[(size_t)m] = (int64_t)(cells_[ci].ty.bytes() / 2);
            m++;
        }
        if (rc == 0 && m > 0)
            rc = digest_batch_f16(m, xs.data(), ns.data(), scratch + (size_t)done * 257 * sizeof(int64_t),
                                  scratch + out_bytes, stream_);
        for (int i = done; i < done + m; i++) cells_[cells[i]].pin--;
        if (rc == 0 && m == 0) rc = CACTI_E_OOM;
        done += m;
    }
    if (rc == 0) {
        rc = hip_status(hipMemcpyAsync(host.data(), scratch, out_bytes, hipMemcpyDeviceToHost, stream_), "digest d2h");
        bytes_d2h_ += out_bytes;
    }
    const int rs = hip_status(hipStreamSynchronize(stream_), "digest sync");
    pool_.free(off);
    if (rc) return rc;
    if (rs) return rs;
    for (int i = 0; i < n; i++) {
        memcpy(hist + (size_t)i * 256, host.data() + (size_t)i * 257, 256 * sizeof(int64_t));
        nan[i] = host[(size_t)i * 257 + 256];
    }
    return 0;
}

namespace {
constexpr size_t kIngestChunk = 32u << 20;        // source bytes per staging buffer
constexpr int kIngestThreads = 8;

// pread the whole range, split over a few threads (the page cache copies at a few GB/s per core)
bool read_range(int fd, uint64_t off, char *dst, size_t bytes)
{
    const int nt = bytes >= ((size_t)kIngestThreads << 20) ? kIngestThreads : 1;
    std::vector<std::thread> th;
    std::vector<char> ok((size_t)nt, 1);
    const size_t per = ((bytes + (size_t)nt - 1) / (size_t)nt + 4095) & ~(size_t)4095;
    for (int t = 0; t < nt; t++) {
        const size_t b = std::min(bytes, per * (size_t)t), e = std::min(bytes, b + per);
        auto work = [fd, off, dst, b, e, &ok, t]() {
            size_t done = b;
            while (done < e) {
                const ssize_t r = pread(fd, dst + done, e - done, (off_t)(off + done));
                if (r <= 0) {
                    ok[(size_t)t] = 0;
                    return;
                }
                done += (size_t)r;
            }
        };
        if (t + 1 < nt) th.emplace_back(work);
        else work();
    }
    for (std::thread &x : th) x.join();
    for (char v : ok)
        if (!v) return false;
    return true;
}
}  // namespace

int Ctx::cell_ingest(CellPtr ci, int fd, uint64_t off, size_t bytes, int cast)
{
    CACTI_REQUIRE(ci > 0 && (size_t)ci < cells_.size() && cells_[ci].alive, CACTI_E_INVALID, "cell_ingest: dead cell");
    CACTI_REQUIRE(cast >= 0 && cast <= 2, CACTI_E_INVALID, "cell_ingest: unknown cast %d", cast);
    const size_t dst_bytes = cast == 2 ? bytes / 2 : bytes;
    CACTI_REQUIRE(dst_bytes == cells_[ci].ty.bytes() && (cast == 0 || cells_[ci].ty.dtype == F16), CACTI_E_INVALID,
                  "cell_ingest: %zu source bytes do not fill cell %s", bytes, cells_[ci].name.c_str());
    for (int k = 0; k < 2; k++) {
        if (!ingest_host_[k]) CACTI_HIP(hipHostMalloc(&ingest_host_[k], kIngestChunk, hipHostMallocDefault));
        if (!ingest_ev_[k]) CACTI_HIP(hipEventCreateWithFlags(&ingest_ev_[k], hipEventDisableTiming));
    }
    cells_[ci].pin++;
    int rc = ensure_vmem(ci, false);
    size_t scratch = kNoOffset;
    if (!rc && cast) rc = pool_alloc(2 * kIngestChunk, &scratch);
    char *dst = rc ? nullptr : static_cast<char *>(dev_ptr(cells_[ci].voff));
    int buf = 0;
    for (size_t done = 0; done < bytes && !rc; done += kIngestChunk, buf ^= 1) {
        const size_t n = std::min(kIngestChunk, bytes - done);
        // the upload that last read this staging buffer must have finished
        rc = hip_status(hipEventSynchronize(ingest_ev_[buf]), "ingest wait");
        if (rc) break;
        if (!read_range(fd, off + done, static_cast<char *>(ingest_host_[buf]), n)) {
            set_error("cell_ingest: short read at offset %llu", (unsigned long long)(off + done));
            rc = CACTI_E_IO;
            break;
        }
        char *stage = cast ? static_cast<char *>(dev_ptr(scratch)) + (size_t)buf * kIngestChunk : dst + done;
        rc = hip_status(hipMemcpyAsync(stage, ingest_host_[buf], n, hipMemcpyHostToDevice, stream_), "ingest upload");
        if (!rc) rc = hip_status(hipEventRecord(ingest_ev_[buf], stream_), "ingest record");
        bytes_h2d_ += n;
        if (!rc && cast == 1) rc = cacti_hip_raw_cast_bf16_f16((int64_t)(n / 2), stage, dst + done, stream_);
        if (!rc && cast == 2) rc = cacti_hip_cast_f32_f16((int64_t)(n / 4), stage, dst + done / 2, stream_);
    }
    if (scratch != kNoOffset) pool_.free(scratch);               // reuse is ordered on the stream
    cells_[ci].pin--;
    if (rc) return rc;
    Cell &c = cells_[ci];
    host_free(c);
    c.v_valid = true;
    c.h_valid = false;
    return 0;
}

int Ctx::cell_cast_f16_f32(CellPtr src, CellPtr dst)
{
    CACTI_REQUIRE(src > 0 && dst > 0 && (size_t)src < cells_.size() && (size_t)dst < cells_.size() &&
                      cells_[src].alive && cells_[dst].alive && cells_[src].ty.dtype == F16 &&
                      cells_[dst].ty.dtype == F32 && cells_[src].ty.bytes() * 2 == cells_[dst].ty.bytes(),
                  CACTI_E_INVALID, "cell_cast: wants a live f16 source and an f32 destination of the same shape");
    cells_[src].pin++;
    cells_[dst].pin++;
    int rc = ensure_vmem(src, true);
    if (!rc) rc = ensure_vmem(dst, false);
    if (!rc)
        rc = cacti_hip_cast_f16_f32((int64_t)(cells_[src].ty.bytes() / 2), dev_ptr(cells_[src].voff),
                                    dev_ptr(cells_[dst].voff), stream_);
    cells_[src].pin--;
    cells_[dst].pin--;
    if (!rc) {
        cells_[dst].v_valid = true;
        cells_[dst].h_valid = false;
    }
    return rc;
}

int Ctx::cell_zero(CellPtr c)
{
    CACTI_REQUIRE(c > 0 && (size_t)c < cells_.size() && cells_[c].alive, CACTI_E_INVALID, "cell_zero: dead cell");
    int rc = ensure_vmem(c, false);
    if (rc) return rc;
    CACTI_HIP(hipMemsetAsync(dev_ptr(cells_[c].voff), 0, cells_[c].ty.bytes(), stream_));
    cells_[c].v_valid = true;
    cells_[c].h_valid = false;
    return 0;
}

// The five cells of a tensor must be resident together; with a capped pool the list is cut into
// as many launches as needed.
int Ctx::cells_adamw32(int n, const CellPtr *grads, const CellPtr *avgs, const CellPtr *avg2s,
                       const CellPtr *masters, const CellPtr *params, const float *sc)
{
    CACTI_REQUIRE(n >= 0 && (n == 0 || (grads && avgs && avg2s && masters && params && sc)), CACTI_E_INVALID,
                  "cells_adamw32: null argument");
    if (n == 0) return 0;
    size_t off;
    int rc = pool_alloc(cacti_hip_adamw32_scratch_bytes(n), &off);
    if (rc) return rc;
    std::vector<const void *> g((size_t)n);
    std::vector<void *> a((size_t)n), b((size_t)n), w((size_t)n), p((size_t)n);
    std::vector<int64_t> ns((size_t)n);
    int done = 0;
    while (done < n && rc == 0) {
        int m = 0;
        for (int i = done; i < n; i++) {
            const CellPtr five[5] = {grads[i], avgs[i], avg2s[i], masters[i], params[i]};
            size_t elems = 0;
            for (int k = 0; k < 5 && rc == 0; k++) {
                const CellPtr ci = five[k];
                const bool ok = ci > 0 && (size_t)ci < cells_.size() && cells_[ci].alive &&
                                cells_[ci].ty.dtype == ((k == 0 || k == 4) ? F16 : F32);
                const size_t e = ok ? cells_[ci].ty.bytes() / ((k == 0 || k == 4) ? 2 : 4) : 0;
                if (!ok || (k > 0 && e != elems)) {
                    set_error("cells_adamw32: tensor %d: cell %d has the wrong type, size or is dead", i, ci);
                    rc = CACTI_E_INVALID;
                }
                elems = e;
            }
            if (rc) break;
            int pinned = 0;
            for (; pinned < 5 && rc == 0; pinned++) {
                cells_[five[pinned]].pin++;
                rc = ensure_vmem(five[pinned], pinned != 4);      // the parameter is only written
            }
            if (rc) {
                for (int k = 0; k < pinned; k++) cells_[five[k]].pin--;
                if (m > 0 && rc == CACTI_E_OOM) rc = 0;          // update what fits, then go on
                break;
            }
            g[(size_t)m] = dev_ptr(cells_[five[0]].voff);
            a[(size_t)m] = dev_ptr(cells_[five[1]].voff);
            b[(size_t)m] = dev_ptr(cells_[five[2]].voff);
            w[(size_t)m] = dev_ptr(cells_[five[3]].voff);
            p[(size_t)m] = dev_ptr(cells_[five[4]].voff);
            ns[(size_t)m] = (int64_t)elems;
            m++;
        }
        if (rc == 0 && m > 0)
            rc = cacti_hip_adamw32_step_f16_batch(m, g.data(), a.data(), b.data(), w.data(), p.data(), ns.data(), sc,
                                                  dev_ptr(off), stream_);
        for (int i = done; i < done + m; i++) {
            const CellPtr five[5] = {grads[i], avgs[i], avg2s[i], masters[i], params[i]};
            for (int k = 0; k < 5; k++) cells_[five[k]].pin--;
            if (rc == 0)
                for (int k = 1; k < 5; k++) {
                    cells_[five[k]].v_valid = true;
                    cells_[five[k]].h_valid = false;
                }
        }
        if (rc == 0 && m == 0) rc = CACTI_E_OOM;
        done += m;
    }
    pool_.free(off);                                             // reuse is ordered on the stream
    return rc;
}

// VMem -> Mem: keep (or make) a host copy of the current version, then drop the device
// replica.  PCell::read_loc(.., Locus::Mem) + yeet, src/pctx/nvgpu.rs:2198-2251.
int Ctx::evict(CellPtr ci)
{
    Cell &c = cells_[ci];
    if (c.voff == kNoOffset) return 0;
    if (c.v_ready) {                           // never picked as a victim; a direct call waits for the upload
        CACTI_HIP(hipStreamWaitEvent(stream_, c.v_ready, 0));
        ev_put(c.v_ready);
        c.v_ready = nullptr;
    }
    if (c.v_valid && !c.h_valid) {
        int rc = host_alloc(c);
        if (rc) return rc;
        if (async_spill_) {
            // download on the copy stream, after the compute work queued so far (the cell's producer);
            // the region goes back to the pool when the download is done (reclaim)
            if ((rc = order_after_compute(down_stream_))) return rc;
            if (c.h_busy) CACTI_HIP(hipStreamWaitEvent(down_stream_, c.h_busy, 0));   // earlier users of the buffer
            CACTI_HIP(hipMemcpyAsync(c.hptr, dev_ptr(c.voff), c.ty.bytes(), hipMemcpyDeviceToHost, down_stream_));
            host_mark_busy(c, down_stream_);
            hipEvent_t done = ev_get();
            CACTI_REQUIRE(done, CACTI_E_STATE, "ctx: cannot create an event");
            CACTI_HIP(hipEventRecord(done, down_stream_));
            sum_downloaded_ += c.ty.bytes();
            (in_eager_ ? cyc_eager_ : cyc_demand_down_) += c.ty.bytes();
            pending_.push_back(PendingFree{c.voff, pool_.size_of(c.voff), done});
            pending_bytes_ += pending_.back().bytes;
            c.h_valid = true;
            bytes_d2h_ += c.ty.bytes();
            c.voff = kNoOffset;
            c.v_valid = false;
            n_evict_++;
            return 0;
        }
        CACTI_HIP(hipMemcpyAsync(c.hptr, dev_ptr(c.voff), c.ty.bytes(), hipMemcpyDeviceToHost,
                                 stream_));
        if (!host_pagelocked_) CACTI_HIP(hipStreamSynchronize(stream_));
        host_mark_busy(c, stream_);
        c.h_valid = true;
        bytes_d2h_ += c.ty.bytes();
    }
    if (async_spill_) {
        sum_dropped_ += c.ty.bytes();
        cyc_dropped_ += c.ty.bytes();
    }
    pool_.free(c.voff);          // later users of the region are ordered after the copy
    c.voff = kNoOffset;
    c.v_valid = false;
    n_evict_++;
    return 0;
}

// Regions of evicted cells whose download has finished go back to the pool; with a request that
// does not fit yet, the streams that may reuse a region are made to wait for the unfinished downloads,
// oldest first, and those regions go back too until the request fits (no host wait either way).
void Ctx::reclaim(size_t need)
{
    size_t kept = 0;
    bool busy = false;          // the downloads finish in the order they were queued: one query finds the first unfinished
    for (size_t i = 0; i < pending_.size(); i++) {
        PendingFree &pf = pending_[i];
        bool done = !busy && hipEventQuery(pf.done) == hipSuccess;
        busy = !done;
        if (!done && need && pool_.largest_free() < need) {
            hipStreamWaitEvent(stream_, pf.done, 0);        // whoever gets the region next: a thunk ...
            hipStreamWaitEvent(up_stream_, pf.done, 0);     // ... or an upload
            done = true;
        }
        if (done) {
            pool_.free(pf.off);
            pending_bytes_ -= pf.bytes;
            ev_put(pf.done);
        } else {
            pending_[kept++] = pf;
        }
    }
    pending_.resize(kept);
}

// Entry index of the next use of a cell in the compiled log, from the entry being run on; a cell that
// this cycle does not touch again is needed by the next cycle, where its first use says how soon.
// (uses_ holds 2 * entry + 1 where the entry overwrites the cell without reading it.)
size_t Ctx::next_use(CellPtr c, bool *overwrite) const
{
    if (overwrite) *overwrite = false;
    auto it = uses_.find(c);
    if (it == uses_.end() || it->second.empty()) return 2 * log_.size() + (size_t)c;
    const std::vector<uint32_t> &u = it->second;
    auto p = std::lower_bound(u.begin(), u.end(), (uint32_t)(2 * pc_));
    if (p == u.end()) p = u.begin();
    if (overwrite) *overwrite = (*p & 1) != 0;
    return (p == u.begin() && (*p >> 1) < pc_ ? log_.size() : 0) + (*p >> 1);
}

// The resident, unpinned cell whose next use lies farthest ahead (among those of at least min_bytes);
// without a compiled log, the oldest cell (the reference's creation order, src/pctx/nvgpu.rs:2004-2283).
int Ctx::pick_victim(size_t min_bytes, bool allow_prefetched, int cls) const
{
    int best = 0;
    size_t best_use = 0;
    for (size_t i = 1; i < cells_.size(); i++) {
        const Cell &c = cells_[i];
        if (!c.alive || c.voff == kNoOffset || c.pin > 0 || (c.v_ready && !allow_prefetched)) continue;
        if (pool_.size_of(c.voff) < min_bytes) continue;
        if (!compiled_) return (int)i;
        bool ow = false;
        const size_t u = next_use((CellPtr)i, &ow);
        const bool drop = !c.v_valid || c.h_valid;               // nothing to download
        if (cls == V_DROP && !drop) continue;
        if (cls == V_DOWN_ONLY && (drop || !ow)) continue;
        if (!best || u > best_use) {
            best = (int)i;
            best_use = u;
        }
    }
    return best;
}

// NvGpuMemPool::_try_soft_oom, src/pctx/nvgpu.rs:2004-2283: dead cells are already freed
// at their Unlive entry; here live, unpinned cells are spilled in creation order, first
// only those at least as large as the request, then any.
int Ctx::try_soft_oom(size_t need)
{
    n_soft_oom_++;
    const size_t req = (need + kAllocAlign - 1) / kAllocAlign * kAllocAlign;
    // regions whose download is under way first: finished ones cost nothing, the others a stream wait
    reclaim(0);
    if (pool_.largest_free() >= req) return 0;
    reclaim(req);
    if (pool_.largest_free() >= req) return 0;
    // then victims: those that free their memory at once (nothing to download) and are not needed
    // soon, then by next use alone, first only cells at least as large as the request, then any
    // (a last pass also takes cells that were uploaded ahead of their use)
    for (int pass = -1; pass < 3; pass++) {
        for (;;) {
            const int v = pick_victim(pass <= 0 ? req : 0, pass == 2, pass < 0 ? V_DROP : V_ANY);
            if (!v || (pass <= 0 && compiled_ && next_use((CellPtr)v) < pc_ + 48)) break;
            int rc = evict((CellPtr)v);
            if (rc) return rc;
            reclaim(req);
            if (pool_.largest_free() >= req) return 0;
        }
    }
    return CACTI_E_OOM;
}

// Before a thunk runs on a pool that has already run out once: evict ahead of need, so that the
// downloads overlap the thunks in between and allocations find free memory instead of waiting.
int Ctx::keep_reserve()
{
    if (!async_spill_ || n_soft_oom_ == 0 || !compiled_) return 0;
    reclaim(0);
    const size_t reserve = reserve_bytes();
    while (pool_.cap() - pool_.used() + pending_bytes_ < reserve) {
        // the class that has carried less so far first, then the other, then any cell
        const int first = sum_dropped_ <= sum_downloaded_ ? V_DROP : V_DOWN_ONLY;
        int v = pick_victim(0, false, first);
        if (!v || next_use((CellPtr)v) < pc_ + 48) v = pick_victim(0, false, first == V_DROP ? V_DOWN_ONLY : V_DROP);
        if (!v || next_use((CellPtr)v) < pc_ + 48) v = pick_victim(0);
        if (!v) break;
        // nothing is gained by evicting what the next thunks use
        if (next_use((CellPtr)v) < pc_ + 24) break;
        int rc = evict((CellPtr)v);
        if (rc) return rc;
    }
    return 0;
}

// One spilled cell back into memory that is free now, on the upload stream; 1 when there is no room.
int Ctx::upload_ahead(Cell &c, bool *ordered)
{
    const size_t off = pool_.alloc(c.ty.bytes(), c.stable);
    if (off == kNoOffset) return 1;
    n_alloc_++;
    if (!*ordered) {
        // the region may have belonged to a cell that queued compute work still reads
        int rc = order_after_compute(up_stream_);
        if (rc) {
            pool_.free(off);
            return rc;
        }
        *ordered = true;
    }
    c.voff = off;
    if (c.h_busy) CACTI_HIP(hipStreamWaitEvent(up_stream_, c.h_busy, 0));
    CACTI_HIP(hipMemcpyAsync(dev_ptr(off), c.hptr, c.ty.bytes(), hipMemcpyHostToDevice, up_stream_));
    host_mark_busy(c, up_stream_);
    c.v_ready = ev_get();
    CACTI_REQUIRE(c.v_ready, CACTI_E_STATE, "ctx: cannot create an event");
    CACTI_HIP(hipEventRecord(c.v_ready, up_stream_));
    c.v_valid = true;
    n_upload_++;
    bytes_h2d_ += c.ty.bytes();
    return 0;
}

// Upload, on the upload stream, the spilled cells that coming thunks read, into memory that is free
// now (never by evicting: a prefetch must not push out what is needed sooner).  The next 16 thunks
// are looked at before every thunk, past the end of the log into the start of the next cycle (which
// replays this one); entries farther ahead are gone through once, by a cursor that stops where an
// upload would leave less than the reserve free: the backward pass frees memory as it goes, and an
// upload takes longer than the thunks that wait for it, so it has to start that early.
int Ctx::prefetch_ahead()
{
    if (!async_spill_ || n_soft_oom_ == 0 || !compiled_) return 0;
    bool ordered = false;
    auto reads = [&](const Entry &f, bool far) -> int {
        for (size_t k = 0; k < f.args.size() + f.outs.size(); k++) {
            const bool is_out = k >= f.args.size();
            const CellPtr ci = is_out ? f.outs[k - f.args.size()] : f.args[k];
            if (is_out && !((f.acc_mask >> (k - f.args.size())) & 1)) continue;      // written, not read
            Cell &c = cells_[ci];
            if (!c.alive || c.voff != kNoOffset || !c.h_valid) continue;
            if (far && pool_.cap() - pool_.used() < c.ty.bytes() + reserve_bytes()) return 1;
            int rc = upload_ahead(c, &ordered);
            if (rc) return rc;
        }
        return 0;
    };
    int thunks = 0;
    const size_t n = log_.size();
    for (size_t j = pc_ + 1; j < pc_ + n && thunks < 16; j++) {
        const Entry &f = log_[j < n ? j : j - n];
        if (f.kind != E_APPLY) continue;
        thunks++;
        int rc = reads(f, false);
        if (rc) return rc < 0 ? rc : 0;                                              // no room now: later
    }
    if (pf_cursor_ < pc_ + 1) pf_cursor_ = pc_ + 1;
    for (const size_t end = std::min(n, pc_ + 1 + 640); pf_cursor_ < end; pf_cursor_++) {
        const Entry &f = log_[pf_cursor_];
        if (f.kind != E_APPLY) continue;
        int rc = reads(f, true);
        if (rc) return rc < 0 ? rc : 0;
    }
    return 0;
}

int Ctx::spill_eagerly(const Entry &e)
{
    if (!async_spill_ || eager_left_ == 0 || e.kind != E_APPLY) return 0;
    for (CellPtr o : e.outs) {
        Cell &c = cells_[o];
        if (!c.alive || !c.stable || c.voff == kNoOffset || c.pin > 0 || c.v_ready || !c.v_valid || c.h_valid)
            continue;
        if (c.ty.bytes() > eager_left_) continue;
        bool ow = false;
        if (next_use(o, &ow) < log_.size() || !ow) continue;
        eager_left_ -= c.ty.bytes();
        in_eager_ = true;
        int rc = evict(o);
        in_eager_ = false;
        if (rc) return rc;
    }
    return 0;
}

int Ctx::pool_alloc(size_t bytes, size_t *off, bool high)
{
    size_t o = pool_.alloc(bytes, high);
    if (o == kNoOffset) {
        int rc = try_soft_oom(bytes);
        if (rc == 0) o = pool_.alloc(bytes, high);
        if (o == kNoOffset) {
            // the reference dumps the pool's usage before it panics (src/pctx/nvgpu.rs:2424-2440); here the
            // full table goes to stderr and the status message carries the pool's line of it
            const std::string rep = usage_report();
            fprintf(stderr, "cacti: device pool exhausted, request of %zu bytes does not fit after eviction\n%s", bytes,
                    rep.c_str());
            size_t pinned = 0;
            for (const Cell &c : cells_)
                if (c.alive && c.voff != kNoOffset && c.pin > 0) pinned += c.ty.bytes();
            set_error("device pool exhausted: request %zu bytes, cap %zu, used %zu, front %zu, largest free %zu, "
                      "pinned by the running thunk %zu, downloads in flight %zu (usage by class of cell on stderr)",
                      bytes, pool_.cap(), pool_.used(), pool_.front(), pool_.largest_free(), pinned, pending_bytes_);
            return CACTI_E_OOM;
        }
    }
    n_alloc_++;
    *off = o;
    return 0;
}

int Ctx::ensure_vmem(CellPtr ci, bool need_value)
{
    CACTI_REQUIRE(is_live(ci), CACTI_E_STATE, "use of dead cell %d", ci);
    Cell &c = cells_[ci];
    if (c.voff == kNoOffset) {
        size_t off;
        int rc = pool_alloc(c.ty.bytes(), &off, c.stable);
        if (rc) return rc;
        cells_[ci].voff = off;
        cells_[ci].v_valid = false;
    }
    Cell &d = cells_[ci];
    if (d.v_ready) {                           // prefetched: the compute stream waits for the upload here
        CACTI_HIP(hipStreamWaitEvent(stream_, d.v_ready, 0));
        ev_put(d.v_ready);
        d.v_ready = nullptr;
    }
    if (need_value && !d.v_valid) {
        CACTI_REQUIRE(d.h_valid, CACTI_E_STATE, "cell %d (%s) is read before it holds a value", ci,
                      d.name.c_str());
        // an upload the prefetch did not get to: on the compute stream, which needs it now (a download
        // of this cell that is still under way on the copy stream comes first)
        if (d.h_busy) CACTI_HIP(hipStreamWaitEvent(stream_, d.h_busy, 0));
        CACTI_HIP(hipMemcpyAsync(dev_ptr(d.voff), d.hptr, d.ty.bytes(), hipMemcpyHostToDevice,
                                 stream_));
        host_mark_busy(d, stream_);
        d.v_valid = true;
        n_upload_++;
        bytes_h2d_ += d.ty.bytes();
    }
    return 0;
}

// ---------------------------------------------------------------------------
// staging

void Ctx::reset()
{
    // CACTI_VERBOSE: the usage dump at every reset, i.e. once per cycle, before the cycle's cells are
    // collected (Ctx::reset, src/ctx.rs:150-167)
    static const bool verbose = getenv("CACTI_VERBOSE") && !getenv("CACTI_SILENT");
    if (verbose && pc_ > 0) fprintf(stderr, "cacti: usage at the end of a cycle\n%s", usage_report().c_str());
    for (size_t i = 1; i < cells_.size(); i++) {
        Cell &c = cells_[i];
        if (c.alive && !c.stable) {
            cell_free_all((CellPtr)i);
            c.alive = false;
        }
    }
    // compact trailing dead cells so ids do not grow without bound across cycles; never below an id
    // that a stable cell has had: its owner may still hold the handle after freeing the cell, and
    // must get "dead cell" for it, not whatever cell a later cycle would put there
    while (cells_.size() > std::max<size_t>(1, stable_end_) && !cells_.back().alive) cells_.pop_back();
    log_.clear();
    uses_.clear();
    if (pc_ > 0) {
        // what the forward pass of the cycle that ends here needed: the early downloads of the cycle
        // before it, and what it evicted itself
        eager_left_ = (prev_eager_ + cyc_demand_down_ + cyc_dropped_) / 2;
        prev_eager_ = cyc_eager_;
    }
    cyc_eager_ = cyc_demand_down_ = cyc_dropped_ = 0;
    pf_cursor_ = 0;
    thunks_.clear();
    kept_.clear();
    adj_.clear();
    adj_wr_.clear();
    pc_ = 0;
    compiled_ = false;
    fwd_end_ = 0;
}

int Ctx::add_thunk(std::unique_ptr<ThunkSpec> spec)
{
    thunks_.push_back(std::move(spec));
    return (int)thunks_.size() - 1;
}

int Ctx::stage_apply(int thunk, const std::vector<CellPtr> &args, std::vector<CellPtr> *outs)
{
    const ThunkSpec &sp = *thunks_[thunk];
    CACTI_REQUIRE((int)args.size() == sp.arity(), CACTI_E_INVALID, "%s: %zu args, arity %d",
                  sp.name(), args.size(), sp.arity());
    std::vector<CellType> aty, oty;
    for (CellPtr a : args) {
        CACTI_REQUIRE(a > 0 && (size_t)a < cells_.size() && cells_[a].alive, CACTI_E_INVALID,
                      "%s: dead or nil argument cell", sp.name());
        aty.push_back(cells_[a].ty);
    }
    int rc = sp.out_ty(aty, oty);
    if (rc) return rc;
    Entry e;
    e.kind = E_APPLY;
    e.thunk = thunk;
    e.args = args;
    for (auto &t : oty) e.outs.push_back(cell_new(t, false, sp.name()));
    if (outs) *outs = e.outs;
    log_.push_back(std::move(e));
    return 0;
}

int Ctx::stage_into(int thunk, const std::vector<CellPtr> &args, const std::vector<CellPtr> &outs,
                    uint32_t acc_mask)
{
    const ThunkSpec &sp = *thunks_[thunk];
    std::vector<CellType> aty, oty;
    for (CellPtr a : args) aty.push_back(cells_[a].ty);
    int rc = sp.out_ty(aty, oty);
    if (rc) return rc;
    CACTI_REQUIRE(oty.size() == outs.size(), CACTI_E_INVALID, "%s: output count mismatch", sp.name());
    for (size_t k = 0; k < outs.size(); k++)
        CACTI_REQUIRE(cells_[outs[k]].ty == oty[k], CACTI_E_INVALID,
                      "%s: output %zu type differs from the target cell %s", sp.name(), k,
                      cells_[outs[k]].name.c_str());
    Entry e;
    e.kind = E_APPLY;
    e.thunk = thunk;
    e.args = args;
    e.outs = outs;
    e.acc_mask = acc_mask;
    log_.push_back(std::move(e));
    return 0;
}

void Ctx::stage_yield_set(CellPtr c)
{
    Entry e;
    e.kind = E_YIELD_SET;
    e.cell = c;
    log_.push_back(std::move(e));
}

void Ctx::adj_seed(CellPtr primal, CellPtr adj)
{
    adj_[primal] = adj;
    adj_wr_[adj] = true;
}

void Ctx::adj_bind(CellPtr primal, CellPtr adj, bool cached)
{
    adj_[primal] = adj;
    // a cached adjoint counts as written: the cycle's first write into it accumulates
    // (SpineEntry::Cache gives the cell this cycle's init_once clock, src/spine.rs:786-805)
    adj_wr_[adj] = cached;
}

CellPtr Ctx::adj_of(CellPtr primal)
{
    if (cells_[primal].konst) return 0;
    auto it = adj_.find(primal);
    if (it != adj_.end()) return it->second;
    CellPtr a = cell_new(cells_[primal].ty, false, ("d:" + cells_[primal].name).c_str());
    adj_[primal] = a;
    adj_wr_[a] = false;
    return a;
}

bool Ctx::adj_written(CellPtr primal)
{
    auto it = adj_.find(primal);
    return it != adj_.end() && adj_wr_[it->second];
}

int Ctx::adj_add(const std::vector<CellPtr> &primals, std::unique_ptr<ThunkSpec> spec,
                 const std::vector<CellPtr> &args)
{
    std::vector<CellPtr> outs;
    uint32_t mask = 0;
    bool any = false;
    for (size_t k = 0; k < primals.size(); k++) {
        CellPtr a = adj_of(primals[k]);
        if (a == 0) {
            // no adjoint wanted for this argument: the fused thunk still needs a target
            a = cell_new(cells_[primals[k]].ty, false, "d:unused");
        } else {
            any = true;
            if (adj_wr_[a]) mask |= 1u << k;
            adj_wr_[a] = true;
        }
        outs.push_back(a);
    }
    if (!any) return 0;
    int t = add_thunk(std::move(spec));
    return stage_into(t, args, outs, mask);
}

int Ctx::vadd_vjp()
{
    fwd_end_ = log_.size();
    for (size_t i = fwd_end_; i-- > 0;) {
        if (log_[i].kind != E_APPLY) continue;
        const Entry e = log_[i];                 // copy: pop_adj appends to the log
        std::vector<CellPtr> out_adj(e.outs.size(), 0);
        bool any = false;
        for (size_t k = 0; k < e.outs.size(); k++) {
            auto it = adj_.find(e.outs[k]);
            if (it != adj_.end() && adj_wr_[it->second]) {
                out_adj[k] = it->second;
                any = true;
            }
        }
        if (!any) continue;
        int rc = thunks_[e.thunk]->pop_adj(*this, e, out_adj);
        if (rc) return rc;
    }
    return 0;
}

// Liveness: a non-stable, non-kept cell dies after its last use; an Unlive entry frees it
// there (Spine::_compile splices Live/Unlive, src/spine.rs:1435-1478).
int Ctx::compile()
{
    // Copy forwarding.  y := copy(x) (the adjoint of an add hands the same gradient to both operands)
    // where x is still read later: if nothing writes x any more and nothing writes y before the last
    // of those reads, the readers may as well read y, which holds the same bytes until then.  x then
    // dies at the copy, and the copy becomes the storage move below instead of a launch.
    static const bool no_forward = getenv("CACTI_NO_COPY_FORWARD") != nullptr;
    for (size_t i = 0; i < log_.size() && !no_forward; i++) {
        const Entry &e = log_[i];
        if (!(e.kind == E_APPLY && thunks_[e.thunk]->is_copy() && e.acc_mask == 0)) continue;
        const CellPtr x = e.args[0], y = e.outs[0];
        if (x == y || cells_[x].stable || cells_[y].stable || cells_[x].ty.bytes() != cells_[y].ty.bytes() ||
            std::find(kept_.begin(), kept_.end(), x) != kept_.end())
            continue;
        size_t last_read = i, first_write_y = log_.size();
        bool ok = true;
        for (size_t j = i + 1; j < log_.size() && ok; j++) {
            const Entry &f = log_[j];
            if (f.kind == E_APPLY) {
                if (std::find(f.outs.begin(), f.outs.end(), x) != f.outs.end()) ok = false;
                if (std::find(f.args.begin(), f.args.end(), x) != f.args.end()) last_read = j;
                if (first_write_y == log_.size() && std::find(f.outs.begin(), f.outs.end(), y) != f.outs.end())
                    first_write_y = j;
            } else if (f.kind == E_YIELD_SET) {
                if (f.cell == x) ok = false;
                if (f.cell == y && first_write_y == log_.size()) first_write_y = j;
            }
        }
        if (!ok || last_read == i || last_read >= first_write_y) continue;
        for (size_t j = i + 1; j <= last_read; j++)
            if (log_[j].kind == E_APPLY)
                for (CellPtr &a : log_[j].args)
                    if (a == x) a = y;
    }
    // The mirror case: y := copy(x) where x is written again later (the gradient of the residual stream,
    // which the next junction accumulates into) but every read of y comes before that write and nothing
    // else writes y: the readers read x, which holds the same bytes until then, and the copy is dropped
    // altogether (y never gets storage).
    for (size_t i = 0; i < log_.size() && !no_forward; i++) {
        const Entry &e = log_[i];
        if (!(e.kind == E_APPLY && thunks_[e.thunk]->is_copy() && e.acc_mask == 0)) continue;
        const CellPtr x = e.args[0], y = e.outs[0];
        if (x == y || cells_[x].stable || cells_[y].stable || cells_[x].ty.bytes() != cells_[y].ty.bytes() ||
            std::find(kept_.begin(), kept_.end(), y) != kept_.end())
            continue;
        size_t last_read_y = i, first_write_x = log_.size();
        bool ok = true, x_read_later = false;
        for (size_t j = i + 1; j < log_.size() && ok; j++) {
            const Entry &f = log_[j];
            if (f.kind == E_APPLY) {
                if (std::find(f.outs.begin(), f.outs.end(), y) != f.outs.end()) ok = false;
                if (std::find(f.args.begin(), f.args.end(), y) != f.args.end()) last_read_y = j;
                if (std::find(f.args.begin(), f.args.end(), x) != f.args.end()) x_read_later = true;
                if (first_write_x == log_.size() && std::find(f.outs.begin(), f.outs.end(), x) != f.outs.end())
                    first_write_x = j;
            } else if (f.kind == E_YIELD_SET) {
                if (f.cell == y) ok = false;
                if (f.cell == x && first_write_x == log_.size()) first_write_x = j;
            }
        }
        // only where x lives on anyway (it is written or read again): otherwise the storage move below
        // already makes the copy free
        if (!ok || last_read_y == i || last_read_y >= first_write_x || !(x_read_later || first_write_x < log_.size()))
            continue;
        for (size_t j = i + 1; j <= last_read_y; j++)
            if (log_[j].kind == E_APPLY)
                for (CellPtr &a : log_[j].args)
                    if (a == y) a = x;
        log_.erase(log_.begin() + (std::ptrdiff_t)i);
        i--;
    }
    std::unordered_map<CellPtr, size_t> last;
    for (size_t i = 0; i < log_.size(); i++) {
        const Entry &e = log_[i];
        if (e.kind == E_APPLY) {
            for (CellPtr a : e.args) last[a] = i;
            for (CellPtr o : e.outs) last[o] = i;
        } else if (e.kind == E_YIELD_SET) {
            last[e.cell] = i;
        }
    }
    for (CellPtr k : kept_) last.erase(k);
    std::vector<std::vector<CellPtr>> dies(log_.size());
    for (auto &kv : last)
        if (!cells_[kv.first].stable) dies[kv.second].push_back(kv.first);
    std::vector<Entry> out;
    out.reserve(log_.size() * 2);
    for (size_t i = 0; i < log_.size(); i++) {
        Entry &e = log_[i];
        // first-write copy (the memcpy adjoint) of a cell that is used nowhere else afterwards:
        // same bytes under a new name, so the output adopts the source's storage
        if (e.kind == E_APPLY && thunks_[e.thunk]->is_copy() && e.acc_mask == 0 &&
            !cells_[e.args[0]].stable && !cells_[e.outs[0]].stable && e.args[0] != e.outs[0] &&
            cells_[e.args[0]].ty.bytes() == cells_[e.outs[0]].ty.bytes() &&
            std::find(dies[i].begin(), dies[i].end(), e.args[0]) != dies[i].end())
            e.move = true;
        out.push_back(std::move(log_[i]));
        std::sort(dies[i].begin(), dies[i].end());
        for (CellPtr c : dies[i]) {
            Entry u;
            u.kind = E_UNLIVE;
            u.cell = c;
            out.push_back(std::move(u));
        }
    }
    log_.swap(out);
    uses_.clear();
    for (size_t i = 0; i < log_.size(); i++) {
        const Entry &e = log_[i];
        if (e.kind != E_APPLY) continue;
        for (CellPtr a : e.args)
            if (uses_[a].empty() || (uses_[a].back() >> 1) != (uint32_t)i) uses_[a].push_back((uint32_t)(2 * i));
        for (size_t k = 0; k < e.outs.size(); k++) {
            const CellPtr o = e.outs[k];
            if (!uses_[o].empty() && (uses_[o].back() >> 1) == (uint32_t)i) continue;     // also read here
            uses_[o].push_back((uint32_t)(2 * i + (((e.acc_mask >> k) & 1) || e.move ? 0 : 1)));
        }
    }
    compiled_ = true;
    pc_ = 0;
    return 0;
}

const char *Ctx::entry_name(size_t i) const
{
    const Entry &e = log_[i];
    if (e.kind == E_APPLY) return thunks_[e.thunk]->name();
    return e.kind == E_YIELD_SET ? "yield_set" : "unlive";
}

int Ctx::run_entry(const Entry &e)
{
    if (e.move) {
        const CellPtr si = e.args[0], di = e.outs[0];
        int rc = ensure_vmem(si, true);           // re-uploads a spilled source
        if (rc) return rc;
        Cell &src = cells_[si], &dst = cells_[di];
        CACTI_REQUIRE(dst.alive, CACTI_E_STATE, "move into dead cell %d (%s)", di, dst.name.c_str());
        if (dst.voff != kNoOffset) pool_.free(dst.voff);
        dst.voff = src.voff;
        dst.v_valid = true;
        dst.h_valid = false;
        src.voff = kNoOffset;
        src.v_valid = false;
        n_moved_++;
        return 0;
    }
    const ThunkSpec &sp = *thunks_[e.thunk];
    std::vector<CellType> aty, oty;
    for (CellPtr a : e.args) cells_[a].pin++;
    for (CellPtr o : e.outs) cells_[o].pin++;
    int rc = 0;
    std::vector<void *> ap, op;
    for (CellPtr a : e.args) {
        if ((rc = ensure_vmem(a, true))) break;
        aty.push_back(cells_[a].ty);
    }
    for (size_t k = 0; !rc && k < e.outs.size(); k++) {
        if ((rc = ensure_vmem(e.outs[k], (e.acc_mask >> k) & 1))) break;
        oty.push_back(cells_[e.outs[k]].ty);
    }
    size_t ws_off = kNoOffset, ws_bytes = 0;
    if (!rc) {
        ws_bytes = sp.workspace(aty);
        if (ws_bytes) rc = pool_alloc(ws_bytes, &ws_off);
    }
    if (!rc) {
        // resolve pointers only now: eviction during allocation cannot move pinned cells
        for (CellPtr a : e.args) ap.push_back(dev_ptr(cells_[a].voff));
        for (CellPtr o : e.outs) op.push_back(dev_ptr(cells_[o].voff));
        hipEvent_t e0 = ev0_, e1 = ev1_;
        int timing = timing_;
        std::string key;
        if (timing == 2) {
            key = sp.key(aty, e.acc_mask);
            if (!timing_filter_.empty() && key.compare(0, timing_filter_.size(), timing_filter_) != 0)
                timing = 0;
            else if (timing_seen_++ % (uint64_t)timing_every_ != 0)
                timing = 0;
        }
        if (timing == 2) {
            if (ev_keys_.size() == ev_pool_.size()) {
                hipEvent_t a = nullptr, b = nullptr;
                if (hipEventCreate(&a) != hipSuccess || hipEventCreate(&b) != hipSuccess) {
                    if (a) hipEventDestroy(a);
                    timing = 0;                          // this launch goes unsampled
                } else {
                    ev_pool_.emplace_back(a, b);
                }
            }
            if (timing) {
                e0 = ev_pool_[ev_keys_.size()].first;
                e1 = ev_pool_[ev_keys_.size()].second;
                ev_keys_.push_back(key);
            }
        }
        if (timing) {
            // operand bytes of one launch: every argument read once, every output written once,
            // an output that is accumulated into read as well
            uint64_t b = 0;
            for (auto &t : aty) b += t.bytes();
            for (size_t k = 0; k < oty.size(); k++) b += oty[k].bytes() * (((e.acc_mask >> k) & 1) ? 2 : 1);
            op_bytes_[timing == 2 ? key : sp.key(aty, e.acc_mask)] = b;
        }
        if (timing) hipEventRecord(e0, stream_);
        rc = sp.run(*this, aty, ap.data(), oty, op.data(), e.acc_mask,
                    ws_off == kNoOffset ? nullptr : dev_ptr(ws_off), ws_bytes);
        if (timing) hipEventRecord(e1, stream_);
        if (timing == 1 && !rc) {
            hipEventSynchronize(e1);
            float ms = 0;
            hipEventElapsedTime(&ms, e0, e1);
            auto &t = times_[sp.key(aty, e.acc_mask)];
            t.first += ms;
            t.second++;
        }
        n_run_++;
    }
    if (ws_off != kNoOffset) pool_.free(ws_off);      // reuse is ordered on the stream
    if (!rc)
        for (CellPtr o : e.outs) {
            cells_[o].v_valid = true;
            cells_[o].h_valid = false;
        }
    for (CellPtr a : e.args) cells_[a].pin--;
    for (CellPtr o : e.outs) cells_[o].pin--;
    return rc;
}

int Ctx::collect_timings()
{
    CACTI_HIP(hipStreamSynchronize(stream_));
    for (size_t i = 0; i < ev_keys_.size(); i++) {
        float ms = 0;
        if (hipEventElapsedTime(&ms, ev_pool_[i].first, ev_pool_[i].second) != hipSuccess) continue;
        auto &t = times_[ev_keys_[i]];
        t.first += ms;
        t.second++;
    }
    ev_keys_.clear();
    return 0;
}

int Ctx::resume(CellPtr *yield_cell)
{
    CACTI_REQUIRE(compiled_, CACTI_E_STATE, "resume before compile");
    while (pc_ < log_.size()) {
        const Entry &e = log_[pc_];
        if (e.kind == E_YIELD_SET) {
            if (yield_cell) *yield_cell = e.cell;
            return R_YIELD;                           // pc_ advances in resume_put
        }
        if (e.kind == E_UNLIVE) {
            cell_free_all(e.cell);
            cells_[e.cell].alive = false;
        } else {
            int rc = keep_reserve();
            if (!rc) rc = prefetch_ahead();
            if (!rc) rc = run_entry(e);
            if (rc) return rc < 0 ? rc : -1000 - rc;  // keep 0/1 for DONE/YIELD
            pc_++;
            if ((rc = spill_eagerly(e))) return rc;
            continue;
        }
        pc_++;
    }
    return R_DONE;
}

int Ctx::resume_put(CellPtr c, const void *host, size_t bytes)
{
    CACTI_REQUIRE(pc_ < log_.size() && log_[pc_].kind == E_YIELD_SET && log_[pc_].cell == c,
                  CACTI_E_STATE, "resume_put: the spine is not waiting for cell %d", c);
    int rc = cell_put(c, host, bytes);
    if (rc) return rc;
    pc_++;
    return 0;
}

// One line per class of cell: bytes resident on the device (pinned ones apart) and bytes held only
// by a host replica; then the pool's own figures.  The classes follow the cells' roles in the cycle:
// parameters, gradients and optimiser state live across cycles and are what a capped pool spills;
// everything else is an activation or an adjoint of the running cycle.
std::string Ctx::usage_report() const
{
    struct Row { const char *what; size_t n = 0, dev = 0, pinned = 0, host_only = 0, largest = 0; };
    Row rows[5];
    rows[0].what = "parameters";
    rows[1].what = "gradients";
    rows[2].what = "optimiser state";
    rows[3].what = "tables, inputs, caches";
    rows[4].what = "cycle cells";
    for (size_t i = 1; i < cells_.size(); i++) {
        const Cell &c = cells_[i];
        if (!c.alive) continue;
        int k = 4;
        if (c.stable) {
            const std::string &n = c.name;
            if (n.compare(0, 5, "grad:") == 0) k = 1;
            else if (n.compare(0, 7, "master:") == 0 || n.compare(0, 9, "grad_avg:") == 0 || n.compare(0, 10, "grad2_avg:") == 0) k = 2;
            else if (n == "cos" || n == "sin" || n.compare(0, 3, "in_") == 0 || n.find("cache") != std::string::npos ||
                     n.compare(0, 6, "cached") == 0) k = 3;
            else k = 0;
        }
        Row &r = rows[k];
        const size_t b = c.ty.bytes();
        r.n++;
        if (c.voff != kNoOffset) {
            r.dev += b;
            if (c.pin > 0) r.pinned += b;
            r.largest = std::max(r.largest, b);
        } else if (c.hptr && c.h_valid) {
            r.host_only += b;
        }
    }
    char line[256];
    std::string out;
    snprintf(line, sizeof line, "pool: cap=%zu used=%zu peak=%zu front=%zu largest_free=%zu pending_downloads=%zu (%zu regions) "
             "host=%zu\n", pool_.cap(), pool_.used(), pool_.peak(), pool_.front(), pool_.largest_free(), pending_bytes_,
             pending_.size(), (size_t)host_bytes_);
    out += line;
    for (const Row &r : rows) {
        snprintf(line, sizeof line, "  %-24s cells=%zu device=%zu (pinned %zu, largest %zu) host_only=%zu\n", r.what, r.n, r.dev,
                 r.pinned, r.largest, r.host_only);
        out += line;
    }
    snprintf(line, sizeof line, "  evictions=%llu uploads=%llu d2h=%llu h2d=%llu soft_oom=%llu entry=%zu/%zu\n",
             (unsigned long long)n_evict_, (unsigned long long)n_upload_, (unsigned long long)bytes_d2h_,
             (unsigned long long)bytes_h2d_, (unsigned long long)n_soft_oom_, pc_, log_.size());
    out += line;
    return out;
}

void Ctx::stats(Stats *s) const
{
    s->pool_cap = pool_.cap();
    s->pool_used = pool_.used();
    s->pool_peak = pool_.peak();
    s->pool_front = pool_.front();
    s->n_alloc = n_alloc_;
    s->n_evict = n_evict_;
    s->n_upload = n_upload_;
    s->bytes_d2h = bytes_d2h_;
    s->bytes_h2d = bytes_h2d_;
    s->n_soft_oom = n_soft_oom_;
    s->n_entries = log_.size();
    s->n_thunks_run = n_run_;
    s->host_bytes = host_bytes_;
}

}  // namespace cacti
