/*
 * cacti_hip_runtime.h -- C ABI of the host runtime inside libcacti_gpu_hip_ffi.so:
 * the HIP device context (pooled allocator + host spill), the spine
 * (reset / compile / resume / resume_put) and the LLaMA step staged on it.
 *
 * The kernel-level entry points are in cacti_gpu_hip_ffi.h; this header is the
 * layer a host program drives, with the reference's control flow:
 *   reset(); stage...; vadd_vjp; compile(); resume() <-> resume_put(); read outputs
 * (examples/open_llama_3b_train.rs:203-531).  Status codes as in cacti_gpu_hip_ffi.h.
 * One thread per context (src/ctx.rs:21-29).
 */
#ifndef CACTI_HIP_RUNTIME_H
#define CACTI_HIP_RUNTIME_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct cacti_ctx cacti_ctx;
typedef struct cacti_llama cacti_llama;

/* LlamaConfig, src/librarium/llama.rs:28-105 (batch ubat_sz = 1, q_group = 1). */
typedef struct {
    int64_t S;   /* seq_cap          */
    int64_t D;   /* num_head*head_dim */
    int64_t H;   /* num_head         */
    int64_t Dh;  /* head_dim         */
    int64_t F;   /* mlp_inner_dim    */
    int64_t V;   /* tok_dim          */
    int64_t L;   /* num_layer        */
    float eps;   /* rms_norm_eps     */
} cacti_llama_cfg;

typedef struct {
    uint64_t pool_cap, pool_used, pool_peak, pool_front;
    uint64_t n_alloc, n_evict, n_upload, bytes_d2h, bytes_h2d, n_soft_oom;
    uint64_t n_entries, n_thunks_run, host_bytes;
} cacti_stats;

/* ---- device context: replaces NvGpuPCtx + NvGpuMemPool, src/pctx/nvgpu.rs:163-306,
 * 1377-2002.  pool_bytes = 0 reserves 90.01 % of the device (src/ctx.rs:43); otherwise the
 * cap in bytes (the CACTI_VMEM_SOFT_LIMIT analogue, src/pctx/nvgpu.rs:1434-1463).  The pool
 * is ONE hipMalloc; when it is exhausted live cells are spilled to host memory
 * (_try_soft_oom, src/pctx/nvgpu.rs:2004-2283) and re-uploaded on their next use.
 * host_pagelocked: 1 = hipHostMalloc, 0 = malloc (CACTI_NVGPU_MEM_ALLOC, :995-1002),
 * -1 = what the environment says (cacti_env_host_pagelocked).  With pool_bytes = 0 the
 * environment variable CACTI_VMEM_SOFT_LIMIT, when set, gives the reserve
 * (cacti_vmem_soft_limit). */
int cacti_ctx_create(cacti_ctx **ctx, int dev, size_t pool_bytes, int host_pagelocked);

/* ---- configuration from the environment (cacti_cfg_env/src/lib.rs:47-234), as plain functions
 * so that the rules can be checked without a device.
 * cacti_parse_byte_size: "10 KB" = 10000, "16 KiB" = 16384, "0.2 MiB" = 209715, "123k" = 123000:
 * a decimal number (fraction, exponent, '_' and blanks allowed), an optional prefix K M G T P E
 * (powers of 1000; of 1024 when an 'i' follows), an optional B; results round to nearest
 * (src/algo/str/parse_size.rs:262-400).  CACTI_E_INVALID for no number, a character that does
 * not belong, or a result beyond 64 bits.
 * cacti_vmem_soft_limit: the size of the device reserve for a CACTI_VMEM_SOFT_LIMIT text
 * (NULL or "" = the default 90.01 % of `total`): a text that reads as a decimal number is a
 * fraction of `total`, held to [0, 1] and to avail - 32 MiB; else a byte size; else the
 * default; rounded down to 64 KiB (NvGpuMemPool::new, src/pctx/nvgpu.rs:1434-1463).  A bare
 * integer reads as a decimal number, so a size in bytes needs its unit ("17179869184B").
 * cacti_env_host_pagelocked: 1 when CACTI_GPU_MEM_ALLOC (else the reference's name,
 * CACTI_NVGPU_MEM_ALLOC) is "pagelocked" (src/pctx/nvgpu.rs:995-1002), else 0. */
int cacti_parse_byte_size(const char *text, uint64_t *bytes);
int cacti_vmem_soft_limit(const char *text, size_t avail, size_t total, size_t *reserve);
int cacti_env_host_pagelocked(void);
int cacti_ctx_destroy(cacti_ctx *ctx);
int cacti_ctx_stats(cacti_ctx *ctx, cacti_stats *out);
/* The pool's usage as text (NvGpuPCtx::_dump_usage / _dump_sizes / _dump_free,
 * src/pctx/nvgpu.rs:690-742): one line for the pool (cap, used, peak, front, largest free region,
 * downloads in flight, host bytes), one per class of cell (parameters, gradients, optimiser state,
 * tables and inputs, the running cycle's cells: count, bytes on the device, of those pinned, largest,
 * bytes held by a host replica only) and the spill counters.  The same text goes to stderr when the pool
 * is exhausted with everything else pinned (the reference dumps and panics, :2424-2440; here the call
 * returns CACTI_E_OOM) and, with CACTI_VERBOSE set, at every reset, i.e. once per cycle
 * (src/ctx.rs:150-167).  The buffer must hold the text (4 KiB is enough), else CACTI_E_INVALID. */
int cacti_ctx_usage_report(cacti_ctx *ctx, char *buf, size_t cap);
int cacti_ctx_sync(cacti_ctx *ctx);      /* stream sync + token-range status check */
void *cacti_ctx_stream(cacti_ctx *ctx);                 /* the hipStream_t all work runs on */
/* per-thunk device times (CACTI_DEBUG_TIMING, src/ctx.rs:114-133).  mode 1 syncs after
 * every thunk; mode 2 records a HIP event pair around every launch without syncing and
 * reads them back in the report, so a run is measured undisturbed; 0 switches timing off
 * and clears the totals.  The report is text, one "label count total_ms operand_bytes" line
 * per label (operand bytes of one launch: every argument read once, every output written
 * once, an accumulated output read as well); GEMM labels carry the transposes and
 * nblk x M x N x K.  A filter restricts mode 2 to the
 * launches whose label starts with the given text (an event pair costs a few microseconds
 * of stream time per launch, about 10 % of a whole step when every launch carries one);
 * NULL or "" matches every launch; of the matching launches every `every`-th is timed
 * (1 = all). */
int cacti_ctx_set_timing(cacti_ctx *ctx, int on);
int cacti_ctx_set_timing_filter(cacti_ctx *ctx, const char *label_prefix, int every);
int cacti_ctx_timing_report(cacti_ctx *ctx, char *buf, size_t cap);

/* ---- the pool's placement policy alone, over a plain offset range (no device memory is
 * touched, so it can be exercised on a host without a GPU): first fit over the coalesced
 * free regions, else bump the front cursor; 256-byte granules; freeing the last region
 * retracts the cursor (src/pctx/nvgpu.rs:30, 1633-1655).  alloc returns the offset, or
 * UINT64_MAX when the request does not fit.  alloc_high is the mirror image from the top of
 * the range (highest hole first, else a back cursor that moves down): the runtime places
 * the cells that live across cycles (parameters, gradients) there, so that a cycle's
 * short-lived regions are not scattered between them; the reference has one front
 * allocator and no counterpart.  Either kind takes a hole of the other end before it
 * reports that the request does not fit. */
typedef struct cacti_mempool cacti_mempool;
int cacti_mempool_create(cacti_mempool **pool, uint64_t cap);
int cacti_mempool_destroy(cacti_mempool *pool);
uint64_t cacti_mempool_alloc(cacti_mempool *pool, uint64_t bytes);
uint64_t cacti_mempool_alloc_high(cacti_mempool *pool, uint64_t bytes);
int cacti_mempool_free(cacti_mempool *pool, uint64_t offset);
/* out[0..4] = cap, used, peak, front cursor, largest request that fits now */
int cacti_mempool_stats(cacti_mempool *pool, uint64_t out[5]);

/* ---- spine: src/ctx.rs:326-373, src/spine.rs:1193-1991 */
int cacti_reset(cacti_ctx *ctx);
int cacti_compile(cacti_ctx *ctx);
/* returns 0 = ran to the end, 1 = yielded: *yield_cell must be supplied with
 * cacti_resume_put before resuming; negative = error */
int cacti_resume(cacti_ctx *ctx, int *yield_cell);
int cacti_resume_put(cacti_ctx *ctx, int cell, const void *host, size_t bytes);
int cacti_cell_bytes(cacti_ctx *ctx, int cell, size_t *bytes);
int cacti_cell_get(cacti_ctx *ctx, int cell, void *host, size_t bytes);   /* with_mem, src/op.rs:2203 */
/* number of log entries and the name of entry i ("matmul", "rms_norm_bwd", "unlive", ...) */
int cacti_log_len(cacti_ctx *ctx);
const char *cacti_log_name(cacti_ctx *ctx, int i);

/* ---- model: Llama::{from, init_constants, apply}, src/librarium/llama.rs:223-548.
 * Parameters (3 + 9 L tensors, f16) and their gradients are stable cells; order:
 * embed, per layer {pre_norm, q, k, v, o, post_norm, gate, up, down}, head_norm, lm_head. */
int cacti_llama_create(cacti_ctx *ctx, const cacti_llama_cfg *cfg, cacti_llama **model);
int cacti_llama_destroy(cacti_llama *model);
int cacti_llama_num_params(cacti_llama *model);
int cacti_llama_param_info(cacti_llama *model, int i, char *name, size_t name_cap,
                           int64_t *rows, int64_t *cols, int *param_cell, int *grad_cell);
int cacti_llama_param_put(cacti_llama *model, int i, const void *host, size_t bytes);
int cacti_llama_grad_get(cacti_llama *model, int i, void *host, size_t bytes);
/* Numerical-health digests of every parameter (of_grads = 0) or gradient (1), in parameter
 * order: hist [num_params][256] and nan [num_params], int64, host memory.  What the reference's
 * example computes each cycle with p.abs_log2_hist8(), p.nan_count(), g.abs_log2_hist8(),
 * g.nan_count() (examples/open_llama_3b_train.rs:409-424, read at :587-650); bins as in
 * cacti_hip_abs_log2_hist8_f16.  One stream synchronisation for the whole call. */
int cacti_llama_digests(cacti_llama *model, int of_grads, int64_t *hist, int64_t *nan);
/* AdamW32 with f32 master weights and moment averages, as the reference's example sets it up
 * (examples/open_llama_3b_train.rs:189-205, 230-243): adamw_init creates, per parameter, the f32
 * cells master (= set_cast of the parameter), grad_avg and grad2_avg (= set_zeros).  adamw_step
 * runs one step of every parameter from its current gradient (the loop at :252-268: adamw.step,
 * then p.set_lossy_cast(master)) in one launch and returns without synchronising; skip_embed = 1
 * leaves the embedding untouched as the example does (:262-263).  The new parameters are what the
 * next cacti_llama_step reads.  adamw_state_get copies master (which = 0), grad_avg (1) or
 * grad2_avg (2) of parameter i to host memory. */
typedef struct {
    float grad_scale;          /* <= 0: gradients are not scaled */
    float lr, wd, a1, a2, eps;
} cacti_adamw32;
int cacti_llama_adamw_init(cacti_llama *model);
int cacti_llama_adamw_step(cacti_llama *model, int iter_nr, const cacti_adamw32 *opt, int skip_embed);
int cacti_llama_adamw_state_get(cacti_llama *model, int i, int which, void *host, size_t bytes);
/* ---- weight ingest: TensorsDir (src/util/safetensor.rs:45-160), CellMatcher (src/util/cell.rs:47-112),
 * Llama::match_pickle_dir (src/librarium/llama.rs:284-302), resume_put (src/spine.rs:1714-1745).
 *
 * tensors_dir_open: `path` is a safetensors file, or a directory holding model.safetensors or the
 * shards model-*-of-*.safetensors (taken in sorted order).  The files are memory-mapped, the
 * headers parsed; a tensor name that occurs twice, a byte range that does not fit the file or the
 * tensor's type, or a malformed header is CACTI_E_FORMAT, a missing file CACTI_E_IO.
 * tensors_dir_entry: entry i in byte-wise sorted name order (the order CellMatcher scans): name,
 * dtype as spelled in the file ("F16", "BF16", "F32", ...), shape (at most 8 dims), a pointer into
 * the mapping (valid until close) and its length; a name or dtype longer than its buffer is
 * CACTI_E_INVALID. */
typedef struct cacti_tensors_dir cacti_tensors_dir;
int cacti_tensors_dir_open(const char *path, cacti_tensors_dir **dir);
int cacti_tensors_dir_close(cacti_tensors_dir *dir);
int cacti_tensors_dir_count(cacti_tensors_dir *dir);
int cacti_tensors_dir_entry(cacti_tensors_dir *dir, int i, char *name, size_t name_cap, char *dtype,
                            size_t dtype_cap, int *ndim, int64_t *shape8, const void **data,
                            uint64_t *bytes);
/* PickleDir::open / open_with_prefix / get (src/util/safepickle.rs:52-195), the reader the training
 * example opens its checkpoint with (examples/open_llama_3b_train.rs:91).  `path` is one torch
 * checkpoint file, or a directory holding <prefix>.bin or the shards <prefix>-*-of-*.bin (sorted);
 * prefix NULL or "" means "pytorch_model".  Each file is a ZIP archive (ZIP64 included) whose
 * data.pkl is scanned without executing anything; every top-level entry of the state dictionary
 * that is a tensor (bare or wrapped as a parameter) joins the table.  The handle is the one
 * tensors_dir_open returns: count, entry, close and llama_load_tensors_dir apply unchanged, with
 * dtypes spelled as in safetensors ("F16", "BF16", "F32", ...).  As in the reference, a tensor whose
 * strides are not the packed ones is refused (CACTI_E_NOTIMPL), as is a storage type outside
 * src/cell/mod.rs:1553-1574; a first byte that is not 64-byte aligned, a tensor that does not fit
 * its storage, a duplicate name, a legacy (non-ZIP) file or an unknown pickle opcode is
 * CACTI_E_FORMAT. */
int cacti_pickle_dir_open(const char *path, const char *prefix, cacti_tensors_dir **dir);
/* CellMatcher::match_: rule r (components separated by '/', "#12" = the integer 12, anything else
 * a string) takes the first key, in sorted order and not taken by an earlier rule, whose
 * '.'-separated tokens consume the rule left to right: an integer needs a token equal to its
 * decimal text, a string a token that equals or contains it.  match[r] = index into keys, or -1. */
int cacti_cell_matcher_match(const char *const *keys, int nkeys, const char *const *rules, int nrules,
                             int *match);
/* Matches the model's parameters against the directory with the rules of Llama::match_pickle_dir
 * and stores every matched tensor into its parameter cell: F16 as it is (resume_put), BF16 and F32
 * through the device casts set_lossy_cast stages (src/op.rs:1112-1135).  A matched tensor whose
 * shape differs from the parameter's is CACTI_E_INVALID (the reference panics on mismatched types),
 * another dtype CACTI_E_NOTIMPL.  Parameters without a match keep their value; *n_matched counts the
 * matched ones. */
int cacti_llama_load_tensors_dir(cacti_llama *model, cacti_tensors_dir *dir, int *n_matched);
/* ---- KV-cached forward pass: LlamaCached, src/librarium/llama.rs:561-963 (batch 1, q_group 1).
 * cached_create shares the model's parameters and position tables (LlamaCached::from(Llama) /
 * from_train, llama.rs:618-686) and adds zeroed k / v caches [seq_cap, H, Dh] per layer and an
 * input token cell [seq_cap] (u16, zeros = pad); seq_cap % 8 == 0, seq_cap <= the model's S.
 * reset_state zeroes the caches (llama.rs:784-789).  set_tokens writes the first n input tokens
 * and pads the rest with 0 (the example's resume_put_mem_with, open_llama_3b_deploy.rs:221-231).
 * apply runs positions prev .. next-1 (llama.rs:805-963): embeds in_tok[prev .. next], adds the new
 * keys and values to the caches, attends over the cache with the row-causal mask, and keeps logit
 * [T,V] f16, tok [T] u16 (arg max) and, if asked, prob [T,V] f32 for the T = next - prev rows; the
 * token generated for the last row is added to in_tok[next] when next < seq_cap.  It returns with
 * the work queued on the context's stream.  outputs copies what the last apply kept (any pointer
 * may be NULL) and synchronises; a token id >= V is reported there as CACTI_E_INDEX. */
typedef struct cacti_llama_cached cacti_llama_cached;
int cacti_llama_cached_create(cacti_llama *model, int64_t seq_cap, cacti_llama_cached **cached);
int cacti_llama_cached_destroy(cacti_llama_cached *cached);
int cacti_llama_cached_reset_state(cacti_llama_cached *cached);
int cacti_llama_cached_set_tokens(cacti_llama_cached *cached, const uint16_t *tok, int64_t n);
int cacti_llama_cached_get_tokens(cacti_llama_cached *cached, uint16_t *tok);
int cacti_llama_cached_apply(cacti_llama_cached *cached, int64_t prev, int64_t next, int want_prob);
int cacti_llama_cached_outputs(cacti_llama_cached *cached, void *logit_f16, float *prob, uint16_t *tok);
/* cells of the inputs (tok u16 [S], lm_tok u16 [S], loss_scale f32 [S]) and of the kept
 * outputs of the last staged cycle (logit f16 [S,V], loss f32 [S], amax u16 [S],
 * prob f32 [S,V] or 0) */
int cacti_llama_io_cells(cacti_llama *model, int *tok, int *lm_tok, int *loss_scale, int *logit,
                         int *loss, int *amax, int *prob);
/* How the attention block of a layer (src/librarium/llama.rs:501-507) is staged from the next cycle on:
 * 0 (default) one fused thunk, cacti_hip_attention_fwd / _bwd, which keeps the [S, H, S] scores and
 * probabilities in registers; 1 the reference's chain of separate thunks (block product, causal softmax,
 * block product and their adjoints), which materialises them.  Same rounding points either way. */
int cacti_llama_set_attention(cacti_llama *model, int mode);
/* How the projections that share an input are staged from the next cycle on (a pointer-array batch: the
 * reference's cublasGemmBatchedEx shape, cacti_gpu_cu_ffi/src/lib.rs:793-885).  0: one matmul thunk per
 * product as src/librarium/llama.rs:478-497 stages them.  1 (default): the up and gate projections of a layer
 * as one thunk and one launch, their adjoints as for separate thunks.  2: also the query, key and value
 * projections, and the weight gradients of both groups as one thunk each.  Every product is computed by the
 * same tiles in the same order in all three and the adjoint's accumulations keep their order, so the results
 * are identical bit for bit; measured on the 3B step on one MI355X, same box: 52.80, 52.68 and 53.35 ms
 * (the batched weight gradients run 4 % slower than their separate launches). */
int cacti_llama_set_product_groups(cacti_llama *model, int on);
/* Stages one cycle on a freshly reset spine: mem_set_yield_ of the three inputs,
 * Llama::apply, and (want_grad) sink.add(loss, loss_scale) + vadd_vjp over all parameters
 * (examples/open_llama_3b_train.rs:350-389).  want_grad = 1 overwrites the gradients; want_grad = 2
 * is g.cache() on every gradient first (the micro-batch accumulation of :334-345; SpineEntry::Cache,
 * src/spine.rs:786-805): this cycle's gradients are added, in f16 as every accumulation of the
 * path, to the values the cells hold.  CACTI_E_STATE if no cycle has written them yet. */
int cacti_llama_stage(cacti_llama *model, int want_prob, int want_grad);
/* reset + stage + compile + resume/resume_put.  With loss_out [S] f32 the call syncs, checks
 * the token-range status and copies the loss back; with loss_out = NULL it returns while the
 * cycle still runs on the stream (results and a CACTI_E_INDEX status are then observed by the
 * next synchronizing call: cacti_ctx_sync, cacti_cell_get, cacti_llama_grad_get). */
int cacti_llama_step(cacti_llama *model, const uint16_t *tok, const uint16_t *lm_tok,
                     const float *loss_scale, int want_prob, int want_grad, float *loss_out);

#ifdef __cplusplus
}
#endif
#endif /* CACTI_HIP_RUNTIME_H */
