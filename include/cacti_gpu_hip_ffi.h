/*
 * cacti_gpu_hip_ffi.h -- C ABI of libcacti_gpu_hip_ffi.so
 *
 * The MI355X (gfx950) counterpart of cacti's `cacti_gpu_cu_ffi` crate plus the
 * kernels its thunks dispatch to.  Every entry point is plain C: raw device
 * pointers, integer sizes, a stream handle passed as `void*` (a hipStream_t;
 * NULL = the null stream, which is the stream the reference computes on,
 * src/pctx/nvgpu.rs:263).  No C++ or torch types cross this boundary.
 *
 * Conventions
 *   - every function returns an int status: 0 = success, a positive value = the
 *     hipError_t of the failing runtime call, a negative value = CACTI_E_*.
 *     (reference: C level integer status, 0 = ok; Rust wrappers map it to
 *     Result<_, code>, cacti_gpu_cu_ffi/src/lib.rs:98-885.)
 *   - kernels are asynchronous on `stream`; results are complete at stream sync
 *     (the reference syncs the stream around every thunk, src/thunk/mod.rs:3480,3536).
 *   - pointers are borrowed for the duration of the call; nothing is freed or
 *     retained by the library (src/thunk/op.rs:4574-4578 convention: the caller
 *     owns and pre-allocates outputs).
 *   - f16 tensors are IEEE binary16, row-major, contiguous unless a leading
 *     dimension is given.  `acc` arguments: 0 = Apply (output is first written),
 *     1 = Accumulate (output += result, added in the output dtype; for GEMMs
 *     beta = 1 is added in fp32 before the single output rounding), mirroring
 *     ThunkImpl::{apply,accumulate}, src/thunk/mod.rs:347-351.
 *   - calls on one device context are not re-entrant (one thread per context,
 *     as in the reference, src/ctx.rs:21-29).
 */
#ifndef CACTI_GPU_HIP_FFI_H
#define CACTI_GPU_HIP_FFI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CACTI_OK 0
#define CACTI_E_INVALID (-1)   /* bad shape / null pointer / misaligned operand      */
#define CACTI_E_NOTIMPL (-2)   /* shape outside what the kernel supports             */
#define CACTI_E_INDEX (-3)     /* token / key id out of range (reference: assert)     */
#define CACTI_E_OOM (-4)       /* pool exhausted even after eviction                  */
#define CACTI_E_STATE (-5)     /* call not valid in the current state                 */
#define CACTI_E_IO (-6)        /* a file cannot be opened or mapped                   */
#define CACTI_E_FORMAT (-7)    /* a file does not have the expected layout            */

/* Human-readable text for the last non-zero status returned on this thread. */
const char *cacti_hip_last_error(void);

/* ------------------------------------------------------------------------- */
/* Device, memory, streams, events.                                           */
/* Replaces cacti_gpu_cu_ffi/src/lib.rs:98-131 (device), :204-268 (memory),   */
/* :332-399 (runtime), :401-565 (events, streams).                            */

int cacti_hip_device_count(int *count);                         /* lib.rs:98, :332  */
int cacti_hip_device_get(int *dev);                             /* lib.rs:341       */
int cacti_hip_device_set(int dev);                              /* lib.rs:350       */
int cacti_hip_device_attribute(int dev, int attr, int *value);  /* lib.rs:116       */
int cacti_hip_device_sync(void);                                /* lib.rs:368       */
int cacti_hip_mem_get_info(size_t *free_bytes, size_t *total_bytes); /* lib.rs:358  */
int cacti_hip_mem_alloc(void **dptr, size_t bytes);             /* lib.rs:204       */
int cacti_hip_mem_free(void *dptr);                             /* lib.rs:222       */
int cacti_hip_mem_alloc_host(void **ptr, size_t bytes);         /* lib.rs:213 (hipHostMalloc) */
int cacti_hip_mem_free_host(void *ptr);                         /* lib.rs:230       */
int cacti_hip_memcpy_d2h(void *dst, const void *src, size_t bytes);                 /* lib.rs:238 */
int cacti_hip_memcpy_async(void *dst, const void *src, size_t bytes, void *stream); /* lib.rs:246 */
int cacti_hip_memcpy_h2d_async(void *dst, const void *src, size_t bytes, void *stream); /* :254 */
int cacti_hip_memcpy_d2h_async(void *dst, const void *src, size_t bytes, void *stream); /* :262 */
int cacti_hip_memset_async(void *dst, int byte, size_t bytes, void *stream);
int cacti_hip_primary_ctx_retain(int dev, void **pctx);         /* lib.rs:177 (hipDevicePrimaryCtxRetain) */
int cacti_hip_primary_ctx_release(int dev);                     /* lib.rs:159       */
/* set_flags on a primary context that is already active returns the runtime's error as its positive
 * hipError_t (a status, never an abort).  reset destroys everything on the device, so it is refused with CACTI_E_STATE
 * while a cacti_ctx of this library exists on `dev`; after a reset the library looks its per-device
 * state (kernel attributes, the address of its built-in scratch array) up again on the next launch.
 * Memory, streams and events the caller created on the device are the caller's to forget. */
int cacti_hip_primary_ctx_set_flags(int dev, unsigned flags);   /* lib.rs:186       */
int cacti_hip_primary_ctx_reset(int dev);                       /* lib.rs:169       */
void *cacti_hip_stream_null(void);                              /* lib.rs:512: the null stream's handle (NULL) */
int cacti_hip_stream_create(void **stream);                     /* lib.rs:518       */
int cacti_hip_stream_create_nonblocking(void **stream);         /* lib.rs:529       */
int cacti_hip_stream_destroy(void *stream);                     /* lib.rs:493       */
int cacti_hip_stream_sync(void *stream);                        /* lib.rs:540       */
int cacti_hip_stream_wait_event(void *stream, void *event);     /* lib.rs:548       */
int cacti_hip_event_create(void **event, int enable_timing);    /* lib.rs:431       */
int cacti_hip_event_destroy(void *event);                       /* lib.rs:415       */
int cacti_hip_event_record(void *event, void *stream);          /* lib.rs:442       */
int cacti_hip_event_query(void *event);                         /* lib.rs:453       */
int cacti_hip_event_sync(void *event);                          /* lib.rs:461       */
int cacti_hip_event_elapsed_ms(void *start, void *stop, float *ms);

/* ------------------------------------------------------------------------- */
/* GEMM: C = alpha * op(A) op(B) + beta * C, f16 x f16 -> fp32 accumulate ->   */
/* f16 out, hand-written MFMA kernels.                                         */

/* Row-major form.  op(A) is M x K: stored [M,K] (ta = 0) or [K,M] (ta = 1);
 * op(B) is K x N: stored [K,N] (tb = 0) or [N,K] (tb = 1); C is [M,N].
 * Leading dimensions in elements.  beta must be 0 or 1.
 * Replaces MatrixMulF16F32GpuThunkImpl::_enter, src/thunk/op.rs:4423-4700. */
int cacti_hip_gemm_f16(int ta, int tb, int64_t M, int64_t N, int64_t K, float alpha,
                       const void *A, int64_t lda, const void *B, int64_t ldb, float beta,
                       void *C, int64_t ldc, void *stream);

/* `nblk` independent blocks, block h at A + h*stride_a etc. (strides in
 * elements).  This is how the per-head blocks of [B,S,H,Dh] / [B,S,H,S]
 * tensors are addressed; it replaces the pointer-array staging of
 * BlockMatrixMulF16F32GpuThunkImpl::_enter, src/thunk/op.rs:5027-5471
 * (cublasGemmBatchedEx, cacti_gpu_cu_ffi/src/lib.rs:793-885).  No padding of
 * the inner dimension is needed (the reference pads Dh 100 -> 104,
 * src/op.rs:1454-1482).  When the blocks of a not transposed B lie side by side in
 * its rows (stride_b < ldb), a block's product may read columns of the neighbouring
 * blocks in the same row, never anything outside the columns
 * [0, (nblk - 1) * stride_b + N) of B's rows; C is written only inside each block. */
int cacti_hip_gemm_f16_strided_batched(int ta, int tb, int64_t nblk, int64_t M, int64_t N,
                                       int64_t K, float alpha, const void *A, int64_t lda,
                                       int64_t stride_a, const void *B, int64_t ldb,
                                       int64_t stride_b, float beta, void *C, int64_t ldc,
                                       int64_t stride_c, void *stream);

/* Measurement aid with no counterpart in the reference (bench.py --workload mfma-power): one launch of
 * `blocks` workgroups of 8 waves that do nothing but MFMAs on register fragments, `iters` (even) iterations
 * of 262144 flops per wave.  shape 0: v_mfma_f32_32x32x16_f16, 1: v_mfma_f32_16x16x32_f16; lds_reads: 0, 4
 * or 6 fragments (16 bytes per lane each) refreshed from LDS per iteration; random_operands 0: all operands
 * zero.  out: blocks * 512 floats of device memory.  Run for a second or more it shows the rate the device
 * sustains under its power limit, which depends on all three. */
int cacti_hip_mfma_probe(int shape, int lds_reads, int random_operands, int blocks, int64_t iters,
                         unsigned seed, void *out, void *stream);

/* Pointer-array batch, the shape of cublasGemmBatchedEx (cacti_gpu_cu_ffi/src/lib.rs:793-885):
 * nblk products of one shape, block z on A[z], B[z], C[z] (host arrays of device pointers, read
 * before the call returns).  With every operand 16-byte aligned up to four products share a launch,
 * otherwise they run one after another.  (Sharing a launch saves launches, not time: measured on the
 * three 2048 x 3200 x 3200 projections of a layer, 600 whole tiles on 256 CUs take three tile times
 * either way.)  Results equal those of nblk calls of cacti_hip_gemm_f16. */
int cacti_hip_gemm_f16_batched(int ta, int tb, int64_t nblk, int64_t M, int64_t N, int64_t K,
                               float alpha, const void *const *A, int64_t lda, const void *const *B,
                               int64_t ldb, float beta, void *const *C, int64_t ldc, void *stream);

/* The same with the triangular structure of causal attention made explicit, so that the
 * half of each sequence x sequence product that the causal mask discards is never computed:
 *   tri = 0  none (identical to the call above);
 *   tri = 1  only the lower triangle (column <= row) of C is wanted (M == N): tiles wholly
 *            above the diagonal are skipped and their part of C is left UNWRITTEN
 *            (S = a Q K^T and dP = dO V^T feed the causal softmax, which never reads there);
 *   tri = 2  A is lower triangular, not transposed (M == K): O = P V, dQ = a dS K;
 *   tri = 3  A is lower triangular, transposed (M == K): dV = P^T dO, dK = a dS^T Q.
 * For 2 and 3 the entries of A above the diagonal must be zero up to the next multiple of
 * 256 columns (the causal softmax kernels write them so); beyond that A is not read.
 * The reference computes these products densely (src/thunk/op.rs:5027-5471). */
int cacti_hip_gemm_f16_strided_batched_tri(int ta, int tb, int64_t nblk, int64_t M, int64_t N,
                                           int64_t K, float alpha, const void *A, int64_t lda,
                                           int64_t stride_a, const void *B, int64_t ldb,
                                           int64_t stride_b, float beta, void *C, int64_t ldc,
                                           int64_t stride_c, int tri, void *stream);

/* Column-major, cuBLAS-shaped form with host alpha/beta pointers, the call the
 * reference makes (cublas_gemm, cacti_gpu_cu_ffi/src/lib.rs:727-791; row-major
 * callers pass the operands swapped, src/thunk/op.rs:4469-4491).  tr_* = 0 (N)
 * or 1 (T).  Only f16 in / f16 out / fp32 compute is provided. */
int cacti_hip_gemm_colmajor_f16(int tr_a, int tr_b, int m, int n, int k, const float *alpha,
                                const void *a, int lda, const void *b, int ldb,
                                const float *beta, void *c, int ldc, void *stream);

/* ------------------------------------------------------------------------- */
/* accumulate_1d_{f32,f16,u16}: dst[i] += src[i]                               */
/* Replaces the NVRTC kernels of src/pctx/nvgpu.rs:2598-2668 (n <= INT32_MAX). */

int cacti_hip_accumulate_1d_f32(void *dst, const void *src, int64_t n, void *stream);
int cacti_hip_accumulate_1d_f16(void *dst, const void *src, int64_t n, void *stream);
int cacti_hip_accumulate_1d_u16(void *dst, const void *src, int64_t n, void *stream);

/* ------------------------------------------------------------------------- */
/* Fused thunks.  Each stands for a chain of reference thunks and reproduces   */
/* that chain's rounding points in registers.                                  */

/* RMSNorm, rms_norm closure src/librarium/llama.rs:442-451
 * (Cast op.rs:621, Square :2522, InnerMean :3150, AddScalar :1395, Sqrt :2609,
 *  BroadcastDiv :2358, BroadcastMul :2058, Cast).
 * x, y: [N,D] f16; w: [D] f16.  D % 8 == 0, D <= 8192. */
int cacti_hip_rms_norm_fwd(int64_t N, int64_t D, const void *x, const void *w, float eps,
                           void *y, void *stream);
/* The residual add in front of a norm and the norm in one pass over the rows:
 * sum = f16(a + b) (AddFutThunkSpec, src/thunk/op.rs:1480-1535; x1 = stream + o and
 * x2 = x1 + down in src/librarium/llama.rs:514-533), y = rms_norm(sum, w) as above.  Both
 * outputs are written; the results equal those of cacti_hip_add_f16 followed by
 * cacti_hip_rms_norm_fwd bit for bit. */
int cacti_hip_add_rms_norm_fwd(int64_t N, int64_t D, const void *a, const void *b, const void *w,
                               float eps, void *sum, void *y, void *stream);

/* Adjoint of the chain above (src/spine.rs:447-690 over the same thunks).
 * dx [N,D] f16 receives the two f16 contributions of the reference in order
 * (dx_acc: 0 first write, 1 dx already holds the residual gradient).
 * dw [D] f16 (dw_acc likewise).  workspace: device scratch of at least
 * cacti_hip_rms_norm_bwd_workspace(N, D) bytes, contents undefined on return. */
size_t cacti_hip_rms_norm_bwd_workspace(int64_t N, int64_t D);
int cacti_hip_rms_norm_bwd(int64_t N, int64_t D, const void *x, const void *w, float eps,
                           const void *dy, void *dx, int dx_acc, void *dw, int dw_acc,
                           void *workspace, size_t workspace_bytes, void *stream);

/* The same adjoint for callers that cannot allocate device memory or carry a workspace (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in
 * the reference.  The fp32 partial rows of dw go to a buffer built into the library, of
 * cacti_hip_rms_norm_bwd_static_max_bytes() = 8 MiB per device, held until the process ends; shapes
 * with cacti_hip_rms_norm_bwd_workspace(N, D) above that are CACTI_E_INVALID.  The call allocates
 * nothing and frees nothing.  All calls on one device share the one buffer: calls that overlap on a
 * device (two streams, two threads) race; calls on one stream are ordered and safe.  Results are
 * bit-identical to cacti_hip_rms_norm_bwd. */
size_t cacti_hip_rms_norm_bwd_static_max_bytes(void);
int cacti_hip_rms_norm_bwd_static(int64_t N, int64_t D, const void *x, const void *w, float eps,
                                  const void *dy, void *dx, int dx_acc, void *dw, int dw_acc,
                                  void *stream);

/* RoPE tables, Llama::init_constants src/librarium/llama.rs:389-411.
 * cos16, sin16: [S,Dh] f16 (two identical halves of width Dh/2). */
int cacti_hip_rope_tables(int64_t S, int64_t Dh, void *cos16, void *sin16, void *stream);

/* symplectic_embed src/librarium/llama.rs:463-465 and its adjoint
 * (InnerSymplecticMapFutThunkSpec :975-1049, BroadcastMul, Add).
 * x, y, dy, dx: [S,H,Dh] f16 (heads are the middle dimension); Dh even, H*Dh % 8 == 0. */
int cacti_hip_rope_fwd(int64_t S, int64_t H, int64_t Dh, const void *x, const void *cos16,
                       const void *sin16, void *y, void *stream);
int cacti_hip_rope_bwd(int64_t S, int64_t H, int64_t Dh, const void *dy, const void *cos16,
                       const void *sin16, void *dx, int dx_acc, void *stream);
/* The same on two tensors of one shape in one launch: the query and the key of a layer
 * (src/librarium/llama.rs:483, 490 apply the map to both), results as from two calls. */
int cacti_hip_rope_fwd_pair(int64_t S, int64_t H, int64_t Dh, const void *x0, const void *x1,
                            const void *cos16, const void *sin16, void *y0, void *y1, void *stream);
int cacti_hip_rope_bwd_pair(int64_t S, int64_t H, int64_t Dh, const void *dy0, const void *dy1,
                            const void *cos16, const void *sin16, void *dx0, int dx0_acc, void *dx1,
                            int dx1_acc, void *stream);

/* SiLU gate, src/librarium/llama.rs:526-527: h = f16(f16(silu(g)) * u)
 * (StandardSiluFutThunkSpec op.rs:2867-2909, MulFutThunkSpec :2001-2055), and
 * the adjoint: du (+)= f16(y*dh); dg (+)= f16(f16(dh*u) * c), c per :2901-2908.
 * All [n] f16, n % 8 == 0. */
int cacti_hip_silu_gate_fwd(int64_t n, const void *g, const void *u, void *h, void *stream);
int cacti_hip_silu_gate_bwd(int64_t n, const void *g, const void *u, const void *dh, void *dg,
                            int dg_acc, void *du, int du_acc, void *stream);

/* Causal softmax over attention scores, src/librarium/llama.rs:501-505:
 * P16 = f16(softmax_j(mask(f32(S16)))) with mask j > i -> -inf
 * (Cast, BlockTriElemAffineFutThunkSpec op.rs:4189-4278, InnerSoftmaxFutThunkSpec
 * :3257-3383), and its adjoint dS16 = f16(tril(T - (sum_j T) P')), T = P' * f32(dP16),
 * P' recomputed in fp32 (InnerSoftmaxPostAdjFutThunkSpec :3386-3457).
 * s16, p16, dp16, ds16: [S,H,S] f16 (row i, head, column j).  S % 8 == 0, S <= 8192.
 * Inputs are read only at j <= i; outputs are written at j <= i and as zeros from there to
 * the next multiple of 256 columns (what the tri = 2 / 3 GEMMs read); entries further right
 * are left untouched. */
int cacti_hip_causal_softmax_fwd(int64_t S, int64_t H, const void *s16, void *p16, void *stream);
int cacti_hip_causal_softmax_bwd(int64_t S, int64_t H, const void *s16, const void *dp16,
                                 void *ds16, void *stream);

/* Causal attention of one layer, fused: O = f16(P16 V), P16 = f16(softmax_j(mask(f32(S16)))),
 * S16 = f16(alpha Q K^T) -- the chain block_matmul_scale -> cast -> BlockTriElemAffine -> InnerSoftmax ->
 * cast -> block_matmul of src/librarium/llama.rs:501-507 (src/thunk/op.rs:4719-5471, 4189-4278,
 * 3257-3383) with every rounding point of the chain kept -- and its adjoint
 * (pop_adj src/thunk/op.rs:4882-4912, InnerSoftmaxPostAdj :3386-3457):
 *   dV (+)= f16(P16^T dO), dQ (+)= f16(alpha dS16 K), dK (+)= f16(alpha dS16^T Q),
 *   dS16 = f16(tril(T - (sum_j T) P')), T = P' f32(f16(dO V^T)).
 * The sequence x sequence tensors S16, P16, dP16, dS16 never reach memory (the reference, and the
 * separate entry points above, keep them: 4 x H S^2 f16); the adjoint recomputes S16, P' and dP16
 * tile by tile and forms the row sums sum_j T from the rounded dP16 as the reference does.
 * q, k, v, o, dO, dq, dk, dv: [S, H, Dh] f16 with row stride ld (elements), 8-byte aligned;
 * Dh % 4 == 0, Dh <= 128, ld % 4 == 0.  stats: cacti_hip_attention_stats_bytes(S, H) bytes of device
 * memory, written by the forward call (row maximum and sum per head and row, f32) and read by the
 * adjoint; workspace: cacti_hip_attention_bwd_workspace(S, H) bytes, contents undefined on return.
 * Faster with every tensor of the call 16-byte aligned, ld % 8 == 0 and, for Dh % 8 == 4, an even number of
 * heads filling the row (every head then lies inside whole 16-byte pieces of its row that start at or 8 bytes
 * before it): the kernels move all their tiles, operands and results, as whole row segments between memory and
 * LDS, 20 % less time at 32 heads x 100.  In that form a head's
 * products run over those whole pieces, the elements of the neighbouring head in them multiplied by zeros: for
 * finite inputs the same values; a non-finite element in the 4 columns next to a head makes that head's
 * result non-finite as well (the reference: the neighbour's only, until the output projection mixes them).
 * *_acc: 0 first write, 1 the product is added to the tensor in fp32 before the one rounding (the
 * GEMMs' beta = 1).
 * o (adjoint): the forward call's output, or NULL.  With it a block of 128 queries whose rows all have their
 * probability spread (sum_j exp(S16_ij - m_i) >= 8, i.e. no probability above 1/8) takes its row sums
 * sum_j T_ij as sum_d dO_id O_id and skips the pass over the keys that forms them from the rounded dP16; the
 * two agree to 2^-11 |dP| sqrt(sum_j P_ij^2), below the rounding of dS16.  Blocks with a concentrated row
 * (the first of a sequence always: row 0 sees one key), o = NULL and the exactly rounded forms keep the pass.
 * Arithmetic between the rounding points.  By default a probability is formed as
 * 2^(s log2 e - c) with one fp32 offset c = m log2 e + log2 l per row (row maximum m, row sum l): the
 * rounding of c is an error common to the row, at most half an ulp of c times ln 2 relative -- 3e-6 for
 * |m| < 90, 2e-5 at |m| = 500 -- and in a row whose probability sits on one key it breaks the exact
 * cancellation dP - sigma = 0 the reference has there.  Results agree with the reference's chain to 1e-4
 * relative L2 for row maxima up to some hundreds; beyond that (|m| in the thousands: measured 7e-3 on dQ
 * at |m| = 1500 .. 2600) call cacti_hip_attention_set_exact(1): every later launch of this process uses
 * the exactly rounded forms of the separate softmax kernels (range-reduced exp of s - m, correctly
 * rounded quotient by l) at 5 % / 12 % more time forward / adjoint; 0 restores the default. */
int cacti_hip_attention_set_exact(int on);
size_t cacti_hip_attention_stats_bytes(int64_t S, int64_t H);
int cacti_hip_attention_fwd(int64_t S, int64_t H, int64_t Dh, float alpha, const void *q, const void *k,
                            const void *v, int64_t ld, void *o, void *stats, void *stream);
size_t cacti_hip_attention_bwd_workspace(int64_t S, int64_t H);
int cacti_hip_attention_bwd(int64_t S, int64_t H, int64_t Dh, float alpha, const void *q, const void *k,
                            const void *v, const void *o, const void *dO, int64_t ld, const void *stats,
                            void *dq, int dq_acc, void *dk, int dk_acc, void *dv, int dv_acc,
                            void *workspace, size_t workspace_bytes, void *stream);

/* Row-causal softmax of the cached forward pass, src/librarium/llama.rs:905-907:
 * P16 = f16(softmax_j(mask(f32(S16)))) with mask j > t + initial_row -> -inf
 * (Cast, RowCausalAttentionMaskFutThunkSpec src/librarium/llama.rs:1052-1112, InnerSoftmax, Cast).
 * s16, p16: [T,H,ld] f16, columns 0 .. C-1 of each row used (C % 8 == 0, ld % 8 == 0, ld >= C);
 * row (t, h) belongs to sequence position t + initial_row.  All C columns of p16 are written
 * (zeros at the masked ones). */
int cacti_hip_row_causal_softmax_fwd(int64_t T, int64_t H, int64_t C, int64_t ld, int64_t initial_row,
                                     const void *s16, void *p16, void *stream);
/* One to four rows through a chain of small thunks and a weight matrix in ONE pass over the
 * weights (decoding), with the rounding points of the separate thunks:
 *   r = x                      or f16(x + x2), which is also stored to sum_out (AddFutThunkSpec)
 *   a = rms_norm(r, w_norm)    as cacti_hip_rms_norm_fwd; skipped (a = r) when w_norm is NULL
 *   C = f16(a B^T)             matmul(false, B, true), src/librarium/llama.rs:857-937
 *   or, with B_mul:  C = f16(f16(silu(f16(a B^T))) * f16(a B_mul^T))   the gate / up pair and
 *                    standard_silu + mul of src/librarium/llama.rs:926-935
 * x, x2, sum_out: [M,K] f16; w_norm: [K]; B, B_mul: [N,K]; C: [M,N]; all contiguous, 16-byte
 * aligned; 1 <= M <= 4, K % 8 == 0, K <= 8192. */
int cacti_hip_rows_norm_matmul_f16(int64_t M, int64_t N, int64_t K, const void *x, const void *x2,
                                   const void *w_norm, float eps, void *sum_out, const void *B,
                                   const void *B_mul, void *C, void *stream);

/* The head of a cached attention block for one to four rows in ONE launch
 * (src/librarium/llama.rs:855-893): a = rms_norm(x or f16(x + x2), w_norm) as above, then
 *   q_rot                = symplectic_embed(f16(a Wq^T))
 *   k_cache_rows        += symplectic_embed(f16(a Wk^T))
 *   v_cache_rows        += f16(a Wv^T)
 * with the rounding points of the separate thunks (product, cos / sin products, their sum, the
 * accumulation into the cache).  x, x2, sum_out, q_rot: [M, H*Dh] f16; Wq, Wk, Wv: [H*Dh, H*Dh];
 * cos16, sin16: rows of the position tables for the M positions ([M, Dh]); k_cache_rows,
 * v_cache_rows: the cache rows of the M positions ([M, H*Dh]).  Dh % 4 == 0, H*Dh <= 8192. */
int cacti_hip_rows_qkv_rope_cache_f16(int64_t M, int64_t H, int64_t Dh, const void *x, const void *x2,
                                      const void *w_norm, float eps, void *sum_out, const void *Wq,
                                      const void *Wk, const void *Wv, const void *cos16, const void *sin16,
                                      void *q_rot, void *k_cache_rows, void *v_cache_rows, void *stream);

/* Attention of T = 1..4 new positions over the key / value cache in three small launches: the chain
 * block_matmul_scale(q, k_cache^T, alpha) -> f32 -> row-causal mask -> softmax -> f16 ->
 * block_matmul(., v_cache) of src/librarium/llama.rs:895-915 with its rounding points (f16 scores
 * and probabilities, fp32 accumulation, one rounding of the output).  q: [T, ldq] f16 with head h
 * at columns h*Dh..; k_cache, v_cache: element (position j, head h, d) at j*ldkv + h*head_stride + d
 * (the reference's [C, H, Dh] layout is ldkv = H*Dh, head_stride = Dh; positions beyond
 * T + initial_row - 1 are not read); out: [T, ldo] f16.  Dh % 4 == 0, Dh <= 100; pointers 8-byte
 * aligned, pitches multiples of 4; C <= 8192.  workspace: cacti_hip_attn_decode_workspace bytes,
 * 16-byte aligned, contents undefined on return. */
size_t cacti_hip_attn_decode_workspace(int64_t T, int64_t H, int64_t Dh, int64_t C);
int cacti_hip_attn_decode_f16(int64_t T, int64_t H, int64_t Dh, int64_t C, int64_t initial_row, float alpha,
                              const void *q, int64_t ldq, const void *k_cache, const void *v_cache,
                              int64_t ldkv, int64_t head_stride, void *out, int64_t ldo, void *workspace,
                              size_t workspace_bytes, void *stream);
/* in_tok[pos] += out_tok[last] (u16): the token generated for the last position appended to the
 * input sequence on the device, src/librarium/llama.rs:958-959. */
int cacti_hip_append_token_u16(void *in_tok, int64_t pos, const void *out_tok, int64_t last, void *stream);

/* LM loss, src/librarium/llama.rs:541-546 on logit16 [N,V] f16, tok [N] u16:
 * prob [N,V] f32 = softmax(f32(logit)) (InnerSoftmax), loss [N] f32
 * (InnerSoftmaxCategoricalNLLFutThunkSpec op.rs:3460-3569), amax [N] u16
 * (InnerArgMaxFutThunkSpec :806-880, first index of the maximum).
 * prob / loss / amax may each be NULL.  status [1] i32 on the device is set to
 * 1 + row if a token id is >= V (the reference asserts, op.rs:3538); it must be
 * zero-initialised by the caller, or NULL to skip the check. */
int cacti_hip_softmax_ce_fwd(int64_t N, int64_t V, const void *logit16, const void *tok,
                             void *prob, void *loss, void *amax, void *status, void *stream);

/* Adjoint: dlogit16 (+)= f16(scale[n] * (softmax(f32(logit)) - one_hot(tok)))
 * (pop_adj op.rs:3555-3568 with InnerOneHot :883-997, Sub :1782, BroadcastMul, Cast).
 * scale [N] f32 is the sink seed (examples/open_llama_3b_train.rs:384). */
int cacti_hip_softmax_ce_bwd(int64_t N, int64_t V, const void *logit16, const void *tok,
                             const void *scale, void *dlogit16, int acc, void *stream);

/* Embedding, OuterSelectFutThunkSpec src/thunk/op.rs:1229-1314: y[s] = W[tok[s]]
 * (bit-exact gather) and its adjoint: dW[v] (+)= sum of dy rows with tok[s] == v,
 * summed in position order with one rounding.  W, dW: [V,D] f16; tok: [S] u16;
 * y, dy: [S,D] f16.  D % 8 == 0.  With acc = 0 rows never selected are zeroed.
 * status as in cacti_hip_softmax_ce_fwd. */
int cacti_hip_embed_fwd(int64_t V, int64_t D, const void *W, int64_t S, const void *tok,
                        void *y, void *status, void *stream);
int cacti_hip_embed_bwd(int64_t V, int64_t D, int64_t S, const void *tok, const void *dy,
                        void *dW, int acc, void *stream);

/* f16 residual add y = a + b (AddFutThunkSpec src/thunk/op.rs:1480-1535); y may alias a or b. */
int cacti_hip_add_f16(int64_t n, const void *a, const void *b, void *y, void *stream);

/* Wave-level reduction self-test: fills out[0..3] (f32, device) with the 64-lane
 * sum and max of lane-dependent values computed two ways (cross-lane DPP path and
 * LDS path).  Returns the kernel launch status only; the caller compares. */
int cacti_hip_selftest_wave_reduce(void *out4, void *stream);

/* ---------------------------------------------------------------------------
 * Numerical-health digests of an f16 tensor of n elements (any shape, contiguous), integer-exact.
 * The reference's training example takes both of every parameter and gradient each cycle
 * (examples/open_llama_3b_train.rs:409-424).
 *
 * nan_count: *count_i64 = number of NaNs (exponent field all ones, mantissa not zero);
 * NanCountFutThunkSpec, src/thunk/op.rs:273-349 (output: i64 scalar).
 * abs_log2_hist8: hist_i64_256[b] = number of elements of class b, where b = 255 for inf and nan,
 * 0 for +-0 and floor(log2 |x|) + 127 otherwise (103..112 subnormal, 113..142 normal);
 * AbsLog2Hist8FutThunkSpec, src/thunk/op.rs:351-441 (output: i64[256]).
 * The outputs are device memory, overwritten; x must be 16-byte aligned. */
int cacti_hip_nan_count_f16(int64_t n, const void *x, void *count_i64, void *stream);
int cacti_hip_abs_log2_hist8_f16(int64_t n, const void *x, void *hist_i64_256, void *stream);

/* Both digests of `count` tensors in one launch and one read of each tensor (the example's loop
 * over all parameters and gradients, examples/open_llama_3b_train.rs:409-424, as one call):
 * out_i64[257 * i + b] = abs_log2_hist8 class b of tensor i, out_i64[257 * i + 256] = its NaN
 * count.  xs[i] (device, 16-byte aligned) holds ns[i] >= 0 f16 elements; xs and ns are host
 * arrays read before the call returns.  out_i64 (count * 257 values) and scratch
 * (cacti_hip_digests_scratch_bytes(count) bytes) are device memory, 8-byte aligned. */
size_t cacti_hip_digests_scratch_bytes(int count);
int cacti_hip_digests_f16_batch(int count, const void *const *xs, const int64_t *ns, void *out_i64,
                                void *scratch, void *stream);

/* ---------------------------------------------------------------------------
 * Optimiser thunks of AdamW32 (src/librarium/adamw.rs:45-60).  They are Initialize-mode thunks:
 * the output is read and overwritten in place.  n elements, contiguous, 16-byte aligned; every
 * f32 operation is rounded on its own, in the order the reference's lambda is written.
 *
 * online_average_scale: v += rate * (src_scale * f32(u) - v); OnlineAverageScaleInitFutThunkSpec,
 *   src/thunk/op.rs:3884-3939 (init_online_average_scale, src/op.rs:950-966).
 * online_average_square_scale: v += rate * ((src_scale * f32(u)) * (src_scale * f32(u)) - v);
 *   OnlineAverageSquareScaleInitFutThunkSpec, src/thunk/op.rs:3941-4002.
 * online_adamw_update: w += signed_lr * (lr_unbias * (u / (sqrt(v) + eps)) + lamda * w);
 *   OnlineAdamWUpdateInitFutThunkSpec, src/thunk/op.rs:4004-4062.
 * cast_f32_f16 / cast_f16_f32: CastFutThunkSpec, src/thunk/op.rs:621-663, as staged by
 *   set_lossy_cast / set_cast (src/op.rs:1085-1135); f32 -> f16 rounds to nearest even. */
int cacti_hip_online_average_scale_f16_f32(int64_t n, const void *src_f16, void *dst_f32,
                                           float src_scale, float rate, void *stream);
int cacti_hip_online_average_square_scale_f16_f32(int64_t n, const void *src_f16, void *dst_f32,
                                                  float src_scale, float rate, void *stream);
int cacti_hip_online_adamw_update_f32(int64_t n, const void *grad1_avg_f32, const void *grad2_avg_f32,
                                      void *master_f32, float signed_lr, float lr_unbias, float lamda,
                                      float eps, void *stream);
int cacti_hip_cast_f32_f16(int64_t n, const void *src_f32, void *dst_f16, void *stream);
int cacti_hip_cast_f16_f32(int64_t n, const void *src_f16, void *dst_f32, void *stream);

/* Host arithmetic of one AdamW32 step (AdamW32::step, src/librarium/adamw.rs:45-60, and
 * init_online_adamw_update32, src/op.rs:984-1023): out7 = {grad_unscale, a1, a2, signed_lr,
 * lr_unbias, lamda, eps * unbias2}, all f32, the powers taken as f32::powi does.  grad_scale <= 0
 * stands for None.  iter_nr <= 0 is CACTI_E_INVALID (the reference panics). */
int cacti_adamw32_scalars(int iter_nr, float grad_scale, float lr, float wd, float a1, float a2,
                          float eps, float *out7);

/* One AdamW32 step of `count` tensors in one launch: for each tensor the three thunks above and the
 * cast of the master weights back to the f16 parameter (the loop of
 * examples/open_llama_3b_train.rs:252-268), each element read and written once; bit-identical to
 * the four separate thunks.  grads (f16, read), avgs, avg2s, masters (f32, updated), params (f16,
 * written), ns (element counts) are host arrays of device pointers / sizes, read before the call
 * returns; scalars7 as cacti_adamw32_scalars fills it; scratch: device memory of
 * cacti_hip_adamw32_scratch_bytes(count) bytes, 8-byte aligned. */
size_t cacti_hip_adamw32_scratch_bytes(int count);
int cacti_hip_adamw32_step_f16_batch(int count, const void *const *grads_f16, void *const *avgs_f32,
                                     void *const *avg2s_f32, void *const *masters_f32,
                                     void *const *params_f16, const int64_t *ns, const float *scalars7,
                                     void *scratch, void *stream);

/* ---------------------------------------------------------------------------
 * bf16 held as raw u16 bit patterns <-> f16 / f32 (what set_lossy_cast stages for a bf16 source,
 * src/op.rs:1112-1135).  n elements, contiguous, 16-byte aligned.
 * bf16_f16: f16(f32 from (u << 16)), round to nearest even, overflow to inf;
 *   RawCastBf16F16FutThunkSpec, src/thunk/op.rs:665-698.
 * bf16_f32: f32 from (u << 16), exact; RawCastBf16F32FutThunkSpec, src/thunk/op.rs:700-733.
 * f32_bf16: upper 16 bits of the f32 (truncation); RawCastF32Bf16FutThunkSpec, src/thunk/op.rs:735-768.
 * f16_bf16: upper 16 bits of f32(x); RawCastF16Bf16FutThunkSpec, src/thunk/op.rs:770-803. */
int cacti_hip_raw_cast_bf16_f16(int64_t n, const void *src_u16, void *dst_f16, void *stream);
int cacti_hip_raw_cast_bf16_f32(int64_t n, const void *src_u16, void *dst_f32, void *stream);
int cacti_hip_raw_cast_f32_bf16(int64_t n, const void *src_f32, void *dst_u16, void *stream);
int cacti_hip_raw_cast_f16_bf16(int64_t n, const void *src_f16, void *dst_u16, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* CACTI_GPU_HIP_FFI_H */
