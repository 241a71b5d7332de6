"""Host-side handles for the runtime C ABI (include/cacti_hip_runtime.h): the device
context with its capped pool and host spill, the spine calls, and the LLaMA step.

Mirrors the reference's control flow (reset / stage / vadd_vjp / compile / resume /
resume_put, examples/open_llama_3b_train.rs:203-531); arrays cross as numpy.
"""
import ctypes as C

import numpy as np

from . import ffi

DONE, YIELD = 0, 1


class MemPool:
    """The pool's placement policy over a plain offset range (no GPU involved)."""

    def __init__(self, cap):
        self._p = C.c_void_p()
        ffi.call("cacti_mempool_create", C.byref(self._p), cap)

    def alloc(self, nbytes, high=False):
        """high: packed downwards from the top (cells that live across cycles)."""
        f = ffi.lib().cacti_mempool_alloc_high if high else ffi.lib().cacti_mempool_alloc
        off = f(self._p, nbytes)
        return None if off == 2 ** 64 - 1 else off

    def free(self, off):
        ffi.call("cacti_mempool_free", self._p, off)

    def stats(self):
        out = (C.c_uint64 * 5)()
        ffi.call("cacti_mempool_stats", self._p, out)
        return dict(zip(("cap", "used", "peak", "front", "largest_free"), list(out)))

    def __del__(self):
        if getattr(self, "_p", None):
            ffi.lib().cacti_mempool_destroy(self._p)
            self._p = None


class Ctx:
    def __init__(self, dev=0, pool_bytes=0, host_pagelocked=True):
        self._c = C.c_void_p()
        self.operand_bytes = {}   # label -> operand bytes of one launch (filled by timing_report)
        ffi.call("cacti_ctx_create", C.byref(self._c), dev, pool_bytes, int(host_pagelocked))

    def close(self):
        if self._c:
            ffi.lib().cacti_ctx_destroy(self._c)
            self._c = None

    def __del__(self):
        self.close()

    def stats(self):
        s = ffi.Stats()
        ffi.call("cacti_ctx_stats", self._c, C.byref(s))
        return {n: getattr(s, n) for n, _ in ffi.Stats._fields_}

    def usage_report(self):
        buf = C.create_string_buffer(4096)
        ffi.call("cacti_ctx_usage_report", self._c, buf, C.c_size_t(len(buf)))
        return buf.value.decode()

    def sync(self):
        ffi.call("cacti_ctx_sync", self._c)

    @property
    def stream(self):
        return ffi.lib().cacti_ctx_stream(self._c)

    def set_timing(self, mode):
        """0 off (clears totals), 1 sync per thunk, 2 event pairs without syncing."""
        ffi.call("cacti_ctx_set_timing", self._c, int(mode))

    def set_timing_filter(self, prefix, every=1):
        """Mode 2 then times only every `every`-th launch whose label starts with prefix
        ('' = all labels)."""
        ffi.call("cacti_ctx_set_timing_filter", self._c, (prefix or "").encode(), int(every))

    def timing_report(self):
        buf = C.create_string_buffer(1 << 18)
        ffi.call("cacti_ctx_timing_report", self._c, buf, len(buf))
        out = {}
        for line in buf.value.decode().splitlines():
            name, cnt, ms, nbytes = line.rsplit(" ", 3)
            out[name] = (int(cnt), float(ms))
            self.operand_bytes[name] = int(nbytes)
        return out

    # ---- spine
    def reset(self):
        ffi.call("cacti_reset", self._c)

    def compile(self):
        ffi.call("cacti_compile", self._c)

    def resume(self):
        """Returns (DONE, None) or (YIELD, cell)."""
        y = C.c_int(0)
        rc = ffi.lib().cacti_resume(self._c, C.byref(y))
        if rc < 0:
            ffi.check(rc)
        return (rc, y.value if rc == YIELD else None)

    def resume_put(self, cell, arr):
        arr = np.ascontiguousarray(arr)
        ffi.call("cacti_resume_put", self._c, cell, arr.ctypes.data, arr.nbytes)

    def cell_get(self, cell, dtype, shape):
        out = np.empty(shape, dtype)
        ffi.call("cacti_cell_get", self._c, cell, out.ctypes.data, out.nbytes)
        return out

    def log_names(self):
        n = ffi.lib().cacti_log_len(self._c)
        return [ffi.lib().cacti_log_name(self._c, i).decode() for i in range(n)]


class Llama:
    """Llama::{from, apply} + the training cycle (src/librarium/llama.rs:223-548)."""

    def __init__(self, ctx, S, D, H, Dh, F, V, L, eps=1e-6):
        self.ctx = ctx
        self.cfg = ffi.LlamaCfg(S, D, H, Dh, F, V, L, eps)
        self._m = C.c_void_p()
        ffi.call("cacti_llama_create", ctx._c, C.byref(self.cfg), C.byref(self._m))
        self.params = []          # (name, shape)
        for i in range(ffi.lib().cacti_llama_num_params(self._m)):
            name = C.create_string_buffer(64)
            r, c = C.c_int64(), C.c_int64()
            ffi.call("cacti_llama_param_info", self._m, i, name, 64, C.byref(r), C.byref(c), None,
                     None)
            shape = (r.value,) if name.value.endswith(b"norm") else (r.value, c.value)
            self.params.append((name.value.decode(), shape))

    def close(self):
        if self._m:
            ffi.lib().cacti_llama_destroy(self._m)
            self._m = None

    def set_attention(self, mode):
        """"fused" (default): one thunk per layer, nothing of size S x S stored; "thunks": the reference's
        chain of separate thunks."""
        ffi.call("cacti_llama_set_attention", self._m, {"fused": 0, "thunks": 1}[mode])

    def set_product_groups(self, on):
        """0: one matmul thunk per product; 1 (default): the up and gate projections of a layer as one thunk and
        launch; 2: also q, k, v, and the weight gradients of both groups.  Bit-identical results."""
        ffi.call("cacti_llama_set_product_groups", self._m, int(on))

    def put_param(self, i, arr):
        arr = np.ascontiguousarray(arr, dtype=np.float16)
        assert arr.shape == self.params[i][1], (arr.shape, self.params[i])
        ffi.call("cacti_llama_param_put", self._m, i, arr.ctypes.data, arr.nbytes)

    def put_params_flat(self, flat):
        o = 0
        for i, (_, shp) in enumerate(self.params):
            n = int(np.prod(shp))
            self.put_param(i, flat[o:o + n].reshape(shp))
            o += n
        assert o == flat.size

    def grad(self, i):
        out = np.empty(self.params[i][1], np.float16)
        ffi.call("cacti_llama_grad_get", self._m, i, out.ctypes.data, out.nbytes)
        return out

    def grads(self):
        return {name: self.grad(i) for i, (name, _) in enumerate(self.params)}

    def digests(self, of_grads=False):
        """(hist int64 [num_params, 256], nan int64 [num_params]) of every parameter or gradient:
        abs_log2_hist8 and nan_count as the reference's example takes them each cycle
        (examples/open_llama_3b_train.rs:409-424)."""
        n = len(self.params)
        hist, nan = np.zeros((n, 256), np.int64), np.zeros(n, np.int64)
        ffi.call("cacti_llama_digests", self._m, int(of_grads), hist.ctypes.data, nan.ctypes.data)
        return hist, nan

    def param(self, i):
        """Current value of parameter i (f16), read back from its cell."""
        cell = C.c_int(0)
        ffi.call("cacti_llama_param_info", self._m, i, None, 0, None, None, C.byref(cell), None)
        return self.ctx.cell_get(cell.value, np.float16, self.params[i][1])

    def load_tensors_dir(self, tensors_dir):
        """Stores every tensor of an open ingest.TensorsDir or ingest.PickleDir that Llama::match_pickle_dir's rules match
        into its parameter (src/librarium/llama.rs:284-302); returns how many were matched."""
        n = C.c_int(0)
        ffi.call("cacti_llama_load_tensors_dir", self._m, tensors_dir._d, C.byref(n))
        return n.value

    def adamw_init(self):
        """master = set_cast(param), grad_avg = grad2_avg = 0 (examples/open_llama_3b_train.rs:230-243)."""
        ffi.call("cacti_llama_adamw_init", self._m)

    def adamw_step(self, iter_nr, grad_scale=None, lr=1e-3, wd=0.0, a1=0.1, a2=1e-3, eps=1e-8, skip_embed=False):
        """One AdamW32 step of every parameter from its current gradient, then the cast of the master
        weights back to f16 (examples/open_llama_3b_train.rs:252-268; defaults: AdamW32::default)."""
        opt = ffi.AdamW32(grad_scale or 0.0, lr, wd, a1, a2, eps)
        ffi.call("cacti_llama_adamw_step", self._m, int(iter_nr), C.byref(opt), int(skip_embed))

    def adamw_state(self, i, which):
        """master / grad_avg / grad2_avg (f32) of parameter i."""
        out = np.empty(self.params[i][1], np.float32)
        ffi.call("cacti_llama_adamw_state_get", self._m, i, ("master", "grad_avg", "grad2_avg").index(which),
                 out.ctypes.data, out.nbytes)
        return out

    def io_cells(self):
        v = [C.c_int(0) for _ in range(7)]
        ffi.call("cacti_llama_io_cells", self._m, *[C.byref(x) for x in v])
        return dict(zip(("tok", "lm_tok", "loss_scale", "logit", "loss", "amax", "prob"),
                        [x.value for x in v]))

    def stage(self, want_prob=False, want_grad=True):
        ffi.call("cacti_llama_stage", self._m, int(want_prob), int(want_grad))

    def step(self, tok, lm_tok, loss_scale, want_prob=False, want_grad=True, want_loss=True, accumulate=False):
        """One fwd + loss + bwd cycle; returns the per-position loss (f32 [S]) or None.  accumulate:
        the gradients are cached first (g.cache(), examples/open_llama_3b_train.rs:334-345), so this
        cycle's gradients add to the ones held."""
        tok = np.ascontiguousarray(tok, dtype=np.uint16)
        lm_tok = np.ascontiguousarray(lm_tok, dtype=np.uint16)
        loss_scale = np.ascontiguousarray(loss_scale, dtype=np.float32)
        S = self.cfg.S
        assert tok.size == S and lm_tok.size == S and loss_scale.size == S
        loss = np.empty(S, np.float32) if want_loss else None
        ffi.call("cacti_llama_step", self._m, tok.ctypes.data, lm_tok.ctypes.data,
                 loss_scale.ctypes.data, int(want_prob), 2 if (want_grad and accumulate) else int(want_grad),
                 loss.ctypes.data if want_loss else None)
        return loss

    def step_explicit(self, tok, lm_tok, loss_scale, want_prob=False, want_grad=True):
        """The same cycle driven call by call, as the reference's example drives the spine."""
        c = self.ctx
        c.reset()
        self.stage(want_prob, want_grad)
        c.compile()
        io = self.io_cells()
        feed = {io["tok"]: np.asarray(tok, np.uint16), io["lm_tok"]: np.asarray(lm_tok, np.uint16),
                io["loss_scale"]: np.asarray(loss_scale, np.float32)}
        while True:
            rc, cell = c.resume()
            if rc == DONE:
                break
            c.resume_put(cell, feed[cell])
        S, V = self.cfg.S, self.cfg.V
        out = dict(loss=c.cell_get(io["loss"], np.float32, (S,)),
                   logit=c.cell_get(io["logit"], np.float16, (S, V)),
                   amax=c.cell_get(io["amax"], np.uint16, (S,)))
        if want_prob:
            out["prob"] = c.cell_get(io["prob"], np.float32, (S, V))
        return out


class LlamaCached:
    """LlamaCached (src/librarium/llama.rs:561-963) on the parameters of a Llama: incremental forward
    passes over a key / value cache."""

    def __init__(self, model, seq_cap):
        self.model = model
        self.cap = int(seq_cap)
        self._k = C.c_void_p()
        ffi.call("cacti_llama_cached_create", model._m, self.cap, C.byref(self._k))
        self._rows, self._prob = 0, False

    def close(self):
        if self._k:
            ffi.lib().cacti_llama_cached_destroy(self._k)
            self._k = None

    def reset_state(self):
        ffi.call("cacti_llama_cached_reset_state", self._k)

    def set_tokens(self, tok):
        tok = np.ascontiguousarray(tok, dtype=np.uint16)
        ffi.call("cacti_llama_cached_set_tokens", self._k, tok.ctypes.data, tok.size)

    def tokens(self):
        out = np.empty(self.cap, np.uint16)
        ffi.call("cacti_llama_cached_get_tokens", self._k, out.ctypes.data)
        return out

    def apply(self, prev, next_, want_prob=False):
        """Queues positions prev .. next_-1; read the results with outputs()."""
        ffi.call("cacti_llama_cached_apply", self._k, int(prev), int(next_), int(want_prob))
        self._rows, self._prob = int(next_) - int(prev), bool(want_prob)

    def outputs(self, want_logit=True):
        """dict(logit [T,V] f16 or None, tok [T] u16, prob [T,V] f32 or None) of the last apply."""
        T, V = self._rows, self.model.cfg.V
        logit = np.empty((T, V), np.float16) if want_logit else None
        prob = np.empty((T, V), np.float32) if self._prob else None
        tok = np.empty(T, np.uint16)
        ffi.call("cacti_llama_cached_outputs", self._k, logit.ctypes.data if want_logit else None,
                 prob.ctypes.data if self._prob else None, tok.ctypes.data)
        return dict(logit=logit, tok=tok, prob=prob)

