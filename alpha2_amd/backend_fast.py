"""`FastHipBackend`: the same `Backend` interface as `HipBackend` (packages/core/src/interfaces.ts:38-151), with the fast mode
kept entirely behind it -- callers still see "f32" TensorData (the reference's Dtype has no bf16, packages/core/src/types.ts:6)
and still issue one call per op, as the reference's tape-driven trainer does (packages/autograd/src/ops.ts:197-234,426-487;
packages/train/src/trainer.ts:1188-1273,1761-1784).  Behind the interface:

  * activations that only feed matrix products are STORED as bf16 (LayerNorm outputs, linear-layer outputs, attention
    outputs, their gradients); the residual stream, parameters, gradients of parameters and optimizer state stay f32;
  * every 2-D parameter has a bf16 shadow that `adamwStep` refreshes in the same pass (the MFMA operand of the next step);
  * a linear layer's product is held back by ONE call, so that the op the reference issues next can become its epilogue:
        gelu(matmulTransposed(x, W))                   -> AH_EPI_GELU_GRAD (ops.ts:426-487 issues exactly these two calls): the
                                                          launch saves gelu'(pre) and leaves pre itself as a recipe
        geluBackward(pre, matmul(g, W))                -> AH_EPI_MUL_AUX with that derivative (AH_EPI_GELU_BWD from a written pre)
        add(x, reshape(matmulTransposed(h, W)))        -> AH_EPI_RESIDUAL  (gpt.ts:280-281,331-332 via residualDropoutAdd)
    anything else that touches the held-back product simply launches it as it is;
  * weight gradients dW = G^T X (matmulTransposedA) are held back until something reads one of them (in the trainer: the
    gradient norm), then computed by ONE grouped launch over all of them, accumulating straight into an existing gradient
    when the tape's addInplace asked for that;
  * clone() is copy-on-write (the tape clones every first gradient, tape.ts:126).

Everything not named here runs the inherited f32 kernels after an on-the-fly cast, so the whole interface keeps working.
"""
from __future__ import annotations

import ctypes as C
from typing import List, Optional, Sequence

import numpy as np

from . import _ffi as ffi
from ._ffi import check
from .backend import HipBackend, TensorData, _Buf, shapeSize

BF16, F32 = ffi.BF16, ffi.F32


class _HeldGemm:
    """A product whose launch is held back by one call.  It holds a reference on its operands' buffers and on its output
    buffer until it is launched (or dropped, when nobody but this record still refers to the output)."""
    __slots__ = ("layout", "a_ptr", "b_ptr", "out_buf", "out_off", "m", "n", "k", "lda", "ldb", "holds", "a_planes", "gelu_grad")

    def __init__(self, layout, a_ptr, b_ptr, out, m, n, k, lda, ldb, holds):
        self.layout, self.a_ptr, self.b_ptr, self.out_buf, self.out_off = layout, a_ptr, b_ptr, out._buf, out._off
        self.m, self.n, self.k, self.lda, self.ldb, self.holds = m, n, k, lda, ldb, holds
        # A lies in planes (an unwritten sum of scatterSlice results): (columns per plane, elements from plane to plane), a_ptr
        # the first plane, lda its row stride
        self.a_planes = None
        # gelu was asked of this product: its derivative at the product's values, saved by the launch that made the activation
        # (a buffer of the record's own, released with it); the product itself was not written
        self.gelu_grad = None

    @property
    def out_ptr(self) -> int:
        return self.out_buf.ptr + self.out_off


class _HeldWeightGrad:
    __slots__ = ("g_ptr", "x_ptr", "out_buf", "out_off", "m", "n", "k", "holds", "into", "add_after", "planes", "dst")

    def __init__(self, g_ptr, x_ptr, out, m, n, k, holds):
        self.g_ptr, self.x_ptr, self.out_buf, self.out_off, self.m, self.n, self.k, self.holds = g_ptr, x_ptr, out._buf, out._off, m, n, k, holds
        self.planes = None                # G lies in planes: (columns per plane, bytes from plane to plane); one problem per plane
        self.dst = None                   # set at launch: where the product (all of its problems) is written
        self.into = None                  # (buffer, offset) of an existing gradient to accumulate into instead
        self.add_after = None             # set at launch: the same, when the product had to be computed into its own tensor


class _HeldLayerNormBwd:
    """A layerNormBackward that has been asked for and not launched yet.  The tape's next call usually adds its dx to the gradient
    already flowing along the residual stream (tape.ts:116-127): that gradient then becomes the kernel's own residual input
    and the sum costs no pass of its own."""

    def __init__(self, x_ptr, w_ptr, g_ptr, dx, dw, db, rows, dim, eps, holds):
        self.x_ptr, self.w_ptr, self.g_ptr = x_ptr, w_ptr, g_ptr
        self.outs = (dx._buf, dw._buf, db._buf)
        self.rows, self.dim, self.eps, self.holds = rows, dim, eps, holds


class _HeldCrossEntropy:
    """A crossEntropy that has been asked for and not launched: if the next call on its logits is crossEntropyBackward (the
    last entry of the tape is the first one its backward pass visits, tape.ts:60-157), loss and gradient come out of one pass
    over the logits instead of two."""

    def __init__(self, logits_ptr, targets_ptr, logits_buf, out, lse, n, c, holds):
        self.logits_ptr, self.targets_ptr, self.logits_buf = logits_ptr, targets_ptr, logits_buf
        self.out, self.out_buf, self.lse_buf = out, out._buf, lse._buf      # (the tensor itself only to hand it its read-back ticket)
        self.n, self.c, self.holds = n, c, holds


class _HeldScatter:
    """scatterSlice results that have been asked for and not written: column blocks of a [rows, cols] bf16 matrix that is zero
    elsewhere.  The tape adds the three blocks of d(qkv) to one another (ops.ts:816-858, tape.ts:116-127): sums of held scatters
    with disjoint columns are merged, and the matrix is written once, each block copied to its place."""

    def __init__(self, rows, cols, parts, srcs, out):
        self.rows, self.cols = rows, cols
        self.parts = parts                  # [(source address, first column, width)]
        self.srcs, self.out = srcs, out     # held buffers: the sources, the (unwritten) result

    def disjoint(self, other) -> bool:
        return all(c0 + w <= d0 or d0 + v <= c0 for _, c0, w in self.parts for _, d0, v in other.parts)


class _HeldFlash:
    """A flashAttention that has been asked for and not launched (gpt.ts:247-254 reshapes its result to [B, H, T, D] and
    transposes (1, 2) next: launched from that transpose, the kernel writes the transposed layout itself through its output
    strides).  Afterwards the record says where the result lies: `twin` = (buffer, B, H) of the [B, T, H, D] copy while the
    [B H, T, D] tensor the caller holds is still unwritten (it is written from the twin if anybody reads it)."""
    __slots__ = ("q", "k", "v", "o_buf", "lse_buf", "BH", "T", "D", "scale", "cap", "holds", "twin", "launched")

    def __init__(self, q, k, v, o_buf, lse_buf, BH, T, D, scale, cap, holds):
        self.q, self.k, self.v, self.o_buf, self.lse_buf, self.BH, self.T, self.D = q, k, v, o_buf, lse_buf, BH, T, D
        self.scale, self.cap, self.holds, self.twin, self.launched = scale, cap, holds, None, False


class _LazyTranspose:
    """transpose(1, 2) of a 4-D bf16 tensor that has been asked for and not written: in the backward pass of the slab wiring its
    consumer is flashAttentionBackward, which reads the source through strides instead."""
    __slots__ = ("src_ptr", "src_shape", "out_buf", "holds")

    def __init__(self, src_ptr, src_shape, out_buf, holds):
        self.src_ptr, self.src_shape, self.out_buf, self.holds = src_ptr, tuple(src_shape), out_buf, holds


class FastHipBackend(HipBackend):
    name = "hip"

    def __init__(self, device: int = 0, group_weight_grads: bool = True, stream_bf16: bool = True, gelu_saves_derivative: bool = True):
        super().__init__(device)
        # gelu of a held-back product saves gelu'(pre) for the backward product's epilogue (one multiply per element there); False:
        # it saves the pre-activation itself, as the reference's matmulTransposedGelu contract reads, and backward evaluates gelu'
        self.geluSavesDerivative = gelu_saves_derivative
        # the residual stream (the running sum the residual adds produce) and the gradient flowing back along it are stored in
        # bf16 like every other activation; False keeps both in f32
        self.streamBf16 = stream_bf16
        self._held: Optional[_HeldGemm] = None
        self._wgrads: List[_HeldWeightGrad] = []
        self._wq_out, self._wq_into = set(), set()   # id(_Buf) of the queued gradients' results / of the tensors they will be added into
        self._group = group_weight_grads
        self._plans = {}                 # (epilogue, shapes) -> grouped plan id
        # products that became another op's epilogue and were never written themselves: computed only if somebody reads them
        self._orphans = {}               # id(_Buf) -> _HeldGemm
        # adamwStep calls of one optimizer pass, launched together (one kernel per 48 tensors) when anything needs their result
        self._adam_q: List[tuple] = []   # (p, g, m, v, shadow, n, weight decay) as device addresses
        self._adam_key = None
        self._adam_flush_at = 1
        self._adam_holds: List[_Buf] = []
        self._adam_bufs = set()          # id(_Buf) of every buffer a queued update reads or writes
        self._ssq_args = None            # (addresses, sizes, their ctypes arrays) of the last totalSumOfSquares call
        self._scatters = {}              # id(_Buf) of an unwritten scatterSlice result -> _HeldScatter
        self._planes_ok = {}             # (layout, m, n, k, plane extents) -> does ah_gemm_planes take it
        # unwritten results whose making is still open: id(_Buf) -> _HeldFlash (under its output's and its LSE's buffer) or _LazyTranspose
        self._lazy = {}
        self._pending_flash: Optional[_HeldFlash] = None
        self._held_ce: Optional[_HeldCrossEntropy] = None
        self._held_ln: Optional[_HeldLayerNormBwd] = None
        # dx tensors whose LayerNorm backward went straight into a sum and that were never written themselves: id(_Buf) -> recipe
        self._ln_unwritten = {}

    # ------------------------------------------------------------------ storage helpers
    def _hold(self, *bufs):
        for b in bufs:
            b.refs += 1
        return list(bufs)

    def _unhold(self, holds):
        for b in holds:
            b.release()

    def _is_held(self, t: TensorData) -> bool:
        h = self._held
        return h is not None and t._buf is h.out_buf

    def _is_queued(self, buf) -> bool:
        return id(buf) in self._wq_out

    def _ptr(self, t: TensorData) -> int:
        if not t._dev_valid and t._buf is not None:
            t._shadow = None                                    # the host wrote new contents: the bf16 shadow is stale
        if self._adam_q and t._buf is not None and id(t._buf) in self._adam_bufs:
            self._flush_adam()
        if t._buf is not None:
            if self._held_ln is not None and any(t._buf is b for b in self._held_ln.holds):
                self._launch_ln()
            elif self._ln_unwritten and id(t._buf) in self._ln_unwritten:
                h = self._ln_unwritten.pop(id(t._buf))           # somebody reads the dx that only ever existed inside a sum
                scratch = _Buf(self.lib, 8 * h.dim)
                check(self.lib.ah_layernorm_bwd(h.x_ptr, h.w_ptr, h.g_ptr, BF16, 0, 0, h.outs[0].ptr, scratch.ptr, scratch.ptr + 4 * h.dim,
                                                h.rows, h.dim, h.eps, 0, BF16))
                scratch.release()
                self._unhold(h.holds)
            if self._scatters and id(t._buf) in self._scatters:
                self._write_scatter(t._buf)
            if self._lazy and id(t._buf) in self._lazy:
                self._materialise(t._buf)
            if self._held_ce is not None and any(t._buf is b for b in self._held_ce.holds):
                self._launch_ce()
            if self._held is not None and t._buf is self._held.out_buf:
                self._launch_held()
            elif self._wgrads and (id(t._buf) in self._wq_out or id(t._buf) in self._wq_into):
                self._launch_weight_grads()
            elif self._orphans and id(t._buf) in self._orphans:
                h = self._orphans.pop(id(t._buf))
                self._run_held(h, h.out_ptr)
                self._unhold(h.holds)
        return super()._ptr(t)

    def _download(self, t: TensorData):
        tk = getattr(t, "_early", None)
        if tk:                                                  # its copy to the host was started when it was computed
            t._early = None
            out = np.empty(1, dtype=np.float32)
            if t._dev_valid and t.store == "f32" and t.size == 1 and self.lib.ah_download_end(tk, out.ctypes.data_as(C.c_void_p), 4) == 0:
                return out
        self._ptr(t)
        # the host is about to wait for the device: whatever is queued and will be needed anyway (the weight gradients once
        # backward has been issued) goes out first, so the device has work while the host reads and carries on
        self._launch_weight_grads()
        return super()._download(t)

    def _f32(self, *ts):
        """Ops inherited from HipBackend take f32 storage: a bf16-stored operand gets an f32 copy of its own."""
        for t in ts:
            if t.dtype != "f32":
                raise TypeError(f"op expects f32 tensors, got {t.dtype}")
            if t.store == "bf16":
                src = self._ptr(t)
                buf = _Buf(self.lib, t.size * 4)
                check(self.lib.ah_cast(src, BF16, buf.ptr, F32, t.size))
                t._buf.release()
                t._buf, t._off, t.store = buf, 0, "f32"

    def _words(self, *ts):
        """Inherited data-movement kernels copy 4-byte elements: a bf16-stored tensor gets f32 storage first."""
        self._f32(*[t for t in ts if t.store == "bf16"])

    def _dirty(self, t: TensorData):
        super()._dirty(t)
        t._shadow = None
        t._early = None

    # ---- data movement on bf16 storage.  The kernels behind slice / transpose / scatter copy 4-byte words and never look
    # inside them, so a bf16 tensor whose innermost dimension is even and is left whole (or cut at even columns) is moved as
    # the tensor of half that width: q, k, v and the head transposes of the reference's attention branch (gpt.ts:232-253) stay
    # in bf16 instead of being widened to f32 first.
    def _takes_planes(self, layout, m, n, k, lda, ldb, ldc, c_planes=(0, 0), a_planes=(0, 0)) -> bool:
        key = (layout, m, n, k, lda, ldb, ldc, c_planes, a_planes)
        ok = self._planes_ok.get(key)
        if ok is None:                                          # asked once per shape: nothing is launched
            g = ffi.AhGemm(layout, BF16, BF16, ffi.EPI_NONE, m, n, k, lda, ldb, ldc, 1, 0, 0, 0, 256, 256, 256, 0)
            ok = self._planes_ok[key] = self.lib.ah_gemm_planes(C.byref(g), *c_planes, *a_planes, 1) == 0
        return ok

    def _plane_views(self, count: int, shape) -> list:
        """`count` bf16 tensors of one shape that lie one behind the other in one allocation."""
        n = shapeSize(shape)
        buf = _Buf(self.lib, count * n * 2)
        buf.refs = count
        out = []
        for p in range(count):
            v = TensorData(shape, "f32")
            v.store, v._buf, v._off, v._dev_valid, v._backend = "bf16", buf, p * n * 2, True, self
            out.append(v)
        return out

    def sliceQkv(self, a: TensorData):
        rows, c3 = a.shape
        d = c3 // 3
        if a.store != "bf16" or d % 2 or c3 != 3 * d:
            return super().sliceQkv(a)
        h = self._held
        if h is not None and a._buf is h.out_buf and a._off == h.out_off and h.layout == ffi.GEMM_NT and h.a_planes is None \
                and (h.m, h.n) == (rows, c3) and self._takes_planes(ffi.GEMM_NT, h.m, h.n, h.k, h.lda, h.ldb, d, c_planes=(d, rows * d)):
            # the projection is still to be launched: it writes q, k and v as three matrices itself (ah_gemm_planes)
            self._held = None
            q, k, v = self._plane_views(3, (rows, d))
            self._gemm(ffi.GEMM_NT, h.a_ptr, h.b_ptr, q._buf.ptr, h.m, h.n, h.k, h.lda, h.ldb, d, in_dtype=BF16, out_dtype=BF16,
                       planes=(d, rows * d, 0, 0))
            if h.out_buf.refs > 1:
                self._orphans[id(h.out_buf)] = h                # the [rows, 3d] product itself was not written: keep the recipe
            else:
                self._unhold(h.holds)
            return [q, k, v]
        q, k, v = (self._new((rows, d), "f32", "bf16") for _ in range(3))
        check(self.lib.ah_slice_qkv(self._ptr(a), q._buf.ptr, k._buf.ptr, v._buf.ptr, rows, d // 2))
        return [q, k, v]

    def transpose(self, a: TensorData, dim0: int, dim1: int) -> TensorData:
        nd = len(a.shape)
        d0, d1 = self._axis(dim0, nd), self._axis(dim1, nd)
        if a.store != "bf16" or nd < 3 or nd - 1 in (d0, d1) or a.shape[-1] % 2:
            return super().transpose(a, dim0, dim1)
        ns = list(a.shape)
        ns[d0], ns[d1] = a.shape[d1], a.shape[d0]
        if nd == 4 and (d0, d1) == (1, 2) and a._buf is not None and a._dev_valid and a.size > 0:
            rec = self._lazy.get(id(a._buf))
            if isinstance(rec, _HeldFlash) and not rec.launched and a._buf is rec.o_buf and a._off == 0 \
                    and a.shape[0] * a.shape[1] == rec.BH and (a.shape[2], a.shape[3]) == (rec.T, rec.D):
                out = self._new(ns, a.dtype, "bf16")            # the attention kernel writes [B, T, H, D] itself
                self._launch_flash(rec, twin=(out._buf, a.shape[0], a.shape[1]))
                return out
            src = self._ptr(a)                                  # (whatever still has to produce `a` runs now)
            out = self._new(ns, a.dtype, "bf16")
            self._lazy[id(out._buf)] = _LazyTranspose(src, a.shape, out._buf, self._hold(a._buf, out._buf))
            return out
        half = list(a.shape)
        half[-1] //= 2
        out = self._new(ns, a.dtype, "bf16")
        check(self.lib.ah_transpose(self._ptr(a), out._buf.ptr, nd, ffi.shape_arr(half), d0, d1))
        return out

    def slice(self, a: TensorData, starts, ends) -> TensorData:
        if a.store != "bf16" or not a.shape or a.shape[-1] % 2 or starts[-1] % 2 or ends[-1] % 2:
            return super().slice(a, starts, ends)
        halve = lambda xs: list(xs[:-1]) + [xs[-1] // 2]
        out = self._new([e - s for s, e in zip(starts, ends)], a.dtype, "bf16")
        check(self.lib.ah_slice(self._ptr(a), out._buf.ptr, len(a.shape), ffi.shape_arr(halve(a.shape)), ffi.shape_arr(halve(starts)),
                                ffi.shape_arr(halve(ends))))
        return out

    def scatterSlice(self, grad: TensorData, origShape, starts, ends) -> TensorData:
        if grad.store != "bf16" or not grad.shape or grad.shape[-1] % 2 or origShape[-1] % 2 or starts[-1] % 2:
            return super().scatterSlice(grad, origShape, starts, ends)
        if len(origShape) == 2 and len(grad.shape) == 2 and starts[0] == 0 and grad.shape[0] == origShape[0] and grad.size > 0 \
                and starts[1] + grad.shape[1] <= origShape[1]:
            gp = self._ptr(grad)                                # a column block of whole rows: held back
            out = self._new(origShape, grad.dtype, "bf16")
            grad._buf.refs += 1
            out._buf.refs += 1
            self._scatters[id(out._buf)] = _HeldScatter(origShape[0], origShape[1], [(gp, starts[1], grad.shape[1])], [grad._buf], out._buf)
            return out
        halve = lambda xs: list(xs[:-1]) + [xs[-1] // 2]
        out = self._new(origShape, grad.dtype, "bf16")
        check(self.lib.ah_scatter_slice(self._ptr(grad), out._buf.ptr, len(origShape), ffi.shape_arr(halve(grad.shape)),
                                        ffi.shape_arr(halve(origShape)), ffi.shape_arr(halve(starts))))
        return out

    def _write_scatter(self, buf):
        h = self._scatters.pop(id(buf))
        parts = sorted(h.parts, key=lambda p: p[1])
        dst = ffi.shape_arr([h.rows, h.cols // 2])
        covered = parts[0][1] == 0 and parts[-1][1] + parts[-1][2] == h.cols and all(a[1] + a[2] == b[1] for a, b in zip(parts, parts[1:]))
        for i, (src, c0, w) in enumerate(parts):
            blk = ffi.shape_arr([h.rows, w // 2])
            if i == 0 and not covered:                          # the first block brings the zeros of everything that is no block
                check(self.lib.ah_scatter_slice(src, buf.ptr, 2, blk, dst, ffi.shape_arr([0, c0 // 2])))
            else:
                check(self.lib.ah_cat_part(src, buf.ptr, 2, blk, dst, 1, c0 // 2))
        self._unhold(h.srcs + [h.out])

    def _drop_scatter(self, buf):
        h = self._scatters.pop(id(buf))
        self._unhold(h.srcs + [h.out])

    def _operand(self, t: TensorData):
        """Device address of `t` as a bf16 matrix operand, and the buffer that must outlive the launch."""
        if t.store == "bf16":
            return self._ptr(t), t._buf
        p = self._ptr(t)
        sh = getattr(t, "_shadow", None)
        if sh is None or sh.ptr == 0:
            sh = _Buf(self.lib, t.size * 2)
            check(self.lib.ah_cast(p, F32, sh.ptr, BF16, t.size))
            t._shadow = sh
        return sh.ptr, sh

    def releaseGpuTensor(self, t: TensorData):
        if t is None or t._buf is None:
            return
        if self._adam_q and id(t._buf) in self._adam_bufs:
            self._flush_adam()
        sh = getattr(t, "_shadow", None)
        if sh is not None:
            sh.release()
            t._shadow = None
        buf = t._buf
        super().releaseGpuTensor(t)
        if buf.refs == 1:                                       # only a held-back record still refers to it: nobody will read it
            if self._held is not None and buf is self._held.out_buf:
                h, self._held = self._held, None
                self._unhold(h.holds)
            elif self._orphans and id(buf) in self._orphans:
                self._unhold(self._orphans.pop(id(buf)).holds)
            elif self._ln_unwritten and id(buf) in self._ln_unwritten:
                self._unhold(self._ln_unwritten.pop(id(buf)).holds)
            elif self._scatters and id(buf) in self._scatters:
                self._drop_scatter(buf)
            elif self._lazy and id(buf) in self._lazy:
                self._drop_lazy(buf)
            elif self._wgrads:
                for i, w in enumerate(self._wgrads):
                    if buf is w.out_buf and w.into is None:
                        del self._wgrads[i]
                        self._wq_out.discard(id(buf))
                        self._unhold(w.holds)
                        break

    def _view(self, t: TensorData, shape, byte_off: int = 0) -> TensorData:
        if t._buf is not None and t._dev_valid and (self._is_held(t) or id(t._buf) in self._orphans or self._is_queued(t._buf)
                                                    or id(t._buf) in self._scatters or id(t._buf) in self._lazy):
            v = TensorData(shape, t.dtype)                      # a view of a held-back product stays held back
            v.store, v._buf, v._off = t.store, t._buf, t._off + byte_off
            t._buf.refs += 1
            v._dev_valid, v._backend = True, self
            return v
        return super()._view(t, shape, byte_off)

    # ------------------------------------------------------------------ held-back linear-layer products
    def _launch_held(self, epilogue=ffi.EPI_NONE, aux: int = 0, out: Optional[TensorData] = None, out_dtype=BF16):
        h, self._held = self._held, None
        if h is None:
            return
        if out is None and h.out_buf.refs == 1:                 # every tensor that named this product has been released
            self._unhold(h.holds)
            return
        dst = h.out_ptr if out is None else out._buf.ptr + out._off
        self._run_held(h, dst, epilogue, aux, out_dtype)
        if out is not None and epilogue != ffi.EPI_GELU and h.out_buf.refs > 1:
            self._orphans[id(h.out_buf)] = h                    # the plain product was not written: keep the recipe
        else:
            self._unhold(h.holds)

    def _run_held(self, h: _HeldGemm, dst: int, epilogue=ffi.EPI_NONE, aux: int = 0, out_dtype=BF16):
        if h.a_planes is not None:
            if epilogue == ffi.EPI_NONE and out_dtype == BF16:
                self._gemm(h.layout, h.a_ptr, h.b_ptr, dst, h.m, h.n, h.k, h.lda, h.ldb, h.n, in_dtype=BF16, out_dtype=BF16,
                           planes=(0, 0) + h.a_planes)
                return
            # an epilogue (or an f32 result) wants A as one matrix: the planes are copied side by side first
            w, step = h.a_planes
            whole = _Buf(self.lib, h.m * h.k * 2)
            for p in range(h.k // w):
                check(self.lib.ah_cat_part(h.a_ptr + p * step * 2, whole.ptr, 2, ffi.shape_arr([h.m, w // 2]), ffi.shape_arr([h.m, h.k // 2]), 1, p * w // 2))
            self._gemm(h.layout, whole.ptr, h.b_ptr, dst, h.m, h.n, h.k, h.k, h.ldb, h.n, in_dtype=BF16, out_dtype=out_dtype,
                       epilogue=epilogue, aux=aux)
            whole.release()                                      # (stream-ordered: reusable only by later work)
            return
        self._gemm(h.layout, h.a_ptr, h.b_ptr, dst, h.m, h.n, h.k, h.lda, h.ldb, h.n, in_dtype=BF16, out_dtype=out_dtype,
                   epilogue=epilogue, aux=aux)

    def _scatter_planes(self, t: TensorData):
        """`t` as an unwritten sum of scatterSlice results (the three parts of d(qkv), ops.ts:826-834) whose sources are equally
        wide, cover every column and lie equally far apart: (first source, columns each, bytes apart, count, record)."""
        if not self._scatters or t._buf is None or t._off != 0 or not t._dev_valid:
            return None
        h = self._scatters.get(id(t._buf))
        if h is None or tuple(t.shape) != (h.rows, h.cols) or not 2 <= len(h.parts) <= 3:
            return None
        parts = sorted(h.parts, key=lambda p: p[1])
        w, step = parts[0][2], parts[1][0] - parts[0][0]
        if any(p[2] != w or p[1] != i * w or p[0] != parts[0][0] + i * step for i, p in enumerate(parts)) or w * len(parts) != h.cols \
                or step <= 0 or step % 16 or parts[0][0] % 16:
            return None
        return parts[0][0], w, step, len(parts), h

    def _hold_gemm(self, layout, a: TensorData, b: TensorData, oshape, m, n, k, lda, ldb) -> TensorData:
        self._launch_held()
        ap, ah = self._operand(a)
        bp, bh = self._operand(b)
        out = self._new(oshape, "f32", "bf16")
        self._held = _HeldGemm(layout, ap, bp, out, m, n, k, lda, ldb, self._hold(ah, bh, out._buf))
        return out

    def matmulTransposed(self, a: TensorData, b: TensorData) -> TensorData:
        if len(a.shape) != 2 or len(b.shape) != 2:
            return super().matmulTransposed(a, b)
        M, K, N = a.shape[0], a.shape[1], b.shape[0]
        if b.shape[1] != K:
            raise ValueError(f"matmul shape mismatch: [{a.shape}] x [{b.shape}]^T")
        if K % 8:                                               # the bf16 kernels contract in 16-byte pieces: such a product runs in f32
            return super().matmulTransposed(a, b)
        return self._hold_gemm(ffi.GEMM_NT, a, b, (M, N), M, N, K, K, K)

    def matmul(self, a: TensorData, b: TensorData) -> TensorData:
        if len(a.shape) != 2 or len(b.shape) != 2:
            return super().matmul(a, b)
        M, K, N = a.shape[0], a.shape[1], b.shape[1]
        if b.shape[0] != K:
            raise ValueError(f"matmul shape mismatch: [{a.shape}] x [{b.shape}]")
        if K % 8:
            return super().matmul(a, b)
        sp = self._scatter_planes(a)
        if sp is not None and self._takes_planes(ffi.GEMM_NN, M, N, K, sp[1], N, N, a_planes=(sp[1], sp[2] // 2)):
            # dX of the fused projection: the three gradients are read where they lie, their sum is never written
            base, w, step, _, rec = sp
            self._launch_held()
            bp, bh = self._operand(b)
            out = self._new((M, N), "f32", "bf16")
            h = _HeldGemm(ffi.GEMM_NN, base, bp, out, M, N, K, w, N, self._hold(*rec.srcs, bh, out._buf))
            h.a_planes = (w, step // 2)
            self._held = h
            return out
        return self._hold_gemm(ffi.GEMM_NN, a, b, (M, N), M, N, K, K, N)

    def gelu(self, a: TensorData) -> TensorData:
        h = self._held
        if self._is_held(a) and h.layout == ffi.GEMM_NT and not self.geluSavesDerivative:
            out = self._new(a.shape, "f32", "bf16")             # `a` receives the pre-activation, as the caller expects
            self._launch_held(ffi.EPI_GELU, aux=a._buf.ptr + a._off, out=out)
            return out
        if self._is_held(a) and h.layout == ffi.GEMM_NT and h.a_planes is None and a._off == h.out_off:
            # One launch gives gelu(product) and gelu'(product); the derivative is what backward needs (geluBackward multiplies
            # by it), so it is what is saved.  `a` itself, the pre-activation the caller may still read (ops.ts:426-487), is not
            # written: the record stays as its recipe and computes it if anybody asks.
            out = self._new(a.shape, "f32", "bf16")
            h.gelu_grad = _Buf(self.lib, a.size * 2)
            h.holds.append(h.gelu_grad)
            self._launch_held(ffi.EPI_GELU_GRAD, aux=h.gelu_grad.ptr, out=out)
            return out
        return super().gelu(a)

    def geluBackward(self, x: TensorData, g: TensorData) -> TensorData:
        rec = self._orphans.get(id(x._buf)) if self._orphans and x._buf is not None else None
        if rec is not None and rec.gelu_grad is not None and self._is_held(g) and x.store == "bf16" and x.shape == g.shape \
                and x._off == rec.out_off and self._held.a_planes is None:
            out = self._new(g.shape, "f32", "bf16")             # g * gelu'(x) with the saved derivative: one multiply per element
            self._launch_held(ffi.EPI_MUL_AUX, aux=rec.gelu_grad.ptr, out=out)
            return out
        if self._is_held(g) and x.store == "bf16" and x.shape == g.shape and not self._is_held(x):
            pre = self._ptr(x)
            out = self._new(g.shape, "f32", "bf16")
            self._launch_held(ffi.EPI_GELU_BWD, aux=pre, out=out)
            return out
        return super().geluBackward(x, g)

    def add(self, a: TensorData, b: TensorData) -> TensorData:
        for res, prod in ((a, b), (b, a)):
            if self._is_held(prod) and res.store in ("f32", "bf16") and tuple(res.shape) == tuple(prod.shape) and res.dtype == "f32" \
                    and not self._is_held(res):
                if self.streamBf16 and res.size % 8 == 0:
                    # the residual stream in bf16, like every other activation: the sum is rounded once, to bf16
                    rp, keep = self._operand(res)
                    out = self._new(res.shape, "f32", "bf16")
                    self._launch_held(ffi.EPI_RESIDUAL, aux=rp, out=out, out_dtype=BF16)
                    del keep
                    return out
                if res.store == "f32":
                    out = self._new(res.shape)
                    rp = self._ptr(res)
                    self._launch_held(ffi.EPI_RESIDUAL, aux=rp, out=out, out_dtype=F32)
                    return out
        if a.store == b.store == "bf16" and tuple(a.shape) == tuple(b.shape):        # e.g. the three scattered parts of d(qkv)
            pa, pb = self._ptr(a), self._ptr(b)
            if (pa | pb) % 16 == 0:
                out = self._new(a.shape, "f32", "bf16")
                check(self.lib.ah_add_bf16(pa, pb, out._buf.ptr, a.size))
                return out
        return super().add(a, b)

    def residualDropoutAdd(self, residual, projected, mask) -> TensorData:
        if mask is None:
            return self.add(residual, projected)
        return super().residualDropoutAdd(residual, projected, mask)

    # ------------------------------------------------------------------ weight gradients, grouped
    def matmulTransposedA(self, a: TensorData, b: TensorData) -> TensorData:
        """A[M,K]^T @ B[M,N] -> [K,N]: in the trainer, dW = G^T X over M = tokens."""
        if len(a.shape) != 2 or len(b.shape) != 2:
            return super().matmulTransposedA(a, b)
        M, K, N = a.shape[0], a.shape[1], b.shape[1]
        if b.shape[0] != M:
            raise ValueError(f"matmul shape mismatch: [{a.shape}]^T x [{b.shape}]")
        if M % 8:                                               # (the contraction runs over the rows here)
            return super().matmulTransposedA(a, b)
        sp = self._scatter_planes(a) if self._group and M % 64 == 0 and N % 8 == 0 else None
        if sp is not None and sp[1] % 8 == 0:
            # dW of the fused projection: one problem of the grouped launch per gradient, each writing its rows of dW
            bp, bh = self._operand(b)
            out = self._new((K, N))
            wg = _HeldWeightGrad(sp[0], bp, out, K, N, M, self._hold(*sp[4].srcs, bh, out._buf))
            wg.planes = (sp[1], sp[2])
            self._wgrads.append(wg)
            self._wq_out.add(id(out._buf))
            return out
        ap, ah = self._operand(a)
        bp, bh = self._operand(b)
        out = self._new((K, N))
        self._wgrads.append(_HeldWeightGrad(ap, bp, out, K, N, M, self._hold(ah, bh, out._buf)))
        self._wq_out.add(id(out._buf))
        if not self._group:
            self._launch_weight_grads()
        return out

    def _launch_weight_grads(self):
        self._run_weight_grads(*self._take_weight_grads())

    def _take_weight_grads(self):
        """Empties the queue: (the queued products, [(epilogue, descriptors, as one grouped launch?)]).  A product that was
        re-targeted to accumulate into an existing gradient (addInplace) while its own tensor is still alive - the tape
        releases it at once, another caller may not - is computed into its own tensor after all, and added from there:
        its entry in ws carries the sum still to be made."""
        ws, self._wgrads = self._wgrads, []
        self._wq_out, self._wq_into = set(), set()
        descs = []
        for w in ws:
            w.add_after, w.dst = None, None
            if w.into is None and w.out_buf.refs == 1:          # released unread
                continue
            if w.into is not None and w.out_buf.refs > 1:       # (the queue's own hold is one reference)
                w.add_after, w.into = w.into, None
            dst, epi = (w.out_buf.ptr + w.out_off, ffi.EPI_NONE) if w.into is None else (w.into[0].ptr + w.into[1], ffi.EPI_ACCUM)
            w.dst = dst
            if w.planes is None:
                descs.append(ffi.AhGemm(ffi.GEMM_TN, BF16, F32, epi, w.m, w.n, w.k, w.m, w.n, w.n, 1, 0, 0, 0, w.g_ptr, w.x_ptr, dst, 0))
            else:
                cols, step = w.planes
                for p in range(w.m // cols):
                    descs.append(ffi.AhGemm(ffi.GEMM_TN, BF16, F32, epi, cols, w.n, w.k, cols, w.n, w.n, 1, 0, 0, 0, w.g_ptr + p * step, w.x_ptr,
                                            dst + p * cols * w.n * 4, 0))
        groupable = all(d.k % 64 == 0 and d.m % 8 == 0 and d.n % 8 == 0 for d in descs)
        parts = []
        for epi in (ffi.EPI_NONE, ffi.EPI_ACCUM):
            part = [d for d in descs if d.epilogue == epi]
            if part:
                parts.append((epi, part, groupable and len(part) > 1))
        return ws, parts

    def _run_weight_grads(self, ws, parts, sumsq: int = 0):
        """Launches them; with sumsq, the grouped launches add the sum of the squares of what they leave to that device float."""
        for epi, part, grouped in parts:
            if grouped:
                # one plan per list of shapes; the gradients are new tensors every step, so its tables are rewritten every time
                # (also when nothing moved: a step plan wants the same launches from every step)
                key = (epi,) + tuple((d.m, d.n, d.k) for d in part)
                plan = self._plans.get(key)
                arr = (ffi.AhGemm * len(part))(*part)
                if plan is None:
                    if len(self._plans) >= 8:
                        for p in self._plans.values():
                            check(self.lib.ah_gemm_grouped_destroy(p))
                        self._plans = {}
                    pid = C.c_uint64()
                    check(self.lib.ah_gemm_grouped_plan(arr, len(part), C.byref(pid)))
                    plan = self._plans[key] = pid.value
                else:
                    check(self.lib.ah_gemm_grouped_update(plan, arr, len(part)))

                def run():
                    if sumsq:
                        check(self.lib.ah_gemm_grouped_run_sumsq(plan, epi, sumsq))
                    else:
                        check(self.lib.ah_gemm_grouped_run(plan, epi))
                timed = getattr(self, "_timed", None)
                if timed is None:
                    run()
                else:
                    e0, e1 = self._event(), self._event()
                    check(self.lib.ah_event_record(e0))
                    run()
                    check(self.lib.ah_event_record(e1))
                    kernel, nsplit = self.lastGemmKernel()
                    timed.append({"kind": "gemm", "kernel": kernel, "nsplit": nsplit, "layout": ffi.GEMM_TN, "dtype": BF16, "m": 0, "n": 0,
                                  "k": part[0].k, "batch": 1, "flops": sum(2.0 * d.m * d.n * d.k for d in part), "e0": e0, "e1": e1})
            else:
                for d in part:
                    check(self.lib.ah_gemm(C.byref(d)))
        for w in ws:
            if w.add_after is not None:
                check(self.lib.ah_add_inplace(w.add_after[0].ptr + w.add_after[1], w.out_buf.ptr + w.out_off, w.m * w.n))
            self._unhold(w.holds)

    def addInplace(self, a: TensorData, b: TensorData):
        if self._wgrads and b._buf is not None and id(b._buf) in self._wq_out:
            for w in self._wgrads:
                if b._buf is w.out_buf and w.into is None and a.store == "f32" and a.size == b.size and a._buf is not None and a._dev_valid \
                        and a._buf.refs == 1 and id(a._buf) not in self._wq_out and id(a._buf) not in self._wq_into \
                        and not any(a._buf is x for x in w.holds):      # (`a` may be an operand of the very product: it cannot be written while it is read)
                    w.into = (a._buf, a._off)                    # the grouped launch adds into `a`; `b` itself is never computed
                    a._buf.refs += 1
                    w.holds.append(a._buf)
                    self._wq_into.add(id(a._buf))
                    self._dirty(a)
                    return
        if self._scatters and a._buf is not None and b._buf is not None and a._buf is not b._buf:
            sa, sb = self._scatters.get(id(a._buf)), self._scatters.get(id(b._buf))
            if sa is not None and sb is not None and a._off == 0 and b._off == 0 and a.size == b.size == sa.rows * sa.cols \
                    and (sa.rows, sa.cols) == (sb.rows, sb.cols) and a._dev_valid and sa.disjoint(sb):
                for x in sb.srcs:
                    x.refs += 1
                if a._buf.refs > 2:                              # (its own name and the record's hold are two) shared with a clone:
                    for x in sa.srcs:                            # the sum gets a buffer and a record of its own
                        x.refs += 1
                    nb = _Buf(self.lib, a.size * 2)
                    nb.refs += 1
                    self._scatters[id(nb)] = _HeldScatter(sa.rows, sa.cols, sa.parts + sb.parts, sa.srcs + sb.srcs, nb)
                    a._buf.release()
                    a._buf = nb
                else:
                    sa.parts = sa.parts + sb.parts
                    sa.srcs = sa.srcs + sb.srcs
                self._dirty(a)
                return
        h = self._held_ln
        if h is not None and b._buf is h.outs[0] and b._off == 0 and b.size == h.rows * h.dim and a.store == "bf16" and a.size == b.size \
                and a._buf is not None and a._dev_valid and not any(a._buf is x for x in h.holds):
            self._launch_held()
            pa = self._ptr(a)
            if self._held_ln is h and pa % 16 == 0:
                buf = _Buf(self.lib, a.size * 2)                 # (never in place: `a` usually shares its buffer with a clone)
                self._launch_ln(residual=pa, dx_ptr=buf.ptr)
                a._buf.release()
                a._buf, a._off = buf, 0
                self._dirty(a)
                return
        self._launch_held()
        self._ptr(a), self._ptr(b)                               # launches whatever still has to produce (or add into) them
        if a.store == b.store == "bf16" and a.size == b.size and a._dev_valid and (self._ptr(a) | self._ptr(b)) % 16 == 0:
            pa, pb = self._ptr(a), self._ptr(b)
            if a._buf.refs > 1:                                  # copy-on-write, as below
                buf = _Buf(self.lib, a.size * 2)
                check(self.lib.ah_add_bf16(pa, pb, buf.ptr, a.size))
                a._buf.release()
                a._buf, a._off = buf, 0
            else:
                check(self.lib.ah_add_bf16(pa, pb, pa, a.size))
            self._dirty(a)
            return
        if a._buf is not None and a._buf.refs > 1 and a._dev_valid and a.store == "f32" and b.store == "f32":
            # copy-on-write: `a` shares its buffer (clone): the sum goes to a buffer of its own in one pass
            pa, pb = self._ptr(a), self._ptr(b)
            buf = _Buf(self.lib, a.size * 4)
            check(self.lib.ah_binary(ffi.ADD, pa, pb, buf.ptr, a.size))
            a._buf.release()
            a._buf, a._off = buf, 0
            self._dirty(a)
            return
        self._f32(a, b)
        self._own(a)
        super().addInplace(a, b)

    def _own(self, t: TensorData):
        """Before an in-place write: give `t` a buffer nobody else shares."""
        self._launch_flash()                                    # (a pending attention reads its operands as they are now)
        if t._buf is not None and t._buf.refs > 1 and t._dev_valid:
            n = t.size * ffi.DTYPE_BYTES[t.store]
            buf = _Buf(self.lib, n)
            check(self.lib.ah_copy(buf.ptr, self._ptr(t), n))
            t._buf.release()
            t._buf, t._off = buf, 0

    def scaleInplace(self, a: TensorData, s: float):
        self._f32(a)
        self._own(a)
        super().scaleInplace(a, s)

    def clone(self, a: TensorData) -> TensorData:
        """Copy-on-write: the copy shares the buffer until one side is written in place (addInplace / scaleInplace /
        adamwStep copy first).  A host-created tensor is uploaded by _view, as the eager clone would."""
        return self._view(a, a.shape)

    # ------------------------------------------------------------------ nn with bf16 storage
    def _ln_bf16_ok(self, x: TensorData) -> bool:
        dim = x.shape[-1] if x.shape else 0
        return x.store == "bf16" and dim % 4 == 0 and 0 < dim <= 2048

    def layerNorm(self, x, weight, bias, eps) -> TensorData:
        if x.store == "bf16" and not self._ln_bf16_ok(x):
            self._f32(x)
        if x.store not in ("f32", "bf16"):
            return super().layerNorm(x, weight, bias, eps)
        dim = x.shape[-1]
        if weight.size != dim or bias.size != dim:
            raise ValueError("layerNorm: weight/bias length must equal the last dimension")
        out = self._new(x.shape, "f32", "bf16")
        check(self.lib.ah_layernorm(self._ptr(x), self._ptr(weight), self._ptr(bias), out._buf.ptr, x.size // max(1, dim), dim, eps, BF16,
                                    ffi.DTYPE_CODE[x.store]))
        return out

    def layerNormBackward(self, x, weight, gradOutput, eps) -> dict:
        dim = x.shape[-1]
        rows = x.size // max(1, dim)
        if self._ln_bf16_ok(x) and rows > 0:
            # the residual stream is kept in bf16: its gradient, which the tape adds dx to, is kept in bf16 as well
            if gradOutput.store != "bf16":
                gradOutput = self.castStore(gradOutput, "bf16")
            self._launch_ln()
            gp, xp, wp = self._ptr(gradOutput), self._ptr(x), self._ptr(weight)
            dx, dw, db = self._new(x.shape, "f32", "bf16"), self._new(weight.shape), self._new(weight.shape)
            self._held_ln = _HeldLayerNormBwd(xp, wp, gp, dx, dw, db, rows, dim, eps,
                                              self._hold(x._buf, weight._buf, gradOutput._buf, dx._buf, dw._buf, db._buf))
            return {"dx": dx, "dw": dw, "db": db}
        if x.store != "f32":
            return super().layerNormBackward(x, weight, gradOutput, eps)
        gp = self._ptr(gradOutput)
        dx, dw, db = self._new(x.shape), self._new(weight.shape), self._new(weight.shape)
        check(self.lib.ah_layernorm_bwd(self._ptr(x), self._ptr(weight), gp, ffi.DTYPE_CODE[gradOutput.store], 0, dx._buf.ptr, 0, dw._buf.ptr,
                                        db._buf.ptr, rows, dim, eps, 0, ffi.F32))
        return {"dx": dx, "dw": dw, "db": db}

    def _launch_ln(self, residual: int = 0, dx_ptr: int = 0):
        """Launches the held LayerNorm backward: plainly, or (residual, dx_ptr given) with its dx added to `residual` into dx_ptr."""
        h, self._held_ln = self._held_ln, None
        if h is None:
            return
        if not dx_ptr and all(b.refs == 1 for b in h.outs):     # every result was released unread
            self._unhold(h.holds)
            return
        check(self.lib.ah_layernorm_bwd(h.x_ptr, h.w_ptr, h.g_ptr, BF16, residual, 0, dx_ptr or h.outs[0].ptr, h.outs[1].ptr, h.outs[2].ptr,
                                        h.rows, h.dim, h.eps, 0, BF16))
        if dx_ptr:                                               # the bare dx was not written: keep the recipe until its tensor is released
            self._ln_unwritten[id(h.outs[0])] = h
        else:
            self._unhold(h.holds)

    def _early_loss(self, out: TensorData):
        # The reference's trainer reads the loss after it has issued the whole backward pass (trainer.ts:1247): the copy to the
        # host starts as soon as the loss exists, and reading it later waits for this copy only, not for the backward pass.
        if out._buf is None:
            return
        tk = C.c_uint64(0)
        if self.lib.ah_download_begin(out._buf.ptr + out._off, 4, C.byref(tk)) == 0:
            out._early = tk.value

    def _launch_ce(self):
        """The held cross-entropy on its own (somebody needs the loss, or touches its operands, before any backward call)."""
        h, self._held_ce = self._held_ce, None
        if h is None:
            return
        if not (h.out_buf.refs == 1 and h.lse_buf.refs == 1):     # (both released unread otherwise)
            check(self.lib.ah_cross_entropy(h.logits_ptr, BF16, h.targets_ptr, h.out_buf.ptr, h.lse_buf.ptr, h.n, h.c))
            if h.out._buf is h.out_buf:
                self._early_loss(h.out)
        self._unhold(h.holds)

    def crossEntropy(self, logits: TensorData, targets: TensorData) -> TensorData:
        N, Cc = logits.shape
        out, lse = self._new(()), self._new((N,))
        self._launch_ce()
        lp, tp = self._ptr(logits), self._ptr(targets)
        logits._ce_lse = lse
        if logits.store == "bf16" and N > 0 and Cc > 0:
            self._held_ce = _HeldCrossEntropy(lp, tp, logits._buf, out, lse, N, Cc, self._hold(logits._buf, targets._buf, out._buf, lse._buf))
            return out
        check(self.lib.ah_cross_entropy(lp, ffi.DTYPE_CODE[logits.store], tp, out._buf.ptr, lse._buf.ptr, N, Cc))
        self._early_loss(out)
        return out

    def crossEntropyBackward(self, logits, targets, gradOutput) -> TensorData:
        h = self._held_ce
        if h is not None and logits._buf is h.logits_buf and logits.store == "bf16" and tuple(logits.shape) == (h.n, h.c) \
                and gradOutput._buf is not None and not any(gradOutput._buf is b for b in h.holds):
            gp = self._ptr(gradOutput)
            if self._held_ce is h:                              # (still held: loss, gradient and LSE in one pass over the logits)
                self._held_ce = None
                out = self._new((h.n, h.c), "f32", "bf16")
                check(self.lib.ah_cross_entropy_fwd_bwd(h.logits_ptr, BF16, h.targets_ptr, h.out_buf.ptr, h.lse_buf.ptr, gp, 1.0,
                                                        out._buf.ptr, h.n, h.c))
                if h.out._buf is h.out_buf:
                    self._early_loss(h.out)
                self._unhold(h.holds)
                return out
        lse = getattr(logits, "_ce_lse", None)
        if lse is None or lse._buf is None or logits.store != "bf16":
            self._f32(logits)
            return super().crossEntropyBackward(logits, targets, gradOutput)
        N, Cc = logits.shape
        out = self._new((N, Cc), "f32", "bf16")
        check(self.lib.ah_cross_entropy_bwd(self._ptr(logits), BF16, self._ptr(targets), self._ptr(lse), self._ptr(gradOutput), 1.0,
                                            out._buf.ptr, N, Cc))
        return out

    def flashAttention(self, Q, K, V, T, scale, softCap) -> dict:
        if not (Q.store == K.store == V.store):
            self._words(Q, K, V)
        if Q.store != "bf16" or Q.size == 0 or len(Q.shape) != 3 or Q.shape[2] % 8 or not 8 <= Q.shape[2] <= 128:
            return super().flashAttention(Q, K, V, T, scale, softCap)      # (also what the library refuses: it says so at once)
        self._flash_desc(Q, K, V, T, scale, softCap)            # (the shape checks)
        self._launch_flash()
        BH, _, D = Q.shape
        q, k, v = self._ptr(Q), self._ptr(K), self._ptr(V)
        out, lse = self._new(Q.shape, "f32", "bf16"), self._new((BH, T))
        rec = _HeldFlash(q, k, v, out._buf, lse._buf, BH, T, D, scale, softCap, self._hold(Q._buf, K._buf, V._buf, out._buf, lse._buf))
        self._lazy[id(out._buf)] = self._lazy[id(lse._buf)] = self._pending_flash = rec
        return {"output": out, "lse": lse}

    def _flash_strides(self, f: ffi.AhFlash, B: int, H: int, T: int, D: int, o_heads: bool):
        """q, k, v (and their gradients) as [B H, T, D] slabs; o (and dO) as slabs too, or as [B, T, H, D]."""
        f.batch, f.heads, f.seq, f.head_dim = B, H, T, D
        for nm in ("q", "k", "v", "o"):
            setattr(f, nm + "_sb", H * T * D), setattr(f, nm + "_sh", T * D), setattr(f, nm + "_st", D)
        if o_heads:
            f.o_sb, f.o_sh, f.o_st = T * H * D, D, H * D

    def _launch_flash(self, rec: Optional[_HeldFlash] = None, twin=None):
        """Launches the pending attention: into the [B H, T, D] tensor the caller holds, or -- twin = (buffer, B, H) -- as
        [B, T, H, D] into that buffer, leaving the caller's tensor unwritten."""
        rec = rec or self._pending_flash
        if rec is None or rec.launched:
            return
        if self._pending_flash is rec:
            self._pending_flash = None
        self._lazy.pop(id(rec.lse_buf), None)
        if twin is None and rec.o_buf.refs == 1 and rec.lse_buf.refs == 1:      # both results released unread
            self._lazy.pop(id(rec.o_buf), None)
            rec.launched = True
            self._unhold(rec.holds)
            return
        f = ffi.AhFlash()
        f.dtype, f.scale, f.soft_cap, f.bwd_variant = BF16, rec.scale, rec.cap, self.flashBackwardVariant
        f.q, f.k, f.v, f.lse = rec.q, rec.k, rec.v, rec.lse_buf.ptr
        if twin is None:
            self._flash_strides(f, rec.BH, 1, rec.T, rec.D, False)
            f.o = rec.o_buf.ptr
        else:
            self._flash_strides(f, twin[1], twin[2], rec.T, rec.D, True)
            f.o = twin[0].ptr
        check(self.lib.ah_flash_fwd(C.byref(f)))
        rec.launched = True
        self._unhold(rec.holds)
        rec.holds = []
        if twin is None:
            self._lazy.pop(id(rec.o_buf), None)
        else:                                                   # the caller's tensor now stands for "the twin, transposed back"
            rec.twin = twin
            rec.holds = self._hold(rec.o_buf, twin[0])

    def _materialise(self, buf):
        rec = self._lazy.get(id(buf))
        if isinstance(rec, _HeldFlash):
            if not rec.launched:
                self._launch_flash(rec)
            elif buf is rec.o_buf and rec.twin is not None:     # somebody reads the slabs after all: transposed back from the twin
                tb, B, H = rec.twin
                self._lazy.pop(id(buf), None)
                check(self.lib.ah_transpose(tb.ptr, buf.ptr, 4, ffi.shape_arr([B, rec.T, H, rec.D // 2]), 1, 2))
                self._unhold(rec.holds)
        elif isinstance(rec, _LazyTranspose):
            self._lazy.pop(id(buf), None)
            half = list(rec.src_shape)
            half[-1] //= 2
            check(self.lib.ah_transpose(rec.src_ptr, buf.ptr, 4, ffi.shape_arr(half), 1, 2))
            self._unhold(rec.holds)

    def _drop_lazy(self, buf):
        """`buf` has been released by everybody but its record."""
        rec = self._lazy.get(id(buf))
        if isinstance(rec, _HeldFlash) and not rec.launched:
            if rec.o_buf.refs == 1 and rec.lse_buf.refs == 1:   # (its other result may still be read: then it has to be computed)
                self._launch_flash(rec)
            return
        self._lazy.pop(id(buf), None)
        if rec is not None:
            self._unhold(rec.holds)

    def flashAttentionBackward(self, Q, K, V, O, dO, lse, T, scale, softCap) -> dict:
        if not (Q.store == K.store == V.store == O.store == dO.store):
            self._words(Q, K, V, O, dO)
        if Q.store != "bf16":
            return super().flashAttentionBackward(Q, K, V, O, dO, lse, T, scale, softCap)
        # the three gradients one behind the other in one allocation: what consumes their scattered sum (the projection's dX
        # and dW products) can then read them in place
        f = self._flash_desc(Q, K, V, T, scale, softCap)
        f.dtype = BF16
        orec = self._lazy.get(id(O._buf)) if O._buf is not None else None
        drec = self._lazy.get(id(dO._buf)) if dO._buf is not None else None
        if isinstance(orec, _HeldFlash) and orec.twin is not None and isinstance(drec, _LazyTranspose) and O._off == 0 and dO._off == 0 \
                and O._buf is orec.o_buf and drec.src_shape == (orec.twin[1], T, orec.twin[2], Q.shape[2]):
            # the forward result exists as [B, T, H, D] and so does its gradient (the transposes around the slabs were never
            # run): the kernels read both through strides
            self._flash_strides(f, orec.twin[1], orec.twin[2], T, Q.shape[2], True)
            f.q, f.k, f.v, f.lse = self._ptr(Q), self._ptr(K), self._ptr(V), self._ptr(lse)
            f.o, f.d_o = orec.twin[0].ptr, drec.src_ptr
        else:
            f.q, f.k, f.v, f.o, f.lse, f.d_o = self._ptr(Q), self._ptr(K), self._ptr(V), self._ptr(O), self._ptr(lse), self._ptr(dO)
        dQ, dK, dV = self._plane_views(3, Q.shape)
        f.dq, f.dk, f.dv = dQ._buf.ptr + dQ._off, dK._buf.ptr + dK._off, dV._buf.ptr + dV._off
        check(self.lib.ah_flash_bwd(C.byref(f)))
        return {"dQ": dQ, "dK": dK, "dV": dV}

    def attentionQkvBackward(self, qkv, out, dOut, lse, Bt, T, nHead, scale, softCap) -> TensorData:
        if not (qkv.store == out.store == dOut.store):
            self._words(qkv, out, dOut)
        return super().attentionQkvBackward(qkv, out, dOut, lse, Bt, T, nHead, scale, softCap)

    # ------------------------------------------------------------------ optimizer
    def totalSumOfSquares(self, tensors: Sequence[TensorData]) -> TensorData:
        self._launch_held()
        self._launch_ln()
        # The device is idle while this runs (the trainer has just read the loss back, trainer.ts:1247,1345-1349): with nothing
        # pending and every gradient resident in f32, the addresses are read straight off the tensors, and the argument
        # arrays of the last call are reused when the gradient set sits where it sat then.
        def addresses():
            if self._orphans or self._ln_unwritten:
                return (None,)
            try:
                return tuple([t._buf.ptr + t._off if t._dev_valid and t.store == "f32" else None for t in tensors])
            except AttributeError:                              # a tensor without a device buffer
                return (None,)
        if self._wgrads and not self._adam_q:
            # The queued weight gradients are about to be computed by grouped launches: let those sum the squares of what
            # they store, and read only the other gradients again.  Every queued product must then go out in a grouped launch
            # (one that runs on its own would be read by the list before it is computed) and every result must be one of the
            # listed tensors, whole; otherwise the launches run as they are and the list is read as usual.
            key = addresses()
            if None not in key and len(set(key)) == len(key):
                ws, parts = self._take_weight_grads()
                covered = {w.dst: w.m * w.n for w in ws if w.dst is not None} if all(grouped for _, _, grouped in parts) else {}
                listed = {k: t.size for k, t in zip(key, tensors)}
                if covered and all(grouped for _, _, grouped in parts) and all(listed.get(a) == n for a, n in covered.items()) \
                        and not any(w.add_after is not None for w in ws):
                    total = self._new((1,))
                    rest = [(k, t.size) for k, t in zip(key, tensors) if k not in covered]
                    if rest:
                        self._sum_sq_list(tuple(k for k, _ in rest), [n for _, n in rest], total._buf.ptr)
                    else:
                        check(self.lib.ah_fill_f32(total._buf.ptr, 0.0, 1))
                    self._run_weight_grads(ws, parts, total._buf.ptr)
                    return total
                self._run_weight_grads(ws, parts)
        self._launch_weight_grads()
        self._flush_adam()
        key = addresses()
        if None not in key and len(key) > 0:
            total = self._new((1,))
            self._sum_sq_list(key, [t.size for t in tensors], total._buf.ptr)
            return total
        return super().totalSumOfSquares(tensors)

    def _sum_sq_list(self, ptrs, sizes, out: int):
        c = self._ssq_args
        if c is None or c[0] != ptrs or c[1] != sizes:
            c = self._ssq_args = (ptrs, sizes, (C.c_uint64 * len(ptrs))(*ptrs), (C.c_uint64 * len(ptrs))(*sizes))
        check(self.lib.ah_sum_sq_list(c[2], c[3], len(ptrs), out))

    def adamwStep(self, params, grads, m, v, lr, beta1, beta2, eps, weightDecay, bc1, bc2, gradScale=1.0):
        """Queued: the optimizer calls this once per parameter tensor with the same scalars (optimizers.ts:54-94); the updates of
        a pass are launched together when the first of their tensors is read, written or released."""
        self._launch_held()
        self._f32(params, grads, m, v)
        if not (params.size == grads.size == m.size == v.size):
            raise ValueError("adamwStep: params, grads, m, v must have the same size")
        key = (lr, beta1, beta2, eps, bc1, bc2, gradScale)
        if self._adam_q and key != self._adam_key:
            self._flush_adam()
        for t in (params, m, v):
            self._own(t)
        ptrs = [self._ptr(t) for t in (params, grads, m, v)]    # (launches whatever still has to produce the gradient)
        if not self._adam_q:
            if key != self._adam_key:
                self._adam_flush_at = 1                         # a new optimizer pass
            self._adam_key = key
            self._adam_hyper(lr, beta1, beta2, eps, 0.0, bc1, bc2, gradScale)      # the device copy of the scalars, once per pass
        sh = getattr(params, "_shadow", None)
        if sh is not None and self._orphans:
            # a product whose plain result was never written (its epilogue went elsewhere) and whose tensor is still alive
            # would be computed later from this shadow, which the update rewrites in place: compute it from the old weights now
            for key in [k for k, h in self._orphans.items() if any(b is sh for b in h.holds)]:
                h = self._orphans.pop(key)
                self._run_held(h, h.out_ptr)
                self._unhold(h.holds)
        self._adam_q.append((*ptrs, sh.ptr if sh is not None else 0, params.size, weightDecay))
        for b in (params._buf, grads._buf, m._buf, v._buf) + ((sh,) if sh is not None else ()):
            b.refs += 1
            self._adam_holds.append(b)
            self._adam_bufs.add(id(b))
        for t in (params, m, v):
            HipBackend._dirty(self, t)                          # host copies are stale; the shadow is refreshed by the kernel
        if len(self._adam_q) >= self._adam_flush_at:            # the device is usually idle here (the norm was just read back):
            self._flush_adam()                                  # give it the first tensor at once, then 16 while the host queues
            self._adam_flush_at = 16 if self._adam_flush_at == 1 else 48      # the rest, then a launch's full table at a time
            check(self.lib.ah_step_kick())                      # (inside a step plan: launch now, do not wait for a full segment)

    def _flush_adam(self):
        q, self._adam_q = self._adam_q, []
        if not q:
            return
        holds, self._adam_holds, self._adam_bufs = self._adam_holds, [], set()
        lr, beta1, beta2, eps, bc1, bc2, gradScale = self._adam_key
        h, dev = self._adam_hyper(lr, beta1, beta2, eps, 0.0, bc1, bc2, gradScale)
        items = (ffi.AhAdamWItem * len(q))(*[ffi.AhAdamWItem(p, g, m, v, sh, n, wd, 0) for p, g, m, v, sh, n, wd in q])
        check(self.lib.ah_adamw_list(items, len(q), C.byref(h), dev, 0))
        for b in holds:
            b.release()

    def lionStep(self, params, grads, m, *a, **kw):
        self._own(params), self._own(m)
        super().lionStep(params, grads, m, *a, **kw)

    def sgdStep(self, params, grads, *a, **kw):
        self._own(params)
        super().sgdStep(params, grads, *a, **kw)

    def adafactorStep2d(self, params, grads, vr, vc, *a, **kw):
        self._own(params), self._own(vr), self._own(vc)
        super().adafactorStep2d(params, grads, vr, vc, *a, **kw)

    def adafactorStepFlat(self, params, grads, v, *a, **kw):
        self._own(params), self._own(v)
        super().adafactorStepFlat(params, grads, v, *a, **kw)

    def flush(self):
        self._launch_held()
        self._launch_flash()
        self._launch_ln()
        self._launch_ce()
        self._launch_weight_grads()
        self._flush_adam()
        super().flush()

    def syncGpu(self):
        self._launch_held()
        self._launch_flash()
        self._launch_ln()
        self._launch_ce()
        self._launch_weight_grads()
        self._flush_adam()
        super().syncGpu()
