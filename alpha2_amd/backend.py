"""`HipBackend`: the reference's `Backend` op interface (packages/core/src/interfaces.ts:38-151) implemented over
libalpha_hip.so.  Method names, argument order, shape rules and error behaviour follow the reference so that its
callers (autograd / model / train) and its tests carry over unchanged; this module is the Python twin of the
TypeScript shim a Bun process would load (same C symbols, same call sequence).

Residency follows the reference GPU backend's contract (packages/helios/src/backend.ts is NOT ported; only the
behaviour its callers rely on: packages/helios/src/backend.ts:596-729,1143-1171):
  * a TensorData created by the caller on the host (params, optimizer moments, token batches) is uploaded on first
    use and stays resident, keyed by object identity;
  * outputs live on the device; `.data` reads back lazily and caches until an in-place op invalidates it;
  * `reshape` shares the device buffer (reference-counted); `releaseGpuTensor` returns it to the pool.
"""
from __future__ import annotations

import ctypes as C
import math
from typing import List, Optional, Sequence, Tuple

import numpy as np

from . import _ffi as ffi
from ._ffi import check

_NP = {"f32": np.float32, "i32": np.int32, "f16": np.uint16, "bf16": np.uint16, "f64": np.float64}


def shapeSize(shape) -> int:
    s = 1
    for d in shape:
        s *= int(d)
    return s


def shapeStrides(shape) -> List[int]:
    st, s = [0] * len(shape), 1
    for i in range(len(shape) - 1, -1, -1):
        st[i] = s
        s *= int(shape[i])
    return st


class _Buf:
    """One ah_alloc block, shared by views."""
    __slots__ = ("ptr", "nbytes", "refs", "lib")

    def __init__(self, lib, nbytes: int):
        out = C.c_uint64(0)
        check(lib.ah_alloc(max(1, nbytes), C.byref(out)))
        self.ptr, self.nbytes, self.refs, self.lib = out.value, nbytes, 1, lib

    def release(self):
        self.refs -= 1
        if self.refs == 0 and self.ptr:
            self.lib.ah_free(self.ptr)
            self.ptr = 0

    def __del__(self):          # backstop, like the reference's FinalizationRegistry
        try:
            if self.ptr and self.refs > 0:
                self.lib.ah_free(self.ptr)
                self.ptr = 0
        except Exception:
            pass


class TensorData:
    """shape + dtype + data (packages/core/src/interfaces.ts:31-35).  `data` is a flat numpy array; for a
    device-resident tensor it is fetched on demand."""

    def __init__(self, shape, dtype: str = "f32", data: Optional[np.ndarray] = None):
        self.shape: Tuple[int, ...] = tuple(int(s) for s in shape)
        self.dtype = dtype
        self._host: Optional[np.ndarray] = None if data is None else np.ascontiguousarray(data, dtype=_NP[dtype]).reshape(-1)
        self._buf: Optional[_Buf] = None
        self._off = 0               # byte offset into _buf
        self._host_valid = data is not None
        self._dev_valid = False
        self._backend: Optional["HipBackend"] = None
        self.store = dtype          # device storage type ("bf16" for fast-mode activations)

    @property
    def size(self) -> int:
        return shapeSize(self.shape)

    @property
    def data(self) -> np.ndarray:
        if not self._host_valid:
            if self._buf is None or not self._dev_valid:
                raise RuntimeError("TensorData has neither host nor device contents (released?)")
            self._host = self._backend._download(self)
            self._host_valid = True
        return self._host

    @data.setter
    def data(self, arr):
        self._host = np.ascontiguousarray(arr, dtype=_NP[self.dtype]).reshape(-1)
        self._host_valid, self._dev_valid = True, False


class HipBackend:
    name = "hip"

    def __init__(self, device: int = 0):
        self.lib = ffi.load()
        check(self.lib.ah_init(device))
        self._min_gpu_size = 0
        self._step_graphs, self._step_open, self._step_key = False, False, 0
        self.lastStepHow, self.lastStepNote = "eager", ""
        self.stepFallbackNotes: List[str] = []
        self._hyper_dev, self._hyper_key = None, None
        self.planeProducts = 0                 # products issued through ah_gemm_planes (an operand in planes, no copy around it)
        self.flashBackwardVariant = 0          # AhFlash.bwd_variant for the bf16 backward kernels (1: one pass over the scores)

    # ------------------------------------------------------------------ residency helpers
    def _new(self, shape, dtype="f32", store: Optional[str] = None) -> TensorData:
        t = TensorData(shape, dtype)
        t.store = store or dtype
        t._buf = _Buf(self.lib, shapeSize(shape) * ffi.DTYPE_BYTES[t.store])
        t._dev_valid, t._backend = True, self
        return t

    def _ptr(self, t: TensorData) -> int:
        """Device address of `t`, uploading a host-created tensor on first use."""
        if t._buf is None or not t._dev_valid:
            if not t._host_valid:
                raise RuntimeError("use of a released tensor")
            if t._buf is None:
                t._buf = _Buf(self.lib, t._host.nbytes)
                t._off = 0
            t._backend = self
            if t._host.nbytes:
                check(self.lib.ah_upload(t._buf.ptr + t._off, t._host.ctypes.data_as(C.c_void_p), t._host.nbytes))
            t._dev_valid = True
        return t._buf.ptr + t._off

    def _download(self, t: TensorData) -> np.ndarray:
        n = shapeSize(t.shape)
        if t.store == "bf16":       # internal storage, surfaced to callers as f32 (the interface has no bf16)
            raw = np.empty(n, dtype=np.uint16)
            if n:
                check(self.lib.ah_download(raw.ctypes.data_as(C.c_void_p), t._buf.ptr + t._off, raw.nbytes))
            return (raw.astype(np.uint32) << 16).view(np.float32)
        out = np.empty(n, dtype=_NP[t.dtype])
        if n:
            check(self.lib.ah_download(out.ctypes.data_as(C.c_void_p), t._buf.ptr + t._off, out.nbytes))
        return out

    def _dirty(self, t: TensorData):
        """An in-place device op changed `t`: the cached host copy is stale (backend.ts:706-729)."""
        t._host_valid = False
        t._host = None

    def _view(self, t: TensorData, shape, byte_off: int = 0) -> TensorData:
        self._ptr(t)
        v = TensorData(shape, t.dtype)
        v.store = t.store
        v._buf, v._off = t._buf, t._off + byte_off
        t._buf.refs += 1
        v._dev_valid, v._backend = True, self
        return v

    def releaseGpuTensor(self, t: TensorData):
        """packages/train/src/trainer.ts:1003-1006.  Stream-ordered: safe to call right after enqueueing uses."""
        if t is None or t._buf is None:
            return
        t._buf.release()
        t._buf, t._dev_valid = None, False

    def flush(self):
        """The trainer's end-of-step call (trainer.ts:1776-1784).  Work is already on the stream in call order, so there
        is nothing to submit; with step graphs enabled it is the seam between two steps: the open step plan is closed
        (recorded, replayed or fallen back) and the next one is opened, so everything the unchanged trainer issues from one
        flush() to the next runs as recorded hipGraph segments from the third step on."""
        if self._step_graphs:
            if self._step_open:
                self.stepEnd()
            self.stepBegin()

    # ------------------------------------------------------------------ step plans (record -> verify -> replay)
    STEP_HOW = ("eager", "recorded", "replayed", "fell-back")

    def enableStepGraphs(self, on: bool = True, key: int = 0):
        """Bracket every flush()-to-flush() interval with ah_step_begin / ah_step_end."""
        if not on and self._step_open:
            self.stepEnd()
        self._step_graphs, self._step_key = bool(on), int(key)

    def stepBegin(self, key: Optional[int] = None):
        check(self.lib.ah_step_begin(self._step_key if key is None else int(key)))
        self._step_open = True

    def stepEnd(self) -> str:
        how = C.c_int32(0)
        self._step_open = False
        check(self.lib.ah_step_end(C.byref(how)))
        self.lastStepHow = self.STEP_HOW[how.value]
        self.lastStepNote = self.lib.ah_step_note().decode("utf-8", "replace")
        if how.value == 3:
            self.stepFallbackNotes.append(self.lastStepNote)
        return self.lastStepHow

    def resetStepPlan(self, key: Optional[int] = None):
        """Forget the recorded plan (the next bracketed step records again)."""
        check(self.lib.ah_step_reset(self._step_key if key is None else int(key)))

    def stepStats(self) -> dict:
        s = self._stats()
        return {"recorded": s.steps_recorded, "replayed": s.steps_replayed, "fellBack": s.steps_fallback, "nodeUpdates": s.step_node_updates}

    def syncGpu(self):
        check(self.lib.ah_sync())

    def purgeBufferPools(self):
        check(self.lib.ah_trim_pool())

    def resetStepOps(self):
        check(self.lib.ah_reset_op_count())

    @property
    def gpuOpsThisStep(self) -> int:
        return self._stats().ops_launched

    def _stats(self) -> ffi.AhStats:
        s = ffi.AhStats()
        check(self.lib.ah_stats(C.byref(s)))
        return s

    def gpuMemStats(self) -> dict:
        """Fields read at packages/train/src/trainer.ts:1821-1843,1922-1930."""
        s = self._stats()
        return {"bufferPoolEntries": s.pool_blocks, "bufferPoolBytes": s.pool_bytes, "outputPoolEntries": 0,
                "outputPoolBytes": 0, "deferredReleases": 0, "pendingDestroys": 0, "liveAllocs": s.live_allocs,
                "liveBytes": s.live_bytes, "totalAllocs": s.device_mallocs, "graphsLive": s.graphs_live}

    def getDeviceInfo(self) -> dict:
        d = ffi.AhDeviceInfo()
        check(self.lib.ah_device_info(C.byref(d)))
        return {"deviceName": d.name.decode(), "arch": d.arch.decode(), "vendorId": 0x1002, "computeUnits": d.compute_units,
                "waveSize": d.wavefront, "clockKHz": d.clock_khz, "hbmBytes": d.hbm_bytes}

    def setMinGpuSize(self, n: int):
        self._min_gpu_size = n       # every op runs on the device; kept for interface compatibility

    # ------------------------------------------------------------------ creation
    def zeros(self, shape, dtype="f32") -> TensorData:
        return self.full(shape, 0, dtype)

    def ones(self, shape, dtype="f32") -> TensorData:
        return self.full(shape, 1, dtype)

    def full(self, shape, value, dtype="f32") -> TensorData:
        t = self._new(shape, dtype)
        n = shapeSize(shape)
        if dtype == "i32":
            check(self.lib.ah_fill_i32(t._buf.ptr, int(value), n))
        elif dtype == "f32":
            check(self.lib.ah_fill_f32(t._buf.ptr, float(value), n))
        else:
            raise ValueError(f"full: dtype {dtype} not supported")
        return t

    def randn(self, shape, dtype="f32") -> TensorData:
        from .rng import SeededRng
        if not hasattr(self, "_rng"):
            self._rng = SeededRng(42)          # cpu_ref.ts:111
        n = shapeSize(shape)
        return TensorData(shape, dtype, np.array([self._rng.nextGauss() for _ in range(n)], dtype=_NP[dtype]))

    def fromArray(self, data, shape, dtype="f32") -> TensorData:
        if len(data) != shapeSize(shape):
            raise ValueError(f"Data length {len(data)} does not match shape size {shapeSize(shape)}")
        return TensorData(shape, dtype, np.asarray(data, dtype=_NP[dtype]))

    # ------------------------------------------------------------------ math
    def _binary(self, op: int, a: TensorData, b: TensorData) -> TensorData:
        self._f32(a, b)
        if a.shape == b.shape:
            out = self._new(a.shape)
            check(self.lib.ah_binary(op, self._ptr(a), self._ptr(b), out._buf.ptr, a.size))
            return out
        nd = max(len(a.shape), len(b.shape))
        sa = (1,) * (nd - len(a.shape)) + a.shape
        sb = (1,) * (nd - len(b.shape)) + b.shape
        res = []
        for da, db in zip(sa, sb):
            if da != db and da != 1 and db != 1:
                raise ValueError(f"Cannot broadcast shapes [{a.shape}] and [{b.shape}]")
            res.append(max(da, db))
        stra, strb = self._bstrides(sa, res), self._bstrides(sb, res)
        if nd > 6:
            raise ValueError("broadcast over more than 6 dims is not supported")
        out = self._new(res)
        check(self.lib.ah_binary_broadcast(op, self._ptr(a), self._ptr(b), out._buf.ptr, nd, ffi.shape_arr(res),
                                           ffi.shape_arr(stra), ffi.shape_arr(strb)))
        return out

    @staticmethod
    def _bstrides(src, target):
        st, s = [0] * len(target), 1
        for i in range(len(target) - 1, -1, -1):
            st[i] = 0 if (src[i] == 1 and target[i] != 1) else s
            s *= src[i]
        return st

    @staticmethod
    def _f32(*ts):
        for t in ts:
            if t.dtype != "f32" or t.store != "f32":
                raise TypeError(f"op expects f32 tensors, got {t.dtype}/{t.store}")

    def _words(self, *ts):
        """The data-movement kernels copy 4-byte elements: a tensor stored in 2 bytes must not reach them as it is."""
        for t in ts:
            if ffi.DTYPE_BYTES[t.store] != 4:
                raise TypeError(f"data-movement op expects 4-byte storage, got {t.dtype}/{t.store}")

    def add(self, a, b): return self._binary(ffi.ADD, a, b)
    def sub(self, a, b): return self._binary(ffi.SUB, a, b)
    def mul(self, a, b): return self._binary(ffi.MUL, a, b)
    def div(self, a, b): return self._binary(ffi.DIV, a, b)

    def _gemm(self, layout, a_ptr, b_ptr, c_ptr, m, n, k, lda, ldb, ldc, batch=1, sa=0, sb=0, sc=0, in_dtype=ffi.F32,
              out_dtype=ffi.F32, epilogue=ffi.EPI_NONE, aux=0, planes=None):
        """planes = (c_plane_cols, c_plane_stride, a_plane_k, a_plane_stride): the product goes through ah_gemm_planes."""
        g = ffi.AhGemm(layout, in_dtype, out_dtype, epilogue, m, n, k, lda, ldb, ldc, batch, sa, sb, sc, a_ptr, b_ptr, c_ptr, aux)
        run = (lambda: check(self.lib.ah_gemm(C.byref(g)))) if planes is None else (lambda: check(self.lib.ah_gemm_planes(C.byref(g), *planes, 0)))
        self.planeProducts += planes is not None
        timed = getattr(self, "_timed", None)
        if timed is None:
            run()
            return
        e0, e1 = self._event(), self._event()
        check(self.lib.ah_event_record(e0))
        run()
        check(self.lib.ah_event_record(e1))
        kernel, nsplit = self.lastGemmKernel()
        timed.append({"kind": "gemm", "kernel": kernel, "nsplit": nsplit, "layout": layout, "dtype": in_dtype, "m": m, "n": n, "k": k,
                      "batch": batch, "flops": 2.0 * m * n * k * batch, "e0": e0, "e1": e1})

    def lastGemmKernel(self):
        """(name, split-K slices) of the kernel the last ah_gemm call launched, named as a profiler prints it."""
        buf, ns = C.create_string_buffer(128), C.c_int32(1)
        check(self.lib.ah_gemm_last_kernel(buf, 128, C.byref(ns)))
        return buf.value.decode(), ns.value

    def _event(self) -> int:
        ev = C.c_uint64()
        check(self.lib.ah_event_create(C.byref(ev)))
        return ev.value

    def startTiming(self):
        """Bracket every GEMM launch with HIP events on the library stream until stopTiming()."""
        self._timed = []

    def stopTiming(self) -> list:
        """Returns one record per launch with its duration in milliseconds (blocks until the work has finished)."""
        recs, self._timed = self._timed or [], None
        ms = C.c_float()
        for r in recs:
            check(self.lib.ah_event_elapsed_ms(r["e0"], r["e1"], C.byref(ms)))
            r["ms"] = ms.value
            for e in (r.pop("e0"), r.pop("e1")):
                check(self.lib.ah_event_destroy(e))
        return recs

    def _batched(self, a: TensorData, b: TensorData, a_mat, b_mat):
        """Resolve broadcast batch dims (cpu_ref.ts:184-243).  Returns (batch_shape, batch, stride_a, stride_b)
        when the batch collapses to one uniform stride per operand, else None."""
        aB, bB = list(a.shape[:-2]), list(b.shape[:-2])
        nb = max(len(aB), len(bB))
        pa, pb = [1] * (nb - len(aB)) + aB, [1] * (nb - len(bB)) + bB
        bs = []
        for x, y in zip(pa, pb):
            if x != y and x != 1 and y != 1:
                raise ValueError(f"matmul batch shape mismatch: [{a.shape}] x [{b.shape}]")
            bs.append(max(x, y))
        batch = shapeSize(bs)
        if batch == 1:
            return bs, 1, 0, 0
        if pa == bs and pb == bs:
            return bs, batch, a_mat, b_mat
        if shapeSize(pa) == 1 and pb == bs:
            return bs, batch, 0, b_mat
        if shapeSize(pb) == 1 and pa == bs:
            return bs, batch, a_mat, 0
        return bs, batch, None, None

    def matmul(self, a: TensorData, b: TensorData) -> TensorData:
        self._f32(a, b)
        if len(a.shape) < 2 or len(b.shape) < 2:
            raise ValueError(f"matmul requires at least 2D tensors, got [{a.shape}] x [{b.shape}]")
        M, K, N = a.shape[-2], a.shape[-1], b.shape[-1]
        if b.shape[-2] != K:
            raise ValueError(f"matmul shape mismatch: [{a.shape}] x [{b.shape}]")
        bs, batch, sa, sb = self._batched(a, b, M * K, K * N)
        if sa is None:      # mixed broadcast: materialise the broadcast operands first
            a = self.broadcast(a, tuple(bs) + (M, K)) if tuple(a.shape[:-2]) != tuple(bs) else a
            b = self.broadcast(b, tuple(bs) + (K, N)) if tuple(b.shape[:-2]) != tuple(bs) else b
            sa, sb = M * K, K * N
        out = self._new(tuple(bs) + (M, N))
        self._gemm(ffi.GEMM_NN, self._ptr(a), self._ptr(b), out._buf.ptr, M, N, K, K, N, N, batch, sa, sb, M * N)
        return out

    def matmulTransposed(self, a: TensorData, b: TensorData) -> TensorData:
        """A[..,M,K] @ B[..,N,K]^T (interfaces.ts:111)."""
        self._f32(a, b)
        M, K, N = a.shape[-2], a.shape[-1], b.shape[-2]
        if b.shape[-1] != K:
            raise ValueError(f"matmul shape mismatch: [{a.shape}] x [{b.shape}]^T")
        bs, batch, sa, sb = self._batched(a, b, M * K, N * K)
        if sa is None:
            raise ValueError("matmulTransposed: mixed batch broadcast is not supported")
        out = self._new(tuple(bs) + (M, N))
        self._gemm(ffi.GEMM_NT, self._ptr(a), self._ptr(b), out._buf.ptr, M, N, K, K, K, N, batch, sa, sb, M * N)
        return out

    def matmulTransposedA(self, a: TensorData, b: TensorData) -> TensorData:
        """A[..,M,K]^T @ B[..,M,N] -> [..,K,N] (interfaces.ts:112; packages/tests/src/gpu-perf.test.ts:211-233)."""
        self._f32(a, b)
        M, K, N = a.shape[-2], a.shape[-1], b.shape[-1]
        if b.shape[-2] != M:
            raise ValueError(f"matmul shape mismatch: [{a.shape}]^T x [{b.shape}]")
        bs, batch, sa, sb = self._batched(a, b, M * K, M * N)
        if sa is None:
            raise ValueError("matmulTransposedA: mixed batch broadcast is not supported")
        out = self._new(tuple(bs) + (K, N))
        # C[K,N] = A^T B with contraction length M: TN layout with (m, n, k) = (K, N, M)
        self._gemm(ffi.GEMM_TN, self._ptr(a), self._ptr(b), out._buf.ptr, K, N, M, K, N, N, batch, sa, sb, K * N)
        return out

    def sum(self, a: TensorData, axis=None, keepdims=False) -> TensorData:
        return self._reduce(a, axis, keepdims, 0)

    def mean(self, a: TensorData, axis=None, keepdims=False) -> TensorData:
        return self._reduce(a, axis, keepdims, 1)

    def _reduce(self, a, axis, keepdims, mean) -> TensorData:
        self._f32(a)
        if axis is None:
            out = self._new(tuple(1 for _ in a.shape) if keepdims else ())
            check(self.lib.ah_sum_all(self._ptr(a), out._buf.ptr, a.size, mean))
            return out
        ax = self._axis(axis, len(a.shape))
        outer, dim, inner = shapeSize(a.shape[:ax]), a.shape[ax], shapeSize(a.shape[ax + 1:])
        oshape = [(1 if i == ax else d) for i, d in enumerate(a.shape)] if keepdims else [d for i, d in enumerate(a.shape) if i != ax]
        out = self._new(oshape)
        check(self.lib.ah_sum_axis(self._ptr(a), out._buf.ptr, outer, dim, inner, mean))
        return out

    @staticmethod
    def _axis(axis, nd):
        a = axis + nd if axis < 0 else axis
        if a < 0 or a >= nd:
            raise ValueError(f"axis {axis} out of range for ndim {nd}")
        return a

    # ------------------------------------------------------------------ element-wise
    def _unary(self, op, a, p0=0.0, p1=0.0) -> TensorData:
        self._f32(a)
        out = self._new(a.shape)
        check(self.lib.ah_unary(op, self._ptr(a), out._buf.ptr, a.size, p0, p1))
        return out

    def neg(self, a): return self._unary(ffi.NEG, a)
    def exp(self, a): return self._unary(ffi.EXP, a)
    def log(self, a): return self._unary(ffi.LOG, a)
    def sqrt(self, a): return self._unary(ffi.SQRT, a)
    def pow(self, a, e): return self._unary(ffi.POW, a, e)
    def scale(self, a, s): return self._unary(ffi.SCALE, a, s)
    def clamp(self, a, lo, hi): return self._unary(ffi.CLAMP, a, lo, hi)
    def gelu(self, a): return self._unary(ffi.GELU, a)
    def relu(self, a): return self._unary(ffi.RELU, a)
    def silu(self, a): return self._unary(ffi.SILU, a)
    def softCap(self, a, cap): return self._unary(ffi.SOFTCAP, a, cap)

    def _unary_bwd(self, op, x, g, p0=0.0, p1=0.0) -> TensorData:
        self._f32(x, g)
        if x.size != g.size:
            raise ValueError("backward: input and gradient sizes differ")
        out = self._new(g.shape)
        check(self.lib.ah_unary_bwd(op, self._ptr(x), self._ptr(g), out._buf.ptr, x.size, p0, p1))
        return out

    def geluBackward(self, x, g): return self._unary_bwd(ffi.GELU_BWD, x, g)
    def reluBackward(self, x, g): return self._unary_bwd(ffi.RELU_BWD, x, g)
    def siluBackward(self, x, g): return self._unary_bwd(ffi.SILU_BWD, x, g)
    def clampBackward(self, x, g, lo, hi): return self._unary_bwd(ffi.CLAMP_BWD, x, g, lo, hi)
    def softCapBackward(self, g, x, cap): return self._unary_bwd(ffi.SOFTCAP_BWD, x, g, cap)

    def siluMul(self, a, b) -> TensorData:
        self._f32(a, b)
        out = self._new(a.shape)
        check(self.lib.ah_silu_mul(self._ptr(a), self._ptr(b), out._buf.ptr, a.size))
        return out

    def siluMulBackward(self, a, b, g):
        self._f32(a, b, g)
        da, db = self._new(a.shape), self._new(b.shape)
        check(self.lib.ah_silu_mul_bwd(self._ptr(a), self._ptr(b), self._ptr(g), da._buf.ptr, db._buf.ptr, a.size))
        return [da, db]

    # ---- per-channel mixtures of activation bases: not part of the reference interface (it composes them from separate
    # ops, gpt.ts:295-321); the model uses these when the backend offers them, the way the reference probes its optionals
    CHANNEL_BASES = ("silu", "relu", "gelu", "identity", "square")

    def _channel_args(self, x, coefs):
        """coefs: {basis name: [1, cols] tensor}.  Returns (mask, handle array, cols, rows)."""
        self._f32(x, *coefs.values())
        cols = x.shape[-1]
        mask, arr = 0, (C.c_uint64 * 5)()
        for name, t in coefs.items():
            k = self.CHANNEL_BASES.index(name)
            if t.size != cols:
                raise ValueError(f"channelAct: coefficient '{name}' has {t.size} entries for {cols} channels")
            mask |= 1 << k
            arr[k] = self._ptr(t)
        return mask, arr, cols, x.size // cols if cols else 0

    def channelAct(self, x: TensorData, coefs: dict) -> TensorData:
        """out = sum over the given bases of coef[channel] * basis(x): the universal / kan_spline MLP activations in one pass."""
        mask, arr, cols, rows = self._channel_args(x, coefs)
        out = self._new(x.shape)
        check(self.lib.ah_channel_act(ffi.F32, self._ptr(x), arr, mask, out._buf.ptr, rows, cols))
        return out

    def channelActBackward(self, x: TensorData, coefs: dict, g: TensorData):
        """Returns (dx, {basis name: d coef [1, cols]})."""
        self._f32(g)
        mask, arr, cols, rows = self._channel_args(x, coefs)
        dx = self._new(x.shape)
        dco = {name: self._new(t.shape) for name, t in coefs.items()}
        darr = (C.c_uint64 * 5)()
        for name, t in dco.items():
            darr[self.CHANNEL_BASES.index(name)] = t._buf.ptr
        check(self.lib.ah_channel_act_bwd(ffi.F32, self._ptr(x), arr, mask, self._ptr(g), dx._buf.ptr, darr, 0, rows, cols))
        return dx, dco

    def residualDropoutAdd(self, residual, projected, mask) -> TensorData:
        self._f32(residual, projected)
        out = self._new(residual.shape)
        check(self.lib.ah_residual_dropout_add(self._ptr(residual), self._ptr(projected), self._ptr(mask) if mask is not None else 0,
                                               out._buf.ptr, residual.size))
        return out

    def dropoutMask(self, shape, seed, counter, p) -> TensorData:
        out = self._new(shape)
        check(self.lib.ah_dropout_mask(out._buf.ptr, shapeSize(shape), _i32(seed), _i32(counter), p))
        return out

    def addInplace(self, a, b):
        self._f32(a, b)
        if a.size != b.size:
            raise ValueError("addInplace: size mismatch")
        check(self.lib.ah_add_inplace(self._ptr(a), self._ptr(b), a.size))
        self._dirty(a)

    def scaleInplace(self, a, s):
        self._f32(a)
        check(self.lib.ah_scale_inplace(self._ptr(a), s, a.size))
        self._dirty(a)

    # ------------------------------------------------------------------ nn
    def embedding(self, weight: TensorData, indices: TensorData) -> TensorData:
        self._f32(weight)
        vocab, dim = weight.shape
        out = self._new(tuple(indices.shape) + (dim,))
        check(self.lib.ah_embedding(self._ptr(weight), self._ptr(indices), out._buf.ptr, indices.size, dim, vocab, ffi.F32))
        return out

    def embeddingBackward(self, indices, gradOutput, vocabSize) -> TensorData:
        self._f32(gradOutput)
        dim = gradOutput.shape[-1]
        out = self._new((vocabSize, dim))
        check(self.lib.ah_embedding_bwd(self._ptr(indices), self._ptr(gradOutput), out._buf.ptr, indices.size, dim, vocabSize, 0))
        return out

    def layerNorm(self, x, weight, bias, eps) -> TensorData:
        self._f32(x, weight, bias)
        dim = x.shape[-1]
        if weight.size != dim or bias.size != dim:
            raise ValueError("layerNorm: weight/bias length must equal the last dimension")
        out = self._new(x.shape)
        check(self.lib.ah_layernorm(self._ptr(x), self._ptr(weight), self._ptr(bias), out._buf.ptr, x.size // max(1, dim), dim, eps, ffi.F32, ffi.F32))
        return out

    def layerNormBackward(self, x, weight, gradOutput, eps) -> dict:
        self._f32(x, weight, gradOutput)
        dim = x.shape[-1]
        dx, dw, db = self._new(x.shape), self._new(weight.shape), self._new(weight.shape)
        check(self.lib.ah_layernorm_bwd(self._ptr(x), self._ptr(weight), self._ptr(gradOutput), ffi.F32, 0, dx._buf.ptr, 0, dw._buf.ptr,
                                        db._buf.ptr, x.size // max(1, dim), dim, eps, 0, ffi.F32))
        return {"dx": dx, "dw": dw, "db": db}

    def softmax(self, a, axis=None) -> TensorData:
        return self._softmax(a, axis, 0)

    def logSoftmax(self, a, axis=None) -> TensorData:
        return self._softmax(a, axis, 1)

    def _softmax(self, a, axis, log) -> TensorData:
        self._f32(a)
        ax = self._axis(len(a.shape) - 1 if axis is None else axis, len(a.shape))
        out = self._new(a.shape)
        check(self.lib.ah_softmax(self._ptr(a), out._buf.ptr, shapeSize(a.shape[:ax]), a.shape[ax], shapeSize(a.shape[ax + 1:]), log))
        return out

    def softmaxBackward(self, s, g) -> TensorData:
        """s * (g - sum(g*s)) over the last dim; one kernel for the five-op chain of ops.ts:688-700."""
        self._f32(s, g)
        out = self._new(s.shape)
        dim = s.shape[-1]
        check(self.lib.ah_softmax_bwd(self._ptr(s), self._ptr(g), out._buf.ptr, s.size // max(1, dim), dim))
        return out

    def crossEntropy(self, logits: TensorData, targets: TensorData) -> TensorData:
        self._f32(logits)
        N, Cc = logits.shape
        out = self._new(())
        lse = self._new((N,))
        check(self.lib.ah_cross_entropy(self._ptr(logits), ffi.F32, self._ptr(targets), out._buf.ptr, lse._buf.ptr, N, Cc))
        out._lse = lse      # kept for crossEntropyBackward on the same logits
        logits._ce_lse = lse
        return out

    def crossEntropyBackward(self, logits, targets, gradOutput) -> TensorData:
        self._f32(logits, gradOutput)
        N, Cc = logits.shape
        lse = getattr(logits, "_ce_lse", None)
        own = False
        if lse is None or lse._buf is None:
            tmp = self._new(())
            lse = self._new((N,))
            own = True
            check(self.lib.ah_cross_entropy(self._ptr(logits), ffi.F32, self._ptr(targets), tmp._buf.ptr, lse._buf.ptr, N, Cc))
            self.releaseGpuTensor(tmp)
        out = self._new((N, Cc))
        check(self.lib.ah_cross_entropy_bwd(self._ptr(logits), ffi.F32, self._ptr(targets), lse._buf.ptr, self._ptr(gradOutput), 1.0,
                                            out._buf.ptr, N, Cc))
        if own:
            self.releaseGpuTensor(lse)
        return out

    # ------------------------------------------------------------------ reshape / slice
    def reshape(self, a: TensorData, shape) -> TensorData:
        if shapeSize(shape) != shapeSize(a.shape):
            raise ValueError(f"Cannot reshape [{a.shape}] to [{tuple(shape)}]: size mismatch")
        return self._view(a, shape)

    def transpose(self, a: TensorData, dim0: int, dim1: int) -> TensorData:
        nd = len(a.shape)
        d0, d1 = self._axis(dim0, nd), self._axis(dim1, nd)
        ns = list(a.shape)
        ns[d0], ns[d1] = a.shape[d1], a.shape[d0]
        self._words(a)
        out = self._new(ns, a.dtype)
        check(self.lib.ah_transpose(self._ptr(a), out._buf.ptr, nd, ffi.shape_arr(a.shape), d0, d1))
        return out

    def slice(self, a: TensorData, starts, ends) -> TensorData:
        self._words(a)
        out = self._new([e - s for s, e in zip(starts, ends)], a.dtype)
        check(self.lib.ah_slice(self._ptr(a), out._buf.ptr, len(a.shape), ffi.shape_arr(a.shape), ffi.shape_arr(starts), ffi.shape_arr(ends)))
        return out

    def scatterSlice(self, grad: TensorData, origShape, starts, ends) -> TensorData:
        self._words(grad)
        out = self._new(origShape, grad.dtype)
        check(self.lib.ah_scatter_slice(self._ptr(grad), out._buf.ptr, len(origShape), ffi.shape_arr(grad.shape), ffi.shape_arr(origShape),
                                        ffi.shape_arr(starts)))
        return out

    def sliceQkv(self, a: TensorData):
        rows, c3 = a.shape
        d = c3 // 3
        self._words(a)
        q, k, v = self._new((rows, d)), self._new((rows, d)), self._new((rows, d))
        check(self.lib.ah_slice_qkv(self._ptr(a), q._buf.ptr, k._buf.ptr, v._buf.ptr, rows, d))
        return [q, k, v]

    def cat(self, tensors: List[TensorData], axis: int) -> TensorData:
        if not tensors:
            raise ValueError("cat: empty tensor list")
        nd = len(tensors[0].shape)
        ax = self._axis(axis, nd)
        oshape = list(tensors[0].shape)
        for t in tensors[1:]:
            for d in range(nd):
                if d == ax:
                    oshape[d] += t.shape[d]
                elif t.shape[d] != oshape[d]:
                    raise ValueError(f"cat: shape mismatch at dim {d}")
        self._words(*tensors)
        out = self._new(oshape, tensors[0].dtype)
        off = 0
        for t in tensors:
            check(self.lib.ah_cat_part(self._ptr(t), out._buf.ptr, nd, ffi.shape_arr(t.shape), ffi.shape_arr(oshape), ax, off))
            off += t.shape[ax]
        return out

    def broadcast(self, a: TensorData, targetShape) -> TensorData:
        nd = len(targetShape)
        src = (1,) * (nd - len(a.shape)) + tuple(a.shape)
        self._words(a)
        out = self._new(targetShape, a.dtype)
        check(self.lib.ah_broadcast(self._ptr(a), out._buf.ptr, nd, ffi.shape_arr(targetShape), ffi.shape_arr(self._bstrides(src, targetShape))))
        return out

    def castDtype(self, a: TensorData, dtype: str) -> TensorData:
        if dtype == a.dtype:
            return a
        out = self._new(a.shape, dtype)
        check(self.lib.ah_cast(self._ptr(a), ffi.DTYPE_CODE[a.store], out._buf.ptr, ffi.DTYPE_CODE[dtype], a.size))
        return out

    def castStore(self, a: TensorData, store: str) -> TensorData:
        """Internal storage cast f32 <-> bf16 (the tensor stays "f32" to callers: packages/core/src/types.ts:6 has no bf16)."""
        if a.store == store:
            return a
        out = self._new(a.shape, a.dtype, store)
        check(self.lib.ah_cast(self._ptr(a), ffi.DTYPE_CODE[a.store], out._buf.ptr, ffi.DTYPE_CODE[store], a.size))
        return out

    # ------------------------------------------------------------------ utility
    def argmax(self, a: TensorData, axis=None) -> TensorData:
        self._f32(a)
        if axis is None:
            out = self._new((), "i32")
            check(self.lib.ah_argmax(self._ptr(a), out._buf.ptr, 1, a.size, 1))
            return out
        ax = self._axis(axis, len(a.shape))
        oshape = [d for i, d in enumerate(a.shape) if i != ax] or [1]
        out = self._new(oshape, "i32")
        check(self.lib.ah_argmax(self._ptr(a), out._buf.ptr, shapeSize(a.shape[:ax]), a.shape[ax], shapeSize(a.shape[ax + 1:])))
        return out

    def topk(self, a: TensorData, k: int, axis=None):
        """Sampling-path helper, never called from the training step: host sort of a device read-back with the
        reference's ordering (descending value; cpu_ref.ts:758-819)."""
        nd = len(a.shape)
        ax = self._axis(nd - 1 if axis is None else axis, nd)
        if k > a.shape[ax]:
            raise ValueError(f"topk: k={k} exceeds axis size {a.shape[ax]}")
        arr = np.moveaxis(a.data.reshape(a.shape), ax, -1)
        idx = np.argsort(-arr, axis=-1, kind="stable")[..., :k]
        vals = np.take_along_axis(arr, idx, -1)
        oshape = list(a.shape)
        oshape[ax] = k
        return {"values": TensorData(oshape, a.dtype, np.moveaxis(vals, -1, ax)),
                "indices": TensorData(oshape, "i32", np.moveaxis(idx, -1, ax).astype(np.int32))}

    def gather(self, a: TensorData, axis: int, indices: TensorData) -> TensorData:
        """Not on the training path (cpu_ref.ts:821-845): host gather of a read-back."""
        ax = self._axis(axis, len(a.shape))
        out = np.take_along_axis(a.data.reshape(a.shape), indices.data.reshape(indices.shape).astype(np.int64), ax)
        return TensorData(indices.shape, a.dtype, out)

    def clone(self, a: TensorData) -> TensorData:
        out = self._new(a.shape, a.dtype, a.store)
        check(self.lib.ah_copy(out._buf.ptr, self._ptr(a), a.size * ffi.DTYPE_BYTES[a.store]))
        return out

    def equal(self, a: TensorData, b: TensorData) -> bool:
        return a.shape == b.shape and a.dtype == b.dtype and bool(np.all(a.data == b.data))

    def allClose(self, a: TensorData, b: TensorData, atol=1e-5, rtol=1e-8) -> bool:
        if a.shape != b.shape:
            return False
        x, y = a.data.astype(np.float64), b.data.astype(np.float64)
        return bool(np.all(~(np.abs(x - y) > atol + rtol * np.abs(y))))

    # ------------------------------------------------------------------ mask
    def causalMask(self, size: int) -> TensorData:
        out = self._new((size, size))
        check(self.lib.ah_causal_mask(out._buf.ptr, size))
        return out

    def maskedFill(self, a: TensorData, mask: TensorData, value: float) -> TensorData:
        self._f32(a, mask)
        out = self._new(a.shape)
        check(self.lib.ah_masked_fill(self._ptr(a), self._ptr(mask), out._buf.ptr, a.size, mask.size, value))
        return out

    # ------------------------------------------------------------------ flash attention
    def _flash_desc(self, Q, K, V, T, scale, softCap) -> ffi.AhFlash:
        BH, T2, D = Q.shape
        if T2 != T or K.shape != Q.shape or V.shape != Q.shape:
            raise ValueError("flashAttention: Q, K, V must all be [B*H, T, D]")
        f = ffi.AhFlash()
        f.dtype, f.batch, f.heads, f.seq, f.head_dim = ffi.F32, BH, 1, T, D
        for p in ("q", "k", "v", "o"):
            setattr(f, p + "_sb", T * D), setattr(f, p + "_sh", 0), setattr(f, p + "_st", D)
        f.scale, f.soft_cap = scale, softCap
        f.bwd_variant = self.flashBackwardVariant
        return f

    def flashAttention(self, Q, K, V, T, scale, softCap) -> dict:
        f = self._flash_desc(Q, K, V, T, scale, softCap)
        f.dtype = ffi.DTYPE_CODE[Q.store]
        out, lse = self._new(Q.shape, "f32", Q.store), self._new((Q.shape[0], T))
        f.q, f.k, f.v, f.o, f.lse = self._ptr(Q), self._ptr(K), self._ptr(V), out._buf.ptr, lse._buf.ptr
        check(self.lib.ah_flash_fwd(C.byref(f)))
        return {"output": out, "lse": lse}

    def flashAttentionBackward(self, Q, K, V, O, dO, lse, T, scale, softCap) -> dict:
        f = self._flash_desc(Q, K, V, T, scale, softCap)
        f.dtype = ffi.DTYPE_CODE[Q.store]
        dQ, dK, dV = (self._new(Q.shape, "f32", Q.store) for _ in range(3))
        f.q, f.k, f.v, f.o, f.lse = self._ptr(Q), self._ptr(K), self._ptr(V), self._ptr(O), self._ptr(lse)
        f.d_o, f.dq, f.dk, f.dv = self._ptr(dO), dQ._buf.ptr, dK._buf.ptr, dV._buf.ptr
        check(self.lib.ah_flash_bwd(C.byref(f)))
        return {"dQ": dQ, "dK": dK, "dV": dV}

    def _qkv_desc(self, qkv: TensorData, Bt, T, H, scale, softCap, store) -> ffi.AhFlash:
        rows, c3 = qkv.shape
        Cc = c3 // 3
        D = Cc // H
        if rows != Bt * T or Cc * 3 != c3 or D * H != Cc:
            raise ValueError(f"attentionQkv: qkv {qkv.shape} does not match B={Bt}, T={T}, H={H}")
        f = ffi.AhFlash()
        f.dtype, f.batch, f.heads, f.seq, f.head_dim = ffi.DTYPE_CODE[store], Bt, H, T, D
        for p in ("q", "k", "v"):
            setattr(f, p + "_sb", T * c3), setattr(f, p + "_sh", D), setattr(f, p + "_st", c3)
        f.o_sb, f.o_sh, f.o_st = T * Cc, D, Cc
        f.scale, f.soft_cap = scale, softCap
        f.bwd_variant = self.flashBackwardVariant
        return f

    def attentionQkv(self, qkv: TensorData, Bt: int, T: int, nHead: int, scale: float, softCap: float) -> dict:
        """Causal multi-head attention on a fused [B*T, 3C] projection, heads addressed through strides; the output is
        [B*T, C] with heads merged.  Same function as the chain at packages/model/src/gpt.ts:255-279."""
        Cc = qkv.shape[1] // 3
        f = self._qkv_desc(qkv, Bt, T, nHead, scale, softCap, qkv.store)
        esz = ffi.DTYPE_BYTES[qkv.store]
        out = self._new((Bt * T, Cc), "f32", qkv.store)
        lse = self._new((Bt * nHead, T))
        base = self._ptr(qkv)
        f.q, f.k, f.v, f.o, f.lse = base, base + Cc * esz, base + 2 * Cc * esz, out._buf.ptr, lse._buf.ptr
        check(self.lib.ah_flash_fwd(C.byref(f)))
        return {"output": out, "lse": lse}

    def attentionQkvBackward(self, qkv, out, dOut, lse, Bt, T, nHead, scale, softCap) -> TensorData:
        Cc = qkv.shape[1] // 3
        f = self._qkv_desc(qkv, Bt, T, nHead, scale, softCap, qkv.store)
        esz = ffi.DTYPE_BYTES[qkv.store]
        dqkv = self._new(qkv.shape, "f32", qkv.store)
        base, dbase = self._ptr(qkv), dqkv._buf.ptr
        f.q, f.k, f.v, f.o, f.lse = base, base + Cc * esz, base + 2 * Cc * esz, self._ptr(out), self._ptr(lse)
        f.d_o, f.dq, f.dk, f.dv = self._ptr(dOut), dbase, dbase + Cc * esz, dbase + 2 * Cc * esz
        check(self.lib.ah_flash_bwd(C.byref(f)))
        return dqkv

    # ------------------------------------------------------------------ reductions / optimizer
    def sumOfSquares(self, data: TensorData) -> TensorData:
        self._f32(data)
        out = self._new((1,))
        check(self.lib.ah_sum_sq(self._ptr(data), data.size, out._buf.ptr))
        return out

    def totalSumOfSquares(self, tensors: Sequence[TensorData]) -> TensorData:
        """One scalar for the whole gradient set (packages/train/src/trainer.ts:1345-1349)."""
        total = self._new((1,))
        for t in tensors:
            self._f32(t)
        n = len(tensors)
        xs = (C.c_uint64 * max(n, 1))(*[self._ptr(t) for t in tensors])
        ns = (C.c_uint64 * max(n, 1))(*[t.size for t in tensors])
        check(self.lib.ah_sum_sq_list(xs, ns, n, total._buf.ptr))
        return total

    def checkFinite(self, data: TensorData) -> TensorData:
        self._f32(data)
        out = self._new((1,))
        check(self.lib.ah_check_finite(self._ptr(data), data.size, out._buf.ptr))
        return out

    def adamwStep(self, params, grads, m, v, lr, beta1, beta2, eps, weightDecay, bc1, bc2, gradScale=1.0):
        self._f32(params, grads, m, v)
        if not (params.size == grads.size == m.size == v.size):
            raise ValueError("adamwStep: params, grads, m, v must have the same size")
        h, dev = self._adam_hyper(lr, beta1, beta2, eps, weightDecay, bc1, bc2, gradScale)
        check(self.lib.ah_adamw(self._ptr(params), self._ptr(grads), self._ptr(m), self._ptr(v), params.size, C.byref(h), dev, 0, 0))
        for t in (params, m, v):
            self._dirty(t)

    def _adam_hyper(self, lr, beta1, beta2, eps, weightDecay, bc1, bc2, gradScale):
        """The optimizer's scalars are the same for every tensor of a step except the weight decay (optimizers.ts:54-94): they
        are written to a small device struct once per step, which the kernel reads, and the by-value argument carries only
        the weight decay.  A recorded step plan then needs no node rewritten when the learning rate moves."""
        key = (lr, beta1, beta2, eps, bc1, bc2, gradScale)
        if self._hyper_dev is None:
            self._hyper_dev = _Buf(self.lib, C.sizeof(ffi.AhAdamW))
        if key != self._hyper_key:
            full = ffi.AhAdamW(lr, beta1, beta2, eps, 0.0, bc1, bc2, gradScale)
            check(self.lib.ah_upload(self._hyper_dev.ptr, C.byref(full), C.sizeof(full)))
            self._hyper_key = key
        return ffi.AhAdamW(0.0, 0.0, 0.0, 0.0, weightDecay, 0.0, 0.0, 0.0), self._hyper_dev.ptr

    # The reference runs its other optimizers as host loops inside the optimizer classes (optimizers.ts:236-593), not
    # through the Backend interface; these device versions keep parameters and state resident.
    def lionStep(self, params, grads, m, lr, beta1, beta2, weightDecay, gradScale=1.0):
        self._f32(params, grads, m)
        if not (params.size == grads.size == m.size):
            raise ValueError("lionStep: params, grads, m must have the same size")
        h = ffi.AhLion(lr, beta1, beta2, weightDecay, gradScale)
        check(self.lib.ah_lion(self._ptr(params), self._ptr(grads), self._ptr(m), params.size, C.byref(h)))
        self._dirty(params), self._dirty(m)

    def sgdStep(self, params, grads, lr, gradScale=1.0):
        self._f32(params, grads)
        if params.size != grads.size:
            raise ValueError("sgdStep: params and grads must have the same size")
        check(self.lib.ah_sgd(self._ptr(params), self._ptr(grads), params.size, lr, gradScale))
        self._dirty(params)

    def adafactorStep2d(self, params, grads, vr, vc, lr, beta2, eps, clipThreshold, weightDecay, gradScale=1.0):
        self._f32(params, grads, vr, vc)
        rows, cols = params.shape
        if grads.size != params.size or vr.size != rows or vc.size != cols:
            raise ValueError("adafactorStep2d: grads / vr / vc do not match the parameter's shape")
        h = ffi.AhAdafactor(lr, beta2, eps, clipThreshold, weightDecay, gradScale)
        check(self.lib.ah_adafactor_2d(self._ptr(params), self._ptr(grads), self._ptr(vr), self._ptr(vc), rows, cols, C.byref(h)))
        for t in (params, vr, vc):
            self._dirty(t)

    def adafactorStepFlat(self, params, grads, v, lr, beta2, eps, clipThreshold, weightDecay, gradScale=1.0):
        self._f32(params, grads, v)
        if not (params.size == grads.size == v.size):
            raise ValueError("adafactorStepFlat: params, grads, v must have the same size")
        h = ffi.AhAdafactor(lr, beta2, eps, clipThreshold, weightDecay, gradScale)
        check(self.lib.ah_adafactor_flat(self._ptr(params), self._ptr(grads), self._ptr(v), params.size, C.byref(h)))
        self._dirty(params), self._dirty(v)


def _i32(x: int) -> int:
    x &= 0xFFFFFFFF
    return x - (1 << 32) if x >= (1 << 31) else x
