"""TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.

Python face of the CPU oracle: a `CpuRef` object whose methods restate the reference's
`CpuRefBackend` (packages/tensor/src/cpu_ref.ts:109-912) one for one, implemented by the C loops
in cpu_ref.c (f32 storage, f64 intermediates, reference loop order).  Tensors are plain
`TD(shape, dtype, data)` records like the reference's `TensorData`
(packages/core/src/interfaces.ts:31-35).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module.
"""
from __future__ import annotations

import ctypes as C
import math
import os
import subprocess
from dataclasses import dataclass
from typing import List, Sequence, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


def build(force: bool = False) -> str:
    """Compile cpu_ref.c -> liboracle.so with gcc (about a second)."""
    src = os.path.join(_HERE, "cpu_ref.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-s", "-C", _HERE, "-B", "liboracle.so"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_rng_next.restype = C.c_double
        _lib.orc_rng_next_gauss.restype = C.c_double
        _lib.orc_binary.restype = C.c_int64
        _lib.orc_cross_entropy.restype = C.c_float
        _lib.orc_sum_sq.restype = C.c_double
        _lib.orc_check_finite.restype = C.c_float
    return _lib


def _fp(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _i64(seq: Sequence[int]):
    arr = (C.c_int64 * max(1, len(seq)))(*[int(x) for x in seq])
    return arr


def _d(x: float):
    return C.c_double(float(x))


def _n(x: int):
    return C.c_int64(int(x))


@dataclass
class TD:
    """Mirror of the reference's TensorData: row-major contiguous typed array + shape."""
    shape: Tuple[int, ...]
    dtype: str
    data: np.ndarray

    def __post_init__(self):
        self.shape = tuple(int(s) for s in self.shape)


def shape_size(shape) -> int:
    s = 1
    for d in shape:
        s *= int(d)
    return s


def f32(data, shape=None) -> TD:
    a = np.ascontiguousarray(np.asarray(data, dtype=np.float32)).reshape(-1)
    if shape is None:
        shape = np.asarray(data).shape
    assert shape_size(shape) == a.size
    return TD(tuple(shape), "f32", a.copy())


def i32(data, shape=None) -> TD:
    a = np.ascontiguousarray(np.asarray(data, dtype=np.int32)).reshape(-1)
    if shape is None:
        shape = np.asarray(data).shape
    return TD(tuple(shape), "i32", a.copy())


def _norm_axis(axis: int, nd: int) -> int:
    a = axis + nd if axis < 0 else axis
    if a < 0 or a >= nd:
        raise ValueError(f"axis {axis} out of range for ndim {nd}")
    return a


class SeededRng:
    """packages/core/src/rng.ts:6-68 (state lives in the C struct)."""

    class _S(C.Structure):
        _fields_ = [("s0", C.c_int32), ("s1", C.c_int32), ("has_spare", C.c_int), ("spare", C.c_double)]

    def __init__(self, seed: int = 42):
        self._s = SeededRng._S()
        self._seed = seed
        lib().orc_rng_seed(C.byref(self._s), C.c_int32(_to_i32(seed)))

    def seed(self, s: int):
        self._seed = s
        lib().orc_rng_seed(C.byref(self._s), C.c_int32(_to_i32(s)))

    def next(self) -> float:
        return lib().orc_rng_next(C.byref(self._s))

    def nextGauss(self) -> float:
        return lib().orc_rng_next_gauss(C.byref(self._s))

    def fill_gauss(self, n: int, std: float) -> np.ndarray:
        out = np.empty(n, dtype=np.float32)
        lib().orc_rng_fill_gauss(C.byref(self._s), _fp(out), _n(n), _d(std))
        return out

    def fill_uniform(self, n: int) -> np.ndarray:
        out = np.empty(n, dtype=np.float64)
        lib().orc_rng_fill_uniform(C.byref(self._s), _fp(out), _n(n))
        return out


def _to_i32(x: int) -> int:
    x &= 0xFFFFFFFF
    return x - (1 << 32) if x >= (1 << 31) else x


class CpuRef:
    """Method-for-method restatement of CpuRefBackend (cpu_ref.ts:109-912)."""

    name = "cpu_ref"

    # -- creation (cpu_ref.ts:115-146) -------------------------------------------------------
    def zeros(self, shape, dtype="f32") -> TD:
        return TD(tuple(shape), dtype, np.zeros(shape_size(shape), dtype=_np_dtype(dtype)))

    def ones(self, shape, dtype="f32") -> TD:
        return TD(tuple(shape), dtype, np.ones(shape_size(shape), dtype=_np_dtype(dtype)))

    def full(self, shape, value, dtype="f32") -> TD:
        return TD(tuple(shape), dtype, np.full(shape_size(shape), value, dtype=_np_dtype(dtype)))

    def fromArray(self, data, shape, dtype="f32") -> TD:
        if len(data) != shape_size(shape):
            raise ValueError(f"Data length {len(data)} does not match shape size {shape_size(shape)}")
        return TD(tuple(shape), dtype, np.asarray(data, dtype=_np_dtype(dtype)).copy())

    # -- math (cpu_ref.ts:150-164) -----------------------------------------------------------
    def _binary(self, op: int, a: TD, b: TD) -> TD:
        nd = max(len(a.shape), len(b.shape))
        res = (C.c_int64 * 8)()
        sa = (C.c_int64 * 8)()
        sb = (C.c_int64 * 8)()
        size = lib().orc_broadcast_shape(_i64(a.shape), len(a.shape), _i64(b.shape), len(b.shape), res, sa, sb)
        if size < 0:
            raise ValueError(f"Cannot broadcast shapes {a.shape} and {b.shape}")
        out = np.empty(size, dtype=np.float32)
        lib().orc_binary(op, _fp(a.data), _i64(a.shape), len(a.shape), _fp(b.data), _i64(b.shape), len(b.shape), _fp(out))
        return TD(tuple(res[i] for i in range(nd)), "f32", out)

    def add(self, a, b): return self._binary(0, a, b)
    def sub(self, a, b): return self._binary(1, a, b)
    def mul(self, a, b): return self._binary(2, a, b)
    def div(self, a, b): return self._binary(3, a, b)

    def matmul(self, a: TD, b: TD) -> TD:
        """cpu_ref.ts:166-258, batch-dim broadcasting resolved here as lines 184-243 do."""
        if len(a.shape) < 2 or len(b.shape) < 2:
            raise ValueError("matmul requires at least 2D tensors")
        M, K = a.shape[-2], a.shape[-1]
        N = b.shape[-1]
        if b.shape[-2] != K:
            raise ValueError(f"matmul shape mismatch: {a.shape} x {b.shape}")
        aB, bB = list(a.shape[:-2]), list(b.shape[:-2])
        nb = max(len(aB), len(bB))
        batch_shape = []
        for i in range(nb):
            ai = aB[len(aB) - 1 - i] if i < len(aB) else 1
            bi = bB[len(bB) - 1 - i] if i < len(bB) else 1
            if ai != bi and ai != 1 and bi != 1:
                raise ValueError("matmul batch shape mismatch")
            batch_shape.insert(0, max(ai, bi))
        batch = shape_size(batch_shape)
        aStr, bStr = [], []
        st = M * K
        for i in range(len(aB) - 1, -1, -1):
            aStr.insert(0, 0 if aB[i] == 1 else st)
            st *= aB[i]
        st = K * N
        for i in range(len(bB) - 1, -1, -1):
            bStr.insert(0, 0 if bB[i] == 1 else st)
            st *= bB[i]
        a_off, b_off = [], []
        for bt in range(batch):
            rem, ao, bo = bt, 0, 0
            for d in range(len(batch_shape) - 1, -1, -1):
                c = rem % batch_shape[d]
                rem = (rem - c) // batch_shape[d]
                ai = d - (len(batch_shape) - len(aB))
                bi = d - (len(batch_shape) - len(bB))
                if ai >= 0:
                    ao += c * aStr[ai]
                if bi >= 0:
                    bo += c * bStr[bi]
            a_off.append(ao)
            b_off.append(bo)
        out = np.empty(batch * M * N, dtype=np.float32)
        lib().orc_matmul(_fp(a.data), _fp(b.data), _fp(out), _n(batch), _i64(a_off), _i64(b_off), _n(M), _n(K), _n(N))
        return TD(tuple(batch_shape) + (M, N), "f32", out)

    def sum(self, a: TD, axis=None, keepdims=False) -> TD:
        return self._reduce(a, axis, keepdims, 0)

    def mean(self, a: TD, axis=None, keepdims=False) -> TD:
        return self._reduce(a, axis, keepdims, 1)

    def _reduce(self, a: TD, axis, keepdims, mean) -> TD:
        if axis is None:
            out = np.empty(1, dtype=np.float32)
            lib().orc_sum_all(_fp(a.data), _n(a.data.size), _fp(out), mean)
            return TD(tuple(1 for _ in a.shape) if keepdims else (), "f32", out)
        ax = _norm_axis(axis, len(a.shape))
        oshape = [d for i, d in enumerate(a.shape) if i != ax]
        out = np.empty(max(1, shape_size(oshape)), dtype=np.float32)
        lib().orc_sum_axis(_fp(a.data), _i64(a.shape), len(a.shape), ax, _fp(out), mean)
        if keepdims:
            oshape = [1 if i == ax else d for i, d in enumerate(a.shape)]
        return TD(tuple(oshape), "f32", out)

    # -- element-wise (cpu_ref.ts:334-360, 422-435) ------------------------------------------
    def _unary(self, op, a: TD, p0=0.0, p1=0.0) -> TD:
        out = np.empty(a.data.size, dtype=np.float32)
        lib().orc_unary(op, _fp(a.data), _fp(out), _n(a.data.size), _d(p0), _d(p1))
        return TD(a.shape, "f32", out)

    def neg(self, a): return self._unary(0, a)
    def exp(self, a): return self._unary(1, a)
    def log(self, a): return self._unary(2, a)
    def sqrt(self, a): return self._unary(3, a)
    def pow(self, a, e): return self._unary(4, a, e)
    def scale(self, a, s): return self._unary(5, a, s)
    def clamp(self, a, lo, hi): return self._unary(6, a, lo, hi)
    def gelu(self, a): return self._unary(7, a)
    def relu(self, a): return self._unary(8, a)
    def silu(self, a): return self._unary(9, a)

    # -- nn (cpu_ref.ts:364-563) -------------------------------------------------------------
    def embedding(self, weight: TD, indices: TD) -> TD:
        dim = weight.shape[1]
        n = indices.data.size
        out = np.empty(n * dim, dtype=np.float32)
        idx = np.ascontiguousarray(indices.data, dtype=np.int32)
        lib().orc_embedding(_fp(weight.data), _n(dim), _n(weight.shape[0]), _fp(idx), _n(n), _fp(out))
        return TD(tuple(indices.shape) + (dim,), "f32", out)

    def layerNorm(self, x: TD, weight: TD, bias: TD, eps: float) -> TD:
        dim = x.shape[-1]
        outer = x.data.size // dim
        out = np.empty(x.data.size, dtype=np.float32)
        lib().orc_layernorm(_fp(x.data), _fp(weight.data), _fp(bias.data), _d(eps), _n(outer), _n(dim), _fp(out))
        return TD(x.shape, "f32", out)

    def softmax(self, a: TD, axis=None) -> TD:
        ax = _norm_axis(len(a.shape) - 1 if axis is None else axis, len(a.shape))
        out = np.empty(a.data.size, dtype=np.float32)
        lib().orc_softmax(_fp(a.data), _i64(a.shape), len(a.shape), ax, _fp(out))
        return TD(a.shape, "f32", out)

    def logSoftmax(self, a: TD, axis=None) -> TD:
        ax = _norm_axis(len(a.shape) - 1 if axis is None else axis, len(a.shape))
        out = np.empty(a.data.size, dtype=np.float32)
        lib().orc_log_softmax(_fp(a.data), _i64(a.shape), len(a.shape), ax, _fp(out))
        return TD(a.shape, "f32", out)

    def crossEntropy(self, logits: TD, targets: TD) -> TD:
        N, Cc = logits.shape
        scratch = np.empty(N * Cc, dtype=np.float32)
        tg = np.ascontiguousarray(targets.data, dtype=np.int32)
        v = lib().orc_cross_entropy(_fp(logits.data), _fp(tg), _n(N), _n(Cc), _fp(scratch))
        return TD((), "f32", np.array([v], dtype=np.float32))

    # -- reshape / slice (cpu_ref.ts:567-694) ------------------------------------------------
    def reshape(self, a: TD, shape) -> TD:
        if shape_size(shape) != shape_size(a.shape):
            raise ValueError(f"Cannot reshape {a.shape} to {tuple(shape)}: size mismatch")
        return TD(tuple(shape), a.dtype, a.data.copy())

    def transpose(self, a: TD, dim0: int, dim1: int) -> TD:
        nd = len(a.shape)
        d0, d1 = _norm_axis(dim0, nd), _norm_axis(dim1, nd)
        ns = list(a.shape)
        ns[d0], ns[d1] = a.shape[d1], a.shape[d0]
        out = np.empty(a.data.size, dtype=np.float32)
        lib().orc_transpose(_fp(a.data), _i64(a.shape), nd, d0, d1, _fp(out))
        return TD(tuple(ns), "f32", out)

    def slice(self, a: TD, starts, ends) -> TD:
        oshape = [e - s for s, e in zip(starts, ends)]
        out = np.empty(shape_size(oshape), dtype=np.float32)
        lib().orc_slice(_fp(a.data), _i64(a.shape), len(a.shape), _i64(starts), _i64(ends), _fp(out))
        return TD(tuple(oshape), "f32", out)

    def scatterSlice(self, grad: TD, origShape, starts, ends) -> TD:
        out = np.empty(shape_size(origShape), dtype=np.float32)
        lib().orc_scatter_slice(_fp(grad.data), _i64(grad.shape), _i64(origShape), len(origShape), _i64(starts), _fp(out))
        return TD(tuple(origShape), "f32", out)

    def cat(self, tensors: List[TD], axis: int) -> TD:
        """cpu_ref.ts:654-694 (pure data movement; numpy concatenate is the same permutation)."""
        if not tensors:
            raise ValueError("cat: empty tensor list")
        ax = _norm_axis(axis, len(tensors[0].shape))
        arrs = [t.data.reshape(t.shape) for t in tensors]
        out = np.concatenate(arrs, axis=ax)
        return TD(out.shape, tensors[0].dtype, np.ascontiguousarray(out).reshape(-1))

    # -- utility (cpu_ref.ts:698-876) --------------------------------------------------------
    def argmax(self, a: TD, axis=None) -> TD:
        if axis is None:
            out = np.empty(1, dtype=np.int32)
            lib().orc_argmax(_fp(a.data), _i64(a.shape), len(a.shape), -1, _fp(out))
            return TD((), "i32", out)
        ax = _norm_axis(axis, len(a.shape))
        oshape = [d for i, d in enumerate(a.shape) if i != ax] or [1]
        out = np.empty(shape_size(oshape), dtype=np.int32)
        lib().orc_argmax(_fp(a.data), _i64(a.shape), len(a.shape), ax, _fp(out))
        return TD(tuple(oshape), "i32", out)

    def clone(self, a: TD) -> TD:
        return TD(a.shape, a.dtype, a.data.copy())

    def equal(self, a: TD, b: TD) -> bool:
        return a.shape == b.shape and a.dtype == b.dtype and bool(np.all(a.data == b.data))

    def allClose(self, a: TD, b: TD, atol=1e-5, rtol=1e-8) -> bool:
        if a.shape != b.shape:
            return False
        diff = np.abs(a.data.astype(np.float64) - b.data.astype(np.float64))
        return bool(np.all(~(diff > atol + rtol * np.abs(b.data.astype(np.float64)))))

    # -- mask (cpu_ref.ts:880-911) -----------------------------------------------------------
    def causalMask(self, size: int) -> TD:
        out = np.empty(size * size, dtype=np.float32)
        lib().orc_causal_mask(_n(size), _fp(out))
        return TD((size, size), "f32", out)

    def maskedFill(self, a: TD, mask: TD, value: float) -> TD:
        out = np.empty(a.data.size, dtype=np.float32)
        lib().orc_masked_fill(_fp(a.data), _n(a.data.size), _fp(mask.data), _n(mask.data.size), _d(value), _fp(out))
        return TD(a.shape, "f32", out)


def _np_dtype(dtype: str):
    return {"f32": np.float32, "f64": np.float64, "i32": np.int32, "f16": np.uint16}[dtype]


# ---- free functions restating CPU fallbacks that live in autograd / train -----------------------

def gelu_backward(x: TD, g: TD, fused: bool = False) -> TD:
    """packages/autograd/src/ops.ts:405-417 (fused=False) / 449-463 (fused=True)."""
    out = np.empty(x.data.size, dtype=np.float32)
    lib().orc_gelu_bwd(_fp(x.data), _fp(g.data), _fp(out), _n(x.data.size), 1 if fused else 0)
    return TD(x.shape, "f32", out)


def relu_backward(x: TD, g: TD) -> TD:
    out = np.empty(x.data.size, dtype=np.float32)
    lib().orc_relu_bwd(_fp(x.data), _fp(g.data), _fp(out), _n(x.data.size))
    return TD(x.shape, "f32", out)


def silu_backward(x: TD, g: TD) -> TD:
    out = np.empty(x.data.size, dtype=np.float32)
    lib().orc_silu_bwd(_fp(x.data), _fp(g.data), _fp(out), _n(x.data.size))
    return TD(x.shape, "f32", out)


def clamp_backward(x: TD, g: TD, lo: float, hi: float) -> TD:
    out = np.empty(x.data.size, dtype=np.float32)
    lib().orc_clamp_bwd(_fp(x.data), _fp(g.data), _fp(out), _n(x.data.size), _d(lo), _d(hi))
    return TD(g.shape, "f32", out)


def layernorm_backward(x: TD, w: TD, g: TD, eps: float):
    """packages/autograd/src/ops.ts:523-569."""
    dim = x.shape[-1]
    n = x.data.size // dim
    dx = np.empty(x.data.size, dtype=np.float32)
    dw = np.empty(dim, dtype=np.float32)
    db = np.empty(dim, dtype=np.float32)
    lib().orc_layernorm_bwd(_fp(x.data), _fp(w.data), _fp(g.data), _d(eps), _n(n), _n(dim), _fp(dx), _fp(dw), _fp(db))
    return TD(x.shape, "f32", dx), TD(w.shape, "f32", dw), TD(w.shape, "f32", db)


def cross_entropy_backward(logits: TD, targets: TD, g_scalar: float) -> TD:
    """packages/autograd/src/ops.ts:713-727."""
    N, Cc = logits.shape
    out = np.empty(N * Cc, dtype=np.float32)
    tg = np.ascontiguousarray(targets.data, dtype=np.int32)
    lib().orc_cross_entropy_bwd(_fp(logits.data), _fp(tg), _d(g_scalar), _n(N), _n(Cc), _fp(out))
    return TD((N, Cc), "f32", out)


def embedding_backward(indices: TD, g: TD, vocab: int) -> TD:
    """packages/autograd/src/ops.ts:495-505."""
    dim = g.shape[-1]
    n = indices.data.size
    out = np.empty(vocab * dim, dtype=np.float32)
    idx = np.ascontiguousarray(indices.data, dtype=np.int32)
    lib().orc_embedding_bwd(_fp(idx), _n(n), _fp(g.data), _n(dim), _n(vocab), _fp(out))
    return TD((vocab, dim), "f32", out)


def sum_sq(a: TD) -> float:
    """packages/train/src/trainer.ts:488-496."""
    return lib().orc_sum_sq(_fp(a.data), _n(a.data.size))


def check_finite(a: TD) -> float:
    return lib().orc_check_finite(_fp(a.data), _n(a.data.size))


def adamw_step(p: TD, g: TD, m: np.ndarray, v: np.ndarray, lr, beta1, beta2, eps, wd, bc1, bc2, grad_scale=1.0):
    """packages/train/src/optimizers.ts:76-92 (in place on p.data, m, v)."""
    lib().orc_adamw(_fp(p.data), _fp(g.data), _fp(m), _fp(v), _n(p.data.size), _d(lr), _d(beta1), _d(beta2),
                    _d(eps), _d(wd), _d(bc1), _d(bc2), _d(grad_scale))


def dropout_mask(seed: int, counter: int, p: float, n: int) -> np.ndarray:
    """packages/autograd/src/ops.ts:41-51,74-81."""
    out = np.empty(n, dtype=np.float32)
    lib().orc_dropout_mask(C.c_int32(_to_i32(seed)), C.c_int32(_to_i32(counter)), _d(p), _fp(out), _n(0), _n(n))
    return out


def dropout_mask_range(seed: int, counter: int, p: float, lo: int, hi: int) -> np.ndarray:
    """Elements [lo, hi) of the mask (the hash depends on the element index only, so a window needs no prefix)."""
    out = np.empty(hi - lo, dtype=np.float32)
    lib().orc_dropout_mask(C.c_int32(_to_i32(seed)), C.c_int32(_to_i32(counter)), _d(p), _fp(out), _n(lo), _n(hi))
    return out
