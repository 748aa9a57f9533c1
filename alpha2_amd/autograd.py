"""Tape autograd over a `Backend` -- the caller of the op boundary, mirroring the reference's
packages/autograd/src/tape.ts:29-201 (Variable, Tape.backward/clear with the explicit-release protocol) and
packages/autograd/src/ops.ts:99-974 (the differentiable ops and which optional backend ops they prefer).

Every op takes a `Ctx(tape, backend, dropoutRng, release)` plus Variables and returns a Variable whose backward
closure issues backend calls only: with HipBackend nothing is read back to the host inside forward or backward.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, List, Optional, Sequence, Tuple

import numpy as np

from .backend import TensorData, shapeSize

Release = Optional[Callable[[TensorData], None]]


class Variable:
    _next_id = 0

    def __init__(self, data: TensorData, requiresGrad: bool = False):
        self.id = Variable._next_id
        Variable._next_id += 1
        self.data = data
        self.grad: Optional[TensorData] = None
        self.requiresGrad = requiresGrad


class _Entry:
    __slots__ = ("output", "inputs", "backward", "cleanup")

    def __init__(self, output, inputs, backward, cleanup=None):
        self.output, self.inputs, self.backward, self.cleanup = output, inputs, backward, cleanup


class Tape:
    def __init__(self):
        self.entries: List[_Entry] = []

    def record(self, output: Variable, inputs: Sequence[Variable], backward, cleanup=None):
        self.entries.append(_Entry(output, list(inputs), backward, cleanup))

    @property
    def size(self) -> int:
        return len(self.entries)

    def backward(self, loss: Variable, backend, releaseTensor: Release = None, initialGrad: Optional[TensorData] = None):
        """tape.ts:60-157: reverse walk; first gradient is cloned, later ones accumulate in place; each consumed
        gradient and each entry's forward activation is released as soon as nothing later can read it."""
        loss.grad = initialGrad if initialGrad is not None else backend.ones(loss.data.shape, loss.data.dtype)
        released = {}        # id -> the tensor itself: keeping it alive keeps its id from being handed to a new object

        def release_once(td):
            if releaseTensor is None or td is None or id(td) in released:
                return
            released[id(td)] = td
            releaseTensor(td)

        for entry in reversed(self.entries):
            out_grad = entry.output.grad
            if out_grad is None:
                if entry.cleanup:
                    entry.cleanup(releaseTensor)
                continue
            needs = None
            if any(not v.requiresGrad for v in entry.inputs):
                needs = [v.requiresGrad for v in entry.inputs]
            grads = entry.backward(out_grad, backend, releaseTensor, needs)
            uses = {}
            for inp, g in zip(entry.inputs, grads):
                if inp.requiresGrad and g is not None:
                    uses[id(g)] = uses.get(id(g), 0) + 1
            for inp, g in zip(entry.inputs, grads):
                if g is None:
                    continue
                if not inp.requiresGrad:
                    if id(g) not in uses:
                        release_once(g)
                    continue
                if inp.grad is not None:
                    if hasattr(backend, "addInplace"):
                        backend.addInplace(inp.grad, g)
                    else:
                        old = inp.grad
                        inp.grad = backend.add(inp.grad, g)
                        release_once(old)
                else:
                    inp.grad = backend.clone(g)
                uses[id(g)] -= 1
                if uses[id(g)] <= 0:
                    release_once(g)
            release_once(out_grad)
            entry.output.grad = None
            if releaseTensor is not None:
                release_once(entry.output.data)
                entry.output.data = None
            if entry.cleanup:
                entry.cleanup(releaseTensor)

    def clear(self, releaseTensor: Release = None, keepOutput: Optional[Variable] = None):
        """tape.ts:175-197."""
        for entry in self.entries:
            if releaseTensor is not None:
                keep = keepOutput is not None and entry.output.id == keepOutput.id
                if not keep and entry.output.data is not None:
                    releaseTensor(entry.output.data)
                if entry.output.grad is not None:
                    releaseTensor(entry.output.grad)
            if entry.cleanup:
                entry.cleanup(releaseTensor)
            entry.output.grad = None
        self.entries = []


def _to_i32(x: int) -> int:
    x = int(x) & 0xFFFFFFFF
    return x - (1 << 32) if x >> 31 else x


class DropoutRng:
    """Counter-based mask parameters (ops.ts:25-82); the mask itself is generated on the device."""

    def __init__(self, seed: int):
        self.seed, self.counter = _to_i32(seed), 0                    # `seed | 0`

    def reset(self, seed: int, counter: int = 0):
        self.seed, self.counter = _to_i32(seed), _to_i32(counter)

    def nextMaskParams(self):
        r = {"seed": self.seed, "counter": self.counter}
        self.counter += 1
        return r

    def saveCounter(self) -> int:
        return self.counter

    def restoreCounter(self, n: int):
        self.counter = n


@dataclass
class Ctx:
    tape: Tape
    backend: object
    dropoutRng: Optional[DropoutRng] = None
    release: Release = None


def _record(ctx: Ctx, data: TensorData, inputs, backward, cleanup=None) -> Variable:
    out = Variable(data, True)
    ctx.tape.record(out, inputs, backward, cleanup)
    return out


def _has(B, name: str) -> bool:
    return callable(getattr(B, name, None))


def _rel(release: Release, *tds):
    if release is not None:
        for t in tds:
            if t is not None:
                release(t)


# ---- helpers (ops.ts:878-935) -------------------------------------------------------------------------------
def _reduce_broadcast(B, grad: TensorData, target, release: Release = None) -> TensorData:
    target = tuple(target)
    if tuple(grad.shape) == target:
        return grad
    if len(target) == 0 or (len(target) == 1 and target[0] == 1 and len(grad.shape) > 1):
        return B.sum(grad)
    result = grad
    while len(result.shape) > len(target):
        prev = result
        result = B.sum(result, 0)
        if prev is not grad:
            _rel(release, prev)
    for i in range(len(target)):
        if target[i] == 1 and result.shape[i] != 1:
            prev = result
            result = B.sum(result, i, True)
            if prev is not grad:
                _rel(release, prev)
    return result


def _broadcast_to(B, t: TensorData, target) -> TensorData:
    target = tuple(target)
    if tuple(t.shape) == target:
        return t
    return B.broadcast(t, target)


# ---- arithmetic (ops.ts:99-161) -----------------------------------------------------------------------------
def add(ctx, a, b):
    sa, sb = a.data.shape, b.data.shape
    return _record(ctx, ctx.backend.add(a.data, b.data), [a, b],
                   lambda g, B, rel, n: [_reduce_broadcast(B, g, sa, rel), _reduce_broadcast(B, g, sb, rel)])


def sub(ctx, a, b):
    sa, sb = a.data.shape, b.data.shape

    def bw(g, B, rel, n):
        neg_g = B.neg(g)
        gb = _reduce_broadcast(B, neg_g, sb, rel)
        if gb is not neg_g:
            _rel(rel, neg_g)
        return [_reduce_broadcast(B, g, sa, rel), gb]
    return _record(ctx, ctx.backend.sub(a.data, b.data), [a, b], bw)


def mul(ctx, a, b):
    ad, bd = a.data, b.data

    def bw(g, B, rel, n):
        gxb, gxa = B.mul(g, bd), B.mul(g, ad)
        ga, gb = _reduce_broadcast(B, gxb, ad.shape, rel), _reduce_broadcast(B, gxa, bd.shape, rel)
        if ga is not gxb:
            _rel(rel, gxb)
        if gb is not gxa:
            _rel(rel, gxa)
        return [ga, gb]
    return _record(ctx, ctx.backend.mul(ad, bd), [a, b], bw)


def div(ctx, a, b):
    ad, bd = a.data, b.data

    def bw(g, B, rel, n):
        ga = B.div(g, bd)
        gxa, bsq = B.mul(g, ad), B.mul(bd, bd)
        ratio = B.div(gxa, bsq)
        gb = B.neg(ratio)
        _rel(rel, gxa, bsq, ratio)
        gar, gbr = _reduce_broadcast(B, ga, ad.shape, rel), _reduce_broadcast(B, gb, bd.shape, rel)
        if gar is not ga:
            _rel(rel, ga)
        if gbr is not gb:
            _rel(rel, gb)
        return [gar, gbr]
    return _record(ctx, ctx.backend.div(ad, bd), [a, b], bw)


def scale(ctx, a, s):
    return _record(ctx, ctx.backend.scale(a.data, s), [a], lambda g, B, rel, n: [B.scale(g, s)])


def neg(ctx, a):
    return _record(ctx, ctx.backend.neg(a.data), [a], lambda g, B, rel, n: [B.neg(g)])


# ---- matmul (ops.ts:165-234, 426-487) -----------------------------------------------------------------------
def matmul(ctx, a, b):
    ad, bd = a.data, b.data

    def bw(g, B, rel, needs):
        ga = gb = None
        if needs is None or needs[0]:
            if _has(B, "matmulTransposed"):
                ga = B.matmulTransposed(g, bd)                 # G @ B^T without materialising the transpose
            else:
                tB = B.transpose(bd, len(bd.shape) - 2, len(bd.shape) - 1)
                ga = B.matmul(g, tB)
                _rel(rel, tB)
        if needs is None or needs[1]:
            if _has(B, "matmulTransposedA"):
                gb = B.matmulTransposedA(ad, g)
            else:
                tA = B.transpose(ad, len(ad.shape) - 2, len(ad.shape) - 1)
                gb = B.matmul(tA, g)
                _rel(rel, tA)
        return [ga, gb]
    return _record(ctx, ctx.backend.matmul(ad, bd), [a, b], bw)


def _mt_forward(B, ad, bd):
    if _has(B, "matmulTransposed"):
        return B.matmulTransposed(ad, bd), None
    tB = B.transpose(bd, len(bd.shape) - 2, len(bd.shape) - 1)
    return B.matmul(ad, tB), tB


def _mt_backward(B, g, ad, bd, rel, needs):
    ga = gb = None
    if needs is None or needs[0]:
        ga = B.matmul(g, bd)
    if needs is None or needs[1]:
        if _has(B, "matmulTransposedA"):
            gb = B.matmulTransposedA(g, ad)
        else:
            tG = B.transpose(g, len(g.shape) - 2, len(g.shape) - 1)
            gb = B.matmul(tG, ad)
            _rel(rel, tG)
    return [ga, gb]


def matmulTransposed(ctx, a, b):
    ad, bd = a.data, b.data
    out, tB = _mt_forward(ctx.backend, ad, bd)
    live = [tB]

    def cleanup(rel):
        _rel(rel, live[0])
        live[0] = None
    return _record(ctx, out, [a, b], lambda g, B, rel, needs: _mt_backward(B, g, ad, bd, rel, needs), cleanup)


def matmulTransposedGelu(ctx, a, b):
    ad, bd = a.data, b.data
    B0 = ctx.backend
    mm, tB = _mt_forward(B0, ad, bd)
    live = [mm, tB]

    def cleanup(rel):
        _rel(rel, live[0], live[1])
        live[0] = live[1] = None

    def bw(g, B, rel, needs):
        dmm = B.geluBackward(mm, g)
        cleanup(rel)
        grads = _mt_backward(B, dmm, ad, bd, rel, needs)
        _rel(rel, dmm)
        return grads
    return _record(ctx, B0.gelu(mm), [a, b], bw, cleanup)


# ---- reductions (ops.ts:238-255) ----------------------------------------------------------------------------
def sum(ctx, a, axis=None, keepdims=False):      # noqa: A001 - mirrors the reference's export name
    sa = a.data.shape
    return _record(ctx, ctx.backend.sum(a.data, axis, keepdims), [a], lambda g, B, rel, n: [_broadcast_to(B, g, sa)])


def mean(ctx, a, axis=None, keepdims=False):
    sa = a.data.shape
    cnt = sa[axis + len(sa) if axis is not None and axis < 0 else axis] if axis is not None else shapeSize(sa)

    def bw(g, B, rel, n):
        ex = _broadcast_to(B, g, sa)
        r = B.scale(ex, 1 / cnt)
        if ex is not g:
            _rel(rel, ex)
        return [r]
    return _record(ctx, ctx.backend.mean(a.data, axis, keepdims), [a], bw)


# ---- element-wise (ops.ts:259-419) --------------------------------------------------------------------------
def exp(ctx, a):
    out = ctx.backend.exp(a.data)
    return _record(ctx, out, [a], lambda g, B, rel, n: [B.mul(g, out)])


def log(ctx, a):
    ad = a.data
    return _record(ctx, ctx.backend.log(ad), [a], lambda g, B, rel, n: [B.div(g, ad)])


def sqrt(ctx, a):
    out = ctx.backend.sqrt(a.data)

    def bw(g, B, rel, n):
        den = B.scale(out, 2)
        r = B.div(g, den)
        _rel(rel, den)
        return [r]
    return _record(ctx, out, [a], bw)


def relu(ctx, a):
    ad = a.data
    return _record(ctx, ctx.backend.relu(ad), [a], lambda g, B, rel, n: [B.reluBackward(ad, g)])


def clamp(ctx, a, lo, hi):
    ad = a.data
    return _record(ctx, ctx.backend.clamp(ad, lo, hi), [a], lambda g, B, rel, n: [B.clampBackward(ad, g, lo, hi)])


def softCap(ctx, a, cap):
    ad = a.data
    return _record(ctx, ctx.backend.softCap(ad, cap), [a], lambda g, B, rel, n: [B.softCapBackward(g, ad, cap)])


def silu(ctx, a):
    ad = a.data
    return _record(ctx, ctx.backend.silu(ad), [a], lambda g, B, rel, n: [B.siluBackward(ad, g)])


def siluMul(ctx, a, b):
    ad, bd = a.data, b.data
    return _record(ctx, ctx.backend.siluMul(ad, bd), [a, b], lambda g, B, rel, n: B.siluMulBackward(ad, bd, g))


def channelAct(ctx, a, coefs: dict):
    """sum_k coef_k[channel] * basis_k(a) in one backend pass (bases: silu, relu, gelu, identity, square); gradients flow to
    `a` and to every coefficient.  Same function as the chain of silu / relu / gelu / mul / add the reference records for its
    universal and kan_spline activations (gpt.ts:295-321)."""
    ad = a.data
    names = list(coefs)
    cds = {n: coefs[n].data for n in names}

    def backward(g, B, rel, needs):
        dx, dco = B.channelActBackward(ad, cds, g)
        return [dx] + [dco[n] for n in names]
    return _record(ctx, ctx.backend.channelAct(ad, cds), [a] + [coefs[n] for n in names], backward)


def gelu(ctx, a):
    ad = a.data
    return _record(ctx, ctx.backend.gelu(ad), [a], lambda g, B, rel, n: [B.geluBackward(ad, g)])


# ---- nn (ops.ts:491-729) ------------------------------------------------------------------------------------
def embedding(ctx, weight, indices: TensorData):
    wd = weight.data
    return _record(ctx, ctx.backend.embedding(wd, indices), [weight],
                   lambda g, B, rel, n: [B.embeddingBackward(indices, g, wd.shape[0])])


def layerNorm(ctx, x, weight, bias, eps):
    xd, wd = x.data, weight.data

    def bw(g, B, rel, n):
        r = B.layerNormBackward(xd, wd, g, eps)
        return [r["dx"], r["dw"], r["db"]]
    return _record(ctx, ctx.backend.layerNorm(xd, wd, bias.data, eps), [x, weight, bias], bw)


def _mask(ctx, shape, p):
    prm = ctx.dropoutRng.nextMaskParams() if ctx.dropoutRng else {"seed": int(np.random.randint(1 << 30)), "counter": 0}
    return ctx.backend.dropoutMask(shape, prm["seed"], prm["counter"], p)


def dropout(ctx, a, p, training):
    if not training or p == 0:
        return a
    mask = _mask(ctx, a.data.shape, p)
    live = [mask]

    def cleanup(rel):
        _rel(rel, live[0])
        live[0] = None
    return _record(ctx, ctx.backend.mul(a.data, mask), [a], lambda g, B, rel, n: [B.mul(g, mask)], cleanup)


def residualDropoutAdd(ctx, residual, projected, p, training):
    if not training or p == 0:
        return add(ctx, residual, projected)
    mask = _mask(ctx, projected.data.shape, p)
    live = [mask]
    rs = residual.data.shape

    def cleanup(rel):
        _rel(rel, live[0])
        live[0] = None
    out = ctx.backend.residualDropoutAdd(residual.data, projected.data, mask)
    return _record(ctx, out, [residual, projected],
                   lambda g, B, rel, n: [_reduce_broadcast(B, g, rs, rel), B.mul(g, mask)], cleanup)


def softmax(ctx, a, axis=None):
    out = ctx.backend.softmax(a.data, axis)
    last = axis is None or axis == -1 or axis == len(a.data.shape) - 1

    def bw(g, B, rel, n):
        if last and _has(B, "softmaxBackward"):
            return [B.softmaxBackward(out, g)]
        sg = B.mul(out, g)
        ssg = B.sum(sg, -1 if axis is None else axis, True)
        ex = _broadcast_to(B, ssg, out.shape)
        diff = B.sub(g, ex)
        r = B.mul(out, diff)
        _rel(rel, sg, ssg, diff)
        if ex is not ssg:
            _rel(rel, ex)
        return [r]
    return _record(ctx, out, [a], bw)


def crossEntropy(ctx, logits, targets: TensorData):
    ld = logits.data
    live = [targets]

    def cleanup(rel):
        _rel(rel, live[0])
        live[0] = None
    return _record(ctx, ctx.backend.crossEntropy(ld, targets), [logits],
                   lambda g, B, rel, n: [B.crossEntropyBackward(ld, targets, g)], cleanup)


# ---- flash attention (ops.ts:741-770) -----------------------------------------------------------------------
def flashAttention(ctx, q, k, v, T, scale_, softCap_):
    B0 = ctx.backend
    if not _has(B0, "flashAttention"):
        raise RuntimeError("flashAttention requires GPU backend")
    r = B0.flashAttention(q.data, k.data, v.data, T, scale_, softCap_)
    output, lse = r["output"], r["lse"]
    live = [lse]

    def cleanup(rel):
        _rel(rel, live[0])
        live[0] = None

    def bw(g, B, rel, needs):
        if live[0] is None:
            raise RuntimeError("flashAttention backward missing LSE buffer")
        d = B.flashAttentionBackward(q.data, k.data, v.data, output, g, lse, T, scale_, softCap_)
        return [d["dQ"] if needs is None or needs[0] else None, d["dK"] if needs is None or needs[1] else None,
                d["dV"] if needs is None or needs[2] else None]
    return _record(ctx, output, [q, k, v], bw, cleanup)


def causalSelfAttention(ctx, qkv, Bt, T, nHead, scale_, softCap_):
    """Multi-head causal attention straight from the fused projection: qkv is [B*T, 3C]; returns [B*T, C].
    Computes exactly what the reference's non-flash branch computes (packages/model/src/gpt.ts:255-279: split,
    head transpose, QK^T*scale, softcap, causal mask, softmax, PV, head merge) with the flash kernel reading
    Q, K, V in place through strides and writing the merged-head layout directly."""
    B0 = ctx.backend
    r = B0.attentionQkv(qkv.data, Bt, T, nHead, scale_, softCap_)
    output, lse = r["output"], r["lse"]
    live = [lse]

    def cleanup(rel):
        _rel(rel, live[0])
        live[0] = None

    def bw(g, B, rel, needs):
        return [B.attentionQkvBackward(qkv.data, output, g, lse, Bt, T, nHead, scale_, softCap_)]
    return _record(ctx, output, [qkv], bw, cleanup)


# ---- slice / view (ops.ts:775-873) --------------------------------------------------------------------------
def slice(ctx, a, starts, ends):                 # noqa: A001
    orig = tuple(a.data.shape)
    return _record(ctx, ctx.backend.slice(a.data, starts, ends), [a],
                   lambda g, B, rel, n: [B.scatterSlice(g, orig, starts, ends)])


def sliceQkv(ctx, a):
    B0 = ctx.backend
    rows, c3 = a.data.shape
    D = c3 // 3
    orig = (rows, c3)
    qd, kd, vd = B0.sliceQkv(a.data)
    mk = lambda data, i: _record(ctx, data, [a], lambda g, B, rel, n: [B.scatterSlice(g, orig, [0, i * D], [rows, (i + 1) * D])])
    return mk(qd, 0), mk(kd, 1), mk(vd, 2)


def reshape(ctx, a, shape):
    orig = a.data.shape
    return _record(ctx, ctx.backend.reshape(a.data, shape), [a], lambda g, B, rel, n: [B.reshape(g, orig)])


def transpose(ctx, a, d0, d1):
    return _record(ctx, ctx.backend.transpose(a.data, d0, d1), [a], lambda g, B, rel, n: [B.transpose(g, d0, d1)])


# ---- mixed precision storage casts (ops.ts:944-974) ---------------------------------------------------------
def castToF16(ctx, x):
    B0 = ctx.backend
    if not _has(B0, "castDtype"):
        return x
    return _record(ctx, B0.castDtype(x.data, "f16"), [x],
                   lambda g, B, rel, n: [B.castDtype(g, "f32") if g.dtype == "f16" else g])


def castToF32(ctx, x):
    B0 = ctx.backend
    if x.data.dtype == "f32" or not _has(B0, "castDtype"):
        return x
    return _record(ctx, B0.castDtype(x.data, "f32"), [x], lambda g, B, rel, n: [B.castDtype(g, "f16")])


# ---- activation checkpointing (packages/autograd/src/checkpoint.ts:34-87) -----------------------------------
def checkpoint(ctx, fn, inp: Variable) -> Variable:
    """Run `fn` without keeping its tape; on backward, recompute it on a private tape and back-propagate.  Parameter
    Variables captured by `fn` receive their gradients during the replay."""
    B0 = ctx.backend
    inner = Ctx(Tape(), B0, ctx.dropoutRng, ctx.release)
    out = fn(inner, inp)
    out_data = out.data
    inner.tape.clear(ctx.release, out)

    def bw(g, B, rel, needs):
        tape2 = Tape()
        x = Variable(inp.data, True)
        y = fn(Ctx(tape2, B, ctx.dropoutRng, rel), x)
        tape2.backward(y, B, rel, B.clone(g))
        gx = x.grad
        tape2.clear(rel)
        return [gx if gx is not None else B.zeros(inp.data.shape, inp.data.dtype)]
    return _record(ctx, out_data, [inp], bw)
