"""TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.

Restatement of the reference's host-side training step as it runs on its CPU backend:
  * Tape / Variable                     packages/autograd/src/tape.ts:29-201
  * differentiable ops + CPU fallbacks  packages/autograd/src/ops.ts:99-974
  * initGPT / transformerBlock / gptForward (the NON-flash branch cpu_ref takes)
                                        packages/model/src/gpt.ts:73-151, 220-333, 344-427
  * the flash branch of transformerBlock (ModelConfig.attention = "reference-flash": what an unchanged gpt.ts runs on a
    backend that offers flashAttention)  packages/model/src/gpt.ts:247-254, with the op's contract
                                        (packages/core/src/interfaces.ts:127-135) restated in closed form, forward and
                                        backward, per [T, D] slab; pinned in tests/test_oracle_model.py against PyTorch
                                        float64 autograd (whole model, and the op alone against torch's fused routine)
  * AdamW.stepParamEntries              packages/train/src/optimizers.ts:54-115
  * sample(): token selection + loop     packages/train/src/sample.ts:36-198 (pinned in tests/test_sample.py by hand-worked
                                        distributions with scripted rng draws)
  * Lion, Adafactor, SGD                packages/train/src/optimizers.ts:246-593 (pinned in tests/test_optimizers.py by
                                        closed forms: Lion's first step, Adafactor on a rank-one gradient, and the
                                        reference's own gradScale / entry-vs-map properties, packages/tests/src/optimizer.test.ts)
  * evaluate()                          packages/train/src/eval.ts:25-60 (pinned in tests/test_eval.py: loss = ln V and
                                        perplexity = V for a model whose logits are all equal; mean over the rng's batches)
  * LR schedule, grad-norm, clip        packages/train/src/trainer.ts:1088-1096,1150-1159,1297,
                                        1332-1349,1650-1656,1761-1784
  * no-decay set                        apps/cli/src/commands/train.ts:319-331
All tensor arithmetic goes through oracle.ref.CpuRef (C loops).  cpu_ref exposes none of the
optional fused backend ops, so every op below takes the fallback branch the reference takes.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import numpy as np

from . import ref
from .ref import TD, CpuRef, SeededRng, shape_size


# ---- tape.ts ------------------------------------------------------------------------------------

class Variable:
    _next = 0

    def __init__(self, data: TD, requiresGrad: bool = False):
        self.id = Variable._next
        Variable._next += 1
        self.data = data
        self.grad: Optional[TD] = None
        self.requiresGrad = requiresGrad


class Tape:
    def __init__(self):
        self.entries = []

    def record(self, output, inputs, backward):
        self.entries.append((output, inputs, backward))

    def backward(self, loss: Variable, B: CpuRef, initialGrad: Optional[TD] = None):
        """tape.ts:60-157 without the release bookkeeping (CPU arrays are garbage collected)."""
        loss.grad = initialGrad if initialGrad is not None else B.ones(loss.data.shape, loss.data.dtype)
        for output, inputs, bw in reversed(self.entries):
            outGrad = output.grad
            if outGrad is None:
                continue
            needs = None
            if any(not v.requiresGrad for v in inputs):
                needs = [v.requiresGrad for v in inputs]
            grads = bw(outGrad, B, needs)
            for inp, g in zip(inputs, grads):
                if g is None or not inp.requiresGrad:
                    continue
                if inp.grad is not None:
                    inp.grad = B.add(inp.grad, g)       # tape.ts:121-123 (no addInplace on cpu_ref)
                else:
                    inp.grad = B.clone(g)               # tape.ts:126
            output.grad = None

    def clear(self):
        for output, _, _ in self.entries:
            output.grad = None
        self.entries = []


class DropoutRng:
    """ops.ts:25-82: masks from a counter hash of (seed, counter, index); the counter advances once per mask."""

    def __init__(self, seed: int):
        self.seed, self.counter = ref._to_i32(seed), 0

    def reset(self, seed: int, counter: int = 0):
        self.seed, self.counter = ref._to_i32(seed), ref._to_i32(counter)

    def nextMask(self, size: int, p: float) -> np.ndarray:
        m = ref.dropout_mask(self.seed, self.counter, p, size)
        self.counter += 1
        return m

    def saveCounter(self) -> int:
        return self.counter

    def restoreCounter(self, n: int):
        self.counter = n


@dataclass
class Ctx:
    tape: Tape
    backend: CpuRef
    dropoutRng: Optional[DropoutRng] = None


def _record(ctx: Ctx, data: TD, inputs, backward) -> Variable:
    out = Variable(data, True)
    ctx.tape.record(out, inputs, backward)
    return out


# ---- ops.ts -------------------------------------------------------------------------------------

def _reduce_broadcast(B: CpuRef, grad: TD, target: Tuple[int, ...]) -> TD:
    """ops.ts:878-900."""
    if tuple(grad.shape) == tuple(target):
        return grad
    if len(target) == 0 or (len(target) == 1 and target[0] == 1 and len(grad.shape) > 1):
        return B.sum(grad)
    result = grad
    while len(result.shape) > len(target):
        result = B.sum(result, 0)
    for i in range(len(target)):
        if target[i] == 1 and result.shape[i] != 1:
            result = B.sum(result, i, True)
    return result


def _broadcast_to(B: CpuRef, t: TD, target: Tuple[int, ...]) -> TD:
    """ops.ts:903-929."""
    if tuple(t.shape) == tuple(target):
        return t
    src = t.data.reshape(t.shape if len(t.shape) else (1,))
    out = np.broadcast_to(src, target).astype(np.float32).reshape(-1).copy()
    return TD(tuple(target), t.dtype, out)


def add(ctx, a, b):
    sa, sb = a.data.shape, b.data.shape
    return _record(ctx, ctx.backend.add(a.data, b.data), [a, b],
                   lambda g, B, n: [_reduce_broadcast(B, g, sa), _reduce_broadcast(B, g, sb)])


def sub(ctx, a, b):
    sa, sb = a.data.shape, b.data.shape

    def bw(g, B, n):
        negG = B.neg(g)
        return [_reduce_broadcast(B, g, sa), _reduce_broadcast(B, negG, sb)]
    return _record(ctx, ctx.backend.sub(a.data, b.data), [a, b], bw)


def mul(ctx, a, b):
    ad, bd = a.data, b.data

    def bw(g, B, n):
        return [_reduce_broadcast(B, B.mul(g, bd), ad.shape), _reduce_broadcast(B, B.mul(g, ad), bd.shape)]
    return _record(ctx, ctx.backend.mul(ad, bd), [a, b], bw)


def div(ctx, a, b):
    ad, bd = a.data, b.data

    def bw(g, B, n):
        ga = B.div(g, bd)
        gb = B.neg(B.div(B.mul(g, ad), B.mul(bd, bd)))
        return [_reduce_broadcast(B, ga, ad.shape), _reduce_broadcast(B, gb, bd.shape)]
    return _record(ctx, ctx.backend.div(ad, bd), [a, b], bw)


def scale(ctx, a, s):
    return _record(ctx, ctx.backend.scale(a.data, s), [a], lambda g, B, n: [B.scale(g, s)])


def neg(ctx, a):
    return _record(ctx, ctx.backend.neg(a.data), [a], lambda g, B, n: [B.neg(g)])


def matmul(ctx, a, b):
    """ops.ts:165-189 (no matmulTransposedA on cpu_ref)."""
    ad, bd = a.data, b.data

    def bw(g, B, needs):
        ga = gb = None
        if needs is None or needs[0]:
            ga = B.matmul(g, B.transpose(bd, len(bd.shape) - 2, len(bd.shape) - 1))
        if needs is None or needs[1]:
            gb = B.matmul(B.transpose(ad, len(ad.shape) - 2, len(ad.shape) - 1), g)
        return [ga, gb]
    return _record(ctx, ctx.backend.matmul(ad, bd), [a, b], bw)


def matmulTransposed(ctx, a, b):
    """ops.ts:197-234, fallback branch: transpose(b) then matmul; dB = transpose(g) @ a."""
    ad, bd = a.data, b.data
    B0 = ctx.backend
    tB = B0.transpose(bd, len(bd.shape) - 2, len(bd.shape) - 1)

    def bw(g, B, needs):
        ga = gb = None
        if needs is None or needs[0]:
            ga = B.matmul(g, bd)
        if needs is None or needs[1]:
            gb = B.matmul(B.transpose(g, len(g.shape) - 2, len(g.shape) - 1), ad)
        return [ga, gb]
    return _record(ctx, B0.matmul(ad, tB), [a, b], bw)


def matmulTransposedGelu(ctx, a, b):
    """ops.ts:426-487, fallback branches."""
    ad, bd = a.data, b.data
    B0 = ctx.backend
    tB = B0.transpose(bd, len(bd.shape) - 2, len(bd.shape) - 1)
    mm = B0.matmul(ad, tB)

    def bw(g, B, needs):
        dMM = ref.gelu_backward(mm, g, fused=True)
        ga = gb = None
        if needs is None or needs[0]:
            ga = B.matmul(dMM, bd)
        if needs is None or needs[1]:
            gb = B.matmul(B.transpose(dMM, len(dMM.shape) - 2, len(dMM.shape) - 1), ad)
        return [ga, gb]
    return _record(ctx, B0.gelu(mm), [a, b], bw)


def sum_(ctx, a, axis=None, keepdims=False):
    sa = a.data.shape
    return _record(ctx, ctx.backend.sum(a.data, axis, keepdims), [a], lambda g, B, n: [_broadcast_to(B, g, sa)])


def mean(ctx, a, axis=None, keepdims=False):
    sa = a.data.shape
    n_ = sa[axis + len(sa) if axis is not None and axis < 0 else axis] if axis is not None else shape_size(sa)
    return _record(ctx, ctx.backend.mean(a.data, axis, keepdims), [a],
                   lambda g, B, n: [B.scale(_broadcast_to(B, g, sa), 1 / n_)])


def exp(ctx, a):
    out = ctx.backend.exp(a.data)
    return _record(ctx, out, [a], lambda g, B, n: [B.mul(g, out)])


def log(ctx, a):
    ad = a.data
    return _record(ctx, ctx.backend.log(ad), [a], lambda g, B, n: [B.div(g, ad)])


def relu(ctx, a):
    ad = a.data
    return _record(ctx, ctx.backend.relu(ad), [a], lambda g, B, n: [ref.relu_backward(ad, g)])


def clamp(ctx, a, lo, hi):
    ad = a.data
    return _record(ctx, ctx.backend.clamp(ad, lo, hi), [a], lambda g, B, n: [ref.clamp_backward(ad, g, lo, hi)])


def softCap(ctx, a, cap):
    """ops.ts:329-340: composed tanh via exp(2x/cap) clamped to [-80, 80]."""
    xs = scale(ctx, a, 2 / cap)
    xc = clamp(ctx, xs, -80, 80)
    e2x = exp(ctx, xc)
    ones = Variable(ctx.backend.ones(e2x.data.shape, e2x.data.dtype), False)
    numer = sub(ctx, e2x, ones)
    denom = add(ctx, e2x, ones)
    return scale(ctx, div(ctx, numer, denom), cap)


def silu(ctx, a):
    ad = a.data
    return _record(ctx, ctx.backend.silu(ad), [a], lambda g, B, n: [ref.silu_backward(ad, g)])


def siluMul(ctx, a, b):
    """ops.ts:364-399 fallback: silu(a)*b; da = siluBackwardCPU(a, g*b), db = g*silu(a)."""
    ad, bd = a.data, b.data
    B0 = ctx.backend
    sa = B0.silu(ad)

    def bw(g, B, n):
        ga = B.mul(g, bd)
        return [ref.silu_backward(ad, ga), B.mul(g, sa)]
    return _record(ctx, B0.mul(sa, bd), [a, b], bw)


def gelu(ctx, a):
    ad = a.data
    return _record(ctx, ctx.backend.gelu(ad), [a], lambda g, B, n: [ref.gelu_backward(ad, g, fused=False)])


def embedding(ctx, weight, indices: TD):
    wd = weight.data
    return _record(ctx, ctx.backend.embedding(wd, indices), [weight],
                   lambda g, B, n: [ref.embedding_backward(indices, g, wd.shape[0])])


def layerNorm(ctx, x, weight, bias, eps):
    xd, wd = x.data, weight.data
    return _record(ctx, ctx.backend.layerNorm(xd, wd, bias.data, eps), [x, weight, bias],
                   lambda g, B, n: list(ref.layernorm_backward(xd, wd, g, eps)))


def softmax(ctx, a, axis=None):
    """ops.ts:688-700."""
    out = ctx.backend.softmax(a.data, axis)

    def bw(g, B, n):
        sg = B.mul(out, g)
        sumSg = B.sum(sg, -1 if axis is None else axis, True)
        diff = B.sub(g, _broadcast_to(B, sumSg, out.shape))
        return [B.mul(out, diff)]
    return _record(ctx, out, [a], bw)


def crossEntropy(ctx, logits, targets: TD):
    ld = logits.data
    return _record(ctx, ctx.backend.crossEntropy(ld, targets), [logits],
                   lambda g, B, n: [ref.cross_entropy_backward(ld, targets, float(g.data[0]))])


def slice_(ctx, a, starts, ends):
    """ops.ts:775-809, zero-pad fallback (equals scatterSlice: same zero-filled placement)."""
    orig = tuple(a.data.shape)
    return _record(ctx, ctx.backend.slice(a.data, starts, ends), [a],
                   lambda g, B, n: [B.scatterSlice(g, orig, starts, ends)])


def sliceQkv(ctx, a):
    rows, cols3 = a.data.shape
    D = cols3 // 3
    return (slice_(ctx, a, [0, 0], [rows, D]), slice_(ctx, a, [0, D], [rows, 2 * D]),
            slice_(ctx, a, [0, 2 * D], [rows, 3 * D]))


def reshape(ctx, a, shape):
    orig = a.data.shape
    return _record(ctx, ctx.backend.reshape(a.data, shape), [a], lambda g, B, n: [B.reshape(g, orig)])


def transpose(ctx, a, d0, d1):
    return _record(ctx, ctx.backend.transpose(a.data, d0, d1), [a], lambda g, B, n: [B.transpose(g, d0, d1)])


def _cpu_mask(ctx, shape, p) -> TD:
    """ops.ts:583-596, 635-647: cpu_ref has no dropoutMask, so the mask comes from DropoutRng.nextMask on the host.  (Without
    a DropoutRng the reference draws Math.random(): not reproducible, not restated.)"""
    if ctx.dropoutRng is None:
        raise ValueError("dropout > 0 needs a DropoutRng")
    return TD(tuple(shape), "f32", ctx.dropoutRng.nextMask(shape_size(shape), p))


def dropout(ctx, a, p, training):
    """ops.ts:574-613."""
    if not training or p == 0:
        return a
    mask = _cpu_mask(ctx, a.data.shape, p)
    return _record(ctx, ctx.backend.mul(a.data, mask), [a], lambda g, B, n: [B.mul(g, mask)])


def residualDropoutAdd(ctx, residual, projected, p, training):
    """ops.ts:615-685, the separate-ops branch (cpu_ref has no fused residualDropoutAdd)."""
    if not training or p == 0:
        return add(ctx, residual, projected)        # ops.ts:624
    mask = _cpu_mask(ctx, projected.data.shape, p)
    rs = residual.data.shape
    out = ctx.backend.add(residual.data, ctx.backend.mul(projected.data, mask))
    return _record(ctx, out, [residual, projected], lambda g, B, n: [_reduce_broadcast(B, g, rs), B.mul(g, mask)])


# ---- gpt.ts -------------------------------------------------------------------------------------

@dataclass
class ModelConfig:
    vocabSize: int
    blockSize: int
    nLayer: int
    nEmbd: int
    nHead: int
    dropout: float = 0.0
    ffnActivation: str = "gelu"
    ffnDim: Optional[int] = None
    softCap: Optional[float] = None
    activationGraph: Optional[dict] = None
    # which branch of gpt.ts:246-280 the block takes: "heads" = the one for a backend WITHOUT flashAttention (cpu_ref,
    # :255-279), "reference-flash" = the one for a backend WITH it (:247-254), restated with materialised attention
    attention: str = "heads"


def _init_weight(rng: SeededRng, shape, std) -> Variable:
    return Variable(TD(tuple(shape), "f32", rng.fill_gauss(shape_size(shape), std)), True)


def initGPT(cfg: ModelConfig, B: CpuRef, rng: SeededRng) -> dict:
    """gpt.ts:73-151.  Draw order: wte, wpe, per layer (mlp weights FIRST, then wqkv, wo), lmHead."""
    V, T, L, Cc = cfg.vocabSize, cfg.blockSize, cfg.nLayer, cfg.nEmbd
    act = cfg.ffnActivation or "gelu"
    std = 0.02
    wte = _init_weight(rng, [V, Cc], std)
    wpe = _init_weight(rng, [T, Cc], std)
    ffn = cfg.ffnDim or (math.ceil((8 / 3) * Cc / 64) * 64 if act == "swiglu" else 4 * Cc)
    layers = []
    for _ in range(L):
        if act == "swiglu":
            mlp = {"fc_gate": _init_weight(rng, [ffn, Cc], std), "fc_up": _init_weight(rng, [ffn, Cc], std),
                   "fc_proj": _init_weight(rng, [Cc, ffn], std / math.sqrt(2 * L))}
        else:
            mlp = {"fc1": _init_weight(rng, [ffn, Cc], std), "fc2": _init_weight(rng, [Cc, ffn], std / math.sqrt(2 * L))}
            if act == "universal":
                mlp["act_gate"] = Variable(B.full([1, ffn], 1.0), True)
                mlp["act_skip"] = Variable(B.full([1, ffn], 0.0), True)
            elif act == "kan_spline":
                for k, v in (("kan_c0", 0.5), ("kan_c1", 0.0), ("kan_c2", 0.5), ("kan_c3", 0.0), ("kan_c4", 0.0)):
                    mlp[k] = Variable(B.full([1, ffn], v), True)
        layers.append({
            "ln1": {"weight": Variable(B.ones([Cc]), True), "bias": Variable(B.zeros([Cc]), True)},
            "attn": {"wqkv": _init_weight(rng, [3 * Cc, Cc], std), "wo": _init_weight(rng, [Cc, Cc], std / math.sqrt(2 * L))},
            "ln2": {"weight": Variable(B.ones([Cc]), True), "bias": Variable(B.zeros([Cc]), True)},
            "mlp": mlp,
        })
    lnF = {"weight": Variable(B.ones([Cc]), True), "bias": Variable(B.zeros([Cc]), True)}
    lmHead = _init_weight(rng, [V, Cc], std)
    return {"wte": wte, "wpe": wpe, "layers": layers, "lnF": lnF, "lmHead": lmHead}


def collectParamEntries(params: dict) -> List[Tuple[str, Variable]]:
    """gpt.ts:433-468."""
    e = [("wte", params["wte"]), ("wpe", params["wpe"]), ("lmHead", params["lmHead"]),
         ("lnF.weight", params["lnF"]["weight"]), ("lnF.bias", params["lnF"]["bias"])]
    for i, l in enumerate(params["layers"]):
        e += [(f"layer.{i}.ln1.weight", l["ln1"]["weight"]), (f"layer.{i}.ln1.bias", l["ln1"]["bias"]),
              (f"layer.{i}.attn.wqkv", l["attn"]["wqkv"]), (f"layer.{i}.attn.wo", l["attn"]["wo"]),
              (f"layer.{i}.ln2.weight", l["ln2"]["weight"]), (f"layer.{i}.ln2.bias", l["ln2"]["bias"])]
        m = l["mlp"]
        if "fc_gate" in m:
            e += [(f"layer.{i}.mlp.fc_gate", m["fc_gate"]), (f"layer.{i}.mlp.fc_up", m["fc_up"]),
                  (f"layer.{i}.mlp.fc_proj", m["fc_proj"])]
        else:
            e += [(f"layer.{i}.mlp.fc1", m["fc1"]), (f"layer.{i}.mlp.fc2", m["fc2"])]
        for k in ("act_gate", "act_skip", "kan_c0", "kan_c1", "kan_c2", "kan_c3", "kan_c4"):
            if k in m:
                e.append((f"layer.{i}.mlp.{k}", m[k]))
    return e


def _eval_activation_graph(ctx, x, node):
    """gpt.ts:170-192: an expression tree whose leaves are the bases silu / relu / gelu / identity / square of the SAME
    input (an unknown basis name evaluates as gelu) and whose inner nodes are scale-by-constant, add and mul."""
    kind = node["type"]
    if kind == "basis":
        op = node["op"]
        if op == "silu":
            return silu(ctx, x)
        if op == "relu":
            return relu(ctx, x)
        if op == "identity":
            return x
        if op == "square":
            return mul(ctx, x, x)
        return gelu(ctx, x)
    if kind == "scale":
        return scale(ctx, _eval_activation_graph(ctx, x, node["child"]), node["factor"])
    lhs = _eval_activation_graph(ctx, x, node["left"])
    rhs = _eval_activation_graph(ctx, x, node["right"])
    if kind == "add":
        return add(ctx, lhs, rhs)
    if kind == "mul":
        return mul(ctx, lhs, rhs)
    raise ValueError(f"activation graph node {kind!r}")


def flash_attention_forward(q: np.ndarray, k: np.ndarray, v: np.ndarray, scl: float, cap: float):
    """Backend.flashAttention (interfaces.ts:127-135): q, k, v [B*H, T, D] -> output [B*H, T, D] and the log-sum-exp of
    every row [B*H, T].  Per [T, D] slab: scores = scl * q k^T, then tanh(s / cap) * cap when cap > 0
    (helios/src/kernels/attention.ts:427-437: the hyperbolic tangent itself, not the clamped-exponential form the
    autograd fallback composes, ops.ts:329-340), keys after the query masked out, softmax, times v.  f32 in and out,
    f64 inside (cpu_ref's convention); the whole [T, T] matrix is materialised."""
    q64, k64, v64 = (np.asarray(x, np.float64) for x in (q, k, v))
    T = q64.shape[1]
    s = scl * (q64 @ k64.transpose(0, 2, 1))
    th = np.tanh(s / cap) if cap > 0 else None
    c = th * cap if cap > 0 else s
    future = np.triu(np.ones((T, T), dtype=bool), 1)
    c = np.where(future[None], -np.inf, c)
    mx = c.max(-1, keepdims=True)
    e = np.exp(c - mx)
    den = e.sum(-1, keepdims=True)
    p = e / den
    return (p @ v64), (mx + np.log(den))[..., 0], p, th


def flash_attention_backward(q, k, v, do, scl: float, cap: float):
    """Backend.flashAttentionBackward (interfaces.ts:131-135), closed form: dV = P^T dO; dP = dO V^T;
    d(capped scores) = P * (dP - rowsum(dP * P)); through the cap: * (1 - tanh^2); dQ = scl * dS K; dK = scl * dS^T Q."""
    q64, k64, v64, do64 = (np.asarray(x, np.float64) for x in (q, k, v, do))
    _, _, p, th = flash_attention_forward(q, k, v, scl, cap)
    dv = p.transpose(0, 2, 1) @ do64
    dp = do64 @ v64.transpose(0, 2, 1)
    dc = p * (dp - (dp * p).sum(-1, keepdims=True))
    ds = dc * (1.0 - th * th) if cap > 0 else dc
    return scl * (ds @ k64), scl * (ds.transpose(0, 2, 1) @ q64), dv


def flashAttention(ctx, q, k, v, T, scl, cap):
    """ops.ts:741-770: records Backend.flashAttention with Backend.flashAttentionBackward as its gradient.  cpu_ref has
    neither (ops.ts:746 throws); the two functions above restate the contract."""
    shp = q.data.shape
    qa, ka, va = (x.data.data.reshape(shp) for x in (q, k, v))
    out = flash_attention_forward(qa, ka, va, scl, cap)[0]

    def bw(g, B, n):
        dq, dk, dv = flash_attention_backward(qa, ka, va, g.data.reshape(shp), scl, cap)
        return [TD(shp, "f32", x.astype(np.float32).reshape(-1)) for x in (dq, dk, dv)]
    return _record(ctx, TD(shp, "f32", out.astype(np.float32).reshape(-1)), [q, k, v], bw)


def _transformer_block(ctx, x, layer, cfg: ModelConfig, Bt, T, mask: TD, training):
    """gpt.ts:220-333.  cfg.attention picks the branch of :246-280: "heads" is the one taken when backend.flashAttention
    is absent (cpu_ref), "reference-flash" the one taken when it is present."""
    H, Cc = cfg.nHead, cfg.nEmbd
    D = Cc // H
    ln1 = layerNorm(ctx, x, layer["ln1"]["weight"], layer["ln1"]["bias"], 1e-5)
    qkv = matmulTransposed(ctx, reshape(ctx, ln1, [Bt * T, Cc]), layer["attn"]["wqkv"])
    qF, kF, vF = sliceQkv(ctx, qkv)
    q = reshape(ctx, qF, [Bt, T, Cc])
    k = reshape(ctx, kF, [Bt, T, Cc])
    v = reshape(ctx, vF, [Bt, T, Cc])
    cap = cfg.softCap if cfg.softCap is not None else 30.0
    if cfg.attention == "reference-flash":
        return _block_tail(ctx, x, layer, cfg, Bt, T, training, _flash_branch(ctx, q, k, v, cfg, Bt, T, cap))
    qH = transpose(ctx, reshape(ctx, q, [Bt, T, H, D]), 1, 2)
    kH = transpose(ctx, reshape(ctx, k, [Bt, T, H, D]), 1, 2)
    vH = transpose(ctx, reshape(ctx, v, [Bt, T, H, D]), 1, 2)
    kT = transpose(ctx, kH, 2, 3)
    raw = scale(ctx, matmul(ctx, qH, kT), 1 / math.sqrt(D))
    scores = softCap(ctx, raw, cap)
    masked = Variable(ctx.backend.maskedFill(scores.data, mask, -1e9), True)
    ctx.tape.record(masked, [scores], lambda g, B, n: [B.maskedFill(g, mask, 0)])
    att = softmax(ctx, masked, -1)
    out = matmul(ctx, dropout(ctx, att, cfg.dropout, training), vH)
    concat = reshape(ctx, transpose(ctx, out, 1, 2), [Bt * T, Cc])
    return _block_tail(ctx, x, layer, cfg, Bt, T, training, concat)


def _flash_branch(ctx, q, k, v, cfg: ModelConfig, Bt, T, cap):
    """gpt.ts:247-254: [B, T, C] is re-read as [B*H, T, D] WITHOUT moving heads next to the batch (slab j of batch entry b
    is rows j*T/H .. (j+1)*T/H of that entry, each row cut into H pieces of D), attention runs per slab, and the result
    [B, H, T, D] is transposed (1, 2) and flattened to [B*T, C]."""
    H, Cc = cfg.nHead, cfg.nEmbd
    D = Cc // H
    qFA = reshape(ctx, q, [Bt * H, T, D])
    kFA = reshape(ctx, k, [Bt * H, T, D])
    vFA = reshape(ctx, v, [Bt * H, T, D])
    out = flashAttention(ctx, qFA, kFA, vFA, T, 1 / math.sqrt(D), cap)
    return reshape(ctx, transpose(ctx, reshape(ctx, out, [Bt, H, T, D]), 1, 2), [Bt * T, Cc])


def _block_tail(ctx, x, layer, cfg: ModelConfig, Bt, T, training, concat):
    """gpt.ts:281-333: output projection, residual, LayerNorm, MLP, residual."""
    Cc = cfg.nEmbd
    proj = reshape(ctx, matmulTransposed(ctx, concat, layer["attn"]["wo"]), [Bt, T, Cc])
    x = residualDropoutAdd(ctx, x, proj, cfg.dropout, training)

    ln2 = layerNorm(ctx, x, layer["ln2"]["weight"], layer["ln2"]["bias"], 1e-5)
    flat = reshape(ctx, ln2, [Bt * T, Cc])
    act = cfg.ffnActivation or "gelu"
    m = layer["mlp"]
    if act == "composed" and cfg.activationGraph:            # gpt.ts:290-294
        h = matmulTransposed(ctx, flat, m["fc1"])
        mlpH = matmulTransposed(ctx, _eval_activation_graph(ctx, h, cfg.activationGraph), m["fc2"])
    elif act == "swiglu":
        gate = matmulTransposed(ctx, flat, m["fc_gate"])
        up = matmulTransposed(ctx, flat, m["fc_up"])
        mlpH = matmulTransposed(ctx, siluMul(ctx, gate, up), m["fc_proj"])
    elif act == "universal":
        h = matmulTransposed(ctx, flat, m["fc1"])
        h_act = add(ctx, mul(ctx, silu(ctx, h), m["act_gate"]), mul(ctx, h, m["act_skip"]))
        mlpH = matmulTransposed(ctx, h_act, m["fc2"])
    elif act == "kan_spline":
        h = matmulTransposed(ctx, flat, m["fc1"])
        hs = mul(ctx, silu(ctx, h), m["kan_c0"])
        hr = mul(ctx, relu(ctx, h), m["kan_c1"])
        hg = mul(ctx, gelu(ctx, h), m["kan_c2"])
        hi = mul(ctx, h, m["kan_c3"])
        hq = mul(ctx, mul(ctx, h, h), m["kan_c4"])
        h_act = add(ctx, add(ctx, add(ctx, add(ctx, hs, hr), hg), hi), hq)
        mlpH = matmulTransposed(ctx, h_act, m["fc2"])
    elif act == "silu":
        mlpH = matmulTransposed(ctx, silu(ctx, matmulTransposed(ctx, flat, m["fc1"])), m["fc2"])
    elif act == "relu":
        mlpH = matmulTransposed(ctx, relu(ctx, matmulTransposed(ctx, flat, m["fc1"])), m["fc2"])
    else:
        mlpH = matmulTransposed(ctx, matmulTransposedGelu(ctx, flat, m["fc1"]), m["fc2"])
    return residualDropoutAdd(ctx, x, reshape(ctx, mlpH, [Bt, T, Cc]), cfg.dropout, training)


def gptForward(cfg: ModelConfig, params: dict, B: CpuRef, tape: Tape, tokens: TD, targets: Optional[TD] = None,
               training: bool = False, dropoutRng: Optional[DropoutRng] = None):
    """gpt.ts:344-427."""
    ctx = Ctx(tape, B, dropoutRng)
    Bt, T = tokens.shape
    tok = embedding(ctx, params["wte"], tokens)
    pos = TD((Bt, T), "i32", np.tile(np.arange(T, dtype=np.int32), Bt))
    x = add(ctx, tok, embedding(ctx, params["wpe"], pos))
    mask = B.causalMask(T)
    for layer in params["layers"]:
        x = _transformer_block(ctx, x, layer, cfg, Bt, T, mask, training)
    x = layerNorm(ctx, x, params["lnF"]["weight"], params["lnF"]["bias"], 1e-5)
    flat = reshape(ctx, x, [Bt * T, cfg.nEmbd])
    logits = reshape(ctx, matmulTransposed(ctx, flat, params["lmHead"]), [Bt, T, cfg.vocabSize])
    loss = None
    if targets is not None:
        tf = TD((Bt * T,), "i32", targets.data)
        loss = crossEntropy(ctx, reshape(ctx, logits, [Bt * T, cfg.vocabSize]), tf)
    return logits, loss


# ---- sample.ts ----------------------------------------------------------------------------------

def select_token(last: np.ndarray, rng, temperature: float, topk: int, topP: float) -> int:
    """sample.ts:85-193, element by element as written there (plain loops: vocabularies in the tests are small).
    `last` is the Float32Array of logits already divided by the temperature."""
    V = last.size
    f32 = np.float32
    if temperature <= 0:
        best, bestVal = 0, last[0]
        for v in range(1, V):
            if last[v] > bestVal:
                bestVal, best = last[v], v
        return best
    if 0 < topk < V:
        order = sorted(range(V), key=lambda i: -float(last[i]))            # stable, descending
        threshold = last[order[topk - 1]]
        for v in range(V):
            if last[v] < threshold:
                last[v] = -np.inf
    if 0 < topP < 1:
        maxVal = -math.inf
        for v in range(V):
            if last[v] > maxVal:
                maxVal = float(last[v])
        if math.isfinite(maxVal):
            probs = np.zeros(V, dtype=f32)
            active, sumExp = [], 0.0
            for v in range(V):
                if math.isfinite(float(last[v])):
                    p = math.exp(float(last[v]) - maxVal)
                    probs[v] = p
                    active.append(v)
                    sumExp += p
            if sumExp > 0 and active:
                active.sort(key=lambda i: -float(probs[i]))
                target = sumExp * topP
                keptMass, keepCount = 0.0, 0
                while keepCount < len(active):
                    keptMass += float(probs[active[keepCount]])
                    if keptMass >= target:
                        keepCount += 1
                        break
                    keepCount += 1
                if keepCount <= 0:
                    keepCount = 1
                if keptMass <= 0:
                    keptMass = float(probs[active[0]])
                r = rng.next() * keptMass
                cum, sampled = 0.0, active[keepCount - 1]
                for i in range(keepCount):
                    cum += float(probs[active[i]])
                    if r < cum:
                        sampled = active[i]
                        break
                return sampled
    maxVal = -math.inf
    for v in range(V):
        if last[v] > maxVal:
            maxVal = float(last[v])
    probs = np.zeros(V, dtype=f32)
    sumExp = 0.0
    for v in range(V):
        probs[v] = math.exp(float(last[v]) - maxVal) if last[v] != -np.inf else 0.0
        sumExp += float(probs[v])
    for v in range(V):
        probs[v] = float(probs[v]) / sumExp
    r = rng.next()
    cum = 0.0
    for v in range(V):
        cum += float(probs[v])
        if r < cum:
            return v
    return 0


def evaluate(cfg: ModelConfig, params: dict, B: CpuRef, tokens, rng, batchSize: int, nBatches: int = 50):
    """packages/train/src/eval.ts:25-60 after tokenisation: nBatches random batches (one DataLoader over the whole token
    array, the caller's rng), forward pass with targets, mean of the batch losses; returns (loss, perplexity = exp(loss))."""
    loader = DataLoader(tokens, rng, batchSize, cfg.blockSize)
    total = 0.0
    for _ in range(nBatches):
        inputs, targets = loader.next_batch()
        tape = Tape()
        _, loss = gptForward(cfg, params, B, tape, inputs, targets)
        total += float(loss.data.data[0])
        tape.clear()
    avg = total / nBatches
    return avg, math.exp(avg)


def sample_tokens(cfg: ModelConfig, params: dict, B: CpuRef, rng, prompt, steps: int, temperature: float, topk: int, topp=1.0) -> np.ndarray:
    """sample.ts:36-198 without the tokenizer."""
    topP = min(1.0, max(0.0, topp)) if (topp is not None and math.isfinite(topp)) else 1.0
    prompt = np.asarray(prompt, dtype=np.int32)
    maxLen = min(prompt.size + steps, cfg.blockSize)
    tokens = np.zeros(maxLen, dtype=np.int32)
    tokens[:prompt.size] = prompt
    cur = int(prompt.size)
    for _ in range(steps):
        if cur >= cfg.blockSize:
            break
        start = max(0, cur - cfg.blockSize)
        ctx = tokens[start:cur].copy()
        logits, _ = gptForward(cfg, params, B, Tape(), TD((1, ctx.size), "i32", ctx))
        last = np.array(logits.data.data.reshape(-1)[(ctx.size - 1) * cfg.vocabSize:], dtype=np.float32)
        if temperature > 0:
            last = (last.astype(np.float64) / temperature).astype(np.float32)
        nxt = select_token(last, rng, temperature, topk, topP)
        if cur < maxLen:
            tokens[cur] = nxt
            cur += 1
    return tokens[:cur]


# ---- optimizers.ts / trainer.ts -----------------------------------------------------------------

def no_decay_names(nLayer: int) -> set:
    """apps/cli/src/commands/train.ts:319-331 ("lmHead.weight" never matches -> lmHead IS decayed)."""
    s = {"wte", "wpe", "lnF.weight", "lnF.bias", "lmHead.weight"}
    for i in range(nLayer):
        s |= {f"layer.{i}.ln1.weight", f"layer.{i}.ln1.bias", f"layer.{i}.ln2.weight", f"layer.{i}.ln2.bias"}
    return s


class AdamW:
    """optimizers.ts:21-115 (CPU loop branch)."""

    def __init__(self, lr=3e-4, beta1=0.9, beta2=0.999, eps=1e-8, weightDecay=0.01, noDecayNames=None):
        self.lr, self.beta1, self.beta2, self.eps, self.wd = lr, beta1, beta2, eps, weightDecay
        self.noDecay = noDecayNames or set()
        self._step = 0
        self._b1p = 1.0
        self._b2p = 1.0
        self.m: Dict[str, np.ndarray] = {}
        self.v: Dict[str, np.ndarray] = {}

    def setLr(self, lr):
        self.lr = lr

    def stepParamEntries(self, entries, gradScale=1.0):
        self._step += 1
        self._b1p *= self.beta1
        self._b2p *= self.beta2
        bc1, bc2 = 1 - self._b1p, 1 - self._b2p
        for name, var in entries:
            if var.grad is None:
                continue
            if name not in self.m:
                self.m[name] = np.zeros(var.data.data.size, dtype=np.float32)
                self.v[name] = np.zeros(var.data.data.size, dtype=np.float32)
            wd = 0.0 if name in self.noDecay else self.wd
            ref.adamw_step(var.data, var.grad, self.m[name], self.v[name], self.lr, self.beta1, self.beta2,
                           self.eps, wd, bc1, bc2, gradScale)

    def state_dict(self) -> dict:
        """optimizers.ts:202-210: "<name>.m" then "<name>.v" per parameter, in moment-map order."""
        bufs = {}
        for name, m in self.m.items():
            bufs[name + ".m"] = TD((m.size,), "f32", m.copy())
            bufs[name + ".v"] = TD((m.size,), "f32", self.v[name].copy())
        return {"step": self._step, "buffers": bufs}

    def load_state_dict(self, state: dict):
        """optimizers.ts:212-229: the beta powers are rebuilt as pow(beta, step)."""
        self._step = state["step"]
        self._b1p, self._b2p = math.pow(self.beta1, self._step), math.pow(self.beta2, self._step)
        self.m, self.v = {}, {}
        for key, td in state["buffers"].items():
            if key.endswith(".m"):
                self.m[key[:-2]] = np.array(td.data, dtype=np.float32)
            elif key.endswith(".v"):
                self.v[key[:-2]] = np.array(td.data, dtype=np.float32)


def _seq_sum(x: np.ndarray) -> float:
    """Left-to-right double sum, the order of the reference's for loops (numpy's own sum is pairwise)."""
    return float(np.cumsum(x.astype(np.float64))[-1]) if x.size else 0.0


class Lion:
    """optimizers.ts:246-336: host loop in double arithmetic, every Float32Array store rounds to f32."""

    def __init__(self, lr=1e-4, beta1=0.9, beta2=0.99, weightDecay=0.01, noDecayNames=None):
        self.lr, self.beta1, self.beta2, self.wd = lr, beta1, beta2, weightDecay
        self.noDecay = noDecayNames or set()
        self._step = 0
        self.m: Dict[str, np.ndarray] = {}

    def setLr(self, lr):
        self.lr = lr

    def _step_tensor(self, name, p: np.ndarray, g32: np.ndarray, gradScale):
        """optimizers.ts:284-311; p (f32) is updated in place."""
        if name not in self.m:
            self.m[name] = np.zeros(p.size, dtype=np.float32)
        m = self.m[name]
        wd = 0.0 if name in self.noDecay else self.wd
        g = g32.astype(np.float64) * gradScale
        if wd > 0:
            p[:] = (p.astype(np.float64) * (1 - self.lr * wd)).astype(np.float32)
        update = self.beta1 * m.astype(np.float64) + (1 - self.beta1) * g
        p[:] = (p.astype(np.float64) - self.lr * np.sign(update)).astype(np.float32)
        m[:] = (self.beta2 * m.astype(np.float64) + (1 - self.beta2) * g).astype(np.float32)

    def stepParamEntries(self, entries, gradScale=1.0):
        self._step += 1
        for name, var in entries:
            if var.grad is not None:
                self._step_tensor(name, var.data.data, var.grad.data, gradScale)

    def state_dict(self) -> dict:
        return {"step": self._step, "buffers": {name + ".m": TD((m.size,), "f32", m.copy()) for name, m in self.m.items()}}


def _js_max(a: float, b: float) -> float:
    """Math.max: NaN if either argument is NaN (Python's max keeps whichever argument the comparison does not displace)."""
    return float("nan") if (a != a or b != b) else max(a, b)


class Adafactor:
    """optimizers.ts:349-543."""

    def __init__(self, lr=1e-3, beta2=0.999, eps=1e-30, clipThreshold=1.0, weightDecay=0.0, noDecayNames=None):
        self.lr, self.beta2, self.eps, self.clip, self.wd = lr, beta2, eps, clipThreshold, weightDecay
        self.noDecay = noDecayNames or set()
        self._step = 0
        self.vr: Dict[str, np.ndarray] = {}
        self.vc: Dict[str, np.ndarray] = {}
        self.v: Dict[str, np.ndarray] = {}

    def setLr(self, lr):
        self.lr = lr

    def _step_tensor(self, name, p: np.ndarray, shape, g32: np.ndarray, gradScale):
        lr, beta2, eps = self.lr, self.beta2, self.eps
        wd = 0.0 if name in self.noDecay else self.wd
        decay = 1 - lr * wd if wd > 0 else 1.0
        g = g32.astype(np.float64).reshape(-1) * gradScale
        size = p.size
        if len(shape) == 2:                                          # optimizers.ts:412-475
            rows, cols = shape
            if name not in self.vr or self.vr[name].size != rows:
                self.vr[name] = np.zeros(rows, dtype=np.float32)
            if name not in self.vc or self.vc[name].size != cols:
                self.vc[name] = np.zeros(cols, dtype=np.float32)
            vr, vc = self.vr[name], self.vc[name]
            g2 = (g * g).reshape(rows, cols)
            for r in range(rows):
                vr[r] = np.float32(beta2 * float(vr[r]) + (1 - beta2) * (_seq_sum(g2[r]) * (1 / cols)) + eps)
            for c in range(cols):
                vc[c] = np.float32(beta2 * float(vc[c]) + (1 - beta2) * (_seq_sum(g2[:, c]) * (1 / rows)) + eps)
            vr_mean = _js_max(_seq_sum(vr) * (1 / rows), eps)
            r_scale = np.sqrt(vr.astype(np.float64) * (1 / vr_mean))
            denom = np.maximum(eps, r_scale[:, None] * np.sqrt(vc.astype(np.float64))[None, :]).reshape(-1)
        else:                                                        # optimizers.ts:478-500
            if name not in self.v or self.v[name].size != size:
                self.v[name] = np.zeros(size, dtype=np.float32)
            v = self.v[name]
            v[:] = (beta2 * v.astype(np.float64) + (1 - beta2) * (g * g) + eps).astype(np.float32)
            denom = np.sqrt(v.astype(np.float64))
        upd = g / denom
        rms = math.sqrt(_seq_sum(upd * upd) / max(1, size))
        clip_den = _js_max(1.0, rms / self.clip) if self.clip > 0 else 1.0
        step_scale = lr / clip_den
        flat = p.reshape(-1)
        if wd > 0:
            flat[:] = (flat.astype(np.float64) * decay).astype(np.float32)
        flat[:] = (flat.astype(np.float64) - step_scale * upd).astype(np.float32)

    def stepParamEntries(self, entries, gradScale=1.0):
        self._step += 1
        for name, var in entries:
            if var.grad is not None:
                self._step_tensor(name, var.data.data, tuple(var.data.shape), var.grad.data, gradScale)

    def state_dict(self) -> dict:
        bufs = {}
        for suffix, table in ((".vr", self.vr), (".vc", self.vc), (".v", self.v)):
            for name, t in table.items():
                bufs[name + suffix] = TD((t.size,), "f32", t.copy())
        return {"step": self._step, "buffers": bufs}


class SGD:
    """optimizers.ts:546-593."""

    def __init__(self, lr=0.01):
        self.lr, self._step = lr, 0

    def setLr(self, lr):
        self.lr = lr

    def stepParamEntries(self, entries, gradScale=1.0):
        self._step += 1
        for _, var in entries:
            if var.grad is not None:
                p = var.data.data
                p[:] = (p.astype(np.float64) - self.lr * (var.grad.data.astype(np.float64) * gradScale)).astype(np.float32)

    def state_dict(self) -> dict:
        return {"step": self._step, "buffers": {}}


@dataclass
class TrainConfig:
    iters: int = 1
    lr: float = 3e-4
    lrMin: float = 0.0
    warmupIters: int = 0
    beta1: float = 0.9
    beta2: float = 0.95
    eps: float = 1e-8
    weightDecay: float = 0.1
    gradClip: float = 1.0
    gradAccumSteps: int = 1
    optimizer: str = "adamw"
    seed: int = 42                    # packages/core/src/types.ts:126


def lr_at(tc: TrainConfig, step: int) -> float:
    """trainer.ts:1088-1096,1150-1159 (runtimeLrScale = 1)."""
    warmup = tc.warmupIters if tc.warmupIters > 0 else (0 if tc.warmupIters < 0 else min(2000, tc.iters // 5))
    lrMin = tc.lr / 10 if (tc.lrMin or 0) == 0 else tc.lrMin
    denom = max(1, tc.iters - warmup)
    if step < warmup:
        base = lrMin + (tc.lr - lrMin) * (step + 1) / warmup
    else:
        decay = (step - warmup) / denom
        base = lrMin + (tc.lr - lrMin) * 0.5 * (1 + math.cos(math.pi * decay))
    return max(lrMin * 0.1, base)


@dataclass
class StepResult:
    loss: float
    gradNorm: float
    clipCoef: float
    lr: float


class Trainer:
    """The arithmetic of one optimizer step of train() (trainer.ts:1146-1784); telemetry omitted."""

    def __init__(self, cfg: ModelConfig, tc: TrainConfig, seed: int = 0):
        self.cfg, self.tc = cfg, tc
        self.B = CpuRef()
        self.rng = SeededRng(seed)
        self.params = initGPT(cfg, self.B, self.rng)
        self.entries = collectParamEntries(self.params)
        nd = no_decay_names(cfg.nLayer)
        kind = getattr(tc, "optimizer", "adamw")                     # apps/cli/src/resolve.ts:25-36
        if kind == "adamw":
            self.opt = AdamW(tc.lr, tc.beta1, tc.beta2, tc.eps, tc.weightDecay, nd)
        elif kind == "lion":
            self.opt = Lion(tc.lr, tc.beta1, tc.beta2, tc.weightDecay, nd)
        elif kind == "adafactor":
            self.opt = Adafactor(lr=tc.lr, beta2=tc.beta2, eps=tc.eps, weightDecay=tc.weightDecay, noDecayNames=nd)
        elif kind == "sgd":
            self.opt = SGD()
        else:
            raise ValueError(f'Unknown optimizer: "{kind}"')
        self.tape = Tape()
        self.step_idx = 0
        self.dropoutRng = DropoutRng(tc.seed)                        # trainer.ts:1106

    def forward_backward(self, inputs: TD, targets: TD, micro: int = 0) -> float:
        self.dropoutRng.reset(self.tc.seed + self.step_idx * 1000 + micro, 0)       # trainer.ts:1169,1202
        _, loss = gptForward(self.cfg, self.params, self.B, self.tape, inputs, targets, True, self.dropoutRng)
        self.tape.backward(loss, self.B)
        val = float(loss.data.data[0])
        self.tape.clear()
        return val

    def step(self, batches: Sequence[Tuple[TD, TD]]) -> StepResult:
        tc = self.tc
        lr = lr_at(tc, self.step_idx)
        self.opt.setLr(lr)
        accum = len(batches)
        loss_val = 0.0
        if accum == 1:
            loss_val = self.forward_backward(*batches[0])
        else:  # trainer.ts:1208-1223: f32 scale by 1/accum then f32 add
            acc = None
            for micro, (inp, tgt) in enumerate(batches):
                lv = TD((), "f32", np.array([self.forward_backward(inp, tgt, micro)], dtype=np.float32))
                s = self.B.scale(lv, 1 / accum)
                acc = s if acc is None else self.B.add(acc, s)
            loss_val = float(acc.data[0])
        gradScale = 1.0 / accum
        sq = 0.0
        for _, v in self.entries:
            if v.grad is not None:
                sq += ref.sum_sq(v.grad)
        gradNorm = math.sqrt(sq) * abs(gradScale)
        clip, eff = 1.0, gradScale
        if tc.gradClip > 0 and gradNorm > tc.gradClip:
            clip = tc.gradClip / gradNorm
            eff *= clip
        self.opt.stepParamEntries(self.entries, eff)
        for _, v in self.entries:
            v.grad = None
        self.step_idx += 1
        return StepResult(loss_val, gradNorm, clip, lr)


def synthetic_batch(seed: int, Bt: int, T: int, vocab: int) -> Tuple[TD, TD]:
    """Uniform token ids: rng=SeededRng(seed); B*(T+1) draws floor(next()*vocab); row b takes draws
    [b*(T+1), (b+1)*(T+1)); inputs = first T, targets = last T (shift by one, as data.ts:110-114)."""
    rng = SeededRng(seed)
    u = rng.fill_uniform(Bt * (T + 1))
    ids = np.floor(u * vocab).astype(np.int32).reshape(Bt, T + 1)
    return (TD((Bt, T), "i32", np.ascontiguousarray(ids[:, :T]).reshape(-1)),
            TD((Bt, T), "i32", np.ascontiguousarray(ids[:, 1:]).reshape(-1)))


class DataLoader:
    """Batch sampler of packages/train/src/data.ts:30-167, slice by slice as written there.
    Random mode (data.ts:94-120): per batch row, start = floor(rng.next() * (N - T)); inputs = tokens[start, start+T),
    targets = tokens[start+1, start+T+1).  Packed mode (data.ts:131-167): cursor b starts at b*floor(N/B) and advances
    T per batch; a window that reaches the end of the corpus continues at token 0, and the target of the corpus'
    last token is its first."""

    def __init__(self, tokens, rng: SeededRng, batchSize: int, blockSize: int, packed: bool = False):
        self.tokens = np.ascontiguousarray(tokens, dtype=np.int32)
        self.rng, self.batchSize, self.blockSize, self.packed = rng, batchSize, blockSize, packed
        self.cursors = [b * (len(self.tokens) // batchSize) for b in range(batchSize)] if packed else None

    def next_batch(self) -> Tuple[TD, TD]:
        Bt, T, tok, N = self.batchSize, self.blockSize, self.tokens, len(self.tokens)
        inputs, targets = np.zeros(Bt * T, np.int32), np.zeros(Bt * T, np.int32)
        if not self.packed:
            if N <= T:
                raise IndexError(f"Token count ({N}) must exceed block size ({T})")
            max_start = N - T
            for b in range(Bt):
                start = int(math.floor(self.rng.next() * max_start))
                inputs[b * T:(b + 1) * T] = tok[start:start + T]
                targets[b * T:(b + 1) * T] = tok[start + 1:start + T + 1]
        else:
            for b in range(Bt):
                pos, remaining, dst = self.cursors[b], T, b * T
                while remaining > 0:
                    span = min(remaining, N - pos)
                    inputs[dst:dst + span] = tok[pos:pos + span]
                    if pos + span < N:
                        targets[dst:dst + span] = tok[pos + 1:pos + span + 1]
                    else:
                        if span > 1:
                            targets[dst:dst + span - 1] = tok[pos + 1:N]
                        targets[dst + span - 1] = tok[0]
                    dst, remaining, pos = dst + span, remaining - span, pos + span
                    if pos == N:
                        pos = 0
                self.cursors[b] = pos
        return TD((Bt, T), "i32", inputs), TD((Bt, T), "i32", targets)


# ------------------------------------------------------------------------------------------------ checkpoint files
def checkpoint_save_bytes(state: dict) -> bytes:
    """packages/train/src/checkpoint.ts:29-94 (saveBinary): "ALPH", uint32 LE header length, header JSON, then the
    float32 payload: parameters ("p.<name>") in insertion order, then optimizer buffers ("o.<name>")."""
    import json
    import struct
    tensors, chunks = [], []
    for name, p in state["params"].items():
        f32 = np.asarray(p["data"], dtype="<f4").reshape(-1)
        tensors.append({"name": "p." + name, "shape": list(p["shape"]), "elements": int(f32.size)})
        chunks.append(f32.tobytes())
    opt = state.get("optimizerState")
    if opt and opt.get("buffers"):
        for name, td in opt["buffers"].items():
            f32 = np.asarray(td.data, dtype="<f4").reshape(-1)
            tensors.append({"name": "o." + name, "shape": list(td.shape), "elements": int(f32.size)})
            chunks.append(f32.tobytes())
    header = {"modelConfig": state.get("modelConfig"), "configHash": state.get("configHash"), "rngState": state.get("rngState"),
              "step": state.get("step")}
    if state.get("tokenizerArtifacts") is not None:
        header["tokenizerArtifacts"] = state["tokenizerArtifacts"]
    header["optimizerStep"] = opt["step"] if opt else 0
    if state.get("symbioActivationGraph") is not None:
        header["symbioActivationGraph"] = state["symbioActivationGraph"]
    header["tensors"] = tensors
    hb = json.dumps(header, separators=(",", ":"), ensure_ascii=False).encode("utf-8")
    return b"ALPH" + struct.pack("<I", len(hb)) + hb + b"".join(chunks)


def checkpoint_load_bytes(raw: bytes) -> dict:
    """checkpoint.ts:98-136 (loadBinary) and :160-189 (format detection, legacy JSON)."""
    import json
    import struct
    if raw[:4] != b"ALPH":
        parsed = json.loads(raw.decode("utf-8"))
        bufs = {k: TD(tuple(v["shape"]), "f32", np.asarray(v["data"], dtype=np.float32))
                for k, v in ((parsed.get("optimizerState") or {}).get("buffers") or {}).items()}
        return {"modelConfig": parsed.get("modelConfig"), "params": parsed.get("params"),
                "optimizerState": {"step": (parsed.get("optimizerState") or {}).get("step") or 0, "buffers": bufs},
                "tokenizerArtifacts": parsed.get("tokenizerArtifacts"), "rngState": parsed.get("rngState"),
                "configHash": parsed.get("configHash"), "step": parsed.get("step")}
    off = 4
    (hlen,) = struct.unpack_from("<I", raw, off)
    off += 4
    header = json.loads(raw[off:off + hlen].decode("utf-8"))
    off += hlen
    params, bufs = {}, {}
    for t in header["tensors"]:
        n = t["elements"]
        f32 = np.frombuffer(raw, dtype="<f4", count=n, offset=off).astype(np.float32)
        off += 4 * n
        if t["name"].startswith("p."):
            params[t["name"][2:]] = {"shape": t["shape"], "data": f32}
        elif t["name"].startswith("o."):
            bufs[t["name"][2:]] = TD(tuple(t["shape"]), "f32", f32)
    return {"modelConfig": header.get("modelConfig"), "params": params,
            "optimizerState": {"step": header.get("optimizerStep") or 0, "buffers": bufs},
            "tokenizerArtifacts": header.get("tokenizerArtifacts"), "rngState": header.get("rngState"),
            "configHash": header.get("configHash"), "step": header.get("step")}


def restore_params(entries, saved: dict):
    """checkpoint.ts:224-259, including the wq / wk / wv -> wqkv concatenation for old checkpoints."""
    for name, var in entries:
        if name in saved:
            src = np.asarray(saved[name]["data"], dtype=np.float32).reshape(-1)
            var.data.data[:] = src[:var.data.data.size]
            continue
        if name.endswith(".attn.wqkv"):
            prefix = name[:-len(".attn.wqkv")]
            parts = [saved.get(f"{prefix}.attn.{w}") for w in ("wq", "wk", "wv")]
            if all(p is not None for p in parts):
                var.data.data[:] = np.concatenate([np.asarray(p["data"], dtype=np.float32).reshape(-1) for p in parts])
