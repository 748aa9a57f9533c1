"""One optimizer step of the reference trainer on a `Backend`: AdamW (packages/train/src/optimizers.ts:21-234), the LR
schedule, micro-step gradient accumulation, gradient-norm clipping folded into the optimizer's gradScale, and
zero-grad (packages/train/src/trainer.ts:1088-1096,1146-1273,1297-1375,1650-1656,1761-1784).  Telemetry, spike
handling, sampling and checkpoint I/O of the reference's train() are outside this module."""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from .autograd import DropoutRng, Tape, Variable
from ._ffi import check
from .backend import HipBackend, TensorData, shapeSize
from .model import ModelConfig, collectParamEntries, gptForward, initGPT


@dataclass
class TrainConfig:
    """The fields of packages/core/src/types.ts:66-142 that the step arithmetic reads."""
    iters: int = 1000
    batchSize: int = 64
    lr: float = 3e-4
    lrMin: float = 0.0
    warmupIters: int = 0
    beta1: float = 0.9
    beta2: float = 0.95
    eps: float = 1e-8
    weightDecay: float = 0.1
    gradClip: float = 1.0
    seed: int = 42
    gradAccumSteps: int = 1
    optimizer: str = "adamw"          # "adamw" | "lion" | "adafactor" | "sgd" (optimizers.ts:596-603)


def noDecayNames(nLayer: int) -> set:
    """apps/cli/src/commands/train.ts:319-331.  "lmHead.weight" never matches the entry name "lmHead", so the head IS
    decayed -- kept as the reference has it."""
    s = {"wte", "wpe", "lnF.weight", "lnF.bias", "lmHead.weight"}
    for i in range(nLayer):
        s |= {f"layer.{i}.ln1.weight", f"layer.{i}.ln1.bias", f"layer.{i}.ln2.weight", f"layer.{i}.ln2.bias"}
    return s


class AdamW:
    """optimizers.ts:21-234.  Moments are host-created TensorData that become device-resident on first use; bias
    corrections come from running products of the betas (optimizers.ts:107-115)."""
    name = "adamw"

    def __init__(self, backend, lr=3e-4, beta1=0.9, beta2=0.999, eps=1e-8, weightDecay=0.01, noDecayNames=None):
        self.backend = backend
        self.lr, self.beta1, self.beta2, self.eps, self.weightDecay = lr, beta1, beta2, eps, weightDecay
        self.noDecayNames = noDecayNames or set()
        self._step = 0
        self._beta1Pow = 1.0
        self._beta2Pow = 1.0
        self._m: Dict[str, TensorData] = {}
        self._v: Dict[str, TensorData] = {}

    def setLr(self, lr: float):
        self.lr = lr

    def _moments(self, name: str, param: TensorData):
        if name not in self._m:
            n = shapeSize(param.shape)
            self._m[name] = TensorData(param.shape, "f32", np.zeros(n, dtype=np.float32))
            self._v[name] = TensorData(param.shape, "f32", np.zeros(n, dtype=np.float32))
        return self._m[name], self._v[name]

    def _next_bias_corrections(self):
        self._step += 1
        self._beta1Pow *= self.beta1
        self._beta2Pow *= self.beta2
        return 1 - self._beta1Pow, 1 - self._beta2Pow

    def stepParamEntries(self, entries, gradScale: float = 1.0):
        bc1, bc2 = self._next_bias_corrections()
        for name, var in entries:
            if var.grad is None:
                continue
            m, v = self._moments(name, var.data)
            wd = 0.0 if name in self.noDecayNames else self.weightDecay
            self.backend.adamwStep(var.data, var.grad, m, v, self.lr, self.beta1, self.beta2, self.eps, wd, bc1, bc2, gradScale)

    def step(self, params: Dict[str, TensorData], grads: Dict[str, TensorData], gradScale: float = 1.0):
        bc1, bc2 = self._next_bias_corrections()
        for name, p in params.items():
            g = grads.get(name)
            if g is None:
                continue
            m, v = self._moments(name, p)
            wd = 0.0 if name in self.noDecayNames else self.weightDecay
            self.backend.adamwStep(p, g, m, v, self.lr, self.beta1, self.beta2, self.eps, wd, bc1, bc2, gradScale)

    def stateDict(self) -> dict:
        """Reads the moments back from the device (the reference copies stale host arrays after any GPU adamwStep,
        optimizers.ts:202-210; that defect is not reproduced)."""
        bufs = {}
        for name, m in self._m.items():
            bufs[name + ".m"] = TensorData((m.size,), "f32", m.data.copy())
            bufs[name + ".v"] = TensorData((m.size,), "f32", self._v[name].data.copy())
        return {"step": self._step, "buffers": bufs}

    def loadStateDict(self, state: dict):
        self._step = state["step"]
        self._beta1Pow, self._beta2Pow = self.beta1 ** self._step, self.beta2 ** self._step
        self._m, self._v = {}, {}
        for key, td in state["buffers"].items():
            tgt = self._m if key.endswith(".m") else self._v
            tgt[key[:-2]] = TensorData(td.shape, "f32", np.array(td.data, dtype=np.float32))


def makeOptimizer(backend, tc: TrainConfig, noDecay: set):
    """apps/cli/src/commands/train.ts:333-340 with apps/cli/src/resolve.ts:25-36: the training configuration's lr / betas /
    eps / weight decay / no-decay names go to AdamW, Lion and Adafactor (each takes the fields it knows: Adafactor's eps
    becomes the training eps, its clip threshold stays 1); SGD comes from the registry with its own default lr, which
    the trainer's setLr overrides before the first step."""
    if tc.optimizer == "adamw":
        return AdamW(backend, tc.lr, tc.beta1, tc.beta2, tc.eps, tc.weightDecay, noDecay)
    from .optimizers import Adafactor, Lion, SGD
    if tc.optimizer == "lion":
        return Lion(backend, lr=tc.lr, beta1=tc.beta1, beta2=tc.beta2, weightDecay=tc.weightDecay, noDecayNames=noDecay)
    if tc.optimizer == "adafactor":
        return Adafactor(backend, lr=tc.lr, beta2=tc.beta2, eps=tc.eps, weightDecay=tc.weightDecay, noDecayNames=noDecay)
    if tc.optimizer == "sgd":
        return SGD(backend)
    raise ValueError(f'Unknown optimizer: "{tc.optimizer}". Available: adamw, lion, adafactor, sgd')


def lrAt(tc: TrainConfig, step: int) -> float:
    """trainer.ts:1088-1096,1150-1159 with runtimeLrScale = 1 and spikeLrMinScale = 0.1."""
    warmup = tc.warmupIters if tc.warmupIters > 0 else (0 if tc.warmupIters < 0 else min(2000, tc.iters // 5))
    lrMin = tc.lr / 10 if (tc.lrMin or 0) == 0 else tc.lrMin
    denom = max(1, tc.iters - warmup)
    if step < warmup:
        base = lrMin + (tc.lr - lrMin) * (step + 1) / warmup
    else:
        base = lrMin + (tc.lr - lrMin) * 0.5 * (1 + math.cos(math.pi * (step - warmup) / denom))
    return max(lrMin * 0.1, base)


def syntheticBatch(seed: int, Bt: int, T: int, vocab: int) -> Tuple[TensorData, TensorData]:
    """Uniform ids from SeededRng(seed): B*(T+1) draws floor(next()*vocab), row b = draws [b(T+1), (b+1)(T+1));
    inputs are the first T, targets the last T (the shift-by-one of packages/train/src/data.ts:110-114)."""
    from .rng import SeededRng
    ids = np.floor(SeededRng(seed).fillUniform(Bt * (T + 1)) * vocab).astype(np.int32).reshape(Bt, T + 1)
    return TensorData((Bt, T), "i32", ids[:, :T]), TensorData((Bt, T), "i32", ids[:, 1:])


def zipfBatch(seed: int, Bt: int, T: int, vocab: int, s: float = 1.1) -> Tuple[TensorData, TensorData]:
    """Token ids Zipf(s) over [0, vocab) by inverse CDF of the seeded uniform stream; targets shifted by one."""
    from .rng import SeededRng
    w = 1.0 / np.power(np.arange(1, vocab + 1, dtype=np.float64), s)
    cdf = np.cumsum(w / w.sum())
    u = SeededRng(seed).fillUniform(Bt * (T + 1))
    ids = np.minimum(np.searchsorted(cdf, u, side="right"), vocab - 1).astype(np.int32).reshape(Bt, T + 1)
    return TensorData((Bt, T), "i32", ids[:, :T]), TensorData((Bt, T), "i32", ids[:, 1:])


def zipfBatches(seed: int, count: int, Bt: int, T: int, vocab: int, s: float = 1.1) -> List[Tuple[TensorData, TensorData]]:
    """`count` successive batches cut from ONE seeded uniform stream (batch k takes draws [k B (T+1), (k+1) B (T+1))).  Streams
    of neighbouring seeds are no substitute for this: the reference's xorshift (packages/core/src/rng.ts:13-50) seeded with s
    and s + 1 gives sequences that correlate at 0.5, i.e. near-copies of the same batch."""
    from .rng import SeededRng
    w = 1.0 / np.power(np.arange(1, vocab + 1, dtype=np.float64), s)
    cdf = np.cumsum(w / w.sum())
    n = Bt * (T + 1)
    u = SeededRng(seed).fillUniform(count * n)
    out = []
    for k in range(count):
        ids = np.minimum(np.searchsorted(cdf, u[k * n:(k + 1) * n], side="right"), vocab - 1).astype(np.int32).reshape(Bt, T + 1)
        out.append((TensorData((Bt, T), "i32", ids[:, :T]), TensorData((Bt, T), "i32", ids[:, 1:])))
    return out


class DataLoader:
    """DataLoader of packages/train/src/data.ts:19-175 with the corpus resident in HBM: the token array is uploaded
    once, a batch is one `ah_token_windows` launch given B window starts.  Random mode draws
    start = floor(rng.next() * (N - T)) per row (data.ts:104-114); packed mode keeps B cursors b*floor(N/B) that advance
    T per batch and wrap at the end of the corpus (data.ts:131-167).  Batches come from a ring of two buffer pairs,
    like the reference's, so a batch stays valid until the call after next."""

    def __init__(self, B: HipBackend, tokens, rng, batchSize: int, blockSize: int, packed: bool = False):
        self.B, self.rng, self.batchSize, self.blockSize, self.packed = B, rng, int(batchSize), int(blockSize), bool(packed)
        tok = np.ascontiguousarray(tokens, dtype=np.int32).reshape(-1)
        self.length = int(tok.size)
        self._corpus = TensorData((max(1, self.length),), "i32", tok if self.length else np.zeros(1, np.int32))
        B._ptr(self._corpus)
        self.cursors = [b * (self.length // self.batchSize) for b in range(self.batchSize)] if packed else None
        self._ring = [(B._new((self.batchSize, self.blockSize), "i32"), B._new((self.batchSize, self.blockSize), "i32")) for _ in range(2)]
        self._ringIdx = 0

    @classmethod
    def fromText(cls, B: HipBackend, text: str, tokenizer, rng, batchSize: int, blockSize: int, packed: bool = False) -> "DataLoader":
        """data.ts:61-87."""
        from .data import encodeText
        return cls(B, encodeText(text, tokenizer), rng, batchSize, blockSize, packed)

    @property
    def stepsPerEpoch(self) -> int:
        return self.length // (self.batchSize * self.blockSize)

    def nextBatch(self) -> Tuple[TensorData, TensorData]:
        Bt, T, N = self.batchSize, self.blockSize, self.length
        if self.packed:
            if N == 0:
                raise IndexError("packed DataLoader over an empty corpus")
            starts = list(self.cursors)
            self.cursors = [(c + T) % N for c in self.cursors]
        else:
            if N <= T:
                raise IndexError(f"Token count ({N}) must exceed block size ({T}) — need at least {T + 1} tokens for input+target windows")
            maxStart = N - T
            starts = [int(math.floor(self.rng.next() * maxStart)) for _ in range(Bt)]
        inputs, targets = self._ring[self._ringIdx]
        self._ringIdx = (self._ringIdx + 1) % len(self._ring)
        for t in (inputs, targets):
            # The trainer releases the device copy of every batch it has consumed (trainer.ts:1267-1272); the reference's
            # ring holds host arrays, so only that copy goes.  Here the ring IS the device copy: a released slot gets a
            # fresh buffer before it is written again.
            B_ = self.B
            if t._buf is None:
                fresh = B_._new(t.shape, "i32")
                t._buf, t._off, t._dev_valid, t._backend = fresh._buf, 0, True, B_
                fresh._buf = None
        st = TensorData((Bt,), "f64", np.asarray(starts, dtype=np.int64).view(np.float64))     # 8-byte slots holding the int64 starts
        B = self.B
        check(B.lib.ah_token_windows(B._ptr(self._corpus), N, B._ptr(st), Bt, T, B._ptr(inputs), B._ptr(targets)))
        B.releaseGpuTensor(st)
        B._dirty(inputs), B._dirty(targets)
        return inputs, targets


@dataclass
class StepResult:
    loss: float
    gradNorm: float
    clipCoef: float
    lr: float


class Trainer:
    """The step body of train() (trainer.ts:1146-1784) over any Backend."""

    def __init__(self, backend, cfg: ModelConfig, tc: TrainConfig, seed: int = 0, rng=None):
        from .rng import SeededRng
        self.backend, self.cfg, self.tc = backend, cfg, tc
        self.rng = rng or SeededRng(seed)
        self.params = initGPT(cfg, backend, self.rng)
        self.entries = collectParamEntries(self.params)
        self.optimizer = makeOptimizer(backend, tc, noDecayNames(cfg.nLayer))
        self.tape = Tape()
        self.dropoutRng = DropoutRng(tc.seed)
        self.stepIdx = 0
        self.release = getattr(backend, "releaseGpuTensor", None)

    def saveCheckpoint(self, path: str, configHash: str = "", tokenizerArtifacts=None):
        """Full training state in the reference's file format (checkpoint.ts:197-221)."""
        from dataclasses import asdict
        from .checkpoint import FileCheckpoint, buildCheckpointState
        self.backend.syncGpu()
        rng_state = getattr(self.rng, "state", lambda: 0)()
        FileCheckpoint().save(path, buildCheckpointState(self.entries, self.optimizer, rng_state, configHash, self.stepIdx,
                                                         asdict(self.cfg), tokenizerArtifacts))

    def loadCheckpoint(self, path: str) -> dict:
        """Resume: parameters, Adam moments and the step counter (trainer.ts:905-960 restores the same three)."""
        from .checkpoint import FileCheckpoint, restoreParams
        st = FileCheckpoint().load(path)
        restoreParams(self.entries, st["params"])
        self.optimizer.loadStateDict(st["optimizerState"])
        self.stepIdx = int(st.get("step") or 0)
        return st

    def step(self, batches: Sequence[Tuple[TensorData, TensorData]]) -> StepResult:
        B, tc = self.backend, self.tc
        lr = lrAt(tc, self.stepIdx)
        self.optimizer.setLr(lr)
        accum = len(batches)
        lossAccum = None
        lossVal = 0.0
        for micro, (inp, tgt) in enumerate(batches):
            self.dropoutRng.reset(tc.seed + self.stepIdx * 1000 + micro, 0)
            loss = gptForward(self.cfg, self.params, B, self.tape, inp, tgt, True, False, False, self.dropoutRng, self.release)["loss"]
            lossRef = loss.data
            if accum > 1:                                   # trainer.ts:1208-1223: stays on the device
                scaled = B.scale(loss.data, 1 / accum)
                if lossAccum is None:
                    lossAccum = scaled
                else:
                    B.addInplace(lossAccum, scaled)
                    self._rel(scaled)
            self.tape.backward(loss, B, self._keep(lossRef) if accum == 1 else self.release)
            if accum == 1:
                lossVal = float(lossRef.data[0])            # host sync #1 (trainer.ts:1247)
                self._rel(lossRef)
            self.tape.clear(self.release)
            self._rel(inp), self._rel(tgt)                  # trainer.ts:1267-1272
        if accum > 1:
            lossVal = float(lossAccum.data[0])
            self._rel(lossAccum)
        gradScale = 1.0 / accum
        grads = [v.grad for _, v in self.entries if v.grad is not None]
        totalSq = B.totalSumOfSquares(grads)
        gradNorm = math.sqrt(float(totalSq.data[0])) * abs(gradScale)     # host sync #2 (trainer.ts:1348)
        self._rel(totalSq)
        clipCoef, eff = 1.0, gradScale
        if tc.gradClip > 0 and gradNorm > tc.gradClip:
            clipCoef = tc.gradClip / gradNorm
            eff *= clipCoef
        if math.isfinite(lossVal) and math.isfinite(gradNorm):
            self.optimizer.stepParamEntries(self.entries, eff)
        for _, v in self.entries:
            if v.grad is not None:
                self._rel(v.grad)
            v.grad = None
        if hasattr(B, "flush"):
            B.flush()
        self.stepIdx += 1
        return StepResult(lossVal, gradNorm, clipCoef, lr)

    def _rel(self, td):
        if self.release is not None and td is not None:
            self.release(td)

    def _keep(self, keep: TensorData):
        """Release callback that spares the loss scalar until the host has read it."""
        rel = self.release
        if rel is None:
            return None
        return lambda td: None if td is keep else rel(td)
