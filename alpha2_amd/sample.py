"""Text generation from a trained model (packages/train/src/sample.ts:23-201): one forward per new token over the last
blockSize tokens, then greedy / top-k / nucleus / full-softmax selection on the host with the reference's arithmetic (f32
storage, double accumulation, stable descending sorts) and its use of the seeded rng (one draw per sampled token)."""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Callable, Optional, Sequence

import numpy as np

from .autograd import Tape
from .backend import TensorData
from .model import ModelConfig, gptForward


@dataclass
class SampleConfig:
    """packages/core/src/types.ts:145-158."""
    steps: int = 200
    temperature: float = 0.8
    topk: int = 40
    topp: Optional[float] = 1.0


def _stable_desc(values: np.ndarray) -> np.ndarray:
    """Indices by descending value; equal values keep their index order (Array.prototype.sort is stable)."""
    return np.argsort(-values.astype(np.float64), kind="stable")


def selectToken(lastLogits: np.ndarray, rng, temperature: float, topk: int, topP: float) -> int:
    """sample.ts:85-193 for one position.  `lastLogits` is the f32 row already divided by the temperature (when
    positive); it is modified in place exactly as the reference modifies its copy."""
    V = lastLogits.size
    if temperature <= 0:                                                    # sample.ts:85-99: first maximum wins
        return int(np.argmax(lastLogits))
    if 0 < topk < V:                                                        # sample.ts:102-109: ties with the k-th value stay
        threshold = lastLogits[_stable_desc(lastLogits)[topk - 1]]
        lastLogits[lastLogits < threshold] = -np.inf
    if 0 < topP < 1:                                                        # sample.ts:112-163
        maxVal = float(np.max(lastLogits))
        if math.isfinite(maxVal):
            fin = np.isfinite(lastLogits)
            p64 = np.where(fin, np.exp(lastLogits.astype(np.float64) - maxVal), 0.0)
            probs = p64.astype(np.float32)
            active = np.nonzero(fin)[0]
            sumExp = float(np.cumsum(p64[active])[-1]) if active.size else 0.0          # sums the unrounded exponentials
            if sumExp > 0 and active.size > 0:
                active = active[_stable_desc(probs[active])]
                target = sumExp * topP
                keptMass, keepCount = 0.0, 0
                while keepCount < active.size:
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
                cum, sampled = 0.0, int(active[keepCount - 1])
                for i in range(keepCount):
                    cum += float(probs[active[i]])
                    if r < cum:
                        sampled = int(active[i])
                        break
                return sampled
    maxVal = float(np.max(lastLogits))                                      # sample.ts:166-188
    probs = np.exp(lastLogits.astype(np.float64) - maxVal).astype(np.float32)
    sumExp = float(np.cumsum(probs.astype(np.float64))[-1])                 # sums the f32-rounded values, left to right
    probs = (probs.astype(np.float64) / sumExp).astype(np.float32)
    r = rng.next()
    cum = np.cumsum(probs.astype(np.float64))
    hit = np.nonzero(r < cum)[0]
    return int(hit[0]) if hit.size else 0


def sampleTokens(config: ModelConfig, params: dict, backend, rng, promptTokens: Sequence[int], sampleConfig: SampleConfig,
                 releaseTensor: Optional[Callable] = None, flushGpu: Optional[Callable] = None) -> np.ndarray:
    """The token loop of sample() (sample.ts:36-198) without the tokenizer: returns prompt + generated ids."""
    steps, temperature, topk = sampleConfig.steps, sampleConfig.temperature, sampleConfig.topk
    topp = sampleConfig.topp
    topP = min(1.0, max(0.0, topp)) if (topp is not None and math.isfinite(topp)) else 1.0
    prompt = np.asarray(promptTokens, dtype=np.int32)
    maxLen = min(prompt.size + steps, config.blockSize)
    tokens = np.zeros(maxLen, dtype=np.int32)
    tokens[: min(prompt.size, maxLen)] = prompt[:maxLen]                    # Int32Array.set of a longer prompt throws in JS;
    if prompt.size > maxLen:                                                # say so instead of truncating silently
        raise ValueError(f"prompt of {prompt.size} tokens exceeds blockSize {config.blockSize}")
    currentLen = int(prompt.size)
    V = config.vocabSize
    i = 0
    while i < steps and currentLen < config.blockSize:
        ctxStart = max(0, currentLen - config.blockSize)
        ctx = tokens[ctxStart:currentLen].copy()
        inputData = TensorData((1, ctx.size), "i32", ctx)
        tape = Tape()
        logits = gptForward(config, params, backend, tape, inputData)["logits"]
        row = backend.slice(logits.data, [0, ctx.size - 1, 0], [1, ctx.size, V]) if hasattr(backend, "slice") else None
        last = np.asarray(row.data if row is not None else logits.data.data.reshape(-1)[(ctx.size - 1) * V:], dtype=np.float32).reshape(-1).copy()
        if row is not None and releaseTensor is not None:
            releaseTensor(row)
        if temperature > 0:
            last = (last.astype(np.float64) / temperature).astype(np.float32)
        tape.clear(releaseTensor)
        if releaseTensor is not None:
            releaseTensor(inputData)
        if flushGpu is not None and (i & 7) == 7:
            flushGpu()
        nxt = selectToken(last, rng, temperature, topk, topP)
        if currentLen < maxLen:
            tokens[currentLen] = nxt
            currentLen += 1
        i += 1
    return tokens[:currentLen]


def sample(config: ModelConfig, params: dict, backend, rng, encode: Callable, decode: Callable, prompt: str, sampleConfig: SampleConfig,
           releaseTensor: Optional[Callable] = None, flushGpu: Optional[Callable] = None) -> str:
    """sample.ts:23-201."""
    return decode(sampleTokens(config, params, backend, rng, encode(prompt), sampleConfig, releaseTensor, flushGpu))
