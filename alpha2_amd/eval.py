"""Validation loss / perplexity (packages/train/src/eval.ts:15-61): `nBatches` random batches of a text file through the
forward pass, mean of the batch losses, perplexity = exp(mean).  The corpus lives on the device (train.DataLoader) and
only one scalar per batch comes back to the host."""
from __future__ import annotations

import math
from dataclasses import dataclass

from .autograd import Tape
from .data import loadText
from .model import ModelConfig, gptForward
from .train import DataLoader


@dataclass
class EvalResult:
    loss: float
    perplexity: float
    nBatches: int


def evaluate(config: ModelConfig, params: dict, backend, tokenizer, rng, dataPath: str, batchSize: int, nBatches: int = 50) -> EvalResult:
    loader = DataLoader.fromText(backend, loadText(dataPath), tokenizer, rng, batchSize, config.blockSize)
    release = getattr(backend, "releaseGpuTensor", None)
    flush = getattr(backend, "flush", None)
    total = 0.0
    for i in range(nBatches):
        inputs, targets = loader.nextBatch()           # (the loader's ring owns these buffers: they are not released here)
        tape = Tape()
        loss = gptForward(config, params, backend, tape, inputs, targets)["loss"]
        if loss is not None:
            total += float(loss.data.data[0])
            if release is not None:
                release(loss.data)
        tape.clear(release)
        if flush is not None and (i & 7) == 7:
            flush()
    if flush is not None:
        flush()
    avg = total / nBatches
    return EvalResult(avg, math.exp(avg), nBatches)
