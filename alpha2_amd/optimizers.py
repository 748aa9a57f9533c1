"""The reference's optimizer registry beyond AdamW (packages/train/src/optimizers.ts:236-603): Lion, Adafactor, SGD, with
the same constructor defaults, method names and state-dict keys, on device-resident parameters and state.

The reference runs these as host loops over Float32Arrays (double arithmetic, one rounding per store); the kernels behind
`HipBackend.lionStep / adafactorStep2d / adafactorStepFlat / sgdStep` compute the same way."""
from __future__ import annotations

from typing import Dict, Optional

import numpy as np

from .backend import TensorData, shapeSize
from .train import AdamW


class Lion:
    """optimizers.ts:246-336."""
    name = "lion"

    def __init__(self, backend, lr=1e-4, beta1=0.9, beta2=0.99, weightDecay=0.01, noDecayNames=None):
        self.backend = backend
        self.lr, self.beta1, self.beta2, self.weightDecay = lr, beta1, beta2, weightDecay
        self.noDecayNames = noDecayNames or set()
        self._step = 0
        self._m: Dict[str, TensorData] = {}

    def setLr(self, lr: float):
        self.lr = lr

    def _stepTensor(self, name, param, grad, gradScale):
        if name not in self._m:
            self._m[name] = TensorData((shapeSize(param.shape),), "f32", np.zeros(shapeSize(param.shape), dtype=np.float32))
        wd = 0.0 if name in self.noDecayNames else self.weightDecay
        self.backend.lionStep(param, grad, self._m[name], self.lr, self.beta1, self.beta2, wd, gradScale)

    def stepParamEntries(self, entries, gradScale: float = 1.0):
        self._step += 1
        for name, var in entries:
            if var.grad is not None:
                self._stepTensor(name, var.data, var.grad, gradScale)

    def step(self, params: Dict[str, TensorData], grads: Dict[str, TensorData], gradScale: float = 1.0):
        self._step += 1
        for name, p in params.items():
            g = grads.get(name)
            if g is not None:
                self._stepTensor(name, p, g, gradScale)

    def stateDict(self) -> dict:
        return {"step": self._step, "buffers": {name + ".m": TensorData((m.size,), "f32", m.data.copy()) for name, m in self._m.items()}}

    def loadStateDict(self, state: dict):
        self._step = state["step"]
        self._m = {}
        for key, td in state["buffers"].items():
            if key.endswith(".m"):
                self._m[key[:-2]] = TensorData((td.size,), "f32", np.array(td.data, dtype=np.float32))


class Adafactor:
    """optimizers.ts:349-543: factored second moments (row / column) for 2-D parameters, a full one otherwise; the update
    is clipped by its RMS; no first moment."""
    name = "adafactor"

    def __init__(self, backend, lr=1e-3, beta2=0.999, eps=1e-30, clipThreshold=1.0, weightDecay=0.0, noDecayNames=None):
        self.backend = backend
        self.lr, self.beta2, self.eps, self.clipThreshold, self.weightDecay = lr, beta2, eps, clipThreshold, weightDecay
        self.noDecayNames = noDecayNames or set()
        self._step = 0
        self._vr: Dict[str, TensorData] = {}
        self._vc: Dict[str, TensorData] = {}
        self._v: Dict[str, TensorData] = {}

    def setLr(self, lr: float):
        self.lr = lr

    @staticmethod
    def _state(table, name, n):
        t = table.get(name)
        if t is None or t.size != n:          # optimizers.ts:417-424,480-483: re-created when the length changes
            t = table[name] = TensorData((n,), "f32", np.zeros(n, dtype=np.float32))
        return t

    def _stepTensor(self, name, param, grad, gradScale):
        wd = 0.0 if name in self.noDecayNames else self.weightDecay
        if len(param.shape) == 2:
            rows, cols = param.shape
            self.backend.adafactorStep2d(param, grad, self._state(self._vr, name, rows), self._state(self._vc, name, cols), self.lr, self.beta2,
                                         self.eps, self.clipThreshold, wd, gradScale)
        else:
            self.backend.adafactorStepFlat(param, grad, self._state(self._v, name, shapeSize(param.shape)), self.lr, self.beta2, self.eps,
                                           self.clipThreshold, wd, gradScale)

    def stepParamEntries(self, entries, gradScale: float = 1.0):
        self._step += 1
        for name, var in entries:
            if var.grad is not None:
                self._stepTensor(name, var.data, var.grad, gradScale)

    def step(self, params: Dict[str, TensorData], grads: Dict[str, TensorData], gradScale: float = 1.0):
        self._step += 1
        for name, p in params.items():
            g = grads.get(name)
            if g is not None:
                self._stepTensor(name, p, g, gradScale)

    def stateDict(self) -> dict:
        bufs = {}
        for suffix, table in ((".vr", self._vr), (".vc", self._vc), (".v", self._v)):       # optimizers.ts:503-514: in this order
            for name, t in table.items():
                bufs[name + suffix] = TensorData((t.size,), "f32", t.data.copy())
        return {"step": self._step, "buffers": bufs}

    def loadStateDict(self, state: dict):
        self._step = state["step"]
        self._vr, self._vc, self._v = {}, {}, {}
        for key, td in state["buffers"].items():
            copy = TensorData((td.size,), "f32", np.array(td.data, dtype=np.float32))
            if key.endswith(".vr"):
                self._vr[key[:-3]] = copy
            elif key.endswith(".vc"):
                self._vc[key[:-3]] = copy
            elif key.endswith(".v"):
                self._v[key[:-2]] = copy


class SGD:
    """optimizers.ts:546-593."""
    name = "sgd"

    def __init__(self, backend, lr=0.01):
        self.backend, self.lr = backend, lr
        self._step = 0

    def setLr(self, lr: float):
        self.lr = lr

    def stepParamEntries(self, entries, gradScale: float = 1.0):
        self._step += 1
        for _, var in entries:
            if var.grad is not None:
                self.backend.sgdStep(var.data, var.grad, self.lr, gradScale)

    def step(self, params: Dict[str, TensorData], grads: Dict[str, TensorData], gradScale: float = 1.0):
        self._step += 1
        for name, p in params.items():
            g = grads.get(name)
            if g is not None:
                self.backend.sgdStep(p, g, self.lr, gradScale)

    def stateDict(self) -> dict:
        return {"step": self._step, "buffers": {}}

    def loadStateDict(self, state: dict):
        self._step = state["step"]


def createOptimizerRegistry(backend) -> Dict[str, object]:
    """optimizers.ts:596-603: name -> factory with the reference's defaults."""
    return {"adamw": lambda **kw: AdamW(backend, **kw), "lion": lambda **kw: Lion(backend, **kw),
            "adafactor": lambda **kw: Adafactor(backend, **kw), "sgd": lambda **kw: SGD(backend, **kw)}
