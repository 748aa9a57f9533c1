"""The reference's checkpoint files (packages/train/src/checkpoint.ts:1-260): the "ALPH" binary container and the legacy
JSON form, plus buildCheckpointState / restoreParams, so that state written by either side loads on the other.

Binary layout (checkpoint.ts:6-11):
    4 bytes  magic "ALPH"
    4 bytes  uint32 LE: byte length of the header
    N bytes  header JSON (UTF-8): modelConfig, configHash, rngState, step, tokenizerArtifacts, optimizerStep,
             [symbioActivationGraph], tensors = [{name, shape, elements}, ...]
    rest     the tensors' float32 data, little endian, concatenated in header order: parameters as "p.<name>", then
             optimizer buffers as "o.<name>" ("<param>.m", "<param>.v" for AdamW, optimizers.ts:202-210).
"""
from __future__ import annotations

import json
import os
import struct
from typing import Dict, Optional

import numpy as np

from .backend import TensorData

MAGIC = b"ALPH"


class CheckpointError(Exception):
    """packages/core CheckpointError: every failure of save / load surfaces as this type (checkpoint.ts:148-156)."""


def _f32(data) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(data, dtype=np.float32).reshape(-1)).astype("<f4", copy=False)


def saveBinary(path: str, state: dict) -> None:
    """checkpoint.ts:29-94: parameters first, then optimizer buffers, one header, raw float32 payload."""
    tensors, arrays = [], []
    for name, p in state["params"].items():
        f32 = _f32(p["data"])
        tensors.append({"name": f"p.{name}", "shape": [int(x) for x in p["shape"]], "elements": int(f32.size)})
        arrays.append(f32)
    opt = state.get("optimizerState")
    if opt and opt.get("buffers"):
        for name, td in opt["buffers"].items():
            f32 = _f32(td.data)
            tensors.append({"name": f"o.{name}", "shape": [int(x) for x in td.shape], "elements": int(f32.size)})
            arrays.append(f32)
    header = {"modelConfig": state.get("modelConfig"), "configHash": state.get("configHash"), "rngState": state.get("rngState"),
              "step": state.get("step")}
    if state.get("tokenizerArtifacts") is not None:          # JSON.stringify drops undefined members
        header["tokenizerArtifacts"] = state["tokenizerArtifacts"]
    header["optimizerStep"] = (opt or {}).get("step", 0)
    if state.get("symbioActivationGraph") is not None:
        header["symbioActivationGraph"] = state["symbioActivationGraph"]
    header["tensors"] = tensors
    hb = json.dumps(header, separators=(",", ":"), ensure_ascii=False).encode("utf-8")
    d = os.path.dirname(path)
    if d:
        os.makedirs(d, exist_ok=True)
    with open(path, "wb") as f:
        f.write(MAGIC)
        f.write(struct.pack("<I", len(hb)))
        f.write(hb)
        for a in arrays:
            f.write(a.tobytes())


def loadBinary(raw: bytes) -> dict:
    """checkpoint.ts:98-136."""
    (hlen,) = struct.unpack_from("<I", raw, 4)
    off = 8
    header = json.loads(raw[off:off + hlen].decode("utf-8"))
    off += hlen
    params: Dict[str, dict] = {}
    buffers: Dict[str, TensorData] = {}
    for t in header["tensors"]:
        n = int(t["elements"])
        if off + 4 * n > len(raw):
            raise ValueError(f"tensor {t['name']} runs past the end of the file")
        f32 = np.frombuffer(raw, dtype="<f4", count=n, offset=off).astype(np.float32)
        off += 4 * n
        if t["name"].startswith("p."):
            params[t["name"][2:]] = {"shape": list(t["shape"]), "data": f32}
        elif t["name"].startswith("o."):
            buffers[t["name"][2:]] = TensorData(t["shape"], "f32", f32)
    out = {"modelConfig": header.get("modelConfig"), "params": params,
           "optimizerState": {"step": header.get("optimizerStep") or 0, "buffers": buffers},
           "tokenizerArtifacts": header.get("tokenizerArtifacts"), "rngState": header.get("rngState"),
           "configHash": header.get("configHash"), "step": header.get("step")}
    if header.get("symbioActivationGraph"):
        out["symbioActivationGraph"] = header["symbioActivationGraph"]
    return out


class FileCheckpoint:
    """checkpoint.ts:146-193.  save() always writes the binary form; load() detects the form from the first bytes."""

    def save(self, path: str, state: dict) -> None:
        try:
            saveBinary(path, state)
        except Exception as e:            # noqa: BLE001 - the reference wraps every cause
            raise CheckpointError(f"Failed to save checkpoint: {e}") from e

    def load(self, path: str) -> dict:
        try:
            with open(path, "rb") as f:
                raw = f.read()
            if len(raw) >= 4 and raw[:4] == MAGIC:
                return loadBinary(raw)
            parsed = json.loads(raw.decode("utf-8"))          # legacy JSON (checkpoint.ts:168-189)
            buffers = {}
            for k, v in ((parsed.get("optimizerState") or {}).get("buffers") or {}).items():
                buffers[k] = TensorData(v["shape"], "f32", np.asarray(v["data"], dtype=np.float32))
            return {"modelConfig": parsed.get("modelConfig"), "params": parsed.get("params"),
                    "optimizerState": {"step": (parsed.get("optimizerState") or {}).get("step") or 0, "buffers": buffers},
                    "tokenizerArtifacts": parsed.get("tokenizerArtifacts"), "rngState": parsed.get("rngState"),
                    "configHash": parsed.get("configHash"), "step": parsed.get("step")}
        except Exception as e:            # noqa: BLE001
            raise CheckpointError(f"Failed to load checkpoint: {e}") from e


def buildCheckpointState(entries, optimizer, rngState, configHash: str, step: int, modelConfig, tokenizerArtifacts=None) -> dict:
    """checkpoint.ts:197-221.  `entries` = collectParamEntries(params); parameter values are read back from the device."""
    params = {name: {"shape": list(v.data.shape), "data": np.array(v.data.data, dtype=np.float32)} for name, v in entries}
    return {"modelConfig": modelConfig, "params": params, "optimizerState": optimizer.stateDict(), "tokenizerArtifacts": tokenizerArtifacts,
            "rngState": rngState, "configHash": configHash, "step": step}


def restoreParams(entries, checkpointParams: Dict[str, dict]) -> None:
    """checkpoint.ts:224-259: copy saved values into the existing parameters; a checkpoint from before the fused QKV
    projection carries wq / wk / wv, which are concatenated into wqkv."""
    for name, var in entries:
        saved = checkpointParams.get(name)
        if saved is not None:
            arr = np.asarray(saved["data"], dtype=np.float32).reshape(-1)
            if arr.size < var.data.size:
                raise ValueError(f"checkpoint tensor {name} has {arr.size} values, the model needs {var.data.size}")
            var.data.data = arr[:var.data.size].copy()        # the setter marks the device copy stale
            continue
        if name.endswith(".attn.wqkv"):
            prefix = name[:-len(".attn.wqkv")]
            parts = [checkpointParams.get(f"{prefix}.attn.{w}") for w in ("wq", "wk", "wv")]
            if all(p is not None for p in parts):
                var.data.data = np.concatenate([np.asarray(p["data"], dtype=np.float32).reshape(-1) for p in parts])
