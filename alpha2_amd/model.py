"""GPT decoder (pre-LN, untied lmHead, bias-free linears) -- the caller side of the backend for one forward pass,
mirroring packages/model/src/gpt.ts: initGPT (:73-151), transformerBlock (:220-333), gptForward (:344-427),
collectParamEntries (:433-468)."""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import numpy as np

from . import autograd as ag
from .autograd import Ctx, Tape, Variable
from .backend import TensorData, shapeSize


@dataclass
class ModelConfig:
    """packages/core/src/types.ts:51-64."""
    vocabSize: int = 256
    blockSize: int = 256
    nLayer: int = 6
    nEmbd: int = 256
    nHead: int = 8
    dropout: float = 0.0
    ffnActivation: str = "gelu"
    ffnDim: Optional[int] = None
    softCap: Optional[float] = None
    activationGraph: Optional[dict] = None
    # "heads": true multi-head attention (what the reference's cpu_ref branch computes, gpt.ts:255-279), run by the
    #          strided flash kernel.  "reference-flash": the reshape-without-head-transpose the reference applies when a
    #          backend exposes flashAttention (gpt.ts:248-254) -- a different function, kept for drop-in fidelity.
    #          "unfused": the op-by-op chain.
    attention: str = "heads"


def _init_weight(rng, shape, std) -> Variable:
    return Variable(TensorData(shape, "f32", rng.fillGauss(shapeSize(shape), std)), True)


def _const(backend, shape, value) -> Variable:
    return Variable(TensorData(shape, "f32", np.full(shapeSize(shape), value, dtype=np.float32)), True)


def ffn_dim(cfg: ModelConfig) -> int:
    act = cfg.ffnActivation or "gelu"
    return cfg.ffnDim or (math.ceil((8 / 3) * cfg.nEmbd / 64) * 64 if act == "swiglu" else 4 * cfg.nEmbd)


def initGPT(cfg: ModelConfig, backend, rng) -> dict:
    """gpt.ts:73-151.  RNG draw order: wte, wpe, then per layer the MLP weights, then wqkv, wo; lmHead last."""
    V, T, L, Cc = cfg.vocabSize, cfg.blockSize, cfg.nLayer, cfg.nEmbd
    act = cfg.ffnActivation or "gelu"
    std = 0.02
    wte = _init_weight(rng, [V, Cc], std)
    wpe = _init_weight(rng, [T, Cc], std)
    F = ffn_dim(cfg)
    layers = []
    for _ in range(L):
        if act == "swiglu":
            mlp = {"fc_gate": _init_weight(rng, [F, Cc], std), "fc_up": _init_weight(rng, [F, Cc], std),
                   "fc_proj": _init_weight(rng, [Cc, F], std / math.sqrt(2 * L))}
        else:
            mlp = {"fc1": _init_weight(rng, [F, Cc], std), "fc2": _init_weight(rng, [Cc, F], std / math.sqrt(2 * L))}
            if act == "universal":
                mlp["act_gate"], mlp["act_skip"] = _const(backend, [1, F], 1.0), _const(backend, [1, F], 0.0)
            elif act == "kan_spline":
                for k, v in (("kan_c0", 0.5), ("kan_c1", 0.0), ("kan_c2", 0.5), ("kan_c3", 0.0), ("kan_c4", 0.0)):
                    mlp[k] = _const(backend, [1, F], v)
        layers.append({
            "ln1": {"weight": _const(backend, [Cc], 1.0), "bias": _const(backend, [Cc], 0.0)},
            "attn": {"wqkv": _init_weight(rng, [3 * Cc, Cc], std), "wo": _init_weight(rng, [Cc, Cc], std / math.sqrt(2 * L))},
            "ln2": {"weight": _const(backend, [Cc], 1.0), "bias": _const(backend, [Cc], 0.0)},
            "mlp": mlp,
        })
    lnF = {"weight": _const(backend, [Cc], 1.0), "bias": _const(backend, [Cc], 0.0)}
    lmHead = _init_weight(rng, [V, Cc], std)
    return {"wte": wte, "wpe": wpe, "layers": layers, "lnF": lnF, "lmHead": lmHead}


def collectParamEntries(params: dict) -> List[Tuple[str, Variable]]:
    """gpt.ts:433-468 (names are what the optimizer's no-decay set is matched against)."""
    e = [("wte", params["wte"]), ("wpe", params["wpe"]), ("lmHead", params["lmHead"]),
         ("lnF.weight", params["lnF"]["weight"]), ("lnF.bias", params["lnF"]["bias"])]
    for i, l in enumerate(params["layers"]):
        e += [(f"layer.{i}.ln1.weight", l["ln1"]["weight"]), (f"layer.{i}.ln1.bias", l["ln1"]["bias"]),
              (f"layer.{i}.attn.wqkv", l["attn"]["wqkv"]), (f"layer.{i}.attn.wo", l["attn"]["wo"]),
              (f"layer.{i}.ln2.weight", l["ln2"]["weight"]), (f"layer.{i}.ln2.bias", l["ln2"]["bias"])]
        m = l["mlp"]
        if "fc_gate" in m:
            e += [(f"layer.{i}.mlp.fc_gate", m["fc_gate"]), (f"layer.{i}.mlp.fc_up", m["fc_up"]), (f"layer.{i}.mlp.fc_proj", m["fc_proj"])]
        else:
            e += [(f"layer.{i}.mlp.fc1", m["fc1"]), (f"layer.{i}.mlp.fc2", m["fc2"])]
        for k in ("act_gate", "act_skip", "kan_c0", "kan_c1", "kan_c2", "kan_c3", "kan_c4"):
            if k in m:
                e.append((f"layer.{i}.mlp.{k}", m[k]))
    return e


def countParams(params: dict) -> int:
    return sum(shapeSize(v.data.shape) for _, v in collectParamEntries(params))


def _eval_activation_graph(ctx, x, node):
    """gpt.ts:170-192: expression tree over {silu, relu, gelu, identity, square} with scale / add / mul nodes."""
    t = node["type"]
    if t == "basis":
        op = node["op"]
        if op == "silu":
            return ag.silu(ctx, x)
        if op == "relu":
            return ag.relu(ctx, x)
        if op == "identity":
            return x
        if op == "square":
            return ag.mul(ctx, x, x)
        return ag.gelu(ctx, x)
    if t == "scale":
        return ag.scale(ctx, _eval_activation_graph(ctx, x, node["child"]), node["factor"])
    left, right = _eval_activation_graph(ctx, x, node["left"]), _eval_activation_graph(ctx, x, node["right"])
    return ag.add(ctx, left, right) if t == "add" else ag.mul(ctx, left, right)


_mask_cache: Dict[Tuple[int, int], TensorData] = {}
_pos_cache: Dict[Tuple[int, int, int], TensorData] = {}


def clearForwardCache():
    _mask_cache.clear()
    _pos_cache.clear()


def flashHeadSize(d: int) -> bool:
    """Head sizes the fused attention kernels take: multiples of 8 up to 128 (others run the same function op by op)."""
    return 8 <= d <= 128 and d % 8 == 0


def transformerBlock(ctx: Ctx, x: Variable, layer: dict, cfg: ModelConfig, Bt: int, T: int, mask, training: bool) -> Variable:
    """gpt.ts:220-333."""
    H, Cc = cfg.nHead, cfg.nEmbd
    D = Cc // H
    Bk = ctx.backend
    ln1 = ag.layerNorm(ctx, x, layer["ln1"]["weight"], layer["ln1"]["bias"], 1e-5)
    qkv = ag.matmulTransposed(ctx, ag.reshape(ctx, ln1, [Bt * T, Cc]), layer["attn"]["wqkv"])
    cap = cfg.softCap if cfg.softCap is not None else 30.0
    scl = 1 / math.sqrt(D)
    if cfg.attention == "heads" and cfg.dropout == 0 and ag._has(Bk, "attentionQkv") and flashHeadSize(D):
        concat = ag.causalSelfAttention(ctx, qkv, Bt, T, H, scl, cap)
    else:
        qF, kF, vF = ag.sliceQkv(ctx, qkv)
        q, k, v = (ag.reshape(ctx, t, [Bt, T, Cc]) for t in (qF, kF, vF))
        if cfg.attention == "reference-flash" and ag._has(Bk, "flashAttention"):
            qFA, kFA, vFA = (ag.reshape(ctx, t, [Bt * H, T, D]) for t in (q, k, v))
            if flashHeadSize(D):
                att = ag.flashAttention(ctx, qFA, kFA, vFA, T, scl, cap)
            else:
                # a head size without a fused kernel: the same function of the same slabs, op by op (no dropout on the
                # attention weights: this branch has none, gpt.ts:247-254)
                scores = ag.scale(ctx, ag.matmul(ctx, qFA, ag.transpose(ctx, kFA, 1, 2)), scl)
                if cap > 0:
                    scores = ag.softCap(ctx, scores, cap)
                masked = Variable(Bk.maskedFill(scores.data, mask, -1e9), True)
                ctx.tape.record(masked, [scores], lambda g, B, rel, n: [B.maskedFill(g, mask, 0)])
                att = ag.matmul(ctx, ag.softmax(ctx, masked, -1), vFA)
            concat = ag.reshape(ctx, ag.transpose(ctx, ag.reshape(ctx, att, [Bt, H, T, D]), 1, 2), [Bt * T, Cc])
        else:
            qH, kH, vH = (ag.transpose(ctx, ag.reshape(ctx, t, [Bt, T, H, D]), 1, 2) for t in (q, k, v))
            kT = ag.transpose(ctx, kH, 2, 3)
            scores = ag.softCap(ctx, ag.scale(ctx, ag.matmul(ctx, qH, kT), scl), cap)
            masked = Variable(Bk.maskedFill(scores.data, mask, -1e9), True)
            ctx.tape.record(masked, [scores], lambda g, B, rel, n: [B.maskedFill(g, mask, 0)])
            att = ag.dropout(ctx, ag.softmax(ctx, masked, -1), cfg.dropout, training)
            concat = ag.reshape(ctx, ag.transpose(ctx, ag.matmul(ctx, att, vH), 1, 2), [Bt * T, Cc])
    proj = ag.reshape(ctx, ag.matmulTransposed(ctx, concat, layer["attn"]["wo"]), [Bt, T, Cc])
    x = ag.residualDropoutAdd(ctx, x, proj, cfg.dropout, training)

    ln2 = ag.layerNorm(ctx, x, layer["ln2"]["weight"], layer["ln2"]["bias"], 1e-5)
    flat = ag.reshape(ctx, ln2, [Bt * T, Cc])
    act = cfg.ffnActivation or "gelu"
    m = layer["mlp"]
    mt = ag.matmulTransposed
    if act == "composed" and cfg.activationGraph:
        h = mt(ctx, flat, m["fc1"])
        mlpH = mt(ctx, _eval_activation_graph(ctx, h, cfg.activationGraph), m["fc2"])
    elif act == "swiglu":
        mlpH = mt(ctx, ag.siluMul(ctx, mt(ctx, flat, m["fc_gate"]), mt(ctx, flat, m["fc_up"])), m["fc_proj"])
    elif act == "universal" and ag._has(Bk, "channelAct"):
        h = mt(ctx, flat, m["fc1"])
        mlpH = mt(ctx, ag.channelAct(ctx, h, {"silu": m["act_gate"], "identity": m["act_skip"]}), m["fc2"])
    elif act == "kan_spline" and ag._has(Bk, "channelAct"):
        h = mt(ctx, flat, m["fc1"])
        coefs = {"silu": m["kan_c0"], "relu": m["kan_c1"], "gelu": m["kan_c2"], "identity": m["kan_c3"], "square": m["kan_c4"]}
        mlpH = mt(ctx, ag.channelAct(ctx, h, coefs), m["fc2"])
    elif act == "universal":
        h = mt(ctx, flat, m["fc1"])
        mlpH = mt(ctx, ag.add(ctx, ag.mul(ctx, ag.silu(ctx, h), m["act_gate"]), ag.mul(ctx, h, m["act_skip"])), m["fc2"])
    elif act == "kan_spline":
        h = mt(ctx, flat, m["fc1"])
        hs, hr = ag.mul(ctx, ag.silu(ctx, h), m["kan_c0"]), ag.mul(ctx, ag.relu(ctx, h), m["kan_c1"])
        hg, hi = ag.mul(ctx, ag.gelu(ctx, h), m["kan_c2"]), ag.mul(ctx, h, m["kan_c3"])
        hq = ag.mul(ctx, ag.mul(ctx, h, h), m["kan_c4"])
        mlpH = mt(ctx, ag.add(ctx, ag.add(ctx, ag.add(ctx, ag.add(ctx, hs, hr), hg), hi), hq), m["fc2"])
    elif act == "silu":
        mlpH = mt(ctx, ag.silu(ctx, mt(ctx, flat, m["fc1"])), m["fc2"])
    elif act == "relu":
        mlpH = mt(ctx, ag.relu(ctx, mt(ctx, flat, m["fc1"])), m["fc2"])
    else:
        mlpH = mt(ctx, ag.matmulTransposedGelu(ctx, flat, m["fc1"]), m["fc2"])
    return ag.residualDropoutAdd(ctx, x, ag.reshape(ctx, mlpH, [Bt, T, Cc]), cfg.dropout, training)


def gptForward(cfg: ModelConfig, params: dict, backend, tape: Tape, tokens: TensorData, targets: Optional[TensorData] = None,
               training: bool = False, activationCheckpointing: bool = False, mixedPrecision: bool = False,
               dropoutRng=None, release=None):
    """gpt.ts:344-427.  Returns {"logits": Variable, "loss": Variable | None}."""
    ctx = Ctx(tape, backend, dropoutRng, release)
    Bt, T = tokens.shape
    tok = ag.embedding(ctx, params["wte"], tokens)
    key = (id(backend), Bt, T)
    pos = _pos_cache.get(key)
    if pos is None:
        pos = TensorData((Bt, T), "i32", np.tile(np.arange(T, dtype=np.int32), Bt))
        _pos_cache[key] = pos
    x = ag.add(ctx, tok, ag.embedding(ctx, params["wpe"], pos))
    mask = None
    if cfg.attention == "unfused" or cfg.dropout != 0 or not ag._has(backend, "attentionQkv") or not flashHeadSize(cfg.nEmbd // cfg.nHead):
        mask = _mask_cache.get((id(backend), T))
        if mask is None:
            mask = backend.causalMask(T)
            _mask_cache[(id(backend), T)] = mask
    for layer in params["layers"]:
        if mixedPrecision and training:
            x = ag.castToF16(ctx, x)
        if activationCheckpointing and training:
            saved = dropoutRng.saveCounter() if dropoutRng else None

            def block(ictx, inp, layer=layer, saved=saved):
                if dropoutRng is not None and saved is not None:
                    dropoutRng.restoreCounter(saved)
                ictx.dropoutRng = dropoutRng
                f32_in = ag.castToF32(ictx, inp) if mixedPrecision else inp
                return transformerBlock(ictx, f32_in, layer, cfg, Bt, T, mask, training)
            x = ag.checkpoint(ctx, block, x)
        else:
            if mixedPrecision and training:
                x = ag.castToF32(ctx, x)
            x = transformerBlock(ctx, x, layer, cfg, Bt, T, mask, training)
    x = ag.layerNorm(ctx, x, params["lnF"]["weight"], params["lnF"]["bias"], 1e-5)
    flat = ag.reshape(ctx, x, [Bt * T, cfg.nEmbd])
    logits = ag.reshape(ctx, ag.matmulTransposed(ctx, flat, params["lmHead"]), [Bt, T, cfg.vocabSize])
    loss = None
    if targets is not None:
        tf = backend.reshape(targets, [Bt * T]) if targets._buf is not None else TensorData((Bt * T,), "i32", targets.data)
        loss = ag.crossEntropy(ctx, ag.reshape(ctx, logits, [Bt * T, cfg.vocabSize]), tf)
    return {"logits": logits, "loss": loss}
