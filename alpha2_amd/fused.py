"""Fast-mode training step: the same GPT step as `train.Trainer` (packages/train/src/trainer.ts:1146-1784 driving
packages/model/src/gpt.ts:344-427), scheduled by hand on flat device arenas, bf16 activations and bf16 shadow weights
for the MFMA operands, fp32 master weights / gradients / Adam moments, and captured once into a hipGraph that is
replayed every step.

Differences from the op-by-op path are layout and fusion only; the arithmetic is the same function:
  * tok+pos embedding and their add are one kernel; the residual adds are GEMM epilogues; GELU (+ saved
    pre-activation) and its derivative are GEMM epilogues; attention reads Q, K, V in place out of the [BT, 3C]
    projection and writes merged heads (attention="heads"), or -- attention="reference-flash", the function gpt.ts:247-254
    computes on a backend with flashAttention -- the projection writes q, k, v as three [BT, C] matrices that are read as
    [B H, T, D] slabs, and its backward reads the three gradients where the attention kernel leaves them;
  * dropout (reference-flash wiring only): the two residualDropoutAdd of a block become one pass each over the projection
    with the mask made on the fly, and so do the two mask multiplies of their backward; the seed of a step's masks is read
    from device memory, so the captured graph draws new masks at every replay;
  * every activation is bf16, by default the residual stream and the gradient flowing back along it too (stream="f32"
    keeps those two in f32: 3 % slower, losses equal to 1e-4 relative);
  * parameters, gradients and Adam moments each live in ONE arena ordered [decayed | not decayed], so the gradient
    norm is one reduction and AdamW is two launches; the clip coefficient never visits the host
    (trainer.ts:1650-1656 computes it on the host from a read-back norm);
  * per-step scalars (lr, bias corrections) are read by the AdamW kernel from a small device struct written before
    each replay, so the captured graph follows the LR schedule.
"""
from __future__ import annotations

import ctypes as C
import math
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import numpy as np

from . import _ffi as ffi
from ._ffi import check
from .backend import HipBackend, TensorData, shapeSize
from .model import ModelConfig, collectParamEntries, ffn_dim, initGPT
from .train import TrainConfig, lrAt, noDecayNames

F32, BF16 = ffi.F32, ffi.BF16


def _align(n: int, a: int = 64) -> int:
    return (n + a - 1) // a * a


def _i32(x: int) -> int:
    x &= 0xFFFFFFFF
    return x - (1 << 32) if x >> 31 else x


@dataclass
class StepStats:
    loss: float
    gradNorm: float
    clipCoef: float
    lr: float
    skipped: bool = False         # loss or gradient norm was not finite: parameters and moments left as they were


class FusedTrainer:
    def __init__(self, backend: HipBackend, cfg: ModelConfig, tc: TrainConfig, batch: int, seed: int = 0, use_graph: bool = True,
                 accum: int = 1, params: Optional[dict] = None, dw_groups: int = 1, stream: str = "bf16",
                 norm_in_epilogue: bool = True, index_in_step: bool = False, micro_per_pass: int = 1):
        self.act = cfg.ffnActivation or "gelu"
        # micro_per_pass = P: the `accum` micro-steps of an optimizer step (trainer.ts:1164-1273: one forward + backward each,
        # gradients summed, the mean of their losses reported) run P at a time as one pass over P x batch sequences.  A pass's
        # loss is the mean of its micro-steps' losses and its gradient their mean, so the step's numbers are the same; what
        # changes is that the products of a pass have P times the rows (at 8 x 1024 rows a 256-row tile kernel has one tile per
        # CU and nothing to overlap its epilogue with).  Batches are still stored and named one micro-batch at a time.
        self.per_pass = int(micro_per_pass)
        if self.per_pass < 1 or accum % self.per_pass:
            raise ValueError(f"micro_per_pass = {micro_per_pass} must divide the {accum} micro-steps of a step")
        self.micro_batch, self.micro_steps = batch, accum
        batch, accum = batch * self.per_pass, accum // self.per_pass      # from here on: a pass and the number of passes
        index_in_step = index_in_step or self.per_pass > 1         # (an index stored with one micro-batch does not cover a pass)
        # index_in_step: the scatter-add index of the token embedding's gradient (a sort of the micro-batch's ids) is built
        # inside every step, on the side stream beside the forward pass, instead of once when a batch is stored: what a loop
        # pays that feeds a new batch every step
        self.index_in_step = bool(index_in_step)
        if self.act not in ("gelu", "silu", "relu", "swiglu", "universal", "kan_spline"):
            raise ValueError("FusedTrainer schedules the gelu / silu / relu / swiglu / universal / kan_spline blocks; "
                             "use train.Trainer for composed activations")
        # Dropout: the two residualDropoutAdd of a block (gpt.ts:281,332), the only places the model's flash branch drops
        # anything.  The multi-head wiring stands for the CPU branch, which also drops attention weights (gpt.ts:276): the fused
        # attention kernel has no such thing, so dropout goes with the reference's own wiring only.
        self.drop = float(cfg.dropout)
        if not 0.0 <= self.drop < 1.0 or (self.drop > 0 and cfg.attention != "reference-flash"):
            raise ValueError("FusedTrainer applies dropout (0 <= p < 1) with attention='reference-flash' only; use train.Trainer otherwise")
        self.B, self.lib, self.cfg, self.tc = backend, backend.lib, cfg, tc
        self.batch, self.T, self.accum, self.use_graph = batch, cfg.blockSize, accum, use_graph
        self.C, self.H, self.L, self.V, self.F = cfg.nEmbd, cfg.nHead, cfg.nLayer, cfg.vocabSize, ffn_dim(cfg)
        self.D = self.C // self.H
        if not (8 <= self.D <= 128 and self.D % 8 == 0) or self.C % 8 or self.F % 64 or self.C % 64 or self.V % 8:
            raise ValueError("FusedTrainer needs a head size that is a multiple of 8 up to 128, nEmbd and ffnDim multiples of 64, vocab multiple of 8")
        self.BT = batch * self.T
        self.BTm = self.micro_batch * self.T
        # Which function the attention sub-layer computes: "heads" = multi-head attention on the columns of the [BT, 3C] projection;
        # "reference-flash" = what gpt.ts:247-254 computes on a backend with flashAttention: q, k, v cut out of the projection
        # as contiguous [BT, C] matrices and re-read as [B H, T, D] slabs without a head transpose.  Here the projection writes
        # the three matrices itself and its backward reads the three gradients where the attention kernel leaves them
        # (ah_gemm_planes), so the wiring moves no data.
        if cfg.attention not in ("heads", "reference-flash"):
            raise ValueError("FusedTrainer computes attention with the fused kernel: attention must be 'heads' or 'reference-flash'")
        self.slabs = cfg.attention == "reference-flash"
        if self.slabs:
            probe = ffi.AhGemm(ffi.GEMM_NT, BF16, BF16, ffi.EPI_NONE, self.BT, 3 * self.C, self.C, self.C, self.C, self.C, 1, 0, 0, 0, 256, 256, 256, 0)
            if self.lib.ah_gemm_planes(C.byref(probe), self.C, self.BT * self.C, 0, 0, 1) != 0:
                raise ValueError("FusedTrainer with attention='reference-flash' needs a shape that ah_gemm_planes takes: "
                                 + self.lib.ah_last_error().decode("utf-8", "replace"))
        self.dw_groups = max(1, min(int(dw_groups), self.L))
        self._want_norm_in_epilogue = bool(norm_in_epilogue)
        # The residual stream x and the gradient that flows back along it: f32, or bf16 like every other activation
        # ("bf16": the residual epilogues and the LayerNorm kernels move half the bytes; each add into the stream then rounds
        # to 8 bits, as in any all-bf16-activation step)
        if stream not in ("f32", "bf16"):
            raise ValueError("stream must be 'f32' or 'bf16'")
        self.stream = stream
        self.SD = F32 if stream == "f32" else BF16
        if stream == "bf16" and (self.C % 4 or self.C > 2048):
            raise ValueError("a bf16 residual stream needs nEmbd % 4 == 0 and nEmbd <= 2048")
        self.cap = cfg.softCap if cfg.softCap is not None else 30.0
        self._bufs: List[int] = []
        self._graph = None
        self._timed = None
        self._snap = None
        self.stepIdx = 0

        # ---- parameters: reference initialisation order (gpt.ts:73-151), then packed [decayed | not decayed]
        if params is None:
            from .rng import SeededRng
            params = initGPT(cfg, backend, SeededRng(seed))
        self.entries = collectParamEntries(params)
        nodecay = noDecayNames(cfg.nLayer)
        order = [e for e in self.entries if e[0] not in nodecay] + [e for e in self.entries if e[0] in nodecay]
        self.off: Dict[str, int] = {}
        pos = 0
        for name, var in order:
            if name in nodecay and "_split" not in self.off:
                self.off["_split"] = pos
            self.off[name] = pos
            pos += _align(var.data.size)
        self.off.setdefault("_split", pos)
        self.nparam = pos
        host = np.zeros(pos, dtype=np.float32)
        for name, var in order:
            host[self.off[name]:self.off[name] + var.data.size] = var.data.data
        self.P, self.G, self.M, self.Vm = (self._alloc(pos * 4) for _ in range(4))
        self.Pb = self._alloc(pos * 2)
        check(self.lib.ah_upload(self.P, host.ctypes.data_as(C.c_void_p), host.nbytes))
        for buf in (self.G, self.M, self.Vm):
            check(self.lib.ah_fill_f32(buf, 0.0, pos))
        check(self.lib.ah_cast(self.P, F32, self.Pb, BF16, pos))
        self.shapes = {name: var.data.shape for name, var in self.entries}

        # ---- activations (all shapes are static, so every buffer is allocated once)
        BT, Cc, Fd, V = self.BT, self.C, self.F, self.V
        a = self._alloc
        self.toks = [a(BT * 4) for _ in range(self.accum)]               # one resident token batch per micro-step
        self.tgts = [a(BT * 4) for _ in range(self.accum)]
        self.tok, self.tgt = self.toks[0], self.tgts[0]
        # positions of every resident batch sorted by token id, built once when the batch arrives: the embedding scatter-add
        # of every step then sums in a fixed order without sorting again (0 bytes = sizes outside that path)
        self._index_bytes = int(self.lib.ah_embedding_index_bytes(BT, V))
        self.tok_index = [a(self._index_bytes) if self._index_bytes else 0 for _ in range(self.accum)]
        ss = 4 if self.SD == F32 else 2
        self.x = [a(BT * Cc * ss) for _ in range(self.L + 1)]           # residual stream entering layer l
        self.xmid = [a(BT * Cc * ss) for _ in range(self.L)]
        self.ln1 = [a(BT * Cc * 2) for _ in range(self.L)]
        self.qkv = [a(BT * 3 * Cc * 2) for _ in range(self.L)]
        self.att = [a(BT * Cc * 2) for _ in range(self.L)]
        self.lse = [a(batch * self.H * self.T * 4) for _ in range(self.L)]
        self.ln2 = [a(BT * Cc * 2) for _ in range(self.L)]
        # MLP (gpt.ts:286-321).  gelu: activation and derivative are epilogues of the fc1 product, the derivative is what is
        # saved.  The other activations save the pre-activation (Fin columns: 2 F for swiglu, whose gate and up weights are
        # adjacent in the arena and therefore ONE [2F, C] operand) and run one element-wise pass each way.
        self.Fin = 2 * Fd if self.act == "swiglu" else Fd
        self.w1 = "mlp.fc_gate" if self.act == "swiglu" else "mlp.fc1"
        self.w2 = "mlp.fc_proj" if self.act == "swiglu" else "mlp.fc2"
        if self.act == "swiglu":
            assert all(self.off[f"layer.{l}.mlp.fc_up"] == self.off[f"layer.{l}.mlp.fc_gate"] + Fd * Cc for l in range(self.L))
        self._act_coefs = {"universal": (("act_gate", 0), ("act_skip", 3)),
                           "kan_spline": (("kan_c0", 0), ("kan_c1", 1), ("kan_c2", 2), ("kan_c3", 3), ("kan_c4", 4))}.get(self.act, ())
        self._act_mask = {"silu": 1, "relu": 2, "universal": 0b01001, "kan_spline": 0b11111}.get(self.act, 0)
        if self.act == "gelu":
            self.hgrad = [a(BT * Fd * 2) for _ in range(self.L)]      # gelu'(fc1 output), saved by the forward epilogue
        else:
            self.hpre = [a(BT * self.Fin * 2) for _ in range(self.L)]
            self.dact = a(BT * Fd * 2)                                # gradient of the activation's output (one layer at a time)
        self.hact = [a(BT * Fd * 2) for _ in range(self.L)]
        self.lnf, self.logits, self.rowlse = a(BT * Cc * 2), a(BT * V * 2), a(BT * 4)
        self.dx = [a(BT * Cc * 4), a(BT * Cc * 4) if self.SD == F32 else 0]      # f32 gradient stream (bf16 stream: only the embedding's)
        self.dlnb, self.datt = a(BT * Cc * 2), a(BT * Cc * 2)
        # Output gradients of the four linears are kept per layer (bf16): every weight gradient dW = dY^T X of the step is
        # computed at the end of backward by ONE grouped GEMM launch over full K = tokens, instead of 4 small split-K
        # GEMMs per layer.  dy_fc2[l] = grad of the layer's output, dy_wo[l] = grad after the MLP branch joins.
        self.dy_fc2 = [a(BT * Cc * 2) for _ in range(self.L)]
        self.dy_wo = [a(BT * Cc * 2) for _ in range(self.L)]
        self.dh = [a(BT * self.Fin * 2) for _ in range(self.L)]
        self.dqkv = [a(BT * 3 * Cc * 2) for _ in range(self.L)]
        self.dxb0 = a(BT * Cc * 2)                # grad of the embedding output in bf16 (written by the last LayerNorm backward, unused)
        if self.drop > 0:
            # a projection before its mask (one at a time), the masked output gradients of the two projections per layer (the
            # operands of their dX and dW products; the unmasked ones stay the residual stream's gradient), and the seed of every
            # micro-step's masks, which the host writes before each step
            self.proj = a(BT * Cc * 2)
            self.dproj_fc2 = [a(BT * Cc * 2) for _ in range(self.L)]
            self.dproj_wo = [a(BT * Cc * 2) for _ in range(self.L)]
            self.seed_dev = a(4 * self.micro_steps)
        self.loss, self.sumsq, self.clip = a(4), a(4), a(16)         # clip: coefficient (NaN = skip), norm, skipped flag
        self.loss_micro = a(4)
        self.hyper = a(ffi.C.sizeof(ffi.AhAdamW))
        self.guard = a(24)                                           # device doubles: beta1^t, beta2^t, steps skipped
        self._write_guard_state()
        self.loss_hist_cap = 4096
        self.loss_hist, self.norm_hist = a(self.loss_hist_cap * 4), a(self.loss_hist_cap * 16)
        self._batches: List[Tuple[int, int, int]] = []
        self._have_batch = False
        # partial column sums of every LayerNorm backward (dw, db), reduced by ONE launch at the end of backward
        part_bytes = int(self.lib.ah_layernorm_bwd_partials_bytes(BT, Cc))
        assert part_bytes > 0
        self._ln_jobs: List[Tuple[str, int]] = [("lnF", a(part_bytes))]
        for l in range(self.L):
            self._ln_jobs += [(f"layer.{l}.ln2", a(part_bytes)), (f"layer.{l}.ln1", a(part_bytes))]
        self._ln_part = dict(self._ln_jobs)
        self._plan_weight_grads()

    def _plan_weight_grads(self):
        """Descriptors of every dW = dY^T X of the step (TN layout: both operands token-major), lmHead first.  With
        dw_groups = 1 they are ONE grouped launch at the end of backward.  With dw_groups = n the layers are cut into n
        runs (the last layers, whose gradients exist first, and lmHead in run 0): run k is launched on the side stream as
        soon as backward has passed its lowest layer, beside the backward kernels of the layers below."""
        BT, Cc, Fd, V, TN = self.BT, self.C, self.F, self.V, ffi.GEMM_TN     # (swiglu: d[gate; up] is one [2F, C] product)

        def desc(dy, x, gname, m, n, row0=0):
            return ffi.AhGemm(TN, BF16, F32, ffi.EPI_NONE, m, n, BT, m, n, n, 1, 0, 0, 0, dy, x, self.g(gname) + row0 * n * 4, 0)

        def layer(l):
            pre = f"layer.{l}."
            dyf, dyw = (self.dproj_fc2[l], self.dproj_wo[l]) if self.drop > 0 else (self.dy_fc2[l], self.dy_wo[l])
            d = [desc(dyf, self.hact[l], pre + self.w2, Cc, Fd), desc(self.dh[l], self.ln2[l], pre + self.w1, self.Fin, Cc),
                 desc(dyw, self.att[l], pre + "attn.wo", Cc, Cc)]
            if self.slabs:      # dq, dk, dv lie apart as [BT, C] matrices: rows [p C, (p + 1) C) of the [3C, C] gradient each
                return d + [desc(self.dqkv[l] + p * BT * Cc * 2, self.ln1[l], pre + "attn.wqkv", Cc, Cc, p * Cc) for p in range(3)]
            return d + [desc(self.dqkv[l], self.ln1[l], pre + "attn.wqkv", 3 * Cc, Cc)]
        n = self.dw_groups
        bounds = [self.L - (self.L * (k + 1)) // n for k in range(n)]          # lowest layer of run k (run n-1 ends at layer 0)
        self._dw_after_layer = {}                                                # layer whose backward completes run k -> k
        groups, hi = [], self.L
        for k, lo in enumerate(bounds):
            d = [desc(self.logits, self.lnf, "lmHead", V, Cc)] if k == 0 else []
            if n == 1:                                                           # the order the single launch has always had
                for l in range(self.L):
                    d += layer(l)
            else:
                for l in reversed(range(lo, hi)):
                    d += layer(l)
            groups.append(d)
            self._dw_after_layer[lo] = k
            hi = lo
        self._dw_descs = [d for g_ in groups for d in g_]
        self._dw_group_descs = groups
        self._dw_flops = [sum(2.0 * d.m * d.n * d.k for d in g_) for g_ in groups]
        self._dw_plans = None
        if BT % 64 == 0:                          # the grouped kernel contracts in k-tiles of 64 tokens
            self._dw_plans = []
            for g_ in groups:
                arr = (ffi.AhGemm * len(g_))(*g_)
                plan = C.c_uint64()
                check(self.lib.ah_gemm_grouped_plan(arr, len(g_), C.byref(plan)))
                self._dw_plans.append(plan.value)
        # With one launch, its epilogue squares and sums the gradients it stores (ah_gemm_grouped_run_sumsq), so the norm
        # only has to read what that launch does not write: the stretches of the gradient arena between its outputs
        # (embeddings, LayerNorm and activation coefficients; the arena's padding is zero and stays zero).
        self._norm_in_epilogue = self._want_norm_in_epilogue and n == 1 and self._dw_plans is not None
        self._norm_done = False                   # the backward pass of this step has left the norm's square in self.sumsq
        if self._norm_in_epilogue:
            written = sorted((d.c, d.m * d.n * 4) for d in self._dw_descs)
            gaps, at = [], self.G
            for start, nbytes in written + [(self.G + self.nparam * 4, 0)]:
                assert start >= at
                if start > at:
                    gaps.append((at, (start - at) // 4))
                at = start + nbytes
            self._norm_rest = ((C.c_uint64 * len(gaps))(*[a_ for a_, _ in gaps]), (C.c_uint64 * len(gaps))(*[n_ for _, n_ in gaps]), len(gaps))

    def _weight_grads(self, epilogue: int, k: int, sumsq: int = 0):
        """Run k of the weight gradients (all of them when dw_groups = 1); with sumsq, the sum of the squares of the gradients
        the run leaves is added to that device float."""
        def run():
            if sumsq:
                check(self.lib.ah_gemm_grouped_run_sumsq(self._dw_plans[k], epilogue, sumsq))
            else:
                check(self.lib.ah_gemm_grouped_run(self._dw_plans[k], epilogue))
        side = self.dw_groups > 1 and self._timed is None
        if side:
            check(self.lib.ah_side_begin())
        try:
            if self._dw_plans is None:            # odd token counts: one general GEMM per weight
                for d in self._dw_group_descs[k]:
                    self._gemm(d.layout, d.a, d.b, d.c, d.m, d.n, d.k, d.lda, d.ldb, d.ldc, F32, epilogue)
            elif self._timed is None:
                run()
            else:
                e0, e1 = self.B._event(), self.B._event()
                check(self.lib.ah_event_record(e0))
                run()
                check(self.lib.ah_event_record(e1))
                kernel, nsplit = self.B.lastGemmKernel()
                self._timed.append({"kind": "gemm", "kernel": kernel, "nsplit": nsplit, "layout": ffi.GEMM_TN, "m": 0, "n": 0, "k": self.BT,
                                    "flops": self._dw_flops[k], "e0": e0, "e1": e1})
        finally:
            if side:
                check(self.lib.ah_side_end())

    # ------------------------------------------------------------------ helpers
    def _alloc(self, nbytes: int) -> int:
        p = C.c_uint64()
        check(self.lib.ah_alloc(max(16, nbytes), C.byref(p)))
        self._bufs.append(p.value)
        return p.value

    def _coef_handles(self, l: int, where):
        """The five per-channel coefficient (or gradient) vectors of layer l's activation; 0 = none."""
        arr = (C.c_uint64 * 5)()
        for name, k in self._act_coefs:
            arr[k] = where(f"layer.{l}.mlp.{name}")
        return arr

    def p(self, name: str, bf16: bool = False) -> int:
        return (self.Pb + self.off[name] * 2) if bf16 else (self.P + self.off[name] * 4)

    def g(self, name: str) -> int:
        return self.G + self.off[name] * 4

    def _gemm(self, layout, a, b, c, m, n, k, lda, ldb, ldc, out=BF16, epi=ffi.EPI_NONE, aux=0, c_planes=None, a_planes=None):
        """One product; c_planes / a_planes = (extent, stride) of the planes C's columns / A's contraction lie in."""
        g = ffi.AhGemm(layout, BF16, out, epi, m, n, k, lda, ldb, ldc, 1, 0, 0, 0, a, b, c, aux)
        if c_planes or a_planes:
            cp, ap = c_planes or (0, 0), a_planes or (0, 0)
            run = lambda: check(self.lib.ah_gemm_planes(C.byref(g), cp[0], cp[1], ap[0], ap[1], 0))
        else:
            run = lambda: check(self.lib.ah_gemm(C.byref(g)))
        if self._timed is None:
            run()
            return
        e0, e1 = self.B._event(), self.B._event()
        check(self.lib.ah_event_record(e0))
        run()
        check(self.lib.ah_event_record(e1))
        kernel, nsplit = self.B.lastGemmKernel()
        self._timed.append({"kind": "gemm", "kernel": kernel, "nsplit": nsplit, "layout": layout, "m": m, "n": n, "k": k,
                            "flops": 2.0 * m * n * k, "e0": e0, "e1": e1})

    def _dropout(self, x: int, residual: int, out: int, out_dtype: int, micro: int, counter: int):
        """out = residual + x * mask (residual 0: the mask multiply of the backward pass); x bf16, mask number `counter` of the
        micro-step (ops.ts:25-82), its seed read from device memory when the kernel runs."""
        n, rs = self.BTm * self.C, 4 if out_dtype == F32 else 2
        for seg in range(self.per_pass):                              # every micro-batch of the pass with the seed of its own micro-step
            check(self.lib.ah_dropout_apply(x + seg * n * 2, BF16, residual + seg * n * rs if residual else 0, out + seg * n * rs, out_dtype, n,
                                            self.seed_dev + 4 * (micro * self.per_pass + seg), counter, self.drop))

    def _flash(self, l: int, bwd: bool):
        Cc, T, D = self.C, self.T, self.D
        f = ffi.AhFlash()
        f.dtype, f.batch, f.heads, f.seq, f.head_dim = BF16, self.batch, self.H, T, D
        # where q, k, v (and their gradients) of (batch b, head h, position t) lie: in columns h D .. of row b T + t of the
        # [BT, 3C] projection, or -- slabs -- in row t of slab b H + h of a contiguous [BT, C] matrix read as [B H, T, D]
        sb, sh, st, nxt = (T * Cc, T * D, D, self.BT * Cc * 2) if self.slabs else (T * 3 * Cc, D, 3 * Cc, Cc * 2)
        for nm in ("q", "k", "v"):
            setattr(f, nm + "_sb", sb), setattr(f, nm + "_sh", sh), setattr(f, nm + "_st", st)
        f.o_sb, f.o_sh, f.o_st = T * Cc, D, Cc            # (the slabs' result transposed back, gpt.ts:254, is this same layout)
        f.scale, f.soft_cap = 1 / math.sqrt(D), self.cap
        q = self.qkv[l]
        f.q, f.k, f.v, f.o, f.lse = q, q + nxt, q + 2 * nxt, self.att[l], self.lse[l]
        if bwd:
            d = self.dqkv[l]
            f.d_o, f.dq, f.dk, f.dv = self.datt, d, d + nxt, d + 2 * nxt
        t0 = None
        if self._timed is not None:
            t0 = self.B._event()
            check(self.lib.ah_event_record(t0))
        check((self.lib.ah_flash_bwd if bwd else self.lib.ah_flash_fwd)(C.byref(f)))
        if t0 is not None:
            t1 = self.B._event()
            check(self.lib.ah_event_record(t1))
            fl = 4.0 * self.batch * self.H * T * T * D * (2 if bwd else 1)
            self._timed.append({"kind": "flash_bwd" if bwd else "flash_fwd", "flops": fl, "e0": t0, "e1": t1})

    # ------------------------------------------------------------------ the step
    def _forward_backward(self, first_micro: bool, micro: int = 0, last_micro: bool = True):
        self.tok, self.tgt = self.toks[micro], self.tgts[micro]
        lib, BT, Cc, Fd, V, L = self.lib, self.BT, self.C, self.F, self.V, self.L
        NN, NT, TN = ffi.GEMM_NN, ffi.GEMM_NT, ffi.GEMM_TN
        acc = 0 if first_micro else 1
        wepi = ffi.EPI_NONE if first_micro else ffi.EPI_ACCUM
        SD = self.SD
        if self._index_bytes and self.index_in_step:      # one workgroup's work: beside the forward pass, joined before its use
            check(lib.ah_side_begin())
            check(lib.ah_embedding_index(self.tok, BT, V, self.tok_index[micro]))
            check(lib.ah_side_end())
        check(lib.ah_embedding_tok_pos(self.p("wte"), self.p("wpe"), self.tok, self.x[0], BT, self.T, Cc, V, SD))
        for l in range(L):
            pre = f"layer.{l}."
            check(lib.ah_layernorm(self.x[l], self.p(pre + "ln1.weight"), self.p(pre + "ln1.bias"), self.ln1[l], BT, Cc, 1e-5, BF16, SD))
            if self.slabs:
                self._gemm(NT, self.ln1[l], self.p(pre + "attn.wqkv", True), self.qkv[l], BT, 3 * Cc, Cc, Cc, Cc, Cc, c_planes=(Cc, BT * Cc))
            else:
                self._gemm(NT, self.ln1[l], self.p(pre + "attn.wqkv", True), self.qkv[l], BT, 3 * Cc, Cc, Cc, Cc, 3 * Cc)
            self._flash(l, False)
            if self.drop > 0:
                self._gemm(NT, self.att[l], self.p(pre + "attn.wo", True), self.proj, BT, Cc, Cc, Cc, Cc, Cc)
                self._dropout(self.proj, self.x[l], self.xmid[l], SD, micro, 2 * l)
            else:
                self._gemm(NT, self.att[l], self.p(pre + "attn.wo", True), self.xmid[l], BT, Cc, Cc, Cc, Cc, Cc, SD, ffi.EPI_RESIDUAL, self.x[l])
            check(lib.ah_layernorm(self.xmid[l], self.p(pre + "ln2.weight"), self.p(pre + "ln2.bias"), self.ln2[l], BT, Cc, 1e-5, BF16, SD))
            if self.act == "gelu":
                self._gemm(NT, self.ln2[l], self.p(pre + "mlp.fc1", True), self.hact[l], BT, Fd, Cc, Cc, Cc, Fd, BF16, ffi.EPI_GELU_GRAD, self.hgrad[l])
            else:
                Fin = self.Fin
                self._gemm(NT, self.ln2[l], self.p(pre + self.w1, True), self.hpre[l], BT, Fin, Cc, Cc, Cc, Fin)
                if self.act == "swiglu":
                    check(lib.ah_swiglu(BF16, self.hpre[l], self.hact[l], BT, Fd))
                else:
                    check(lib.ah_channel_act(BF16, self.hpre[l], self._coef_handles(l, self.p), self._act_mask, self.hact[l], BT, Fd))
            if self.drop > 0:
                self._gemm(NT, self.hact[l], self.p(pre + self.w2, True), self.proj, BT, Cc, Fd, Fd, Fd, Cc)
                self._dropout(self.proj, self.xmid[l], self.x[l + 1], SD, micro, 2 * l + 1)
            else:
                self._gemm(NT, self.hact[l], self.p(pre + self.w2, True), self.x[l + 1], BT, Cc, Fd, Fd, Fd, Cc, SD, ffi.EPI_RESIDUAL, self.xmid[l])
        check(lib.ah_layernorm(self.x[L], self.p("lnF.weight"), self.p("lnF.bias"), self.lnf, BT, Cc, 1e-5, BF16, SD))
        self._gemm(NT, self.lnf, self.p("lmHead", True), self.logits, BT, V, Cc, Cc, Cc, V)
        # loss and dlogits (in place) from one read of the logits
        if self.accum == 1:
            check(lib.ah_cross_entropy_fwd_bwd(self.logits, BF16, self.tgt, self.loss, self.rowlse, 0, 1.0, self.logits, BT, V))
        else:                                     # reported loss = mean of the micro-step losses (trainer.ts:1270-1273)
            check(lib.ah_cross_entropy_fwd_bwd(self.logits, BF16, self.tgt, self.loss_micro, self.rowlse, 0, 1.0, self.logits, BT, V))
            if first_micro:
                check(lib.ah_fill_f32(self.loss, 0.0, 1))
            check(lib.ah_axpy_inplace(self.loss, self.loss_micro, 1.0 / self.accum, 1))

        self._gemm(NN, self.logits, self.p("lmHead", True), self.dlnb, BT, Cc, V, V, Cc, Cc)
        cur = 0
        f32s = SD == F32                           # f32 stream: gradient in dx[cur] with bf16 copies; bf16 stream: the copies are the stream
        check(lib.ah_layernorm_bwd_deferred(self.x[L], self.p("lnF.weight"), self.dlnb, BF16, 0, self.dx[cur] if f32s else 0, self.dy_fc2[L - 1],
                                            self._ln_part["lnF"], BT, Cc, 1e-5, SD))
        for l in reversed(range(L)):
            pre = f"layer.{l}."
            # MLP: x_out = x_mid + fc2(gelu(fc1(ln2(x_mid))))
            dyf = self.dy_fc2[l]
            if self.drop > 0:                      # the projection's own gradient is the stream's times the mask it was dropped with
                dyf = self.dproj_fc2[l]
                self._dropout(self.dy_fc2[l], 0, dyf, BF16, micro, 2 * l + 1)
            if self.act == "gelu":
                self._gemm(NN, dyf, self.p(pre + "mlp.fc2", True), self.dh[l], BT, Fd, Cc, Cc, Fd, Fd, BF16, ffi.EPI_MUL_AUX, self.hgrad[l])
            else:
                self._gemm(NN, dyf, self.p(pre + self.w2, True), self.dact, BT, Fd, Cc, Cc, Fd, Fd)
                if self.act == "swiglu":
                    check(lib.ah_swiglu_bwd(BF16, self.hpre[l], self.dact, self.dh[l], BT, Fd))
                else:
                    check(lib.ah_channel_act_bwd(BF16, self.hpre[l], self._coef_handles(l, self.p), self._act_mask, self.dact, self.dh[l],
                                                 self._coef_handles(l, self.g), acc, BT, Fd))
            self._gemm(NN, self.dh[l], self.p(pre + self.w1, True), self.dlnb, BT, Cc, self.Fin, self.Fin, Cc, Cc)
            check(lib.ah_layernorm_bwd_deferred(self.xmid[l], self.p(pre + "ln2.weight"), self.dlnb, BF16, self.dx[cur] if f32s else self.dy_fc2[l],
                                                self.dx[cur ^ 1] if f32s else 0, self.dy_wo[l], self._ln_part[pre + "ln2"], BT, Cc, 1e-5, SD))
            cur ^= f32s
            # attention: x_mid = x_in + wo(attn(wqkv(ln1(x_in))))
            dyw = self.dy_wo[l]
            if self.drop > 0:
                dyw = self.dproj_wo[l]
                self._dropout(self.dy_wo[l], 0, dyw, BF16, micro, 2 * l)
            self._gemm(NN, dyw, self.p(pre + "attn.wo", True), self.datt, BT, Cc, Cc, Cc, Cc, Cc)
            self._flash(l, True)
            if self.slabs:
                self._gemm(NN, self.dqkv[l], self.p(pre + "attn.wqkv", True), self.dlnb, BT, Cc, 3 * Cc, Cc, Cc, Cc, a_planes=(Cc, BT * Cc))
            else:
                self._gemm(NN, self.dqkv[l], self.p(pre + "attn.wqkv", True), self.dlnb, BT, Cc, 3 * Cc, 3 * Cc, Cc, Cc)
            check(lib.ah_layernorm_bwd_deferred(self.x[l], self.p(pre + "ln1.weight"), self.dlnb, BF16, self.dx[cur] if f32s else self.dy_wo[l],
                                                self.dx[cur ^ 1] if f32s else (self.dx[0] if l == 0 else 0),      # the embeddings take their gradient in f32
                                                self.dy_fc2[l - 1] if l > 0 else self.dxb0, self._ln_part[pre + "ln1"], BT, Cc, 1e-5, SD))
            cur ^= f32s
            if self.dw_groups > 1 and l in self._dw_after_layer:
                self._weight_grads(wepi, self._dw_after_layer[l])
        jobs = (ffi.AhColsumJob * len(self._ln_jobs))(*[
            ffi.AhColsumJob(part, self.g(name + ".weight"), self.g(name + ".bias"), BT, Cc, acc, 0) for name, part in self._ln_jobs])
        check(lib.ah_layernorm_colsums(jobs, len(self._ln_jobs)))
        if self._index_bytes:
            if self.index_in_step:
                check(lib.ah_side_join())
            check(lib.ah_embedding_bwd_indexed(self.tok_index[micro], self.dx[cur], self.g("wte"), BT, Cc, V, acc))
        else:
            check(lib.ah_embedding_bwd(self.tok, self.dx[cur], self.g("wte"), BT, Cc, V, acc))
        check(lib.ah_pos_embedding_bwd(self.dx[cur], self.g("wpe"), self.batch, self.T, Cc, acc))
        if self.dw_groups == 1:
            if last_micro and self._norm_in_epilogue:     # the norm of the step's gradient: the other gradients first, the launch adds its own
                xs, ns, count = self._norm_rest
                check(lib.ah_sum_sq_list(xs, ns, count, self.sumsq))
                self._weight_grads(wepi, 0, self.sumsq)
                self._norm_done = True
            else:
                self._weight_grads(wepi, 0)
        if self.dw_groups > 1:                    # the next micro-step overwrites the operands, the optimizer reads the results
            check(lib.ah_side_join())

    def _optimizer(self):
        lib, tc = self.lib, self.tc
        split = self.off["_split"]
        if not self._norm_done:
            check(lib.ah_sum_sq(self.G, self.nparam, self.sumsq))           # arena padding is zero and stays zero
        self._norm_done = False
        # clip coefficient, non-finite guard and the bias corrections, all on the device (trainer.ts:1248-1262,1495-1522,1650-1656)
        check(lib.ah_step_guard(self.sumsq, self.loss, 1.0 / self.accum, tc.gradClip, tc.beta1, tc.beta2, self.guard, self.hyper, self.clip))
        h = ffi.AhAdamW(tc.lr, tc.beta1, tc.beta2, tc.eps, tc.weightDecay, 1.0, 1.0, 1.0 / self.accum)
        if split > 0:
            check(lib.ah_adamw(self.P, self.G, self.M, self.Vm, split, C.byref(h), self.hyper, self.clip, self.Pb))
        h.weight_decay = 0.0
        n2 = self.nparam - split
        if n2 > 0:
            check(lib.ah_adamw(self.P + split * 4, self.G + split * 4, self.M + split * 4, self.Vm + split * 4, n2, C.byref(h), self.hyper,
                               self.clip, self.Pb + split * 2))

    def _whole_step(self):
        for m in range(self.accum):               # gradients of the micro-steps are summed in place; scaled once in the optimizer
            self._forward_backward(m == 0, m, m == self.accum - 1)
        self._optimizer()

    def _upload_batch(self, inputs: TensorData, targets: TensorData, ti: int, tt: int):
        n = self.BTm * 4
        a, b = np.ascontiguousarray(inputs.data, dtype=np.int32), np.ascontiguousarray(targets.data, dtype=np.int32)
        if a.size != self.BTm or b.size != self.BTm:
            raise ValueError(f"batch must be [{self.micro_batch}, {self.T}]")
        check(self.lib.ah_upload(ti, a.ctypes.data_as(C.c_void_p), n))
        check(self.lib.ah_upload(tt, b.ctypes.data_as(C.c_void_p), n))

    def set_batch(self, inputs: TensorData, targets: TensorData, micro: int = 0):
        """Upload one [B, T] token batch straight into the resident slot of micro-step `micro` (nothing is retained: a loop
        that feeds a fresh batch every step allocates nothing); step() trains on the resident slots until they change."""
        at = (micro % self.per_pass) * self.BTm * 4             # micro-step `micro` is slot micro % P of pass micro // P
        self._upload_batch(inputs, targets, self.toks[micro // self.per_pass] + at, self.tgts[micro // self.per_pass] + at)
        if self._index_bytes and not self.index_in_step:
            check(self.lib.ah_embedding_index(self.toks[micro], self.BT, self.V, self.tok_index[micro]))
        self._have_batch = True

    def add_batch(self, inputs: TensorData, targets: TensorData) -> int:
        """Store a batch on the device for later steps (step(batch_index)); stored batches live until drop_batches()."""
        n = self.BTm * 4
        ti, tt = self._alloc(n), self._alloc(n)
        self._upload_batch(inputs, targets, ti, tt)
        ix = 0
        if self._index_bytes and not self.index_in_step:
            ix = self._alloc(self._index_bytes)
            check(self.lib.ah_embedding_index(ti, self.BT, self.V, ix))
        self._batches.append((ti, tt, ix))
        return len(self._batches) - 1

    def drop_batches(self):
        for pair in self._batches:
            for b in pair:
                if b:
                    check(self.lib.ah_free(b))
                    self._bufs.remove(b)
        self._batches = []

    def _use_batch(self, i, micro: int = 0):
        """Copy stored batch i into the resident slot of micro-step `micro` (a sequence fills slots 0, 1, ...)."""
        if isinstance(i, (list, tuple)):
            if len(i) != self.micro_steps:
                raise ValueError(f"need {self.micro_steps} batch indices, one per micro-step")
            for m, bi in enumerate(i):
                self._use_batch(bi, m)
            return
        ti, tt, ix = self._batches[i]
        at = (micro % self.per_pass) * self.BTm * 4
        check(self.lib.ah_copy(self.toks[micro // self.per_pass] + at, ti, self.BTm * 4))
        check(self.lib.ah_copy(self.tgts[micro // self.per_pass] + at, tt, self.BTm * 4))
        if ix:
            check(self.lib.ah_copy(self.tok_index[micro], ix, self._index_bytes))
        self._have_batch = True

    def _write_guard_state(self, b1p: float = 1.0, b2p: float = 1.0, skipped: float = 0.0):
        st = (C.c_double * 3)(b1p, b2p, skipped)
        check(self.lib.ah_upload(self.guard, st, 24))
        tc = self.tc
        h = ffi.AhAdamW(tc.lr, tc.beta1, tc.beta2, tc.eps, tc.weightDecay, 1 - b1p, 1 - b2p, 1.0 / self.accum)
        check(self.lib.ah_upload(self.hyper, C.byref(h), C.sizeof(h)))

    def _write_hyper(self) -> float:
        """The learning rate of this step: the first field of the device AhAdamW.  Its bias corrections are kept by
        ah_step_guard on the device, which advances them on applied steps only."""
        lr = lrAt(self.tc, self.stepIdx)
        v = C.c_float(lr)
        check(self.lib.ah_upload(self.hyper, C.byref(v), 4))
        if self.drop > 0:                          # the masks of this step's micro-steps (trainer.ts:1169,1202), as int32 like `seed | 0`
            seeds = (C.c_int32 * self.micro_steps)(*[_i32(self.tc.seed + self.stepIdx * 1000 + m) for m in range(self.micro_steps)])
            check(self.lib.ah_upload(self.seed_dev, seeds, 4 * self.micro_steps))
        return lr

    def step(self, batch_index=None) -> int:
        """Enqueue one optimizer step (no host synchronisation); returns the step index whose loss / grad-norm can be
        read later with history().  `batch_index`: a stored batch, or with gradient accumulation a sequence of `accum`
        stored batches (micro-steps run in that order); None keeps the resident ones."""
        if batch_index is not None:
            self._use_batch(batch_index)
        elif not self._have_batch:
            raise RuntimeError("no batch set")
        self._write_hyper()
        if self.use_graph:
            if self._graph is None:
                self.prepare()
                self._whole_step()                       # eager once: fills the allocator pool, raises any argument error
                self.B.syncGpu()
                self._restore_after_warm_step()
                check(self.lib.ah_graph_begin())
                try:
                    self._whole_step()
                finally:
                    gid = C.c_uint64()
                    check(self.lib.ah_graph_end(C.byref(gid)))
                self._graph = gid.value
            check(self.lib.ah_graph_launch(self._graph))
        else:
            self._whole_step()
        i = self.stepIdx % self.loss_hist_cap
        check(self.lib.ah_copy(self.loss_hist + i * 4, self.loss, 4))
        check(self.lib.ah_copy(self.norm_hist + i * 16, self.clip, 16))
        self.stepIdx += 1
        return self.stepIdx - 1

    def _restore_after_warm_step(self):
        """The eager run that precedes capture must not count as a training step: put parameters and moments back."""
        check(self.lib.ah_copy(self.P, self._snap[0], self.nparam * 4))
        check(self.lib.ah_copy(self.M, self._snap[1], self.nparam * 4))
        check(self.lib.ah_copy(self.Vm, self._snap[2], self.nparam * 4))
        check(self.lib.ah_copy(self.guard, self._snap[3], 24))
        check(self.lib.ah_copy(self.hyper, self._snap[3] + 32, C.sizeof(ffi.AhAdamW)))
        check(self.lib.ah_cast(self.P, F32, self.Pb, BF16, self.nparam))
        for s in self._snap:
            check(self.lib.ah_free(s))
            self._bufs.remove(s)
        self._snap = None

    def prepare(self):
        """Snapshot state ahead of the warm-up run inside the first step()."""
        self._snap = [self._alloc(self.nparam * 4) for _ in range(3)] + [self._alloc(32 + C.sizeof(ffi.AhAdamW))]
        for dst, src in zip(self._snap, (self.P, self.M, self.Vm)):
            check(self.lib.ah_copy(dst, src, self.nparam * 4))
        check(self.lib.ah_copy(self._snap[3], self.guard, 24))                     # running beta powers, skip count
        check(self.lib.ah_copy(self._snap[3] + 32, self.hyper, C.sizeof(ffi.AhAdamW)))

    def history(self, first: int, count: int) -> List[StepStats]:
        """Blocks; loss, gradient norm and clip coefficient of steps [first, first+count)."""
        self.B.syncGpu()
        out = []
        lo, nm = np.empty(self.loss_hist_cap, np.float32), np.empty(self.loss_hist_cap * 4, np.float32)
        check(self.lib.ah_download(lo.ctypes.data_as(C.c_void_p), self.loss_hist, lo.nbytes))
        check(self.lib.ah_download(nm.ctypes.data_as(C.c_void_p), self.norm_hist, nm.nbytes))
        for s in range(first, first + count):
            i = s % self.loss_hist_cap
            out.append(StepStats(float(lo[i]), float(nm[4 * i + 1]), float(nm[4 * i]), lrAt(self.tc, s), bool(nm[4 * i + 2] != 0)))
        return out

    def timed_step(self) -> list:
        """One eager step with every GEMM and attention launch bracketed by HIP events on the library stream."""
        self.B.syncGpu()
        self._write_hyper()
        self._timed = []
        self._whole_step()
        recs, self._timed = self._timed, None
        ms = C.c_float()
        for r in recs:
            check(self.lib.ah_event_elapsed_ms(r["e0"], r["e1"], C.byref(ms)))
            r["ms"] = ms.value
            for e in (r.pop("e0"), r.pop("e1")):
                check(self.lib.ah_event_destroy(e))
        self.stepIdx += 1
        return recs

    def param(self, name: str) -> np.ndarray:
        n = shapeSize(self.shapes[name])
        out = np.empty(n, np.float32)
        self.B.syncGpu()
        check(self.lib.ah_download(out.ctypes.data_as(C.c_void_p), self.p(name), n * 4))
        return out

    def grad(self, name: str) -> np.ndarray:
        n = shapeSize(self.shapes[name])
        out = np.empty(n, np.float32)
        self.B.syncGpu()
        check(self.lib.ah_download(out.ctypes.data_as(C.c_void_p), self.g(name), n * 4))
        return out

    # ------------------------------------------------------------------ checkpoints (reference file format)
    def _arena_slice(self, arena: int, name: str) -> np.ndarray:
        n = shapeSize(self.shapes[name])
        out = np.empty(n, np.float32)
        check(self.lib.ah_download(out.ctypes.data_as(C.c_void_p), arena + self.off[name] * 4, n * 4))
        return out

    def stateDict(self) -> dict:
        """AdamW.stateDict (optimizers.ts:202-210) read from the moment arenas."""
        self.B.syncGpu()
        bufs = {}
        for name, _ in self.entries:
            n = shapeSize(self.shapes[name])
            bufs[name + ".m"] = TensorData((n,), "f32", self._arena_slice(self.M, name))
            bufs[name + ".v"] = TensorData((n,), "f32", self._arena_slice(self.Vm, name))
        return {"step": self.stepIdx, "buffers": bufs}

    def saveCheckpoint(self, path: str, configHash: str = "", tokenizerArtifacts=None):
        from dataclasses import asdict
        from .checkpoint import FileCheckpoint
        self.B.syncGpu()
        params = {name: {"shape": list(self.shapes[name]), "data": self.param(name)} for name, _ in self.entries}
        FileCheckpoint().save(path, {"modelConfig": asdict(self.cfg), "params": params, "optimizerState": self.stateDict(),
                                     "tokenizerArtifacts": tokenizerArtifacts, "rngState": 0, "configHash": configHash, "step": self.stepIdx})

    def loadCheckpoint(self, path: str) -> dict:
        """Parameters, moments and step counter from a checkpoint written by either trainer (or by the reference)."""
        from .checkpoint import FileCheckpoint
        st = FileCheckpoint().load(path)
        self.B.syncGpu()

        def put(arena, name, data):
            a = np.ascontiguousarray(np.asarray(data, dtype=np.float32).reshape(-1))
            n = shapeSize(self.shapes[name])
            if a.size != n:
                raise ValueError(f"checkpoint tensor {name} has {a.size} values, the model needs {n}")
            check(self.lib.ah_upload(arena + self.off[name] * 4, a.ctypes.data_as(C.c_void_p), n * 4))
        for name, _ in self.entries:
            saved = st["params"].get(name)
            if saved is None and name.endswith(".attn.wqkv"):       # pre-fusion checkpoints (checkpoint.ts:243-257)
                pre = name[:-len(".attn.wqkv")]
                parts = [st["params"].get(f"{pre}.attn.{w}") for w in ("wq", "wk", "wv")]
                if all(p is not None for p in parts):
                    saved = {"data": np.concatenate([np.asarray(p["data"], dtype=np.float32).reshape(-1) for p in parts])}
            if saved is not None:
                put(self.P, name, saved["data"])
        bufs = st["optimizerState"]["buffers"]
        check(self.lib.ah_fill_f32(self.M, 0.0, self.nparam))
        check(self.lib.ah_fill_f32(self.Vm, 0.0, self.nparam))
        for key, td in bufs.items():
            if key[:-2] in self.off and key.endswith((".m", ".v")):
                put(self.M if key.endswith(".m") else self.Vm, key[:-2], td.data)
        check(self.lib.ah_cast(self.P, F32, self.Pb, BF16, self.nparam))
        self.stepIdx = int(st["optimizerState"].get("step") or st.get("step") or 0)
        self._write_guard_state(self.tc.beta1 ** self.stepIdx, self.tc.beta2 ** self.stepIdx)   # optimizers.ts:214-215
        return st

    def close(self):
        self.B.syncGpu()
        if self._graph is not None:
            check(self.lib.ah_graph_destroy(self._graph))
            self._graph = None
        for plan in self._dw_plans or []:
            check(self.lib.ah_gemm_grouped_destroy(plan))
        self._dw_plans = None
        for b in self._bufs:
            self.lib.ah_free(b)
        self._bufs = []
