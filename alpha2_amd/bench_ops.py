"""Per-op microbenchmarks on the shapes of the training step, in the manner of the reference's scripts/bench-ops.ts
(3 warm-up calls, then the mean of `iters` calls; TFLOP/s = flops / time, GB/s = algorithmic bytes / time):

    python -m alpha2_amd.bench_ops [--iters 10] [--only gemm|flash|bandwidth|ceiling|epilogue|issue] [--json]

* GEMM: C = A B^T and both backward products, M = 16384 (batch x context), K = 768, N in {768, 2304, 3072, 50304},
  bf16 operands with fp32 accumulation and fp32 throughout; flops 2 M N K (scripts/bench-ops.ts:302,328).
* `--only epilogue` (not part of the default run): the fc1-shaped product M = 16384, N = 3072, K = 768 (and fc2's dX, K and
  N swapped) with every epilogue the library has, to separate what an epilogue's arithmetic costs from what its second
  operand or second result costs: each epilogue is its own kernel instance, so a counter run sees them apart.
* Causal flash attention forward and backward: B = 16, H = 12, head size 64, T in {256, 1024, 2048}, bf16, with and
  without the soft cap of 30; flops counted non-causal like the reference: 4 B H T^2 D forward, 8 B H T^2 D backward
  (scripts/bench-ops.ts:652,673).
* Bandwidth-bound ops at the GPT-2-small step's sizes: LayerNorm forward / backward, GELU forward / backward, fused
  cross-entropy forward + backward, embedding gather / scatter-add, sum of squares, AdamW; bytes = the algorithmic minimum.
* The matrix pipes alone (`ah_probe_mfma_bf16`: independent 32x32x16 bf16 MFMAs on registers, no memory traffic), on zeros and
  on operands whose bits toggle, for one short launch and sustained: what the part's power limit leaves of the published peak.
* `--only issue` (not part of the default run): what one SIMD issues per nanosecond (`ah_probe_issue`: v_fma_f32, v_exp_f32, a
  mix of the two, an MFMA alone and with vector work behind it, at one, two and four waves per SIMD): the figures the
  attention kernels, whose time goes to per-score vector instructions, are read against.

Every call goes through the C ABI; timing is by HIP events on the library's stream.  Peaks used for the last column:
2.5 PFLOP/s (bf16 MFMA), 157.3 TFLOP/s (fp32 MFMA), 8 TB/s (HBM).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import math
import sys

import numpy as np

from . import HipBackend, _ffi as ffi

PEAK_TFLOPS = {"bf16": 2500.0, "f32": 157.3}
PEAK_GBS = 8000.0


class Bench:
    def __init__(self, iters: int):
        self.B = HipBackend(0)
        self.lib = self.B.lib
        self.iters = iters
        self.rows = []
        self._live = []

    def alloc(self, nbytes: int) -> int:
        p = C.c_uint64()
        ffi.check(self.lib.ah_alloc(max(nbytes, 16), C.byref(p)))
        self._live.append(p.value)
        return p.value

    def release(self):
        for p in self._live:
            self.lib.ah_free(p)
        self._live = []

    def randn(self, n: int, dtype: int, std: float = 1.0, seed: int = 2) -> int:
        """n values N(0, std) on the device in `dtype` (generated in blocks of 16 M on the host)."""
        es = ffi.DTYPE_BYTES["bf16" if dtype == ffi.BF16 else "f32"]
        dst = self.alloc(n * es)
        blk = 1 << 24
        tmp = self.alloc(min(n, blk) * 4)
        host = (np.random.RandomState(seed).standard_normal(min(n, blk)) * std).astype(np.float32)
        ffi.check(self.lib.ah_upload(tmp, host.ctypes.data_as(C.c_void_p), host.nbytes))
        for o in range(0, n, blk):
            m = min(blk, n - o)
            if dtype == ffi.F32:
                ffi.check(self.lib.ah_copy(dst + o * 4, tmp, m * 4))
            else:
                ffi.check(self.lib.ah_cast(tmp, ffi.F32, dst + o * es, dtype, m))
        return dst

    def time(self, fn) -> float:
        """Mean milliseconds per call."""
        for _ in range(3):
            fn()
        e0, e1 = self.B._event(), self.B._event()
        ffi.check(self.lib.ah_event_record(e0))
        for _ in range(self.iters):
            fn()
        ffi.check(self.lib.ah_event_record(e1))
        ms = C.c_float()
        ffi.check(self.lib.ah_event_elapsed_ms(e0, e1, C.byref(ms)))
        for e in (e0, e1):
            ffi.check(self.lib.ah_event_destroy(e))
        return ms.value / self.iters

    def record(self, name: str, ms: float, flops: float = 0.0, nbytes: float = 0.0, dtype: str = "bf16", note: str = ""):
        tf = flops / (ms * 1e-3) / 1e12 if flops else None
        gbs = nbytes / (ms * 1e-3) / 1e9 if nbytes else None
        frac = tf / PEAK_TFLOPS[dtype] if flops else gbs / PEAK_GBS
        self.rows.append({"op": name, "us": ms * 1e3, "tflops": tf, "gbs": gbs, "bound": "mfma" if flops else "hbm", "frac_of_peak": frac, "note": note})
        perf = f"{tf:9.1f} TFLOP/s" if flops else f"{gbs:9.0f} GB/s   "
        print(f"{name:34s} {ms * 1e3:10.1f} us {perf} {100 * frac:5.1f} %  {note}", flush=True)


def bench_gemm(b: Bench):
    M, K = 16384, 768
    for dt, dname in ((ffi.BF16, "bf16"), (ffi.F32, "f32")):
        es = 2 if dt == ffi.BF16 else 4
        for N in (768, 2304, 3072, 50304):
            a, w, g = b.randn(M * K, dt, 0.02), b.randn(N * K, dt, 0.02), b.randn(M * N, dt, 0.02)
            c_fwd, c_da = b.alloc(M * N * es), b.alloc(M * K * es)
            c_db = b.alloc(N * K * 4)                                     # weight gradients are kept in f32
            flops = 2.0 * M * N * K
            cases = (("fwd  C=A.B^T", ffi.GEMM_NT, (M, N, K, K, K, N), (a, w, c_fwd), dt),
                     ("dA   G.B", ffi.GEMM_NN, (M, K, N, N, K, K), (g, w, c_da), dt),
                     ("dB   G^T.A", ffi.GEMM_TN, (N, K, M, N, K, K), (g, a, c_db), ffi.F32))
            for label, layout, (m, n, k, lda, ldb, ldc), (pa, pb, pc), out in cases:
                d = ffi.AhGemm(layout, dt, out, ffi.EPI_NONE, m, n, k, lda, ldb, ldc, 1, 0, 0, 0, pa, pb, pc, 0)
                ms = b.time(lambda: ffi.check(b.lib.ah_gemm(C.byref(d))))
                kern, nsplit = b.B.lastGemmKernel()
                b.record(f"gemm {dname} N={N} {label}", ms, flops=flops, dtype=dname, note=f"{kern}" + (f" split-K x{nsplit}" if nsplit > 1 else ""))
            if dt == ffi.BF16 and N == 2304:
                # the fused q, k, v projection under the reference's attention wiring (gpt.ts:239-254): result columns / the
                # contraction in three planes instead of sliceQkv's copies and the written sum of three scatterSlice results
                d = ffi.AhGemm(ffi.GEMM_NT, dt, dt, ffi.EPI_NONE, M, N, K, K, K, K, 1, 0, 0, 0, a, w, c_fwd, 0)
                ms = b.time(lambda: ffi.check(b.lib.ah_gemm_planes(C.byref(d), K, M * K, 0, 0, 0)))
                b.record("gemm bf16 N=2304 fwd, q k v as planes", ms, flops=flops, dtype=dname, note=b.B.lastGemmKernel()[0])
                d2 = ffi.AhGemm(ffi.GEMM_NN, dt, dt, ffi.EPI_NONE, M, K, N, K, K, K, 1, 0, 0, 0, g, w, c_da, 0)
                ms = b.time(lambda: ffi.check(b.lib.ah_gemm_planes(C.byref(d2), 0, 0, K, M * K, 0)))
                b.record("gemm bf16 N=2304 dA, dq dk dv as planes", ms, flops=flops, dtype=dname, note=b.B.lastGemmKernel()[0])
            b.release()


def bench_epilogues(b: Bench):
    """One product shape, every epilogue.  bytes beside the operands: plain 1 store; GELU 2 stores (7 operations per element:
    C = gelu(acc), aux = acc); GELU_GRAD 2 stores (11 operations: C = gelu(acc), aux = gelu'(acc)); GELU_BWD 1 load + 1 store
    (11 operations); MUL_AUX 1 load + 1 store (1 operation); RESIDUAL 1 f32 load + 1 f32 store (1 operation)."""
    M, K, N = 16384, 768, 3072
    a, w = b.randn(M * K, ffi.BF16, 1.0), b.randn(N * K, ffi.BF16, 0.02)
    g, w2 = b.randn(M * K, ffi.BF16, 0.02, 5), b.randn(K * N, ffi.BF16, 0.02, 6)     # dY [M,768] . W2 [768,3072] (NN)
    aux_bf, aux_f = b.randn(M * N, ffi.BF16, 1.0, 7), b.randn(M * N, ffi.F32, 1.0, 8)
    c_bf, c_f = b.alloc(M * N * 2), b.alloc(M * N * 4)
    flops = 2.0 * M * N * K
    nt, nn = (ffi.GEMM_NT, (M, N, K, K, K, N), a, w), (ffi.GEMM_NN, (M, N, K, K, N, N), g, w2)
    for label, (layout, (m, n, k, lda, ldb, ldc), pa, pb), out, epi, aux, pc in (
            ("fc1 fwd plain", nt, ffi.BF16, ffi.EPI_NONE, 0, c_bf),
            ("fc1 fwd gelu, saves acc", nt, ffi.BF16, ffi.EPI_GELU, aux_bf, c_bf),
            ("fc1 fwd gelu, saves gelu'", nt, ffi.BF16, ffi.EPI_GELU_GRAD, aux_bf, c_bf),
            ("fc1 fwd * aux", nt, ffi.BF16, ffi.EPI_MUL_AUX, aux_bf, c_bf),
            ("fc1 fwd * gelu'(aux)", nt, ffi.BF16, ffi.EPI_GELU_BWD, aux_bf, c_bf),
            ("fc1 fwd plain, f32 out", nt, ffi.F32, ffi.EPI_NONE, 0, c_f),
            ("fc1 fwd + residual, f32 out", nt, ffi.F32, ffi.EPI_RESIDUAL, aux_f, c_f),
            ("fc2 dX plain", nn, ffi.BF16, ffi.EPI_NONE, 0, c_bf),
            ("fc2 dX * aux", nn, ffi.BF16, ffi.EPI_MUL_AUX, aux_bf, c_bf),
            ("fc2 dX * gelu'(aux)", nn, ffi.BF16, ffi.EPI_GELU_BWD, aux_bf, c_bf)):
        d = ffi.AhGemm(layout, ffi.BF16, out, epi, m, n, k, lda, ldb, ldc, 1, 0, 0, 0, pa, pb, pc, aux)
        ms = b.time(lambda: ffi.check(b.lib.ah_gemm(C.byref(d))))
        kern, nsplit = b.B.lastGemmKernel()
        b.record(f"{label}", ms, flops=flops, note=kern)
    b.release()


def bench_flash(b: Bench):
    Bt, H, D = 16, 12, 64
    Cc = H * D
    for T in (256, 1024, 2048):
        qkv, do = b.randn(Bt * T * 3 * Cc, ffi.BF16, 1.0, 3), b.randn(Bt * T * Cc, ffi.BF16, 1.0, 4)
        o, dqkv, lse = b.alloc(Bt * T * Cc * 2), b.alloc(Bt * T * 3 * Cc * 2), b.alloc(Bt * H * T * 4)
        for cap in (0.0, 30.0):
            f = ffi.AhFlash()
            f.dtype, f.batch, f.heads, f.seq, f.head_dim = ffi.BF16, Bt, H, T, D
            for p in ("q", "k", "v"):
                setattr(f, p + "_sb", T * 3 * Cc), setattr(f, p + "_sh", D), setattr(f, p + "_st", 3 * Cc)
            f.o_sb, f.o_sh, f.o_st = T * Cc, D, Cc
            f.scale, f.soft_cap = 1 / math.sqrt(D), cap
            f.q, f.k, f.v, f.o, f.lse = qkv, qkv + Cc * 2, qkv + 2 * Cc * 2, o, lse
            f.d_o, f.dq, f.dk, f.dv = do, dqkv, dqkv + Cc * 2, dqkv + 2 * Cc * 2
            ms = b.time(lambda: ffi.check(b.lib.ah_flash_fwd(C.byref(f))))
            b.record(f"flash fwd T={T} cap={cap:g}", ms, flops=4.0 * Bt * H * T * T * D, note="non-causal flop count; causal work is half")
            ms = b.time(lambda: ffi.check(b.lib.ah_flash_bwd(C.byref(f))))
            b.record(f"flash bwd T={T} cap={cap:g}", ms, flops=8.0 * Bt * H * T * T * D, note="dQ + dK/dV kernels")
        b.release()


def bench_bandwidth(b: Bench):
    lib = b.lib
    rows, dim, F, V, P = 16384, 768, 3072, 50304, 163_037_184
    x, res = b.randn(rows * dim, ffi.F32), b.randn(rows * dim, ffi.F32)
    g16 = b.randn(rows * dim, ffi.BF16)
    w, bias = b.randn(dim, ffi.F32), b.randn(dim, ffi.F32)
    out16, dx, dx16, dw, db = b.alloc(rows * dim * 2), b.alloc(rows * dim * 4), b.alloc(rows * dim * 2), b.alloc(dim * 4), b.alloc(dim * 4)
    ms = b.time(lambda: ffi.check(lib.ah_layernorm(x, w, bias, out16, rows, dim, 1e-5, ffi.BF16, ffi.F32)))
    b.record("layernorm fwd 16384x768", ms, nbytes=rows * dim * 6, note="f32 in, bf16 out")
    ms = b.time(lambda: ffi.check(lib.ah_layernorm_bwd(x, w, g16, ffi.BF16, res, dx, dx16, dw, db, rows, dim, 1e-5, 0, ffi.F32)))
    b.record("layernorm bwd 16384x768", ms, nbytes=rows * dim * 16, note="x f32, g bf16, + residual grad f32 -> dx f32 + bf16; dw, db")
    x16, res16 = b.randn(rows * dim, ffi.BF16, 1.0, 11), b.randn(rows * dim, ffi.BF16, 1.0, 12)
    part = b.alloc(int(lib.ah_layernorm_bwd_partials_bytes(rows, dim)))
    ms = b.time(lambda: ffi.check(lib.ah_layernorm(x16, w, bias, out16, rows, dim, 1e-5, ffi.BF16, ffi.BF16)))
    b.record("layernorm fwd 16384x768, bf16 stream", ms, nbytes=rows * dim * 4, note="bf16 in, bf16 out")
    ms = b.time(lambda: ffi.check(lib.ah_layernorm_bwd_deferred(x16, w, g16, ffi.BF16, res16, 0, dx16, part, rows, dim, 1e-5, ffi.BF16)))
    b.record("layernorm bwd 16384x768, bf16 stream", ms, nbytes=rows * dim * 8, note="x, g, residual grad bf16 -> dx bf16; partial dw, db (column sums put off)")
    b.release()

    # data movement of the reference's flash-attention branch (gpt.ts:232-253) on bf16 storage, moved as 4-byte words
    qkv16, q16 = b.randn(rows * 3 * dim, ffi.BF16), [b.alloc(rows * dim * 2) for _ in range(3)]
    ms = b.time(lambda: ffi.check(lib.ah_slice_qkv(qkv16, q16[0], q16[1], q16[2], rows, dim // 2)))
    b.record("sliceQkv 16384x2304 bf16", ms, nbytes=rows * 3 * dim * 4, note="three column blocks, one launch each")
    tr = b.alloc(rows * dim * 2)
    shp = ffi.shape_arr([16, 12, 1024, 32])
    ms = b.time(lambda: ffi.check(lib.ah_transpose(q16[0], tr, 4, shp, 1, 2)))
    b.record("transpose [16,12,1024,64] bf16, dims 1 and 2", ms, nbytes=rows * dim * 4, note="heads <-> positions, 128-byte rows kept whole")
    # residualDropoutAdd and the mask multiply of its backward with the mask made on the fly (no mask tensor): bf16 stream
    seed = b.alloc(4)
    ffi.check(lib.ah_fill_i32(seed, 42, 1))
    ms = b.time(lambda: ffi.check(lib.ah_dropout_apply(q16[0], ffi.BF16, q16[1], q16[2], ffi.BF16, rows * dim, seed, 3, 0.1)))
    b.record("dropout: residual + x * mask 16384x768 bf16", ms, nbytes=rows * dim * 6, note="mask from the counter hash, seed in device memory")
    ms = b.time(lambda: ffi.check(lib.ah_dropout_apply(q16[0], ffi.BF16, 0, q16[2], ffi.BF16, rows * dim, seed, 3, 0.1)))
    b.record("dropout: x * mask 16384x768 bf16", ms, nbytes=rows * dim * 4)
    b.release()

    h = b.randn(rows * F, ffi.F32)
    gh, oh = b.randn(rows * F, ffi.F32), b.alloc(rows * F * 4)
    ms = b.time(lambda: ffi.check(lib.ah_unary(ffi.GELU, h, oh, rows * F, 0.0, 0.0)))
    b.record("gelu fwd 16384x3072 f32", ms, nbytes=rows * F * 8, note="parity-mode op (the fast path fuses GELU into the GEMM epilogue)")
    ms = b.time(lambda: ffi.check(lib.ah_unary_bwd(ffi.GELU_BWD, h, gh, oh, rows * F, 0.0, 0.0)))
    b.record("gelu bwd 16384x3072 f32", ms, nbytes=rows * F * 12)
    b.release()

    lg = b.randn(rows * V, ffi.BF16, 2.0)
    tg = b.alloc(rows * 4)
    th = np.random.RandomState(5).randint(0, V, rows).astype(np.int32)
    ffi.check(lib.ah_upload(tg, th.ctypes.data_as(C.c_void_p), th.nbytes))
    loss, lse = b.alloc(4), b.alloc(rows * 4)
    ms = b.time(lambda: ffi.check(lib.ah_cross_entropy_fwd_bwd(lg, ffi.BF16, tg, loss, lse, 0, 1.0, lg, rows, V)))
    b.record("cross-entropy fwd+bwd 16384x50304", ms, nbytes=rows * V * 4, note="bf16 logits read once, gradient written in place")
    b.release()

    wte, tok = b.randn(V * dim, ffi.F32, 0.02), b.alloc(rows * 4)
    ffi.check(lib.ah_upload(tok, th.ctypes.data_as(C.c_void_p), th.nbytes))
    eo, gw = b.alloc(rows * dim * 4), b.alloc(V * dim * 4)
    ms = b.time(lambda: ffi.check(lib.ah_embedding(wte, tok, eo, rows, dim, V, ffi.F32)))
    b.record("embedding gather 16384x768", ms, nbytes=rows * dim * 8, note="uniform token ids")
    ms = b.time(lambda: ffi.check(lib.ah_embedding_bwd(tok, eo, gw, rows, dim, V, 0)))
    b.record("embedding scatter-add 16384x768", ms, nbytes=rows * dim * 8 + V * dim * 4, note="uniform ids; includes zero-filling the [50304, 768] gradient")
    from .train import zipfBatch
    zh = np.ascontiguousarray(zipfBatch(4, 16, rows // 16, V)[0].data, dtype=np.int32).reshape(-1)
    ffi.check(lib.ah_upload(tok, zh.ctypes.data_as(C.c_void_p), zh.nbytes))
    ms = b.time(lambda: ffi.check(lib.ah_embedding_bwd(tok, eo, gw, rows, dim, V, 0)))
    b.record("embedding scatter-add, power-law ids", ms, nbytes=rows * dim * 8 + V * dim * 4, note="Zipf(1.1) ids as in the step benchmark; same bytes; sorts the ids in every call")
    ib = int(lib.ah_embedding_index_bytes(rows, V))
    if ib:
        index = b.alloc(ib)
        ffi.check(lib.ah_embedding_index(tok, rows, V, index))
        ms = b.time(lambda: ffi.check(lib.ah_embedding_bwd_indexed(index, eo, gw, rows, dim, V, 0)))
        b.record("embedding scatter-add, ids sorted once", ms, nbytes=rows * dim * 8 + V * dim * 4, note="power-law ids, index of the resident batch built beforehand")
    b.release()

    p, g, m, v, sh = (b.randn(P, ffi.F32, 0.02, s) for s in (6, 7, 8, 9, 10))
    ffi.check(lib.ah_binary(ffi.MUL, v, v, v, P))                       # second moment must be non-negative
    acc = b.alloc(8)
    ms = b.time(lambda: ffi.check(lib.ah_sum_sq(g, P, acc)))
    b.record("sum of squares 163.0M", ms, nbytes=P * 4)
    hyp = ffi.AhAdamW(3e-4, 0.9, 0.95, 1e-8, 0.1, 0.1, 0.05, 1.0)
    ms = b.time(lambda: ffi.check(lib.ah_adamw(p, g, m, v, P, C.byref(hyp), 0, 0, sh)))
    b.record("adamw 163.0M (+bf16 shadow)", ms, nbytes=P * 30, note="reads p g m v, writes p m v + bf16 copy of p")
    b.release()


def bench_ceiling(b: Bench):
    """What the matrix pipes sustain with nothing else going on (operands in registers), by how long they are kept busy and by
    what the operands hold; the rate of the last line is the ceiling a bf16 GEMM on real data can be read against."""
    lib = b.lib
    fl = C.c_double()

    def run(name, waves, iters, launches, random_ops, note=""):
        ffi.check(lib.ah_probe_mfma_bf16(waves, 100, random_ops, C.byref(fl)))       # (first launch of a kernel: code upload)
        ffi.check(lib.ah_sync())
        e0, e1 = b.B._event(), b.B._event()
        ffi.check(lib.ah_event_record(e0))
        for _ in range(launches):
            ffi.check(lib.ah_probe_mfma_bf16(waves, iters, random_ops, C.byref(fl)))
        ffi.check(lib.ah_event_record(e1))
        ms = C.c_float()
        ffi.check(lib.ah_event_elapsed_ms(e0, e1, C.byref(ms)))
        for e in (e0, e1):
            ffi.check(lib.ah_event_destroy(e))
        b.record(name, ms.value / launches, flops=fl.value, note=note)
    run("mfma bf16, zeros, 100 x 3 ms", 1, 30000, 100, 0, "registers only, no memory traffic: the published dense peak")
    run("mfma bf16, random, 1 x 0.15 ms", 1, 1000, 1, 1, "operands whose bits toggle; one short launch after an idle device")
    run("mfma bf16, random, 1 x 4 ms", 1, 30000, 1, 1, "the length of the step's weight-gradient launch")
    run("mfma bf16, random, 100 x 4 ms", 1, 30000, 100, 1, "sustained: what the power limit allows the matrix pipes alone")
    run("mfma bf16, random, 100 x 4 ms, 2 waves", 2, 15000, 100, 1, "two waves per SIMD: the same")
    # the other side of it: the library's GEMM on operands that toggle nothing (the power limit does not bind, the clock stays
    # up), which shows what the kernel's own structure - its traffic through L2 and LDS - allows; compare the rows of the
    # same shapes in the GEMM section, which run on random operands
    M, K, N = 16384, 768, 50304
    a, w, g = b.randn(M * K, ffi.BF16, 0.0), b.randn(N * K, ffi.BF16, 0.0), b.randn(M * N, ffi.BF16, 0.0)
    c_fwd, c_da, c_db = b.alloc(M * N * 2), b.alloc(M * K * 2), b.alloc(N * K * 4)
    for label, layout, (m, n, k, lda, ldb, ldc), (pa, pb, pc), out in (
            ("fwd  C=A.B^T", ffi.GEMM_NT, (M, N, K, K, K, N), (a, w, c_fwd), ffi.BF16),
            ("dA   G.B", ffi.GEMM_NN, (M, K, N, N, K, K), (g, w, c_da), ffi.BF16),
            ("dB   G^T.A", ffi.GEMM_TN, (N, K, M, N, K, K), (g, a, c_db), ffi.F32)):
        d = ffi.AhGemm(layout, ffi.BF16, out, ffi.EPI_NONE, m, n, k, lda, ldb, ldc, 1, 0, 0, 0, pa, pb, pc, 0)
        ms = b.time(lambda: ffi.check(lib.ah_gemm(C.byref(d))))
        b.record(f"gemm bf16 N={N} {label}, zeros", ms, flops=2.0 * M * N * K, note="all-zero operands")
    b.release()


def bench_issue(b: Bench):
    """Time per group of instructions on one SIMD (`ah_probe_issue`), by how many waves share the SIMD."""
    lib = b.lib
    n = C.c_double()
    kinds = ((0, "v_fma_f32"), (1, "v_exp_f32"), (2, "v_exp_f32 + 3 v_fma_f32"), (3, "mfma 32x32x16 bf16"),
             (4, "mfma 32x32x16 bf16 + 8 v_fma_f32"), (5, "mfma 32x32x16 bf16 + 16 v_fma_f32"))
    print(f"{'group of instructions':40s} {'waves/SIMD':>10s} {'ns per group per SIMD':>22s}")
    for kind, name in kinds:
        for waves in ((1, 2, 4) if kind < 3 else (1, 2)):
            ffi.check(lib.ah_probe_issue(kind, waves, 100, C.byref(n)))          # (first launch of a kernel: code upload)
            ffi.check(lib.ah_sync())
            e0, e1 = b.B._event(), b.B._event()
            ffi.check(lib.ah_event_record(e0))
            ffi.check(lib.ah_probe_issue(kind, waves, 20000, C.byref(n)))
            ffi.check(lib.ah_event_record(e1))
            ms = C.c_float()
            ffi.check(lib.ah_event_elapsed_ms(e0, e1, C.byref(ms)))
            for e in (e0, e1):
                ffi.check(lib.ah_event_destroy(e))
            ns = ms.value * 1e6 / n.value
            b.rows.append({"op": f"issue: {name}", "waves_per_simd": waves, "ns_per_group": ns})
            print(f"{name:40s} {waves:10d} {ns:22.2f}", flush=True)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--iters", type=int, default=10)
    ap.add_argument("--only", choices=["gemm", "flash", "bandwidth", "ceiling", "epilogue", "issue"])
    ap.add_argument("--json", action="store_true", help="also print one JSON line with every row")
    args = ap.parse_args(argv)
    b = Bench(args.iters)
    if args.only == "issue":
        bench_issue(b)
        if args.json:
            print(json.dumps(b.rows))
        return 0
    print(f"{'op':34s} {'time':>13s} {'rate':>16s} {'peak':>7s}")
    for name, fn in (("gemm", bench_gemm), ("flash", bench_flash), ("bandwidth", bench_bandwidth), ("ceiling", bench_ceiling)):
        if args.only in (None, name):
            fn(b)
    if args.only == "epilogue":
        bench_epilogues(b)
    if args.json:
        print(json.dumps(b.rows))
    return 0


if __name__ == "__main__":
    sys.exit(main())
