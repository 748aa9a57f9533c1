"""FastHipBackend: the fast mode behind the unchanged `Backend` interface.  The caller (the generic tape-driven Trainer, the
same code that drives the fp32 parity path) issues one call per op; bf16 storage, fused epilogues, grouped weight gradients
and hipGraph replay all happen below the interface.  Bars: step loss within 2e-2 relative of the CPU oracle over 50 steps
(the task's bf16 bar); fused call sequences equal their unfused evaluation to bf16 rounding."""
import math

import numpy as np
import pytest

from oracle import ref
from oracle import ref_model as rm

pytestmark = pytest.mark.gpu

CFG = dict(vocabSize=256, blockSize=64, nLayer=2, nEmbd=128, nHead=4)


@pytest.fixture()
def FB():
    from alpha2_amd import FastHipBackend
    b = FastHipBackend(0)
    b.resetStepPlan()
    yield b
    b.enableStepGraphs(False)
    b.resetStepPlan()


def _td(arr):
    from alpha2_amd import TensorData
    arr = np.asarray(arr, np.float32)
    return TensorData(arr.shape, "f32", arr)


def _bf16(x):
    u = np.asarray(x, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def _close(got, want, what, tol=2e-2):
    got, want = np.asarray(got, np.float64).reshape(-1), np.asarray(want, np.float64).reshape(-1)
    rms = float(np.sqrt(np.mean(want * want))) + 1e-30
    assert np.max(np.abs(got - want)) <= tol * rms * 4 and np.sqrt(np.mean((got - want) ** 2)) <= tol * rms, \
        (what, float(np.max(np.abs(got - want))), rms)


def test_held_back_products_and_their_epilogues(FB):
    """The three call sequences the reference's autograd issues around a linear layer, each against float64 numpy on the
    bf16-rounded operands; then the same sequences with the held-back product read by someone else first (no fusion)."""
    rs = np.random.RandomState(5)
    M, K, N = 192, 128, 320
    x, w, g, res = rs.randn(M, K) * 0.5, rs.randn(N, K) * 0.1, rs.randn(M, N) * 0.3, rs.randn(M, N)
    xb, wb = _bf16(x).astype(np.float64), _bf16(w).astype(np.float64)
    pre = xb @ wb.T
    k = math.sqrt(2 / math.pi)
    gelu = lambda v: 0.5 * v * (1 + np.tanh(k * (v + 0.044715 * v ** 3)))
    dgelu = lambda v: 0.5 * (1 + np.tanh(k * (v + 0.044715 * v ** 3))) + 0.5 * v * (1 - np.tanh(k * (v + 0.044715 * v ** 3)) ** 2) * k * (1 + 3 * 0.044715 * v * v)
    # gelu(matmulTransposed)
    mm = FB.matmulTransposed(_td(x), _td(w))
    out = FB.gelu(mm)
    _close(out.data, gelu(pre), "gelu epilogue")
    _close(mm.data, pre, "pre-activation kept for backward")
    # add(res, reshape(matmulTransposed))
    prod = FB.matmulTransposed(_td(x), _td(w))
    view = FB.reshape(prod, (2, M // 2, N))
    y = FB.add(_td(res.reshape(2, M // 2, N)), view)
    assert y.store == "bf16"                                   # the residual stream is a bf16 activation by default ...
    _close(y.data, _bf16(res).reshape(-1) + pre.reshape(-1), "residual epilogue")
    _close(prod.data, pre, "the product itself, computed only now because somebody asked")
    FB.streamBf16 = False                                      # ... and f32 on request
    prod = FB.matmulTransposed(_td(x), _td(w))
    y = FB.add(_td(res), prod)
    FB.streamBf16 = True
    assert y.store == "f32"
    _close(y.data, res.reshape(-1) + pre.reshape(-1), "residual epilogue, f32 stream")
    # geluBackward(pre, matmul(g, w2))
    w2 = rs.randn(N, K) * 0.1                 # [N, K]: g [M, N] @ w2 -> [M, K]
    pre2 = FB.matmulTransposed(_td(x), _td(rs.randn(K, K) * 0.1))
    pre2_host = pre2.data.astype(np.float64).reshape(M, K)
    dx = FB.matmul(_td(g), _td(w2))
    dpre = FB.geluBackward(pre2, dx)
    _close(dpre.data, (_bf16(g).astype(np.float64) @ _bf16(w2).astype(np.float64)) * dgelu(pre2_host), "gelu-backward epilogue")
    # the pair as the tape issues it (ops.ts:426-487): gelu of a held-back product, later geluBackward of that product and a
    # held-back gradient.  The forward launch saved gelu' and the backward multiplies by it; the pre-activation is never written
    # unless somebody reads it, and is right when they do.
    mm = FB.matmulTransposed(_td(x), _td(w))
    act = FB.gelu(mm)
    assert id(mm._buf) in FB._orphans and FB._orphans[id(mm._buf)].gelu_grad is not None
    w3 = rs.randn(K, N) * 0.1
    dmm = FB.geluBackward(mm, FB.matmul(_td(g[:, :K]), _td(w3)))
    want = (_bf16(g[:, :K]).astype(np.float64) @ _bf16(w3).astype(np.float64)) * _bf16(dgelu(pre)).astype(np.float64)
    _close(dmm.data, want, "gelu-backward from the saved derivative")
    _close(act.data, gelu(pre), "gelu epilogue (saving the derivative)")
    _close(mm.data, pre, "the pre-activation, computed only now")
    assert id(mm._buf) not in FB._orphans
    FB.releaseGpuTensor(mm)
    # no fusion when the product has been read
    mm = FB.matmulTransposed(_td(x), _td(w))
    _ = mm.data
    _close(FB.gelu(mm).data, gelu(_bf16(pre).astype(np.float64)), "gelu of a product already launched")


def test_weight_gradients_are_grouped_and_accumulate_in_place(FB):
    rs = np.random.RandomState(6)
    T = 256
    gs = [rs.randn(T, m) * 0.2 for m in (64, 128, 192)]
    xs = [rs.randn(T, n) * 0.5 for n in (128, 64, 128)]
    wants = [_bf16(g).astype(np.float64).T @ _bf16(x).astype(np.float64) for g, x in zip(gs, xs)]
    outs = [FB.matmulTransposedA(_td(g), _td(x)) for g, x in zip(gs, xs)]
    assert len(FB._wgrads) == 3                                  # nothing launched yet
    grads = [FB.clone(o) for o in outs]                         # what the tape does with a first gradient
    for o in outs:
        FB.releaseGpuTensor(o)
    total = FB.totalSumOfSquares(grads)                         # the trainer's gradient norm reads them: one grouped launch
    assert len(FB._wgrads) == 0
    assert FB.lastGemmKernel()[0].endswith(", true>")           # ... which squares and sums what it stores: nothing is read again
    assert abs(float(total.data[0]) - sum(float((w ** 2).sum()) for w in wants)) <= 1e-3 * sum(float((w ** 2).sum()) for w in wants)
    for gr, w in zip(grads, wants):
        _close(gr.data, w, "grouped weight gradient", tol=1e-3)
    # second micro-step: addInplace re-targets the held-back products to accumulate into the existing gradients
    outs2 = [FB.matmulTransposedA(_td(g), _td(x)) for g, x in zip(gs, xs)]
    for gr, o in zip(grads, outs2):
        FB.addInplace(gr, o)
        FB.releaseGpuTensor(o)
    for gr, w in zip(grads, wants):
        _close(gr.data, 2 * w, "accumulated weight gradient", tol=1e-3)
    # the norm over queued products and other tensors: the launch sums its own, the others are read
    sq = [float((w ** 2).sum()) for w in wants]
    o = [FB.matmulTransposedA(_td(g), _td(x)) for g, x in zip(gs, xs)]
    extra = FB.scale(_td(np.arange(10.0)), 1.0)                 # (resident on the device, as the trainer's gradients are)
    got = float(FB.totalSumOfSquares([o[0], extra, o[1], o[2]]).data[0])
    assert FB.lastGemmKernel()[0].endswith(", true>") and abs(got - (sum(sq) + 285.0)) <= 1e-3 * (sum(sq) + 285.0)
    # a queued product that the list does not name must not count: the launches run as they are, the list is read
    o = [FB.matmulTransposedA(_td(g), _td(x)) for g, x in zip(gs, xs)]
    got = float(FB.totalSumOfSquares([o[0], o[2]]).data[0])
    assert FB.lastGemmKernel()[0].endswith(", false>") and abs(got - (sq[0] + sq[2])) <= 1e-3 * (sq[0] + sq[2])
    _close(o[1].data, wants[1], "the product outside the list", tol=1e-3)
    # accumulating launches count the accumulated values
    o2 = [FB.matmulTransposedA(_td(g), _td(x)) for g, x in zip(gs, xs)]
    for gr, x in zip(grads, o2):
        FB.addInplace(gr, x)
        FB.releaseGpuTensor(x)
    got = float(FB.totalSumOfSquares(grads).data[0])
    assert FB.lastGemmKernel()[0].endswith(", true>") and abs(got - 9 * sum(sq)) <= 1e-3 * 9 * sum(sq)


def test_gradient_norm_with_one_accumulating_and_several_fresh_weight_gradients(FB):
    """One queued product re-targeted by addInplace (a shared weight: a part of one descriptor, launched on its own) beside
    fresh ones (a grouped launch): the norm must see the accumulated gradient after its product has run, as eager execution
    (every product launched when it is asked for) does."""
    rs = np.random.RandomState(16)
    T = 256
    gs = [rs.randn(T, m) * 0.2 for m in (64, 128, 192, 64)]
    xs = [rs.randn(T, n) * 0.5 for n in (128, 64, 128, 128)]
    wants = [_bf16(g).astype(np.float64).T @ _bf16(x).astype(np.float64) for g, x in zip(gs, xs)]
    got = []
    for group in (True, False):
        FB._group = group
        try:
            shared = FB.clone(FB.matmulTransposedA(_td(gs[3]), _td(xs[3])))       # the first use's gradient, resident
            FB.syncGpu()
            fresh = [FB.matmulTransposedA(_td(g), _td(x)) for g, x in zip(gs[:3], xs[:3])]
            again = FB.matmulTransposedA(_td(gs[3]), _td(xs[3]))                  # the second use: added into the first
            FB.addInplace(shared, again)
            FB.releaseGpuTensor(again)
            got.append(float(FB.totalSumOfSquares(fresh + [shared]).data[0]))
            _close(shared.data, 2 * wants[3], "gradient of the shared weight", tol=1e-3)
        finally:
            FB._group = True
    want = sum(float((w ** 2).sum()) for w in wants[:3]) + float(((2 * wants[3]) ** 2).sum())
    assert abs(got[0] - want) <= 1e-3 * want and abs(got[1] - want) <= 1e-3 * want, (got, want)


def test_a_product_kept_past_the_optimizer_step_is_of_the_weights_it_was_asked_with(FB):
    """A product whose epilogue took its place (x W^T + residual) is only a recipe while its own tensor is unread; the recipe
    names the weight's bf16 shadow, which adamwStep rewrites in place: read after the update, the tensor must still be the
    product with the weights of the time of the call (what eager execution, and the reference's backends, give)."""
    rs = np.random.RandomState(21)
    x, w, res = _bf16(rs.randn(64, 128) * 0.5), _bf16(rs.randn(256, 128) * 0.1), _bf16(rs.randn(64, 256))
    W = _td(w)
    prod = FB.matmulTransposed(FB.castStore(_td(x), "bf16"), W)
    out = FB.add(FB.castStore(_td(res), "bf16"), prod)              # the residual epilogue: `prod` itself is not written
    g = _td(np.ones_like(w))
    m, v = _td(np.zeros_like(w)), _td(np.zeros_like(w))
    FB.adamwStep(W, g, m, v, 0.5, 0.9, 0.95, 1e-8, 0.0, 0.1, 0.05, 1.0)
    FB.syncGpu()
    want = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.max(np.abs(W.data.reshape(w.shape) - w)) > 0.1      # the weights did move
    _close(prod.data, want, "the product read after the update", tol=1e-2)
    _close(out.data, want + res, "its residual sum", tol=1e-2)


def test_clone_is_copy_on_write(FB):
    a = _td(np.arange(8.0))
    c = FB.clone(a)
    FB.addInplace(c, _td(np.ones(8)))
    assert np.array_equal(a.data, np.arange(8.0)) and np.array_equal(c.data, np.arange(8.0) + 1)
    d = FB.clone(c)
    FB.scaleInplace(c, 2.0)
    assert np.array_equal(d.data, np.arange(8.0) + 1) and np.array_equal(c.data, 2 * (np.arange(8.0) + 1))


@pytest.mark.parametrize("graphs", [False, True])
def test_reference_flash_branch_on_the_fast_backend_tracks_its_oracle_over_50_steps(FB, graphs):
    """The branch an unchanged gpt.ts takes on a backend with flashAttention (gpt.ts:247-254), run by the generic trainer on
    the fast backend (bf16 words moved by sliceQkv / transpose, the three scatterSlice results of the backward pass merged),
    against the oracle's restatement of that branch: loss within 2e-2 relative at every one of 50 steps, eagerly and replayed
    from a step plan, the two bit-identical."""
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig, Trainer, syntheticBatch
    steps = 50
    cfg = dict(CFG, attention="reference-flash")
    tr = Trainer(FB, ModelConfig(**cfg), TrainConfig(iters=steps), seed=3)
    orc = rm.Trainer(rm.ModelConfig(**cfg), rm.TrainConfig(iters=steps), seed=3)
    for t in (tr, orc):                             # attention weights large enough that the slab wiring shows in the loss
        for n, v in t.entries:
            if n.endswith("attn.wqkv"):
                v.data.data = v.data.data * 8
    FB.enableStepGraphs(graphs)
    before, planes_before = FB.stepStats(), FB.planeProducts
    losses = []
    for s in range(steps):
        r = tr.step([syntheticBatch(50 + s, 4, 64, 256)])
        o = orc.step([rm.synthetic_batch(50 + s, 4, 64, 256)])
        assert math.isfinite(r.loss) and abs(r.loss - o.loss) <= 2e-2 * abs(o.loss), (s, r.loss, o.loss)
        assert abs(r.gradNorm - o.gradNorm) <= 5e-2 * o.gradNorm and abs(r.lr - o.lr) < 1e-15, (s, r.gradNorm, o.gradNorm)
        losses.append((r.loss, r.gradNorm))
    FB.enableStepGraphs(False)
    # at this shape the fused projection writes q, k, v in place of sliceQkv's copies and its backward reads dq, dk, dv where
    # they lie (ah_gemm_planes): two such products per layer and step
    assert FB.planeProducts - planes_before == 2 * cfg["nLayer"] * steps, (FB.planeProducts, planes_before)
    fn = test_reference_flash_branch_on_the_fast_backend_tracks_its_oracle_over_50_steps
    if graphs:
        assert FB.stepStats()["replayed"] - before["replayed"] >= steps - 4, (before, FB.stepStats(), FB.lastStepNote)
        fn.graph_losses = losses
    else:
        fn.eager_losses = losses
    if hasattr(fn, "graph_losses") and hasattr(fn, "eager_losses"):
        assert fn.graph_losses == fn.eager_losses


@pytest.mark.parametrize("graphs", [False, True])
def test_generic_trainer_on_the_fast_backend_tracks_the_oracle_over_50_steps(FB, graphs):
    """The reference's trainer structure (tape-driven, one Backend call per op, host-side norm / clip / schedule) on the
    fast backend: loss within 2e-2 relative of the CPU oracle at every one of 50 steps; with step graphs on, steps are
    replayed from the recorded plan and give bit-identical numbers to eager issue."""
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig, Trainer, syntheticBatch
    steps = 50
    tr = Trainer(FB, ModelConfig(**CFG), TrainConfig(iters=steps), seed=3)
    orc = rm.Trainer(rm.ModelConfig(**CFG), rm.TrainConfig(iters=steps), seed=3)
    FB.enableStepGraphs(graphs)
    before = FB.stepStats()
    losses = []
    for s in range(steps):
        r = tr.step([syntheticBatch(50 + s, 4, 64, 256)])
        o = orc.step([rm.synthetic_batch(50 + s, 4, 64, 256)])
        assert math.isfinite(r.loss) and abs(r.loss - o.loss) <= 2e-2 * abs(o.loss), (s, r.loss, o.loss)
        assert abs(r.gradNorm - o.gradNorm) <= 5e-2 * o.gradNorm and abs(r.lr - o.lr) < 1e-15, (s, r.gradNorm, o.gradNorm)
        losses.append((r.loss, r.gradNorm))
    FB.enableStepGraphs(False)
    after = FB.stepStats()
    if graphs:
        assert after["replayed"] - before["replayed"] >= steps - 4, (before, after, FB.lastStepNote)
        test_generic_trainer_on_the_fast_backend_tracks_the_oracle_over_50_steps.graph_losses = losses
    else:
        test_generic_trainer_on_the_fast_backend_tracks_the_oracle_over_50_steps.eager_losses = losses
    fn = test_generic_trainer_on_the_fast_backend_tracks_the_oracle_over_50_steps
    if hasattr(fn, "graph_losses") and hasattr(fn, "eager_losses"):
        assert fn.graph_losses == fn.eager_losses        # the same kernels in the same order, every sum in a fixed order


def test_accumulation_and_other_model_variants_still_run_on_the_fast_backend(FB):
    """Two micro-steps per step (weight gradients accumulate through the grouped launch) and a model variant whose ops have
    no bf16 kernels (swiglu: inherited f32 kernels after a cast): losses within the bf16 bar of the oracle."""
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig, Trainer, syntheticBatch
    for kw, accum in ((dict(), 2), (dict(ffnActivation="swiglu"), 1), (dict(dropout=0.1), 1),
                      (dict(attention="reference-flash"), 2), (dict(attention="reference-flash", dropout=0.1), 2)):     # (plane products that accumulate)
        cfg = dict(CFG, **kw)
        tr = Trainer(FB, ModelConfig(**cfg), TrainConfig(iters=6, gradAccumSteps=accum), seed=4)
        orc = rm.Trainer(rm.ModelConfig(**cfg), rm.TrainConfig(iters=6, gradAccumSteps=accum), seed=4)
        for s in range(6):
            r = tr.step([syntheticBatch(90 + accum * s + m, 4, 64, 256) for m in range(accum)])
            o = orc.step([rm.synthetic_batch(90 + accum * s + m, 4, 64, 256) for m in range(accum)])
            assert abs(r.loss - o.loss) <= 2e-2 * abs(o.loss), (kw, s, r.loss, o.loss)
            assert abs(r.gradNorm - o.gradNorm) <= 5e-2 * o.gradNorm, (kw, s, r.gradNorm, o.gradNorm)


def test_bf16_tensors_move_as_words_and_the_reference_flash_branch_stays_in_bf16(FB):
    """slice / sliceQkv / transpose / scatterSlice on bf16-stored tensors with an even innermost dimension give exactly what the
    f32 kernels give on the same values (the copies never look inside a word), and the model with the reference's own flash
    branch (gpt.ts:232-253: sliceQkv, reshape to [B*H, T, D] without a head transpose, flashAttention, transpose back) trains on
    the fast backend within the bf16 bar of the same model on the fp32 backend, replayed from a step plan."""
    from alpha2_amd import HipBackend
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig, Trainer, syntheticBatch
    rs = np.random.RandomState(11)
    x = _bf16(rs.randn(6, 5, 4, 8))
    t = FB.castStore(_td(x), "bf16")
    assert np.array_equal(FB.transpose(t, 1, 2).data.reshape(6, 4, 5, 8), x.transpose(0, 2, 1, 3)) and FB.transpose(t, 1, 2).store == "bf16"
    assert np.array_equal(FB.transpose(t, 0, 2).data.reshape(4, 5, 6, 8), x.transpose(2, 1, 0, 3))
    assert np.array_equal(FB.transpose(t, 2, 3).data.reshape(6, 5, 8, 4), x.transpose(0, 1, 3, 2))          # touches the last axis: f32 route
    m = _bf16(rs.randn(10, 24))
    tm = FB.castStore(_td(m), "bf16")
    q, k, v = FB.sliceQkv(tm)
    assert q.store == "bf16" and all(np.array_equal(p.data.reshape(10, 8), m[:, 8 * i:8 * i + 8]) for i, p in enumerate((q, k, v)))
    sl = FB.slice(tm, [2, 4], [9, 20])
    assert sl.store == "bf16" and np.array_equal(sl.data.reshape(7, 16), m[2:9, 4:20])
    assert np.array_equal(FB.slice(tm, [2, 3], [9, 20]).data.reshape(7, 17), m[2:9, 3:20])                    # odd column: f32 route
    sc = FB.scatterSlice(q, (10, 24), [0, 8], [10, 16])
    want = np.zeros((10, 24), np.float32); want[:, 8:16] = m[:, :8]
    assert sc.store == "bf16" and np.array_equal(sc.data.reshape(10, 24), want)

    # sums of bf16-stored tensors stay in bf16 (one rounding), in place as well, also when the target shares its buffer
    y = _bf16(rs.randn(10, 24))
    tm, ty = FB.castStore(_td(m), "bf16"), FB.castStore(_td(y), "bf16")      # (the odd-column slice above widened the old `tm` to f32)
    s2 = FB.add(tm, ty)
    assert s2.store == "bf16" and np.array_equal(s2.data.reshape(10, 24), _bf16(m + y))
    acc = FB.clone(tm)
    FB.addInplace(acc, ty)
    assert acc.store == "bf16" and np.array_equal(acc.data.reshape(10, 24), _bf16(m + y)) and np.array_equal(tm.data.reshape(10, 24), m)
    FB.addInplace(acc, ty)
    assert np.array_equal(acc.data.reshape(10, 24), _bf16(_bf16(m + y) + y))

    cfg = dict(CFG, attention="reference-flash")
    ref_b = HipBackend(0)
    slow = Trainer(ref_b, ModelConfig(**cfg), TrainConfig(iters=6), seed=4)
    fast = Trainer(FB, ModelConfig(**cfg), TrainConfig(iters=6), seed=4)
    want = [slow.step([syntheticBatch(70 + s, 4, 64, 256)]) for s in range(8)]
    FB.enableStepGraphs(True)
    before = FB.stepStats()
    for s, a in enumerate(want):
        b = fast.step([syntheticBatch(70 + s, 4, 64, 256)])
        assert math.isfinite(b.loss) and abs(a.loss - b.loss) <= 2e-2 * abs(a.loss), (s, a.loss, b.loss)
        assert abs(a.gradNorm - b.gradNorm) <= 5e-2 * a.gradNorm, (s, a.gradNorm, b.gradNorm)
    FB.enableStepGraphs(False)
    assert FB.stepStats()["replayed"] - before["replayed"] >= 4, (before, FB.stepStats(), FB.stepFallbackNotes)


def test_layernorm_backward_is_held_until_its_dx_is_added_to_the_stream_gradient(FB):
    """The tape's sequence after a LayerNorm on the residual stream (tape.ts:116-127): layerNormBackward, then addInplace of dx
    into the gradient the residual add left on the stream, then clones of dw and db.  The sum comes out of the LayerNorm kernel
    itself; it, dw and db must equal float64 numpy on the bf16-rounded operands, and the same calls in other orders (dx read
    first, dx read after it went into the sum, everything released unread) must still give the plain results."""
    rs = np.random.RandomState(11)
    rows, dim, eps = 96, 128, 1e-5
    x, w, g, acc = rs.randn(rows, dim), 1 + 0.1 * rs.randn(dim), rs.randn(rows, dim) * 0.3, rs.randn(rows, dim)
    xb, gb, ab = _bf16(x).astype(np.float64), _bf16(g).astype(np.float64), _bf16(acc).astype(np.float64)
    mean = xb.mean(1, keepdims=True)
    rstd = 1 / np.sqrt(((xb - mean) ** 2).mean(1, keepdims=True) + eps)
    xh = (xb - mean) * rstd
    gw = gb * w.astype(np.float32).astype(np.float64)
    dx = rstd * (gw - gw.mean(1, keepdims=True) - xh * (gw * xh).mean(1, keepdims=True))
    dw, db = (gb * xh).sum(0), gb.sum(0)

    def operands():
        return (FB.castStore(_td(x), "bf16"), _td(w), FB.castStore(_td(g), "bf16"), FB.castStore(_td(acc), "bf16"))

    # the tape's order: the sum is one launch, the clone keeps the old contents of the stream gradient
    tx, tw, tg, ta = operands()
    keep = FB.clone(ta)
    r = FB.layerNormBackward(tx, tw, tg, eps)
    assert FB._held_ln is not None
    FB.addInplace(ta, r["dx"])
    assert FB._held_ln is None and ta.store == "bf16"
    gw_, gb_ = FB.clone(r["dw"]), FB.clone(r["db"])
    _close(ta.data, ab + dx, "stream gradient + dx", 1e-2)
    assert np.array_equal(keep.data, ab.astype(np.float32).reshape(keep.data.shape))
    _close(gw_.data, dw, "dw", 1e-4)
    _close(gb_.data, db, "db", 1e-4)
    # dx itself was never written; a reader still gets it
    _close(r["dx"].data, dx, "dx read after it went into the sum", 1e-2)
    FB.releaseGpuTensor(r["dx"])
    assert not FB._ln_unwritten

    # dx read first: the plain kernel, then an ordinary add
    tx, tw, tg, ta = operands()
    r = FB.layerNormBackward(tx, tw, tg, eps)
    _close(r["dx"].data, dx, "dx", 1e-2)
    assert FB._held_ln is None
    FB.addInplace(ta, r["dx"])
    _close(ta.data, ab + dx, "stream gradient + dx, two launches", 1.5e-2)
    _close(r["dw"].data, dw, "dw", 1e-4)

    # a second LayerNorm backward while one is held launches the first
    tx, tw, tg, ta = operands()
    r1 = FB.layerNormBackward(tx, tw, tg, eps)
    r2 = FB.layerNormBackward(tx, tw, tg, eps)
    FB.addInplace(ta, r2["dx"])
    _close(r1["dx"].data, dx, "first of two", 1e-2)
    _close(ta.data, ab + dx, "second of two", 1e-2)
    FB.releaseGpuTensor(r2["dx"])                              # (what the tape does with a gradient it has consumed)

    # released unread: nothing is launched, nothing is left behind
    tx, tw, tg, ta = operands()
    r = FB.layerNormBackward(tx, tw, tg, eps)
    for t in r.values():
        FB.releaseGpuTensor(t)
    FB.flush()
    assert FB._held_ln is None and not FB._ln_unwritten


def test_scattered_column_blocks_are_merged_before_they_are_written(FB):
    """The backward of sliceQkv (ops.ts:816-858): three scatterSlice results, the first cloned and the others added in place
    (tape.ts:116-127).  Held back, the three become one matrix written once; blocks that leave columns uncovered bring their
    zeros; overlapping blocks and blocks read on their own take the ordinary route.  All exact: copies and zeros only."""
    rs = np.random.RandomState(13)
    rows, d = 48, 32
    blocks = [_bf16(rs.randn(rows, d)) for _ in range(3)]
    full = np.concatenate(blocks, axis=1)

    def scatter(i, at=None):
        c0 = d * i if at is None else at
        return FB.scatterSlice(FB.castStore(_td(blocks[i]), "bf16"), (rows, 3 * d), [0, c0], [rows, c0 + d])

    # the tape's sequence, last block first
    s = scatter(2)
    acc = FB.clone(s)
    FB.releaseGpuTensor(s)
    for i in (1, 0):
        s = scatter(i)
        FB.addInplace(acc, s)
        FB.releaseGpuTensor(s)
    assert len(FB._scatters) == 1                                  # one unwritten matrix, three blocks
    assert np.array_equal(acc.data.reshape(rows, 3 * d), full)
    assert not FB._scatters

    # two of three blocks: the rest is zero; a clone taken in between keeps the single block
    s = scatter(0)
    acc = FB.clone(s)
    s2 = scatter(2)
    FB.addInplace(acc, s2)                                         # `s` still names the first buffer: the sum gets its own
    want = full.copy()
    want[:, d:2 * d] = 0
    assert np.array_equal(acc.data.reshape(rows, 3 * d), want)
    only0 = np.zeros_like(full)
    only0[:, :d] = blocks[0]
    assert np.array_equal(s.data.reshape(rows, 3 * d), only0)
    only2 = np.zeros_like(full)
    only2[:, 2 * d:] = blocks[2]
    assert np.array_equal(s2.data.reshape(rows, 3 * d), only2)

    # overlapping blocks are really added
    a, b = scatter(0, at=0), scatter(1, at=d // 2)
    acc = FB.clone(a)
    FB.addInplace(acc, b)
    want = np.zeros((rows, 3 * d), np.float32)
    want[:, :d] += blocks[0]
    want[:, d // 2:d // 2 + d] += blocks[1]
    _close(acc.data, _bf16(want), "overlapping blocks", 1e-2)
    for t in (a, b, acc, s, s2):
        FB.releaseGpuTensor(t)
    assert not FB._scatters


def test_the_fused_projection_and_its_backward_take_their_operands_in_planes(FB):
    """sliceQkv of a projection that has not been launched yet makes the projection write q, k, v itself, and the backward
    products of the projection read dq, dk, dv where flashAttentionBackward leaves them instead of a written sum of three
    scatterSlice results (ops.ts:816-858, 197-234).  Same numbers as the route around copies, to an ulp of the bf16 results
    (at this size the ordinary route runs another kernel) and to f32 summation order for the weight gradient."""
    rs = np.random.RandomState(17)
    rows, d = 512, 128
    x, w = _bf16(rs.randn(rows, d)), _bf16(rs.randn(3 * d, d) * 0.1)
    X, W = FB.castStore(_td(x), "bf16"), _td(w)
    n0 = FB.planeProducts
    # forward
    plain = FB.matmulTransposed(X, W).data.reshape(rows, 3 * d).copy()                 # read at once: written as one matrix
    held = FB.matmulTransposed(X, W)
    q, k, v = FB.sliceQkv(held)
    assert FB.planeProducts == n0 + 1 and q._buf is k._buf is v._buf
    for i, t in enumerate((q, k, v)):
        assert t.store == "bf16"
        _close(t.data.reshape(rows, d), plain[:, i * d:(i + 1) * d], f"plane {i}", 4e-3)         # (another kernel at this size: an ulp of bf16 here and there)
        _close(t.data.reshape(rows, d), _bf16(x.astype(np.float64) @ w[i * d:(i + 1) * d].astype(np.float64).T), f"plane {i} vs f64", 4e-3)
    assert np.array_equal(held.data.reshape(rows, 3 * d), plain)                        # the product itself, asked for after all
    # backward: gradients as flashAttentionBackward allocates them (one behind the other), scattered and summed by the tape
    gs = [_bf16(rs.randn(rows, d)) for _ in range(3)]

    def summed(planes: bool):
        if planes:
            ts = FB._plane_views(3, (rows, d))
            for t, g in zip(ts, gs):
                bits = (g.view(np.uint32) >> 16).astype(np.uint16)
                ffi.check(FB.lib.ah_upload(t._buf.ptr + t._off, bits.ctypes.data_as(C.c_void_p), bits.nbytes))
        else:
            ts = [FB.castStore(_td(g), "bf16") for g in gs]
        sc = [FB.scatterSlice(t, (rows, 3 * d), [0, i * d], [rows, (i + 1) * d]) for i, t in enumerate(ts)]
        acc = FB.clone(sc[2])
        for i in (1, 0):
            FB.addInplace(acc, sc[i])
        for t in sc + ts:
            FB.releaseGpuTensor(t)
        return acc
    import ctypes as C
    from alpha2_amd import _ffi as ffi
    res = FB.castStore(_td(_bf16(rs.randn(rows, d))), "bf16")
    outs = {}
    for planes in (False, True):
        n1 = FB.planeProducts
        if not planes:                                # (three separate allocations may happen to lie equally far apart: then they ARE planes)
            FB._scatter_planes = lambda t: None
        else:
            del FB._scatter_planes
        g = summed(planes)
        dx = FB.matmul(g, W)
        dw = FB.matmulTransposedA(g, X)
        other = FB.matmulTransposedA(FB.castStore(_td(gs[0]), "bf16"), X)               # a second queued product: the launch is grouped
        dxv, dwv, ov = dx.data.reshape(rows, d).copy(), dw.data.reshape(3 * d, d).copy(), other.data.copy()
        assert FB.planeProducts - n1 == (1 if planes else 0)
        assert (id(g._buf) in FB._scatters) == planes                                    # with planes the sum is still unwritten
        with_res = FB.add(res, FB.matmul(g, W)).data.reshape(rows, d).copy()            # an epilogue wants the operand whole
        gv = g.data.reshape(rows, 3 * d).copy()
        outs[planes] = (dxv, dwv, ov, with_res, gv)
        for t in (g, dx, dw, other):
            FB.releaseGpuTensor(t)
        assert not FB._scatters
    _close(outs[True][0], outs[False][0], "dX from planes", 4e-3)
    _close(outs[True][3], outs[False][3], "dX + residual", 4e-3)
    assert np.array_equal(outs[True][4], np.concatenate(gs, axis=1)) and np.array_equal(outs[False][4], outs[True][4])
    assert np.array_equal(outs[True][2], outs[False][2])
    _close(outs[True][1], outs[False][1], "dW from planes", 1e-6)
    _close(outs[True][1], np.concatenate(gs, axis=1).astype(np.float64).T @ x.astype(np.float64), "dW", 1e-5)
    _close(outs[True][0], _bf16(np.concatenate(gs, axis=1).astype(np.float64) @ w.astype(np.float64)), "dX", 4e-3)


def test_the_transposes_around_the_slabs_become_strides_of_the_attention_kernels(FB):
    """gpt.ts:247-254 reshapes flashAttention's [B H, T, D] result to [B, H, T, D] and transposes (1, 2); its backward transposes the
    incoming gradient the other way and hands it to flashAttentionBackward.  Held back, neither transpose runs: the forward kernel
    writes [B, T, H, D] through its output strides and the backward kernels read O and dO in that layout.  Bit for bit what the
    calls give when every result is read at once (which launches each op on its own), and the slab-shaped result is still right
    when somebody reads it afterwards."""
    rs = np.random.RandomState(23)
    Bt, H, T, D = 3, 4, 96, 32
    q, k, v = (_bf16(rs.randn(Bt * H, T, D)) for _ in range(3))
    g = _bf16(rs.randn(Bt, T, H, D))
    scale, cap = 1 / math.sqrt(D), 30.0

    def run(eager: bool):
        Q, K, V, G = (FB.castStore(_td(x), "bf16") for x in (q, k, v, g))
        r = FB.flashAttention(Q, K, V, T, scale, cap)
        O, lse = r["output"], r["lse"]
        if eager:
            O.data
        O4 = FB.reshape(O, (Bt, H, T, D))
        Ot = FB.transpose(O4, 1, 2)
        fwd = Ot.data.reshape(Bt, T, H, D).copy()
        gT = FB.transpose(G, 1, 2)
        if eager:
            gT.data
        g3 = FB.reshape(gT, (Bt * H, T, D))
        d = FB.flashAttentionBackward(Q, K, V, O, g3, lse, T, scale, cap)
        grads = [d[n].data.copy() for n in ("dQ", "dK", "dV")]
        lazy_left = len(FB._lazy)
        slab = O.data.reshape(Bt * H, T, D).copy()
        lsev = lse.data.copy()
        for t in (O, O4, lse, Ot, gT, g3, Q, K, V, G, d["dQ"], d["dK"], d["dV"]):
            FB.releaseGpuTensor(t)
        return fwd, grads, slab, lsev, lazy_left
    e, l = run(True), run(False)
    assert e[4] == 0 and l[4] == 2                               # lazily: O stands for its transposed twin, the gradient's transpose was never written
    assert not FB._lazy
    assert np.array_equal(e[0], l[0]) and np.array_equal(e[2], l[2]) and np.array_equal(e[3], l[3])
    assert np.array_equal(l[0], l[2].reshape(Bt, H, T, D).transpose(0, 2, 1, 3))
    for a, b in zip(e[1], l[1]):
        assert np.array_equal(a, b)
    # a result nobody transposes is launched as it is when it is read; one nobody reads is never launched
    Q, K, V = (FB.castStore(_td(x), "bf16") for x in (q, k, v))
    r = FB.flashAttention(Q, K, V, T, scale, cap)
    assert np.array_equal(r["output"].data.reshape(Bt * H, T, D), e[2]) and not FB._lazy
    r = FB.flashAttention(Q, K, V, T, scale, cap)
    FB.releaseGpuTensor(r["output"])
    assert np.array_equal(r["lse"].data, e[3])                   # (its other result is still wanted)
    r = FB.flashAttention(Q, K, V, T, scale, cap)
    FB.releaseGpuTensor(r["output"]), FB.releaseGpuTensor(r["lse"])
    assert not FB._lazy and FB._pending_flash is None


def test_cross_entropy_is_held_until_its_backward_is_asked_for(FB):
    """crossEntropy followed by crossEntropyBackward on the same bf16 logits (the tape's last entry, visited first by its
    backward pass) is one pass over the logits: loss, LSE and gradient bit-identical to the two-kernel route; a loss that is
    read first, and one that is released unread, take the plain forward (or nothing)."""
    rs = np.random.RandomState(17)
    N, V = 96, 512
    logits = _bf16(rs.randn(N, V) * 2)
    targets = rs.randint(0, V, N).astype(np.int32)
    lf = logits.astype(np.float64)
    m = lf.max(1, keepdims=True)
    lse = (m + np.log(np.exp(lf - m).sum(1, keepdims=True)))[:, 0]
    want_loss = float(np.mean(lse - lf[np.arange(N), targets]))
    p = np.exp(lf - lse[:, None])
    p[np.arange(N), targets] -= 1
    want_grad = p / N * 0.5

    from alpha2_amd import TensorData

    def operands():
        return FB.castStore(_td(logits), "bf16"), TensorData(targets.shape, "i32", targets), _td(np.float32(0.5).reshape(()))

    # fused: nothing is launched by crossEntropy itself
    lg, tg, g = operands()
    loss = FB.crossEntropy(lg, tg)
    assert FB._held_ce is not None
    grad = FB.crossEntropyBackward(lg, tg, g)
    assert FB._held_ce is None
    fused_loss, fused_grad = float(loss.data[0]), grad.data.copy()
    assert abs(fused_loss - want_loss) <= 1e-5 * abs(want_loss)
    assert np.all(np.abs(fused_grad.reshape(N, V) - want_grad) <= 2.0 ** -8 * np.abs(want_grad) + 1e-9)      # a bf16 result

    # the loss read first: forward alone, then the backward kernel; same bits
    lg, tg, g = operands()
    loss = FB.crossEntropy(lg, tg)
    plain_loss = float(loss.data[0])
    assert FB._held_ce is None
    plain_grad = FB.crossEntropyBackward(lg, tg, g).data.copy()
    assert plain_loss == fused_loss and np.array_equal(plain_grad, fused_grad)

    # released unread
    lg, tg, g = operands()
    loss = FB.crossEntropy(lg, tg)
    FB.releaseGpuTensor(loss)
    FB.flush()
    assert FB._held_ce is None


@pytest.mark.parametrize("cfg", [
    dict(vocabSize=7, blockSize=1, nLayer=1, nEmbd=8, nHead=1),                              # one token per row, a vocabulary of 7
    dict(vocabSize=33, blockSize=3, nLayer=2, nEmbd=12, nHead=3),                            # head size 4, nothing a multiple of 8
    dict(vocabSize=96, blockSize=5, nLayer=1, nEmbd=64, nHead=2),                            # 5 or 15 tokens: the weight gradients contract over them
    dict(vocabSize=50, blockSize=17, nLayer=1, nEmbd=32, nHead=1, ffnActivation="swiglu"),
    # the reference's own attention wiring at shapes the plane products do not take (fewer than 256 rows; C not a multiple of 128):
    # sliceQkv and the scattered sum move the data, the transposes around the slabs are still the attention kernels' strides
    dict(vocabSize=96, blockSize=16, nLayer=2, nEmbd=64, nHead=2, attention="reference-flash"),
    dict(vocabSize=64, blockSize=96, nLayer=1, nEmbd=192, nHead=8, attention="reference-flash"),       # (3 x 96 = 288 rows, C = 192, head size 24)
])
@pytest.mark.parametrize("batch,accum", [(1, 1), (3, 2)])
def test_shapes_the_bf16_kernels_do_not_take_run_in_f32_behind_the_interface(FB, cfg, batch, accum):
    """A caller of the interface picks any model shape: products whose contraction length is not a multiple of 8 (the bf16
    kernels load 16 bytes at a time) run through the f32 kernels instead of being refused, head sizes without a flash
    kernel through the unfused chain; two steps track the oracle as every other shape does."""
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig, Trainer, syntheticBatch
    tr = Trainer(FB, ModelConfig(**cfg), TrainConfig(iters=4, gradAccumSteps=accum), seed=2)
    orc = rm.Trainer(rm.ModelConfig(**cfg), rm.TrainConfig(iters=4, gradAccumSteps=accum), seed=2)
    for s in range(2):
        bs = [syntheticBatch(9 + 2 * s + m, batch, cfg["blockSize"], cfg["vocabSize"]) for m in range(accum)]
        ob = [rm.synthetic_batch(9 + 2 * s + m, batch, cfg["blockSize"], cfg["vocabSize"]) for m in range(accum)]
        r, o = tr.step(bs), orc.step(ob)
        assert abs(r.loss - o.loss) <= 2e-2 * abs(o.loss), (s, r.loss, o.loss)
        assert abs(r.gradNorm - o.gradNorm) <= 1e-1 * o.gradNorm, (s, r.gradNorm, o.gradNorm)


def test_a_product_added_into_a_gradient_is_still_its_tensors_value_when_that_is_kept(FB):
    """addInplace(acc, product) makes a queued weight gradient accumulate into `acc` and skips the product's own tensor, which
    the tape releases at once (tape.ts:116-127).  A caller that keeps it must find the product in it all the same, and the sum
    in `acc`."""
    rs = np.random.RandomState(12)
    g, x, a0 = rs.randn(64, 32) * 0.3, rs.randn(64, 48) * 0.5, rs.randn(32, 48)
    want = _bf16(g).astype(np.float64).T @ _bf16(x).astype(np.float64)
    acc = FB.scale(_td(a0), 1.0)
    out = FB.matmulTransposedA(_td(g), _td(x))
    FB.addInplace(acc, out)                                      # `out` is not released
    kept = FB.matmulTransposedA(_td(g), _td(x))                  # a second one, released as the tape does
    FB.addInplace(acc, kept)
    FB.releaseGpuTensor(kept)
    _close(out.data, want, "the product whose tensor was kept", tol=1e-3)
    _close(acc.data, a0 + 2 * want, "the sum", tol=1e-3)


def test_random_op_programs_give_what_eager_execution_gives(FB):
    """Random programs over a pool of [16, 16] tensors - products of all three kinds, gelu and its backward, sums, in-place
    sums and scalings, copy-on-write clones, releases, reads and norms in any order - on the fast backend (held products,
    queued gradients, shared buffers) against the same programs on the eager f32 backend.  A slip of the lazy machinery (a
    stale buffer, a sum made twice, a product never computed) is a difference of the size of the values; bf16 storage a few
    percent of it."""
    from alpha2_amd import HipBackend, TensorData
    HB, N = HipBackend(0), 16
    kinds = ["mmT", "mm", "mmTA", "gelu", "geluB", "add", "addI", "scale", "scaleI", "clone", "release", "read", "ssq", "relu"]
    probs = [.14, .08, .08, .08, .05, .1, .08, .04, .04, .09, .07, .09, .03, .03]

    def run(Bk, init, ops):
        pool, reads = [TensorData((N, N), "f32", v.copy()) for v in init], []
        for kind, i, j, sc in ops:
            a, b = pool[i % len(pool)], pool[j % len(pool)]
            if kind == "mmT": pool.append(Bk.matmulTransposed(a, b))
            elif kind == "mm": pool.append(Bk.matmul(a, b))
            elif kind == "mmTA": pool.append(Bk.matmulTransposedA(a, b))
            elif kind == "gelu": pool.append(Bk.gelu(a))
            elif kind == "geluB": pool.append(Bk.geluBackward(a, b))
            elif kind == "relu": pool.append(Bk.relu(a))
            elif kind == "add": pool.append(Bk.add(a, b))
            elif kind == "addI" and a is not b: Bk.addInplace(a, b)
            elif kind == "scale": pool.append(Bk.scale(a, sc))
            elif kind == "scaleI": Bk.scaleInplace(a, sc * 0.7)
            elif kind == "clone": pool.append(Bk.clone(a))
            elif kind == "release" and len(pool) > 2: Bk.releaseGpuTensor(pool.pop(i % len(pool)))
            elif kind == "read": reads.append(np.array(a.data, dtype=np.float32).reshape(-1).copy())
            elif kind == "ssq": reads.append(np.array(Bk.totalSumOfSquares([a, b] if a is not b else [a]).data, dtype=np.float32).reshape(-1).copy())
        reads += [np.array(t.data, dtype=np.float32).reshape(-1).copy() for t in pool]
        Bk.syncGpu()
        return reads
    for seed in range(120):
        rs = np.random.RandomState(seed)
        init = [rs.randn(N, N).astype(np.float32) * 0.25 for _ in range(4)]
        ops = [(str(rs.choice(kinds, p=probs)), int(rs.randint(0, 1 << 30)), int(rs.randint(0, 1 << 30)), float(rs.uniform(0.5, 1.5))) for _ in range(60)]
        for k, (got, want) in enumerate(zip(run(FB, init, ops), run(HB, init, ops))):
            fin = np.isfinite(want)
            size = float(np.abs(want[fin]).max()) if fin.any() else 1.0
            assert got.shape == want.shape and float(np.abs(got[fin] - want[fin]).max(initial=0)) <= 0.1 * size + 1e-3, (seed, k, size)
