"""Pins the CPU oracle's ops: (1) the reference's own known answers (tests/golden/
reference_known_answers.json, transcribed from packages/tests/src/*.test.ts), (2) PyTorch-CPU float64
library routines on random inputs, (3) closed forms.  No GPU."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import ref
from oracle import ref_model as rm

B = ref.CpuRef()
rs = np.random.RandomState(1234)


def t64(td):
    return torch.tensor(td.data.astype(np.float64)).reshape(td.shape)


def close(a, b, tol=2e-7):
    """f32 outputs of f64 math: agree with the f64 library value to f32 rounding."""
    a = np.asarray(a, dtype=np.float64).reshape(-1)
    b = np.asarray(b, dtype=np.float64).reshape(-1)
    assert a.shape == b.shape
    assert np.all(np.abs(a - b) <= tol * (1 + np.abs(b))), float(np.max(np.abs(a - b)))


# ---- (1) reference known answers ---------------------------------------------------------------

def test_known_tensor(golden):
    g = golden["tensor.test.ts"]
    c = g["matmul_2x2"]
    assert [round(float(v)) for v in B.matmul(B.fromArray(c["a"], c["shape"]), B.fromArray(c["b"], c["shape"])).data] == c["expect"]
    c = g["softmax_row"]
    assert abs(float(B.softmax(B.fromArray(c["x"], c["shape"]), -1).data.sum()) - 1.0) < 1e-5
    c = g["gelu"]
    out = B.gelu(B.fromArray(c["x"], [3])).data
    assert abs(out[0]) < 5e-4 and abs(out[1] - c["expect1"]) < 5e-3
    c = g["embedding"]
    out = B.embedding(B.fromArray(c["weight"], c["wshape"]), B.fromArray(c["indices"], [2], "i32"))
    assert out.shape == (2, 2) and np.allclose(out.data, c["expect"], atol=5e-3)
    c = g["layerNorm"]
    out = B.layerNorm(B.fromArray(c["x"], c["shape"]), B.ones([2]), B.zeros([2]), c["eps"]).data
    assert abs(out[0] + out[1]) < 5e-4 and abs(out[2] + out[3]) < 5e-4
    c = g["crossEntropy"]
    loss = B.crossEntropy(B.fromArray(c["logits"], c["shape"]), B.fromArray(c["targets"], [2], "i32"))
    assert loss.data.size == 1 and loss.data[0] < c["less_than"]
    c = g["causalMask"]
    m = B.causalMask(c["size"]).data
    assert all(m[i] == 0 for i in c["zero_at"]) and all(m[i] == -np.inf for i in c["neg_inf_at"])
    c = g["transpose"]
    t = B.transpose(B.fromArray(c["a"], c["shape"]), 0, 1)
    assert list(t.shape) == c["expect_shape"] and [round(float(v)) for v in t.data] == c["expect"]
    c = g["reshape"]
    r = B.reshape(B.fromArray(c["a"], c["shape"]), c["to"])
    assert list(r.shape) == c["to"] and list(r.data) == c["expect"]
    assert B.sum(B.fromArray(g["sum_all"]["a"], [3])).data[0] == g["sum_all"]["expect"]
    c = g["sum_axis0"]
    s = B.sum(B.fromArray(c["a"], c["shape"]), 0)
    assert s.shape == (2,) and [round(float(v)) for v in s.data] == c["expect"]
    c = g["add"]
    assert list(B.add(B.fromArray(c["a"], [3]), B.fromArray(c["b"], [3])).data) == c["expect"]


def _var(data, shape):
    return rm.Variable(B.fromArray(data, shape), True)


def test_known_autograd(golden):
    g = golden["autograd.test.ts"]
    for key, op in (("add_backward", rm.add), ("mul_backward", rm.mul)):
        c = g[key]
        tape = rm.Tape(); ctx = rm.Ctx(tape, B)
        a, b = _var(c["a"], [len(c["a"])]), _var(c["b"], [len(c["b"])])
        tape.backward(rm.sum_(ctx, op(ctx, a, b)), B)
        assert list(a.grad.data) == c["grad_a"]
        if "grad_b" in c:
            assert list(b.grad.data) == c["grad_b"]
    c = g["broadcast_add"]
    tape = rm.Tape(); ctx = rm.Ctx(tape, B)
    a, b = _var(c["a"], c["ashape"]), _var(c["b"], c["bshape"])
    loss = rm.sum_(ctx, rm.add(ctx, a, b))
    tape.backward(loss, B)
    assert abs(loss.data.data[0] - c["loss"]) < 5e-3
    assert list(a.grad.data) == c["grad_a"] and list(b.grad.data) == c["grad_b"]
    c = g["mean_backward"]
    tape = rm.Tape(); ctx = rm.Ctx(tape, B)
    a = _var(c["a"], c["shape"])
    tape.backward(rm.sum_(ctx, rm.mean(ctx, a, 1, True)), B)
    assert np.allclose(a.grad.data, c["grad_each"], atol=5e-6)
    c = g["ce_backward_shape"]
    tape = rm.Tape(); ctx = rm.Ctx(tape, B)
    lg = _var(c["logits"], c["shape"])
    tape.backward(rm.crossEntropy(ctx, lg, B.fromArray(c["targets"], [2], "i32")), B)
    assert list(lg.grad.shape) == c["shape"]


def test_known_broadcast_grads(golden):
    g = golden["memory-leak.test.ts"]
    c = g["reduce_leading"]
    tape = rm.Tape(); ctx = rm.Ctx(tape, B)
    a, b = _var(list(range(24)), c["ashape"]), _var(c["b"], [4])
    tape.backward(rm.sum_(ctx, rm.add(ctx, a, b)), B)
    assert np.allclose(a.grad.data, c["grad_a_each"]) and np.allclose(b.grad.data, c["grad_b_each"])
    for key, op in (("sub_broadcast", rm.sub), ("mul_broadcast", rm.mul)):
        c = g[key]
        tape = rm.Tape(); ctx = rm.Ctx(tape, B)
        a, b = _var(c["a"], c["ashape"]), _var(c["b"], c["bshape"])
        tape.backward(rm.sum_(ctx, op(ctx, a, b)), B)
        assert list(a.grad.data) == c["grad_a"] and list(b.grad.data) == c["grad_b"]
    c = g["div_broadcast"]
    tape = rm.Tape(); ctx = rm.Ctx(tape, B)
    a, b = _var(c["a"], c["ashape"]), _var(c["b"], c["bshape"])
    tape.backward(rm.sum_(ctx, rm.div(ctx, a, b)), B)
    assert np.allclose(a.grad.data, c["grad_a_each"], atol=5e-5)


def test_known_adamw_gradscale(golden):
    c = golden["optimizer.test.ts"]["adamw_gradscale"]

    def run(prescale):
        p = B.fromArray(c["p"], [4])
        g = B.fromArray(c["g"], [4])
        gs = c["gradScale"]
        if prescale:
            g, gs = B.scale(g, gs), 1.0
        v = rm.Variable(p, True); v.grad = g
        opt = rm.AdamW(lr=c["lr"], weightDecay=c["weightDecay"])
        opt.stepParamEntries([("w", v)], gs)
        return p.data
    assert np.max(np.abs(run(False) - run(True))) < c["tol"]


def test_known_check_finite(golden):
    c = golden["gpu-perf.test.ts"]["checkFinite"]
    for case in c["cases"]:
        x = np.array([float(v) for v in case["x"]], dtype=np.float32)
        assert ref.check_finite(ref.f32(x)) == case["expect"]
    big = (np.arange(c["large"]["size"]) * c["large"]["step"]).astype(np.float32)
    assert ref.check_finite(ref.f32(big)) == c["large"]["expect_clean"]
    big[-1] = np.nan
    assert ref.check_finite(ref.f32(big)) == c["large"]["nan_at_last_expect"]


# ---- (2) library routines in float64 ------------------------------------------------------------

@pytest.mark.parametrize("shape", [(33, 19, 47), (64, 64, 64), (5, 1, 7)])
def test_matmul_vs_torch(shape):
    M, K, N = shape
    a, b = ref.f32(rs.randn(M, K)), ref.f32(rs.randn(K, N))
    close(B.matmul(a, b).data, (t64(a) @ t64(b)).numpy())


def test_matmul_batched_broadcast_vs_torch():
    a, b = ref.f32(rs.randn(2, 3, 5, 4)), ref.f32(rs.randn(3, 4, 6))
    out = B.matmul(a, b)
    assert out.shape == (2, 3, 5, 6)
    close(out.data, (t64(a) @ t64(b)).numpy())
    # transposed operand is a different argument order: catches an A/B swap
    a2, b2 = ref.f32(rs.randn(4, 5)), ref.f32(rs.randn(4, 6))
    with pytest.raises(ValueError):
        B.matmul(a2, b2)


def test_binary_broadcast_vs_numpy():
    a, b = ref.f32(rs.randn(2, 1, 4)), ref.f32(rs.randn(3, 1) + 3)
    for name, fn in (("add", np.add), ("sub", np.subtract), ("mul", np.multiply), ("div", np.divide)):
        out = getattr(B, name)(a, b)
        want = fn(a.data.reshape(a.shape).astype(np.float64), b.data.reshape(b.shape).astype(np.float64))
        assert out.shape == want.shape
        close(out.data, want)
    with pytest.raises(ValueError):
        B.add(ref.f32(rs.randn(2, 3)), ref.f32(rs.randn(4)))


def test_unary_vs_torch():
    x = ref.f32(rs.randn(257) * 3)
    xt = t64(x)
    close(B.gelu(x).data, F.gelu(xt, approximate="tanh").numpy())
    close(B.silu(x).data, F.silu(xt).numpy())
    close(B.relu(x).data, F.relu(xt).numpy())
    close(B.exp(x).data, torch.exp(xt).numpy())
    close(B.neg(x).data, (-xt).numpy())
    close(B.scale(x, 0.37).data, (xt * 0.37).numpy())
    close(B.clamp(x, -0.5, 1.25).data, torch.clamp(xt, -0.5, 1.25).numpy())
    xp = ref.f32(np.abs(rs.randn(100)) + 0.1)
    close(B.log(xp).data, torch.log(t64(xp)).numpy())
    close(B.sqrt(xp).data, torch.sqrt(t64(xp)).numpy())
    close(B.pow(xp, 2.5).data, torch.pow(t64(xp), 2.5).numpy())


def test_reductions_vs_torch():
    a = ref.f32(rs.randn(3, 4, 5))
    at = t64(a)
    close(B.sum(a).data, at.sum().numpy())
    close(B.mean(a).data, at.mean().numpy())
    for ax in (0, 1, 2, -1):
        close(B.sum(a, ax).data, at.sum(ax).numpy())
        close(B.mean(a, ax, True).data, at.mean(ax, keepdim=True).numpy(), 3e-7)
        assert B.sum(a, ax, True).shape == tuple(at.sum(ax, keepdim=True).shape)


def test_layernorm_fwd_bwd_vs_torch():
    x, w, b_, g = ref.f32(rs.randn(7, 48) * 2 + 0.5), ref.f32(rs.randn(48)), ref.f32(rs.randn(48)), ref.f32(rs.randn(7, 48))
    xt, wt, bt = t64(x).requires_grad_(), t64(w).requires_grad_(), t64(b_).requires_grad_()
    y = F.layer_norm(xt, (48,), wt, bt, 1e-5)
    close(B.layerNorm(x, w, b_, 1e-5).data, y.detach().numpy(), 5e-7)
    y.backward(t64(g))
    dx, dw, db = ref.layernorm_backward(x, w, g, 1e-5)
    close(dx.data, xt.grad.numpy(), 2e-6)
    close(dw.data, wt.grad.numpy(), 2e-6)
    close(db.data, bt.grad.numpy(), 2e-6)


def test_softmax_logsoftmax_vs_torch():
    a = ref.f32(rs.randn(3, 5, 9) * 4)
    for ax in (0, 1, 2):
        close(B.softmax(a, ax).data, torch.softmax(t64(a), ax).numpy(), 3e-7)
        close(B.logSoftmax(a, ax).data, torch.log_softmax(t64(a), ax).numpy(), 5e-7)


def test_cross_entropy_fwd_bwd_vs_torch():
    N, Cc = 11, 37
    lg, tg = ref.f32(rs.randn(N, Cc) * 3), ref.i32(rs.randint(0, Cc, N))
    lt = t64(lg).requires_grad_()
    loss = F.cross_entropy(lt, torch.tensor(tg.data.astype(np.int64)))
    close(B.crossEntropy(lg, tg).data, loss.detach().numpy(), 5e-7)
    (loss * 0.7).backward()
    close(ref.cross_entropy_backward(lg, tg, 0.7).data, lt.grad.numpy(), 1e-6)
    # closed form: uniform logits -> ln C
    close(B.crossEntropy(ref.f32(np.zeros((N, Cc))), tg).data, [math.log(Cc)], 2e-7)


def test_embedding_fwd_bwd_vs_torch():
    V, D = 13, 6
    w, idx, g = ref.f32(rs.randn(V, D)), ref.i32(rs.randint(0, V, (3, 5))), ref.f32(rs.randn(3, 5, D))
    out = B.embedding(w, idx)
    assert out.shape == (3, 5, D)
    wt = t64(w).requires_grad_()
    y = F.embedding(torch.tensor(idx.data.astype(np.int64)).reshape(3, 5), wt)
    assert np.array_equal(out.data, w.data.reshape(V, D)[idx.data].reshape(-1))   # bit exact gather
    y.backward(t64(g))
    close(ref.embedding_backward(idx, g, V).data, wt.grad.numpy(), 1e-6)


def test_activation_backwards_vs_torch():
    x, g = ref.f32(rs.randn(300) * 2), ref.f32(rs.randn(300))
    for fwd, bwd in ((lambda t: F.gelu(t, approximate="tanh"), lambda: ref.gelu_backward(x, g)),
                     (lambda t: F.gelu(t, approximate="tanh"), lambda: ref.gelu_backward(x, g, fused=True)),
                     (F.silu, lambda: ref.silu_backward(x, g)), (F.relu, lambda: ref.relu_backward(x, g)),
                     (lambda t: torch.clamp(t, -0.7, 0.9), lambda: ref.clamp_backward(x, g, -0.7, 0.9))):
        xt = t64(x).requires_grad_()
        fwd(xt).backward(t64(g))
        close(bwd().data, xt.grad.numpy(), 1e-6)


def test_data_movement_vs_numpy():
    a = ref.f32(rs.randn(2, 3, 4, 5))
    an = a.data.reshape(a.shape)
    for d0, d1 in ((1, 2), (0, 3), (2, 3), (-1, -2)):
        t = B.transpose(a, d0, d1)
        assert np.array_equal(t.data.reshape(t.shape), np.swapaxes(an, d0, d1))
    s = B.slice(a, [0, 1, 1, 2], [2, 3, 3, 5])
    assert np.array_equal(s.data.reshape(s.shape), an[0:2, 1:3, 1:3, 2:5])
    sc = B.scatterSlice(s, a.shape, [0, 1, 1, 2], [2, 3, 3, 5])
    want = np.zeros_like(an); want[0:2, 1:3, 1:3, 2:5] = an[0:2, 1:3, 1:3, 2:5]
    assert np.array_equal(sc.data.reshape(a.shape), want)
    c = B.cat([a, a], 2)
    assert np.array_equal(c.data.reshape(c.shape), np.concatenate([an, an], 2))
    m = B.causalMask(4)
    mf = B.maskedFill(ref.f32(rs.randn(2, 4, 4)), m, -1e9)
    assert np.all(mf.data.reshape(2, 4, 4)[:, np.triu_indices(4, 1)[0], np.triu_indices(4, 1)[1]] == np.float32(-1e9))


def test_argmax_first_index_and_nan():
    a = ref.f32(np.array([[1, 5, 5, 2], [np.nan, 3, 3, -1], [-np.inf, -np.inf, -np.inf, -np.inf]]))
    assert list(B.argmax(a, 1).data) == [1, 1, 0]
    assert int(B.argmax(a).data[0]) == 1
    r = ref.f32(rs.randn(6, 50))
    assert np.array_equal(B.argmax(r, -1).data, np.argmax(r.data.reshape(6, 50), -1).astype(np.int32))
    assert np.array_equal(B.argmax(r, 0).data, np.argmax(r.data.reshape(6, 50), 0).astype(np.int32))


def test_adamw_vs_torch_and_closed_form():
    n = 64
    p0, g = rs.randn(n).astype(np.float32), rs.randn(n).astype(np.float32)
    p = ref.f32(p0)
    m, v = np.zeros(n, np.float32), np.zeros(n, np.float32)
    pt = torch.tensor(p0.astype(np.float64), requires_grad=True)
    opt = torch.optim.AdamW([pt], lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    b1p = b2p = 1.0
    for step in range(3):
        b1p *= 0.9; b2p *= 0.95
        ref.adamw_step(p, ref.f32(g), m, v, 3e-4, 0.9, 0.95, 1e-8, 0.1, 1 - b1p, 1 - b2p, 0.5)
        pt.grad = torch.tensor(g.astype(np.float64) * 0.5)
        opt.step()
        if step == 0:   # closed form at m=v=0
            want = p0 * (1 - 3e-4 * 0.1) - 3e-4 * np.sign(g) * (np.abs(g * 0.5) / (np.abs(g * 0.5) + 1e-8))
            close(p.data, want, 2e-7)
    close(p.data, pt.detach().numpy(), 1e-6)


def test_sum_sq_and_clip_identity():
    a = ref.f32(rs.randn(1000))
    assert abs(ref.sum_sq(a) - float(np.sum(a.data.astype(np.float64) ** 2))) < 1e-9


# ---- DropoutRng.nextMask (packages/autograd/src/ops.ts:41-51,74-81) --------------------------------------------------------
def test_dropout_hash_mixing_rounds_are_murmur3_fmix32():
    """With counter = index = 0 the hash is the published MurmurHash3 32-bit finaliser of the seed; fmix32(0) = 0,
    fmix32(1) = 0x514E28B7 and fmix32(2) = 0x30F4C306 are its known answers.  A mask value is hash / 2^32 > p."""
    from tests.util import py_dropout_hash
    assert [py_dropout_hash(s, 0, 0) for s in (0, 1, 2)] == [0, 0x514E28B7, 0x30F4C306]
    for seed, want in ((0, 0), (1, 0x514E28B7), (2, 0x30F4C306)):
        for p in (0.1, 0.3, 0.9):
            m = ref.dropout_mask(seed, 0, p, 1)
            assert m[0] == (np.float32(1 / (1 - p)) if want / 2 ** 32 > p else 0)


def test_dropout_mask_equals_the_independent_restatement():
    """Every branch of the first line: small sums (exact), negative seeds (ToInt32 of a negative number), sums past 2^32
    (wrap) and index * 2246822519 past 2^53, where the double has already dropped low bits before the |0 (indices above
    ~4.0 M: there the reference's own GPU kernel, which wraps in u32, gives different masks)."""
    from tests.util import py_dropout_mask
    idx = np.concatenate([np.arange(0, 3000), np.arange(4_000_000, 4_003_000), np.arange(4_009_000_000 // 1000, 4_009_000_000 // 1000 + 10),
                          np.arange(2 ** 31 - 2000, 2 ** 31 - 1)])
    for seed, counter, p in ((0, 0, 0.1), (42, 3, 0.1), (-7, 11, 0.5), (2 ** 31 - 1, 2 ** 21, 0.25), (42 + 17 * 1000 + 1, 5, 0.1)):
        n = int(idx.max()) + 1
        got = np.empty(len(idx), np.float32)
        # the C oracle fills [0, n); evaluate it in windows around the probed indices instead of 2^31 elements
        for lo, hi in ((0, 3000), (4_000_000, 4_003_000), (4_009_000, 4_009_010), (2 ** 31 - 2000, 2 ** 31 - 1)):
            sel = (idx >= lo) & (idx < hi)
            got[sel] = ref.dropout_mask_range(seed, counter, p, lo, hi)
        assert np.array_equal(got, py_dropout_mask(seed, counter, p, idx)), (seed, counter, p)
    m = ref.dropout_mask(42, 0, 0.1, 200_000)
    assert set(np.unique(m)) == {np.float32(0), np.float32(1 / 0.9)}
    assert abs((m == 0).mean() - 0.1) < 0.005                    # drop rate p
    assert not np.array_equal(m, ref.dropout_mask(42, 1, 0.1, 200_000))       # the counter changes the mask


def test_dropout_hash_differs_from_u32_wrapping_beyond_2_to_53():
    """Documents the reference's CPU/GPU divergence: the u32-wrapping kernel (packages/helios/src/kernels/nn.ts:5600-5748)
    equals the CPU hash while index * 2246822519 < 2^53 and not beyond."""
    from tests.util import py_dropout_hash

    def wrap(seed, counter, i):
        h = (seed + counter * 2654435761 + i * 2246822519) & 0xFFFFFFFF
        h = ((h ^ (h >> 16)) * 0x85EBCA6B) & 0xFFFFFFFF
        h = ((h ^ (h >> 13)) * 0xC2B2AE35) & 0xFFFFFFFF
        return h ^ (h >> 16)
    limit = 2 ** 53 // 2246822519
    assert all(py_dropout_hash(42, 3, i) == wrap(42, 3, i) for i in list(range(2000)) + list(range(limit - 2000, limit - 8)))
    assert sum(py_dropout_hash(42, 3, i) != wrap(42, 3, i) for i in range(limit + 10, limit + 2010)) > 500


def test_sum_and_mean_over_an_empty_axis():
    """cpu_ref.ts:272-308: one output per combination of the other dimensions, each the sum of no terms; mean divides it by
    the axis length, 0 / 0 (cpu_ref.ts:325-330)."""
    z = ref.f32(np.zeros((3, 0), np.float32))
    s = B.sum(z, 1)
    assert s.shape == (3,) and np.array_equal(s.data[:3], np.zeros(3, np.float32))
    m = B.mean(z, 1)
    assert m.shape == (3,) and np.all(np.isnan(m.data[:3]))
    s0 = B.sum(ref.f32(np.zeros((0, 8), np.float32)), 0)
    assert s0.shape == (8,) and np.array_equal(s0.data[:8], np.zeros(8, np.float32))
    assert np.isnan(B.mean(ref.f32(np.zeros((0,), np.float32))).data[0])


def test_embedding_with_ids_outside_the_table():
    """cpu_ref.ts:364-385 reads weight[id * dim + d] from a typed array: undefined past either end, stored as NaN; the backward
    loop's store past the end is dropped (ops.ts:491-507).  No access outside the arrays on this side either."""
    w = np.arange(12, dtype=np.float32).reshape(3, 4)
    ids = np.array([2, 3, -1, 0], np.int32)
    out = B.embedding(ref.f32(w), ref.i32(ids)).data.reshape(4, 4)
    assert np.array_equal(out[[0, 3]], w[[2, 0]]) and np.isnan(out[[1, 2]]).all()
    g = np.ones((4, 4), np.float32)
    gw = ref.embedding_backward(ref.i32(ids), ref.f32(g), 3).data.reshape(3, 4)
    assert np.array_equal(gw, np.array([[1] * 4, [0] * 4, [1] * 4], np.float32))
