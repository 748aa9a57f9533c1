"""Per-op parity of the HIP kernels (called through the C ABI via HipBackend) against the CPU oracle on the same
seeded inputs.  Bar: bit-exact for integer / index / pure data-movement results; rel 1e-4 (tests/util.py) for fp32."""
import math

import numpy as np
import pytest

from oracle import ref
from oracle import ref_model as rm
from tests.util import assert_close

pytestmark = pytest.mark.gpu

O = ref.CpuRef()


@pytest.fixture(scope="module")
def B():
    from alpha2_amd import HipBackend
    return HipBackend(0)


def dev(B, arr, dtype="f32"):
    from alpha2_amd import TensorData
    arr = np.asarray(arr)
    return TensorData(arr.shape, dtype, arr)


def orc(arr):
    arr = np.asarray(arr)
    return ref.f32(arr) if arr.dtype != np.int32 else ref.i32(arr)


rs = np.random.RandomState(7)


def test_reference_known_answers_on_device(B, golden):
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
    assert list(B.zeros([2, 3]).data) == [0] * 6 and list(B.ones([3]).data) == [1, 1, 1]
    cf = golden["gpu-perf.test.ts"]["checkFinite"]
    for case in cf["cases"]:
        x = np.array([float(v) for v in case["x"]], dtype=np.float32)
        assert B.checkFinite(dev(B, x)).data[0] == case["expect"]
    big = (np.arange(cf["large"]["size"]) * cf["large"]["step"]).astype(np.float32)
    assert B.checkFinite(dev(B, big)).data[0] == 0.0
    big[-1] = np.nan
    assert B.checkFinite(dev(B, big)).data[0] == 1.0
    la = golden["gpu-perf.test.ts"]["loss_accum"]
    acc = None
    for v in la["losses"]:
        s = B.scale(B.fromArray([v], [1]), 1 / la["accumSteps"])
        acc = s if acc is None else B.add(acc, s)
    assert abs(acc.data[0] - sum(la["losses"]) / la["accumSteps"]) < 5e-5
    nan = B.add(B.scale(B.fromArray([float("nan")], [1]), 0.25), B.fromArray([0.5], [1]))
    assert math.isnan(nan.data[0])


@pytest.mark.parametrize("n", [1, 5, 1024, 100003])
def test_elementwise_vs_oracle(B, n):
    x = (rs.randn(n) * 2).astype(np.float32)
    y = (rs.randn(n) + 3).astype(np.float32)
    for name in ("add", "sub", "mul", "div"):
        assert_close(getattr(B, name)(dev(B, x), dev(B, y)).data, getattr(O, name)(orc(x), orc(y)).data, what=name)
    for name in ("neg", "exp", "gelu", "relu", "silu"):
        assert_close(getattr(B, name)(dev(B, x)).data, getattr(O, name)(orc(x)).data, what=name)
    xp = np.abs(x) + 0.1
    for name in ("log", "sqrt"):
        assert_close(getattr(B, name)(dev(B, xp)).data, getattr(O, name)(orc(xp)).data, what=name)
    assert_close(B.pow(dev(B, xp), 2.5).data, O.pow(orc(xp), 2.5).data, what="pow")
    assert_close(B.scale(dev(B, x), -0.37).data, O.scale(orc(x), -0.37).data, what="scale")
    assert np.array_equal(B.clamp(dev(B, x), -0.5, 1.25).data, O.clamp(orc(x), -0.5, 1.25).data)
    g = rs.randn(n).astype(np.float32)
    assert_close(B.geluBackward(dev(B, x), dev(B, g)).data, ref.gelu_backward(orc(x), orc(g), fused=True).data, what="geluBackward")
    assert_close(B.siluBackward(dev(B, x), dev(B, g)).data, ref.silu_backward(orc(x), orc(g)).data, what="siluBackward")
    assert np.array_equal(B.reluBackward(dev(B, x), dev(B, g)).data, ref.relu_backward(orc(x), orc(g)).data)
    assert np.array_equal(B.clampBackward(dev(B, x), dev(B, g), -0.7, 0.9).data, ref.clamp_backward(orc(x), orc(g), -0.7, 0.9).data)
    # softCap: tanh(x/cap)*cap against the oracle's composed exp form (ops.ts:329-340)
    tape = rm.Tape(); ctx = rm.Ctx(tape, O)
    xv = rm.Variable(orc(x * 20), True)
    sc = rm.softCap(ctx, xv, 30.0)
    assert_close(B.softCap(dev(B, x * 20), 30.0).data, sc.data.data, what="softCap")
    tape.backward(sc, O, orc(g))
    assert_close(B.softCapBackward(dev(B, g), dev(B, x * 20), 30.0).data, xv.grad.data, what="softCapBackward")
    a, b = dev(B, x), dev(B, y)
    B.addInplace(a, b)
    assert_close(a.data, O.add(orc(x), orc(y)).data, what="addInplace")
    B.scaleInplace(a, 0.5)
    assert_close(a.data, O.scale(O.add(orc(x), orc(y)), 0.5).data, what="scaleInplace")
    sm = B.siluMul(dev(B, x), dev(B, y))
    assert_close(sm.data, O.mul(O.silu(orc(x)), orc(y)).data, what="siluMul")
    da, db = B.siluMulBackward(dev(B, x), dev(B, y), dev(B, g))
    assert_close(da.data, ref.silu_backward(orc(x), O.mul(orc(g), orc(y))).data, what="siluMulBackward.da")
    assert_close(db.data, O.mul(orc(g), O.silu(orc(x))).data, what="siluMulBackward.db")
    assert_close(B.residualDropoutAdd(dev(B, x), dev(B, y), dev(B, g)).data, O.add(orc(x), O.mul(orc(y), orc(g))).data, what="rda")


def test_dropout_mask_equals_the_cpu_path_for_every_index(B):
    """Backend.dropoutMask against DropoutRng.nextMask of the reference's CPU path (packages/autograd/src/ops.ts:41-51,74-81),
    bit for bit, over 6 M elements: past index 4 008 862 the product index * 2246822519 exceeds 2^53 and the double has lost
    low bits before the cut to 32 bits, which the kernel reproduces (the reference's own GPU kernel does not)."""
    n = 6_000_000
    for seed, counter, p in ((42, 0, 0.1), (-7, 11, 0.5), (2 ** 31 - 1, 2 ** 21, 0.25), (42 + 3 * 1000 + 1, 2, 0.1)):
        got = B.dropoutMask([n], seed, counter, p).data
        want = ref.dropout_mask(seed, counter, p, n)
        assert np.array_equal(got, want), (seed, counter, p, int((got != want).sum()))
    from tests.util import py_dropout_mask
    idx = list(range(0, 50)) + list(range(4_008_800, 4_008_900)) + list(range(n - 50, n))
    assert np.array_equal(B.dropoutMask([n], 42, 0, 0.1).data[idx], py_dropout_mask(42, 0, 0.1, idx))
    assert B.dropoutMask([0], 1, 0, 0.1).data.size == 0
    with pytest.raises(Exception):
        B.dropoutMask([4], 1, 0, 1.0)


@pytest.mark.parametrize("n", [1, 7, 4096, 1_000_003])
def test_dropout_applied_from_a_seed_in_device_memory_equals_mask_then_multiply_add(B, n):
    """ah_dropout_apply against the reference's own sequence (ops.ts:616-686: dropoutMask, then residual + projected * mask, and
    grad * mask in backward) with DropoutRng's CPU-path mask: f32 in and out exactly; bf16 operands to the one rounding of the
    result; a new seed written to the same device word gives the other mask without anything else changing."""
    import ctypes as C
    from alpha2_amd import _ffi as ffi
    lib = B.lib
    r = np.random.RandomState(n % 1000)
    x, res = r.randn(n).astype(np.float32), r.randn(n).astype(np.float32)
    bits = lambda a: (lambda u: ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16))(a.view(np.uint32).astype(np.uint64))
    widen = lambda h: (h.astype(np.uint32) << 16).view(np.float32)
    live = []

    def up(a):
        p = C.c_uint64()
        ffi.check(lib.ah_alloc(max(a.nbytes, 16), C.byref(p)))
        ffi.check(lib.ah_upload(p.value, a.ctypes.data_as(C.c_void_p), a.nbytes))
        live.append(p.value)
        return p.value

    def down(ptr, dtype):
        out = np.empty(n, dtype)
        ffi.check(lib.ah_download(out.ctypes.data_as(C.c_void_p), ptr, out.nbytes))
        return out
    seed_dev = up(np.array([0], np.int32))
    xf, rf, xb, rb = up(x), up(res), up(bits(x)), up(bits(res))
    of, ob = up(np.zeros(n, np.float32)), up(np.zeros(n, np.uint16))
    for seed, counter, p in ((42, 0, 0.1), (-7 + 3 * 1000 + 1, 5, 0.5)):
        ffi.check(lib.ah_upload(seed_dev, np.array([seed], np.int32).ctypes.data_as(C.c_void_p), 4))
        mask = ref.dropout_mask(seed, counter, p, n)
        ffi.check(lib.ah_dropout_apply(xf, ffi.F32, rf, of, ffi.F32, n, seed_dev, counter, p))
        assert np.array_equal(down(of, np.float32), res + x * mask)
        ffi.check(lib.ah_dropout_apply(xf, ffi.F32, 0, of, ffi.F32, n, seed_dev, counter, p))                  # backward: no residual
        assert np.array_equal(down(of, np.float32), x * mask)
        ffi.check(lib.ah_dropout_apply(xb, ffi.BF16, rb, ob, ffi.BF16, n, seed_dev, counter, p))
        assert np.array_equal(down(ob, np.uint16), bits(widen(bits(res)) + widen(bits(x)) * mask))
        ffi.check(lib.ah_dropout_apply(xb, ffi.BF16, rf, of, ffi.F32, n, seed_dev, counter, p))
        assert np.array_equal(down(of, np.float32), res + widen(bits(x)) * mask)
        ffi.check(lib.ah_dropout_apply(xf, ffi.F32, 0, ob, ffi.BF16, n, seed_dev, counter, p))
        assert np.array_equal(down(ob, np.uint16), bits(x * mask))
        if n > 8:                                                   # operands that are not 16-byte aligned take the one-at-a-time path
            ffi.check(lib.ah_dropout_apply(xb + 2, ffi.BF16, rb + 2, ob + 2, ffi.BF16, n - 1, seed_dev, counter, p))
            assert np.array_equal(down(ob, np.uint16)[1:], bits(widen(bits(res))[1:] + widen(bits(x))[1:] * mask[:-1]))
    assert lib.ah_dropout_apply(xf, ffi.F32, 0, of, ffi.F32, n, seed_dev, 0, 1.0) == 2
    assert lib.ah_dropout_apply(xf, ffi.F32, 0, of, ffi.F32, n, 0, 0, 0.5) == 2
    for p_ in live:
        lib.ah_free(p_)


@pytest.mark.parametrize("rows,cols", [(1, 4), (37, 24), (130, 260), (1000, 512)])
def test_channel_activation_mixtures_match_the_composed_ops(B, rows, cols):
    """channelAct / channelActBackward (one pass) against the oracle running the chain of ops the reference records for its
    universal and kan_spline activations (gpt.ts:295-321): values, dx and every coefficient gradient."""
    x = (rs.randn(rows, cols) * 2).astype(np.float32)
    g = rs.randn(rows, cols).astype(np.float32)
    cases = {"universal": ("silu", "identity"), "kan_spline": ("silu", "relu", "gelu", "identity", "square"), "one basis": ("gelu",)}
    for label, names in cases.items():
        co = {n: (rs.randn(1, cols) * 0.7).astype(np.float32) for n in names}
        tape = rm.Tape(); ctx = rm.Ctx(tape, O)
        xv = rm.Variable(orc(x), True)
        cv = {n: rm.Variable(orc(c), True) for n, c in co.items()}
        basis = {"silu": lambda: rm.silu(ctx, xv), "relu": lambda: rm.relu(ctx, xv), "gelu": lambda: rm.gelu(ctx, xv), "identity": lambda: xv,
                 "square": lambda: rm.mul(ctx, xv, xv)}
        out = None
        for n in names:
            term = rm.mul(ctx, basis[n](), cv[n])
            out = term if out is None else rm.add(ctx, out, term)
        tape.backward(out, O, orc(g))
        cod = {n: dev(B, c) for n, c in co.items()}
        assert_close(B.channelAct(dev(B, x), cod).data, out.data.data, what=label)
        dx, dco = B.channelActBackward(dev(B, x), cod, dev(B, g))
        assert_close(dx.data, xv.grad.data, what=label + ".dx")
        for n in names:
            assert dco[n].shape == (1, cols)
            assert_close(dco[n].data, cv[n].grad.data, what=f"{label}.d{n}", scale=float(np.sqrt(rows)))
    with pytest.raises(ValueError):
        B.channelAct(dev(B, x), {"silu": dev(B, np.ones((1, cols + 4), np.float32))})


def _raw_buf(B, arr, bf16):
    """Device copy of `arr` as f32 or as raw bf16 bits; returns (TensorData that owns it, handle)."""
    from alpha2_amd import TensorData
    t = TensorData(arr.shape, "f16", _bf16_round(arr)[1]) if bf16 else TensorData(arr.shape, "f32", np.ascontiguousarray(arr, np.float32))
    return t, B._ptr(t)


def _raw_read(B, t, bf16):
    B._dirty(t)
    raw = t.data
    return ((raw.astype(np.uint32) << 16).view(np.float32) if bf16 else raw).reshape(t.shape)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("rows,cols", [(3, 8), (130, 260), (517, 384)])
def test_plain_and_bf16_channel_activations_and_accumulated_coefficient_gradients(B, bf16, rows, cols):
    """ah_channel_act / ah_channel_act_bwd through the C ABI: a selected basis without a coefficient vector is the plain
    activation (silu, relu, gelu against the oracle's element-wise ops and their backward, cpu_ref.ts:422-435, ops.ts:284-417);
    bf16 operands give the f32 result of the bf16-rounded inputs, rounded once; `accumulate` adds the coefficient gradients to
    what the vectors hold."""
    import ctypes as C
    from alpha2_amd import _ffi as ffi
    dt = ffi.BF16 if bf16 else ffi.F32
    rnd = (lambda a: _bf16_round(a)[0]) if bf16 else (lambda a: a)
    x, g = rnd((rs.randn(rows, cols) * 2).astype(np.float32)), rnd(rs.randn(rows, cols).astype(np.float32))
    tol = 2.0 ** -8 if bf16 else 2e-5
    tx, px = _raw_buf(B, x, bf16)
    tg, pg = _raw_buf(B, g, bf16)
    for k, name in ((0, "silu"), (1, "relu"), (2, "gelu")):
        tape = rm.Tape(); ctx = rm.Ctx(tape, O)
        xv = rm.Variable(orc(x), True)
        out = getattr(rm, name)(ctx, xv)
        tape.backward(out, O, orc(g))
        to, po = _raw_buf(B, np.zeros((rows, cols), np.float32), bf16)
        td, pd = _raw_buf(B, np.zeros((rows, cols), np.float32), bf16)
        ffi.check(B.lib.ah_channel_act(dt, px, None, 1 << k, po, rows, cols))
        ffi.check(B.lib.ah_channel_act_bwd(dt, px, None, 1 << k, pg, pd, None, 0, rows, cols))
        got, gdx = _raw_read(B, to, bf16), _raw_read(B, td, bf16)
        assert np.max(np.abs(got - out.data.data.reshape(rows, cols)) / (np.abs(out.data.data.reshape(rows, cols)) + 1e-2)) <= tol, name
        assert np.max(np.abs(gdx - xv.grad.data.reshape(rows, cols)) / (np.abs(xv.grad.data.reshape(rows, cols)) + 1e-2)) <= tol, name
    # a mixture with coefficients: the second call accumulates, so the coefficient gradients double while dx stays
    co = {0: (rs.randn(cols) * 0.7).astype(np.float32), 3: (rs.randn(cols) * 0.7).astype(np.float32)}
    arr, darr, keep = (C.c_uint64 * 5)(), (C.c_uint64 * 5)(), []
    for k, v in co.items():
        t, ptr = _raw_buf(B, v, False); keep.append(t); arr[k] = ptr
        t, ptr = _raw_buf(B, np.zeros(cols, np.float32), False); keep.append(t); darr[k] = ptr
    td, pd = _raw_buf(B, np.zeros((rows, cols), np.float32), bf16)
    ffi.check(B.lib.ah_channel_act_bwd(dt, px, arr, 0b01001, pg, pd, darr, 0, rows, cols))
    first = {k: _raw_read(B, keep[2 * i + 1], False).copy() for i, k in enumerate(co)}
    dx1 = _raw_read(B, td, bf16).copy()
    ffi.check(B.lib.ah_channel_act_bwd(dt, px, arr, 0b01001, pg, pd, darr, 1, rows, cols))
    sig = 1.0 / (1.0 + np.exp(-x.astype(np.float64)))
    want = {0: (g * x * sig).sum(0), 3: (g.astype(np.float64) * x).sum(0)}
    for i, k in enumerate(co):
        second = _raw_read(B, keep[2 * i + 1], False)
        assert np.allclose(first[k], want[k], rtol=1e-4, atol=1e-4 * np.sqrt(rows)), k
        assert np.allclose(second, 2 * first[k], rtol=1e-6, atol=1e-6), k
    assert np.array_equal(dx1, _raw_read(B, td, bf16))


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("rows,cols", [(1, 4), (37, 24), (513, 384)])
def test_swiglu_on_the_packed_pre_activation(B, bf16, rows, cols):
    """ah_swiglu / ah_swiglu_bwd on [gate | up] rows against the oracle's siluMul and its backward on the two halves
    (gpt.ts:295-299)."""
    from alpha2_amd import _ffi as ffi
    dt = ffi.BF16 if bf16 else ffi.F32
    rnd = (lambda a: _bf16_round(a)[0]) if bf16 else (lambda a: a)
    gu, g = rnd((rs.randn(rows, 2 * cols) * 2).astype(np.float32)), rnd(rs.randn(rows, cols).astype(np.float32))
    tol = 2.0 ** -8 if bf16 else 2e-5
    tape = rm.Tape(); ctx = rm.Ctx(tape, O)
    a, b = rm.Variable(orc(np.ascontiguousarray(gu[:, :cols])), True), rm.Variable(orc(np.ascontiguousarray(gu[:, cols:])), True)
    out = rm.siluMul(ctx, a, b)
    tape.backward(out, O, orc(g))
    tgu, pgu = _raw_buf(B, gu, bf16)
    tg, pg = _raw_buf(B, g, bf16)
    to, po = _raw_buf(B, np.zeros((rows, cols), np.float32), bf16)
    td, pd = _raw_buf(B, np.zeros((rows, 2 * cols), np.float32), bf16)
    ffi.check(B.lib.ah_swiglu(dt, pgu, po, rows, cols))
    ffi.check(B.lib.ah_swiglu_bwd(dt, pgu, pg, pd, rows, cols))
    got, d = _raw_read(B, to, bf16), _raw_read(B, td, bf16)
    close = lambda x, w: np.max(np.abs(x - w) / (np.abs(w) + 1e-2)) <= tol
    assert close(got, out.data.data.reshape(rows, cols))
    assert close(d[:, :cols], a.grad.data.reshape(rows, cols)) and close(d[:, cols:], b.grad.data.reshape(rows, cols))


def test_fill_at_every_alignment_touches_exactly_its_range(B):
    """ah_fill_f32 / ah_fill_i32 write 16 bytes at a time over the aligned middle of the range: every start offset modulo 16
    bytes and ragged lengths, with sentinels either side."""
    import ctypes
    from alpha2_amd import _ffi as ffi
    total = 4096
    for off in range(0, 5):
        for n in (0, 1, 2, 3, 4, 5, 7, 8, 63, 64, 65, 1000, 4000):
            host = np.full(total, -7.0, np.float32)
            buf = dev(B, host)
            ffi.check(B.lib.ah_fill_f32(B._ptr(buf) + 4 * off, 2.5, n))
            B._dirty(buf)
            got = buf.data
            want = host.copy(); want[off:off + n] = 2.5
            assert np.array_equal(got, want), (off, n)
    ib = dev(B, np.full(100, 9, np.int32), "i32")
    ffi.check(B.lib.ah_fill_i32(B._ptr(ib) + 4, -3, 50))
    B._dirty(ib)
    want = np.full(100, 9, np.int32); want[1:51] = -3
    assert np.array_equal(ib.data, want)
    big = B.full([1 << 20], 1.25)
    assert np.all(big.data == 1.25)


def test_empty_tensors(B):
    e = dev(B, np.zeros((0, 4), np.float32))
    assert B.add(e, e).data.size == 0 and B.gelu(e).data.size == 0
    assert B.sum(dev(B, np.zeros((0,), np.float32))).data[0] == 0.0


def test_empty_extents_give_what_the_cpu_path_gives(B):
    """Tensors with an extent of zero through the ops of the step: the shapes and values of the reference's CPU loops
    (an empty sum is 0, an empty mean 0 / 0 = NaN, a product over an empty k is all zeros), no launch of an empty grid."""
    z = lambda *shape: np.zeros(shape, np.float32)
    cases = {
        "matmul, no rows": lambda X, t: X.matmul(t(z(0, 5)), t(np.ones((5, 3), np.float32))),
        "matmul, empty k": lambda X, t: X.matmul(t(z(4, 0)), t(z(0, 3))),
        "matmul, no columns": lambda X, t: X.matmul(t(np.ones((4, 5), np.float32)), t(z(5, 0))),
        "transpose": lambda X, t: X.transpose(t(z(0, 3)), 0, 1),
        "layerNorm": lambda X, t: X.layerNorm(t(z(0, 8)), t(np.ones(8, np.float32)), t(z(8)), 1e-5),
        "softmax": lambda X, t: X.softmax(t(z(0, 8))),
        "sum over an empty axis": lambda X, t: X.sum(t(z(3, 0)), 1),
        "sum along an axis of an empty tensor": lambda X, t: X.sum(t(z(0, 8)), 0),
        "mean over an empty axis": lambda X, t: X.mean(t(z(3, 0)), 1),
        "mean of nothing": lambda X, t: X.mean(t(z(0))),
        "scale": lambda X, t: X.scale(t(z(0, 2)), 2.0),
        "argmax": lambda X, t: X.argmax(t(z(0, 4)), -1),
        "slice to nothing": lambda X, t: X.slice(t(np.ones((4, 4), np.float32)), [0, 2], [4, 2]),
    }
    for name, fn in cases.items():
        got, want = fn(B, lambda a: dev(B, a)), fn(O, orc)
        assert tuple(got.shape) == tuple(want.shape), (name, got.shape, want.shape)
        assert np.array_equal(np.asarray(got.data).reshape(-1)[:shape_size_of(want)], np.asarray(want.data).reshape(-1)[:shape_size_of(want)], equal_nan=True), (name, got.data, want.data)
    emb = B.embedding(dev(B, np.ones((5, 4), np.float32)), dev(B, np.zeros((0,), np.int32), "i32"))
    assert tuple(emb.shape) == (0, 4) and emb.data.size == 0
    assert float(B.totalSumOfSquares([]).data[0]) == 0.0 and float(B.sumOfSquares(dev(B, z(0))).data[0]) == 0.0
    # the loss over no rows is a mean of nothing (cpu_ref.ts:543-563), its gradient has no entries
    no_rows, no_targets = dev(B, z(0, 8)), dev(B, np.zeros(0, np.int32), "i32")
    assert np.isnan(B.crossEntropy(no_rows, no_targets).data).all() and np.isnan(O.crossEntropy(orc(z(0, 8)), orc(np.zeros(0, np.int32))).data).all()
    assert tuple(B.crossEntropyBackward(no_rows, no_targets, dev(B, np.ones((), np.float32))).shape) == (0, 8)


def shape_size_of(t):
    n = 1
    for d in t.shape:
        n *= d
    return n


def test_broadcast_binary_and_errors(B):
    a, b = rs.randn(2, 1, 4).astype(np.float32), (rs.randn(3, 1) + 3).astype(np.float32)
    for name in ("add", "sub", "mul", "div"):
        got, want = getattr(B, name)(dev(B, a), dev(B, b)), getattr(O, name)(orc(a), orc(b))
        assert got.shape == want.shape
        assert_close(got.data, want.data, what=name)
    with pytest.raises(ValueError):
        B.add(dev(B, rs.randn(2, 3).astype(np.float32)), dev(B, rs.randn(4).astype(np.float32)))
    # [BT,F] * [1,F] -- the per-channel gate of the universal / kan_spline activations
    h, gate = rs.randn(37, 24).astype(np.float32), rs.randn(1, 24).astype(np.float32)
    assert_close(B.mul(dev(B, h), dev(B, gate)).data, O.mul(orc(h), orc(gate)).data)
    t = B.broadcast(dev(B, gate), (5, 24))
    assert np.array_equal(t.data.reshape(5, 24), np.broadcast_to(gate, (5, 24)))


def test_reductions_vs_oracle(B):
    a = rs.randn(3, 40, 5).astype(np.float32)
    assert_close(B.sum(dev(B, a)).data, O.sum(orc(a)).data)
    assert_close(B.mean(dev(B, a)).data, O.mean(orc(a)).data)
    for ax in (0, 1, 2, -1):
        for keep in (False, True):
            got, want = B.sum(dev(B, a), ax, keep), O.sum(orc(a), ax, keep)
            assert got.shape == want.shape
            assert_close(got.data, want.data, what=f"sum{ax}")
            assert_close(B.mean(dev(B, a), ax, keep).data, O.mean(orc(a), ax, keep).data, what=f"mean{ax}")
    big = rs.randn(1_000_003).astype(np.float32)
    assert_close(B.sum(dev(B, big)).data, O.sum(orc(big)).data, rel=1e-5)
    wide = rs.randn(5000, 3).astype(np.float32)        # many short strided lines
    assert_close(B.sum(dev(B, wide), 0).data, O.sum(orc(wide), 0).data)
    assert_close(B.sumOfSquares(dev(B, big)).data, [ref.sum_sq(orc(big))], rel=1e-6)
    parts = [rs.randn(n).astype(np.float32) for n in (1, 7, 4096, 33333)]
    assert_close(B.totalSumOfSquares([dev(B, p) for p in parts]).data, [sum(ref.sum_sq(orc(p)) for p in parts)], rel=1e-6)
    # one launch for a whole gradient set: more tensors than one launch's table holds, an empty one, tensors of several chunks,
    # a view that is not 16-byte aligned; the same call twice gives the same bits (fixed partition, fixed order)
    sizes = [0, 1, 7, 65536, 65537, 200001, 3] + [int(rs.randint(1, 3000)) for _ in range(260)] + [1 << 20]
    parts = [rs.randn(n).astype(np.float32) for n in sizes]
    devs = [dev(B, p) for p in parts]
    odd = dev(B, rs.randn(1001).astype(np.float32))
    devs.append(B.slice(odd, [1], [1000]))
    want = sum(float(np.sum(p.astype(np.float64) ** 2)) for p in parts) + float(np.sum(odd.data[1:1000].astype(np.float64) ** 2))
    got = B.totalSumOfSquares(devs).data
    assert abs(float(got[0]) - want) <= 1e-6 * want
    assert np.array_equal(got, B.totalSumOfSquares(devs).data)
    assert float(B.totalSumOfSquares([]).data[0]) == 0.0


def test_softmax_family_vs_oracle(B):
    a = (rs.randn(3, 5, 300) * 4).astype(np.float32)
    for ax in (0, 1, 2):
        assert_close(B.softmax(dev(B, a), ax).data, O.softmax(orc(a), ax).data, what=f"softmax{ax}")
        assert_close(B.logSoftmax(dev(B, a), ax).data, O.logSoftmax(orc(a), ax).data, what=f"logSoftmax{ax}")
    s = O.softmax(orc(a), -1)
    g = rs.randn(*a.shape).astype(np.float32)
    tape = rm.Tape(); ctx = rm.Ctx(tape, O)
    av = rm.Variable(orc(a), True)
    tape.backward(rm.softmax(ctx, av, -1), O, orc(g))
    assert_close(B.softmaxBackward(dev(B, s.data.reshape(a.shape)), dev(B, g)).data, av.grad.data, what="softmaxBackward")


def test_argmax_bit_exact(B):
    a = np.array([[1, 5, 5, 2], [np.nan, 3, 3, -1], [-np.inf, -np.inf, -np.inf, -np.inf]], dtype=np.float32)
    assert list(B.argmax(dev(B, a), 1).data) == list(O.argmax(orc(a), 1).data) == [1, 1, 0]
    assert int(B.argmax(dev(B, a)).data[0]) == int(O.argmax(orc(a)).data[0])
    r = np.round(rs.randn(64, 50304) * 3, 1).astype(np.float32)       # rounded: many exact ties per row
    assert np.array_equal(B.argmax(dev(B, r), -1).data, O.argmax(orc(r), -1).data)
    r2 = np.round(rs.randn(70, 9, 33) * 2, 1).astype(np.float32)
    for ax in (0, 1, 2):
        got = B.argmax(dev(B, r2), ax)
        assert got.dtype == "i32" and np.array_equal(got.data, O.argmax(orc(r2), ax).data)


def test_data_movement_bit_exact(B):
    a = rs.randn(2, 3, 4, 5).astype(np.float32)
    for d0, d1 in ((1, 2), (0, 3), (2, 3), (-1, -2), (0, 1)):
        got, want = B.transpose(dev(B, a), d0, d1), O.transpose(orc(a), d0, d1)
        assert got.shape == want.shape and np.array_equal(got.data, want.data)
    big = rs.randn(3, 70, 130).astype(np.float32)
    assert np.array_equal(B.transpose(dev(B, big), 1, 2).data, O.transpose(orc(big), 1, 2).data)
    s = B.slice(dev(B, a), [0, 1, 1, 2], [2, 3, 3, 5])
    assert np.array_equal(s.data, O.slice(orc(a), [0, 1, 1, 2], [2, 3, 3, 5]).data)
    sc = B.scatterSlice(s, a.shape, [0, 1, 1, 2], [2, 3, 3, 5])
    assert np.array_equal(sc.data, O.scatterSlice(O.slice(orc(a), [0, 1, 1, 2], [2, 3, 3, 5]), a.shape, [0, 1, 1, 2], [2, 3, 3, 5]).data)
    c = B.cat([dev(B, a), dev(B, a[:, :, :2])], 2)
    assert np.array_equal(c.data, O.cat([orc(a), orc(a[:, :, :2])], 2).data)
    with pytest.raises(ValueError):
        B.cat([dev(B, a), dev(B, a[:, :2])], 2)
    qkv = rs.randn(9, 24).astype(np.float32)
    q, k, v = B.sliceQkv(dev(B, qkv))
    assert np.array_equal(q.data.reshape(9, 8), qkv[:, :8]) and np.array_equal(v.data.reshape(9, 8), qkv[:, 16:])
    r = B.reshape(dev(B, a), (6, 20))
    assert r.shape == (6, 20) and np.array_equal(r.data, a.reshape(-1))
    with pytest.raises(ValueError):
        B.reshape(dev(B, a), (7, 20))
    m = B.causalMask(5)
    assert np.array_equal(m.data, O.causalMask(5).data)
    x = rs.randn(2, 3, 5, 5).astype(np.float32)
    assert np.array_equal(B.maskedFill(dev(B, x), m, -1e9).data, O.maskedFill(orc(x), O.causalMask(5), -1e9).data)
    cl = B.clone(dev(B, a))
    assert np.array_equal(cl.data, a.reshape(-1))
    h = B.castDtype(dev(B, a), "f16")
    assert h.dtype == "f16" and np.array_equal(h.data.view(np.float16), a.reshape(-1).astype(np.float16))
    assert_close(B.castDtype(h, "f32").data, a.reshape(-1).astype(np.float16).astype(np.float32), rel=0)


def test_embedding_fwd_bwd(B):
    V, D = 257, 48
    w = rs.randn(V, D).astype(np.float32)
    idx = rs.randint(0, V, (4, 33)).astype(np.int32)
    idx[0, :8] = 5                          # collisions
    g = rs.randn(4, 33, D).astype(np.float32)
    out = B.embedding(dev(B, w), dev(B, idx, "i32"))
    assert out.shape == (4, 33, D) and np.array_equal(out.data, O.embedding(orc(w), orc(idx)).data)   # gather is bit exact
    gw = B.embeddingBackward(dev(B, idx, "i32"), dev(B, g), V)
    assert_close(gw.data, ref.embedding_backward(orc(idx), orc(g), V).data, what="embeddingBackward")


@pytest.mark.parametrize("n,dim,V", [(1000, 768, 300), (16384, 768, 50304), (131, 1000, 7), (513, 2052, 40), (300, 50, 9)])
def test_embedding_backward_with_heavily_repeated_ids(B, n, dim, V):
    """Power-law ids (the most frequent one takes a large share of the positions, as token ids do), positions that do not
    fill the last block, rows that do not fill the last column group, ids out of range (skipped), and accumulation onto an
    existing gradient; against a float64 scatter-add."""
    from alpha2_amd import _ffi as ffi
    r = np.random.RandomState(n + dim)
    idx = np.minimum((V * r.rand(n) ** 4).astype(np.int64), V - 1).astype(np.int32)
    idx[::97] = -3
    idx[5::89] = V + 2
    g = r.randn(n, dim).astype(np.float32)
    ok = (idx >= 0) & (idx < V)
    want = np.zeros((V, dim), np.float64)
    np.add.at(want, idx[ok], g[ok].astype(np.float64))
    di, dg = dev(B, idx, "i32"), dev(B, g)
    gw = B.zeros((V, dim))
    for k in (1, 2):                                       # the second call accumulates
        ffi.check(B.lib.ah_embedding_bwd(B._ptr(di), B._ptr(dg), B._ptr(gw), n, dim, V, 0 if k == 1 else 1))
        B._dirty(gw)
        assert_close(gw.data.reshape(V, dim), k * want, what=f"scatter-add x{k}")


def test_embedding_backward_is_the_same_from_run_to_run_and_follows_position_order(B):
    """16384 power-law token ids over 50304 rows of 768: the summation order is a function of the ids alone, so repeated
    calls are bit-identical; and an id whose positions all fall into one chunk of 32 sorted positions (every id with up to
    two positions at least... here: every id that occurs at most 8 times and does not straddle a chunk border is checked
    through the closed form below) is summed in position order, f32 add by f32 add, exactly as the reference's loop does
    (packages/autograd/src/ops.ts:491-507)."""
    from alpha2_amd import _ffi as ffi
    n, dim, V = 16384, 768, 50304
    r = np.random.RandomState(11)
    idx = np.minimum((V * r.rand(n) ** 6).astype(np.int64), V - 1).astype(np.int32)
    g = (r.randn(n, dim) * np.exp(r.randn(n, 1) * 3)).astype(np.float32)          # rows of very different size: order matters
    di, dg = dev(B, idx, "i32"), dev(B, g)
    outs = []
    for _ in range(3):
        gw = B.zeros((V, dim))
        ffi.check(B.lib.ah_embedding_bwd(B._ptr(di), B._ptr(dg), B._ptr(gw), n, dim, V, 0))
        B._dirty(gw)
        outs.append(gw.data.reshape(V, dim).copy())
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])
    # position-order f32 sums for the ids whose positions are neighbours in the sorted order AND inside one chunk of 32
    order = np.lexsort((np.arange(n), idx))
    sid = idx[order]
    exact = 0
    for c in range(0, n, 32):
        ids_c = sid[c:c + 32]
        for v in np.unique(ids_c):
            if (c > 0 and sid[c - 1] == v) or (c + 32 < n and sid[c + 32] == v):
                continue                                        # crosses a chunk border: summed as parts
            acc = np.zeros(dim, np.float32)
            for p in order[c:c + 32][ids_c == v]:
                acc = acc + g[p]
            assert np.array_equal(outs[0][v], acc), v
            exact += 1
    assert exact > 3000
    want = np.zeros((V, dim), np.float64)
    np.add.at(want, idx, g.astype(np.float64))
    assert_close(outs[0], want, what="scatter-add")



@pytest.mark.parametrize("n,vocab", [(1, 7), (700, 50304), (1024, 300), (5000, 50304), (16384, 50304), (16384, 3), (20000, 65534), (32768, 50304)])
def test_embedding_index_is_the_stable_order_by_id(B, n, vocab):
    """ah_embedding_index: keys (id << 16 | position) of the valid positions in ascending order -- positions of one id in position
    order, the order ops.ts:491-507 adds them in -- then padding.  Both sort kernels (radix up to 16384 positions, bitonic beyond),
    power-law ids, ids out of range."""
    from alpha2_amd import _ffi as ffi
    lib = B.lib
    ids = (rs.zipf(1.3, size=n) % vocab).astype(np.int32)
    ids[rs.rand(n) < 0.01] = -1
    ids[rs.rand(n) < 0.01] = vocab
    nbytes = lib.ah_embedding_index_bytes(n, vocab)
    assert nbytes >= 4 * n
    tok = dev(B, ids, "i32")
    out = dev(B, np.zeros(nbytes // 4, np.int32), "i32")
    ffi.check(lib.ah_embedding_index(B._ptr(tok), n, vocab, B._ptr(out)))
    B._dirty(out)
    got = out.data.view(np.uint32)
    valid = np.nonzero((ids >= 0) & (ids < vocab))[0]
    order = valid[np.argsort(ids[valid], kind="stable")]
    want = np.full(nbytes // 4, 0xFFFFFFFF, np.uint32)
    want[:len(order)] = (ids[order].astype(np.uint32) << 16) | order.astype(np.uint32)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("rows,dim", [(1, 2), (7, 48), (1024, 128), (333, 768), (5, 1000), (3, 4096)])
def test_layernorm_fwd_bwd(B, rows, dim):
    x = (rs.randn(rows, dim) * 2 + 0.5).astype(np.float32)
    w, b_, g = rs.randn(dim).astype(np.float32), rs.randn(dim).astype(np.float32), rs.randn(rows, dim).astype(np.float32)
    assert_close(B.layerNorm(dev(B, x), dev(B, w), dev(B, b_), 1e-5).data, O.layerNorm(orc(x), orc(w), orc(b_), 1e-5).data, what="ln")
    r = B.layerNormBackward(dev(B, x), dev(B, w), dev(B, g), 1e-5)
    dx, dw, db = ref.layernorm_backward(orc(x), orc(w), orc(g), 1e-5)
    term = float(np.max(np.abs(g * w)) / np.sqrt(np.min(x.var(-1)) + 1e-5))      # size of the terms dx is a difference of
    assert_close(r["dx"].data, dx.data, what="ln.dx", scale=term if dim < 8 else 0.0)
    assert_close(r["dw"].data, dw.data, what="ln.dw")
    assert_close(r["db"].data, db.data, what="ln.db")


@pytest.mark.parametrize("rows,dim", [(3, 8), (130, 260), (333, 768), (64, 2048), (4096, 1024)])
def test_layernorm_on_a_bf16_residual_stream(B, rows, dim):
    """x, the residual gradient and dx in bf16 (ah_layernorm with x_dtype = bf16, ah_layernorm_bwd_deferred with stream_dtype = bf16;
    cpu_ref.ts:387-420, ops.ts:509-571): the f32 arithmetic of the oracle on the bf16-rounded inputs, results rounded once.  The
    f32 copy of dx is written only where asked for.  tok + pos embedding straight to bf16 as well."""
    import ctypes as C
    from alpha2_amd import _ffi as ffi
    lib = B.lib
    x = _bf16_round((rs.randn(rows, dim) * 2 + 0.5).astype(np.float32))[0]
    g, res = _bf16_round(rs.randn(rows, dim).astype(np.float32))[0], _bf16_round(rs.randn(rows, dim).astype(np.float32))[0]
    w, b_ = rs.randn(dim).astype(np.float32), rs.randn(dim).astype(np.float32)
    tx, px = _raw_buf(B, x, True); tg, pg = _raw_buf(B, g, True); tr, pr = _raw_buf(B, res, True)
    wd, bd = dev(B, w), dev(B, b_)
    to, po = _raw_buf(B, np.zeros((rows, dim), np.float32), True)
    ffi.check(lib.ah_layernorm(px, B._ptr(wd), B._ptr(bd), po, rows, dim, 1e-5, ffi.BF16, ffi.BF16))
    want = O.layerNorm(orc(x), orc(w), orc(b_), 1e-5).data.reshape(rows, dim)
    assert_close(_raw_read(B, to, True), want, rel=2.0 ** -8, what="ln16")
    assert lib.ah_layernorm(px, B._ptr(wd), B._ptr(bd), po, rows, dim, 1e-5, ffi.F32, ffi.BF16) != 0          # bf16 in, f32 out: not provided
    dx, dw, db = ref.layernorm_backward(orc(x), orc(w), orc(g), 1e-5)
    want_dx = dx.data.reshape(rows, dim) + res
    nbytes = lib.ah_layernorm_bwd_partials_bytes(rows, dim)
    part = B.zeros((nbytes // 4,))
    td, pd = _raw_buf(B, np.zeros((rows, dim), np.float32), True)
    df = B.zeros((rows, dim))
    dwd, dbd = B.zeros((dim,)), B.zeros((dim,))
    for f32_copy in (0, B._ptr(df)):
        ffi.check(lib.ah_layernorm_bwd_deferred(px, B._ptr(wd), pg, ffi.BF16, pr, f32_copy, pd, B._ptr(part), rows, dim, 1e-5, ffi.BF16))
        term = float(np.max(np.abs(g * w)) / np.sqrt(np.min(x.var(-1)) + 1e-5))
        assert_close(_raw_read(B, td, True), want_dx, rel=2.0 ** -8, what="ln16.dx", scale=term if dim < 16 else 0.0)
    B._dirty(df)
    assert_close(df.data, want_dx, what="ln16.dx f32 copy", scale=term if dim < 16 else 0.0)
    jobs = (ffi.AhColsumJob * 1)(ffi.AhColsumJob(B._ptr(part), B._ptr(dwd), B._ptr(dbd), rows, dim, 0, 0))
    ffi.check(lib.ah_layernorm_colsums(jobs, 1))
    B._dirty(dwd); B._dirty(dbd)
    assert_close(dwd.data, dw.data, what="ln16.dw")
    assert_close(dbd.data, db.data, what="ln16.db")
    # a bf16 stream with f32 gradients is refused
    assert lib.ah_layernorm_bwd_deferred(px, B._ptr(wd), B._ptr(df), ffi.F32, pr, 0, pd, B._ptr(part), rows, dim, 1e-5, ffi.BF16) != 0
    # tok + pos embedding written as bf16
    V, T = 50, 7
    n = (rows // T) * T
    if n:
        wte, wpe = rs.randn(V, dim).astype(np.float32), rs.randn(T, dim).astype(np.float32)
        tok = rs.randint(0, V, size=n).astype(np.int32)
        te, pe = _raw_buf(B, np.zeros((n, dim), np.float32), True)
        wted, wped, tokd = dev(B, wte), dev(B, wpe), dev(B, tok, "i32")
        ffi.check(lib.ah_embedding_tok_pos(B._ptr(wted), B._ptr(wped), B._ptr(tokd), pe, n, T, dim, V, ffi.BF16))
        assert np.array_equal(_raw_read(B, te, True), _bf16_round(wte[tok] + wpe[np.arange(n) % T])[0])


def test_layernorm_backward_with_column_sums_put_off(B):
    """ah_layernorm_bwd_deferred + one ah_layernorm_colsums over several LayerNorms of different sizes gives exactly the dx,
    dw and db of ah_layernorm_bwd, also when accumulating onto existing dw / db; bad jobs are reported."""
    import ctypes as C
    from alpha2_amd import _ffi as ffi
    lib = B.lib
    cases = [(16384, 768), (333, 768), (7, 48), (5, 1000), (1, 2), (4096, 1024)]
    keep, jobs, wants = [], [], []
    for rows, dim in cases:
        x, w, g = (rs.randn(rows, dim) * 2 + 0.5).astype(np.float32), rs.randn(dim).astype(np.float32), rs.randn(rows, dim).astype(np.float32)
        dx_, dw_, db_ = B.zeros((rows, dim)), dev(B, np.full(dim, 3.0, np.float32)), dev(B, np.full(dim, -2.0, np.float32))
        dx2, dw2, db2 = B.zeros((rows, dim)), dev(B, np.full(dim, 3.0, np.float32)), dev(B, np.full(dim, -2.0, np.float32))
        xd, wd, gd = dev(B, x), dev(B, w), dev(B, g)
        nbytes = lib.ah_layernorm_bwd_partials_bytes(rows, dim)
        assert nbytes >= 8 * dim
        part = B.zeros((nbytes // 4,))
        keep += [xd, wd, gd, dx_, dw_, db_, dx2, dw2, db2, part]
        ffi.check(lib.ah_layernorm_bwd(B._ptr(xd), B._ptr(wd), B._ptr(gd), ffi.F32, 0, B._ptr(dx_), 0, B._ptr(dw_), B._ptr(db_), rows, dim, 1e-5, 1, ffi.F32))
        ffi.check(lib.ah_layernorm_bwd_deferred(B._ptr(xd), B._ptr(wd), B._ptr(gd), ffi.F32, 0, B._ptr(dx2), 0, B._ptr(part), rows, dim, 1e-5, ffi.F32))
        jobs.append(ffi.AhColsumJob(B._ptr(part), B._ptr(dw2), B._ptr(db2), rows, dim, 1, 0))
        wants.append((dx_, dw_, db_, dx2, dw2, db2))
    arr = (ffi.AhColsumJob * len(jobs))(*jobs)
    ffi.check(lib.ah_layernorm_colsums(arr, len(jobs)))
    for (rows, dim), ts in zip(cases, wants):
        for t in ts:
            B._dirty(t)
        assert np.array_equal(ts[0].data, ts[3].data), (rows, dim, "dx")
        assert np.array_equal(ts[1].data, ts[4].data), (rows, dim, "dw")
        assert np.array_equal(ts[2].data, ts[5].data), (rows, dim, "db")
        assert not np.array_equal(ts[1].data, np.full(dim, 3.0, np.float32))
    assert lib.ah_layernorm_colsums(arr, 0) == 0
    bad = (ffi.AhColsumJob * 1)(ffi.AhColsumJob(0, 1 << 20, 1 << 20, 4, 4, 0, 0))
    assert lib.ah_layernorm_colsums(bad, 1) != 0 and b"null operand" in lib.ah_last_error()
    assert lib.ah_layernorm_bwd_deferred(1 << 20, 1 << 20, 1 << 20, ffi.F32, 0, 1 << 20, 0, 0, 4, 4, 1e-5, ffi.F32) != 0 and b"null operand" in lib.ah_last_error()


@pytest.mark.parametrize("n,c", [(2, 3), (11, 37), (128, 256), (16, 50304)])
def test_cross_entropy_fwd_bwd(B, n, c):
    lg = (rs.randn(n, c) * 3).astype(np.float32)
    tg = rs.randint(0, c, n).astype(np.int32)
    lgd, tgd = dev(B, lg), dev(B, tg, "i32")
    loss = B.crossEntropy(lgd, tgd)
    assert loss.shape == ()
    assert_close(loss.data, O.crossEntropy(orc(lg), orc(tg)).data, what="ce")
    gs = dev(B, np.array([0.7], np.float32))
    assert_close(B.crossEntropyBackward(lgd, tgd, gs).data, ref.cross_entropy_backward(orc(lg), orc(tg), 0.7).data, what="ce.bwd")
    fresh = dev(B, lg)                      # backward without a preceding forward on the same object
    assert_close(B.crossEntropyBackward(fresh, tgd, gs).data, ref.cross_entropy_backward(orc(lg), orc(tg), 0.7).data, what="ce.bwd2")


@pytest.mark.parametrize("n,c,dtype", [(7, 8, "bf16"), (33, 2056, "bf16"), (12, 50304, "bf16"), (5, 51200, "bf16"), (3, 51208, "bf16"), (9, 100, "bf16"),
                                       (11, 37, "f32")])
def test_cross_entropy_one_pass_equals_forward_then_backward(B, n, c, dtype):
    """ah_cross_entropy_fwd_bwd keeps a bf16 row in registers between the two halves (rows of up to 51200 classes, a multiple
    of 8) and otherwise runs the two kernels: loss, lse and dlogits are bit-identical to the pair either way, also in
    place and with an out-of-range target; the values are checked against the oracle on the logits as stored."""
    from alpha2_amd import _ffi as ffi
    code = ffi.DTYPE_CODE[dtype]
    lg = (rs.randn(n, c) * 3).astype(np.float32)
    logits = lambda: B.castStore(dev(B, lg), dtype)
    seen = np.array(logits().data, dtype=np.float32).reshape(n, c)

    def run(entry, tg, inplace=False):
        src, tgd = logits(), dev(B, tg, "i32")
        loss, lse = B._new(()), B._new((n,))
        dl = src if inplace else B._new((n, c), "f32", dtype)
        if entry == "pair":
            ffi.check(B.lib.ah_cross_entropy(B._ptr(src), code, B._ptr(tgd), B._ptr(loss), B._ptr(lse), n, c))
            ffi.check(B.lib.ah_cross_entropy_bwd(B._ptr(src), code, B._ptr(tgd), B._ptr(lse), 0, 0.7, B._ptr(dl), n, c))
        else:
            ffi.check(B.lib.ah_cross_entropy_fwd_bwd(B._ptr(src), code, B._ptr(tgd), B._ptr(loss), B._ptr(lse), 0, 0.7, B._ptr(dl), n, c))
        B._dirty(dl)
        return [np.array(t.data).copy() for t in (loss, lse, dl)]

    tg = rs.randint(0, c, n).astype(np.int32)
    tg[-1] = c - 1
    bad = tg.copy()
    bad[0] = -1
    for targets in (tg, bad):
        want = run("pair", targets)
        for inplace in (False, True):
            for got, exp, what in zip(run("one", targets, inplace), want, ("loss", "lse", "dlogits")):
                assert np.array_equal(got, exp), (what, inplace)
    loss, _, dl = run("one", tg)
    half = 2.0 ** -8 if dtype == "bf16" else 0.0               # rounding of the stored gradient
    assert_close(loss, O.crossEntropy(orc(seen), orc(tg)).data, what="ce")
    wantg = ref.cross_entropy_backward(orc(seen), orc(tg), 0.7).data
    assert np.all(np.abs(dl - wantg) <= np.abs(wantg) * (half + 1e-4) + 1e-9), "ce.dlogits"


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("scale", [1e3, 1e5, 1e30])
def test_cross_entropy_with_logits_far_from_zero(B, dtype, scale):
    """The reference takes exp(x - max) of the difference (cpu_ref.ts:493-563), so the loss of a row does not depend on
    where the row sits: logits of the size of 1e3, 1e5 or 1e30 (rows with a clear winner, with ties, and rows shifted as a
    whole) must give the oracle's loss.  (An exponent formed as x log2(e) - max log2(e) in one fused multiply-add is off by
    |max| 2^-24: visible from 1e5, infinite at 1e30.)  The gradient is checked to 1e-4 where an f32 log-sum-exp, which is
    what the backward kernels are handed, still resolves it: rows up to 1e3 (half an ulp of 1e3 is 3e-5); at 1e5 to 2 % of a
    row's mass; at 1e30, where log(sum) vanishes beside the maximum in f32 (the reference keeps the two apart in f64), only
    that it is finite."""
    from alpha2_amd import _ffi as ffi
    code = ffi.DTYPE_CODE[dtype]
    n, c = 6, 64
    base = rs.randn(n, c).astype(np.float32)
    lg = base.copy()
    lg[0] *= scale                                   # spread over the whole range: one clear winner
    lg[1] = scale + base[1]                          # a row shifted as a whole
    lg[2] = -scale + 3 * base[2]
    lg[3] = 0.0; lg[3, 5] = scale; lg[3, 9] = scale   # a tie at the top
    lg[4] = scale * np.sign(base[4])                 # half the row at +scale, half at -scale
    lg[5] = base[5]                                  # an ordinary row beside them
    tg = np.array([int(np.argmax(lg[0])), 3, 7, 5, int(np.argmin(lg[4])), 1], np.int32)
    src = B.castStore(dev(B, lg), dtype)
    seen = np.array(src.data, dtype=np.float32).reshape(n, c)
    tgd = dev(B, tg, "i32")
    for entry in ("pair", "one"):
        loss, lse, dl = B._new(()), B._new((n,)), B._new((n, c), "f32", dtype)
        if entry == "pair":
            ffi.check(B.lib.ah_cross_entropy(B._ptr(src), code, B._ptr(tgd), B._ptr(loss), B._ptr(lse), n, c))
            ffi.check(B.lib.ah_cross_entropy_bwd(B._ptr(src), code, B._ptr(tgd), B._ptr(lse), 0, 1.0, B._ptr(dl), n, c))
        else:
            ffi.check(B.lib.ah_cross_entropy_fwd_bwd(B._ptr(src), code, B._ptr(tgd), B._ptr(loss), B._ptr(lse), 0, 1.0, B._ptr(dl), n, c))
        B._dirty(dl)
        want = O.crossEntropy(orc(seen), orc(tg)).data
        want = float(np.asarray(want).reshape(-1)[0])
        assert np.isfinite(want) and abs(float(np.asarray(loss.data).reshape(-1)[0]) - want) <= 1e-5 * abs(want) + 1e-6, (entry, loss.data, want)
        wantg = ref.cross_entropy_backward(orc(seen), orc(tg), 1.0).data.reshape(n, c)
        half = 2.0 ** -8 if dtype == "bf16" else 0.0
        got = np.array(dl.data, dtype=np.float32).reshape(n, c)
        if scale <= 1e3:
            assert np.all(np.abs(got - wantg) <= np.abs(wantg) * (half + 1e-4) + 1e-7), (entry, np.abs(got - wantg).max())
        elif scale <= 1e5:
            assert np.all(np.isfinite(got)) and np.all(np.abs(got.sum(axis=1)) <= 2e-2 / n) and np.all(got[np.arange(n), tg] <= 0), entry
            assert np.all(np.abs(got - wantg) <= 2e-2 / n), (entry, np.abs(got - wantg).max())      # probabilities within 2 % of the row's mass
        else:
            assert np.all(np.isfinite(got)), entry


def test_unary_backward_formulas_at_the_ends_of_the_range(B):
    """Where f32 arithmetic and the reference's f64 could part ways: gelu' of huge inputs (x^3 overflows f32 from 7e12 on; the
    derivative is 1 or 0 there, and 0 x inf = NaN at the infinities themselves, ops.ts:401-419), and relu's backward as a
    product with the 0 / 1 mask (ops.ts:280-290: an infinite gradient where the input was not positive is NaN, not 0)."""
    x = np.array([1e13, -1e13, 3.4e38, -3.4e38, 50.0, -50.0, np.inf, -np.inf, np.nan, 0.5], np.float32)
    for gval in (1.0, -2.5, np.inf):
        g = np.full(x.shape, gval, np.float32)
        got, want = B.geluBackward(dev(B, x), dev(B, g)).data, ref.gelu_backward(orc(x), orc(g)).data
        assert np.array_equal(np.isnan(got), np.isnan(want)), (gval, got, want)
        ok = ~np.isnan(want)
        assert np.allclose(got[ok], want[ok], rtol=1e-5, atol=1e-30), (gval, got, want)
    xr = np.array([1.0, 0.0, -1.0, -0.0, np.nan, 2.0], np.float32)
    gr = np.array([np.inf, np.inf, -np.inf, 3.0, 1.0, np.nan], np.float32)
    got, want = B.reluBackward(dev(B, xr), dev(B, gr)).data, ref.relu_backward(orc(xr), orc(gr)).data
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(got[~np.isnan(want)], want[~np.isnan(want)]), (got, want)
    assert np.isinf(got[0]) and np.isnan(got[1]) and np.isnan(got[2]) and got[3] == 0.0


def test_embedding_of_an_id_outside_the_table_is_a_row_of_nan(B):
    """The reference's gather reads weight[id * dim + d] from a typed array: past either end that is undefined, stored as NaN
    (cpu_ref.ts:364-385).  The device gives the same rows (also from the fused token + position gather) without touching
    memory outside the table; the backward pass skips such ids, as a store past a typed array's end is dropped (ops.ts:491-507)."""
    import ctypes as C
    from alpha2_amd import _ffi as ffi
    w = rs.randn(6, 8).astype(np.float32)
    ids = np.array([0, 5, 6, -1, 3, 1 << 20, -(1 << 20)], np.int32)
    got, want = B.embedding(dev(B, w), dev(B, ids, "i32")).data.reshape(len(ids), 8), O.embedding(orc(w), orc(ids)).data.reshape(len(ids), 8)
    assert np.array_equal(got, want, equal_nan=True)
    assert np.isnan(got[[2, 3, 5, 6]]).all() and np.array_equal(got[[0, 1, 4]], w[[0, 5, 3]])
    wpe = rs.randn(len(ids), 8).astype(np.float32)
    out = B._new((len(ids), 8))
    tw, tp, ti = dev(B, w), dev(B, wpe), dev(B, ids, "i32")
    ffi.check(B.lib.ah_embedding_tok_pos(B._ptr(tw), B._ptr(tp), B._ptr(ti), B._ptr(out), len(ids), len(ids), 8, 6, ffi.F32))
    B._dirty(out)
    both = out.data.reshape(len(ids), 8)
    assert np.isnan(both[[2, 3, 5, 6]]).all() and np.array_equal(both[[0, 1, 4]], (w[[0, 5, 3]] + wpe[[0, 1, 4]]))
    g = rs.randn(len(ids), 8).astype(np.float32)
    assert_close(B.embeddingBackward(dev(B, ids, "i32"), dev(B, g), 6).data, ref.embedding_backward(orc(ids), orc(g), 6).data, what="embedding backward with ids outside")


def test_clamp_keeps_nan(B):
    """max(lo, min(hi, x)) in the reference's arithmetic (cpu_ref.ts:358-360): Math.min / Math.max return NaN for a NaN."""
    x = np.array([np.nan, -3.0, 0.5, 7.0, np.inf, -np.inf], np.float32)
    got, want = B.clamp(dev(B, x), -1.0, 2.0).data, O.clamp(orc(x), -1.0, 2.0).data
    assert np.isnan(got[0]) and np.isnan(want[0]) and np.array_equal(got[1:], want[1:]) and np.array_equal(got[1:], [-1.0, 0.5, 2.0, 2.0, -1.0])


@pytest.mark.parametrize("M,K,N", [(2, 2, 2), (33, 19, 47), (64, 64, 64), (128, 128, 128), (256, 256, 256), (1024, 128, 384), (130, 515, 257)])
def test_gemm_f32_all_layouts(B, M, K, N):
    a, b = rs.randn(M, K).astype(np.float32), rs.randn(K, N).astype(np.float32)
    want = O.matmul(orc(a), orc(b)).data
    assert_close(B.matmul(dev(B, a), dev(B, b)).data, want, what="matmul")
    bt = np.ascontiguousarray(b.T)
    assert_close(B.matmulTransposed(dev(B, a), dev(B, bt)).data, want, what="matmulTransposed")
    at = np.ascontiguousarray(a.T)
    assert_close(B.matmulTransposedA(dev(B, at), dev(B, b)).data, want, what="matmulTransposedA")
    with pytest.raises(ValueError):
        B.matmul(dev(B, a), dev(B, rs.randn(K + 1, N).astype(np.float32)))


@pytest.mark.parametrize("M,K,N", [(256, 4096, 128), (132, 2052, 260), (64, 8192, 64)])
def test_gemm_f32_long_contraction_split_k(B, M, K, N):
    """Few output tiles and a long contraction: the fp32 kernel runs K in slices (as batch entries) and sums the slices
    in fixed order; all three layouts and the accumulating epilogue against a float64 product."""
    from alpha2_amd import _ffi as ffi
    a, b = rs.randn(M, K).astype(np.float32), rs.randn(K, N).astype(np.float32)
    want = a.astype(np.float64) @ b.astype(np.float64)
    scale = float(np.sqrt(K))                                   # size of a result entry
    got = {"nn": B.matmul(dev(B, a), dev(B, b)), "nt": B.matmulTransposed(dev(B, a), dev(B, np.ascontiguousarray(b.T))),
           "tn": B.matmulTransposedA(dev(B, np.ascontiguousarray(a.T)), dev(B, b))}
    for name, t in got.items():
        assert B.lastGemmKernel()[0].startswith("k_gemm_f32")
        assert np.max(np.abs(t.data.reshape(M, N) - want)) <= 2e-6 * K ** 0.5 * scale, name
    assert B.lastGemmKernel()[1] > 1                            # the product above did run in slices
    # accumulate into an existing C through the raw entry point
    import ctypes
    c0 = rs.randn(M, N).astype(np.float32)
    c, at, bb = dev(B, c0), dev(B, np.ascontiguousarray(a.T)), dev(B, b)
    g = ffi.AhGemm(ffi.GEMM_TN, ffi.F32, ffi.F32, ffi.EPI_ACCUM, M, N, K, M, N, N, 1, 0, 0, 0, B._ptr(at), B._ptr(bb), B._ptr(c), 0)
    ffi.check(B.lib.ah_gemm(ctypes.byref(g)))
    B._dirty(c)
    assert B.lastGemmKernel()[1] > 1
    assert np.max(np.abs(c.data.reshape(M, N) - (want + c0))) <= 2e-6 * K ** 0.5 * scale


def test_gemm_f32_batched_and_broadcast(B):
    a, b = rs.randn(2, 3, 40, 16).astype(np.float32), rs.randn(2, 3, 16, 24).astype(np.float32)
    assert_close(B.matmul(dev(B, a), dev(B, b)).data, O.matmul(orc(a), orc(b)).data)
    b1 = rs.randn(16, 24).astype(np.float32)
    got = B.matmul(dev(B, a), dev(B, b1))
    assert got.shape == (2, 3, 40, 24)
    assert_close(got.data, O.matmul(orc(a), orc(b1)).data)
    b2 = rs.randn(3, 16, 24).astype(np.float32)          # mixed broadcast [2,3] x [3]
    assert_close(B.matmul(dev(B, a), dev(B, b2)).data, O.matmul(orc(a), orc(b2)).data)
    bt = np.ascontiguousarray(np.swapaxes(b, 2, 3))
    assert_close(B.matmulTransposed(dev(B, a), dev(B, bt)).data, O.matmul(orc(a), orc(b)).data)
    g = rs.randn(2, 3, 40, 24).astype(np.float32)
    want = O.matmul(O.transpose(orc(a), 2, 3), orc(g)).data
    assert_close(B.matmulTransposedA(dev(B, a), dev(B, g)).data, want)


def _oracle_attention(q, k, v, do, scale, cap):
    """[BH,T,D] attention through the oracle's own op chain (gpt.ts:255-279) and tape."""
    tape = rm.Tape(); ctx = rm.Ctx(tape, O)
    T = q.shape[1]
    qv, kv, vv = (rm.Variable(orc(x), True) for x in (q, k, v))
    s = rm.scale(ctx, rm.matmul(ctx, qv, rm.transpose(ctx, kv, 1, 2)), scale)
    if cap > 0:
        s = rm.softCap(ctx, s, cap)
    mask = O.causalMask(T)
    masked = rm.Variable(O.maskedFill(s.data, mask, -1e9), True)
    tape.record(masked, [s], lambda g, Bk, n: [Bk.maskedFill(g, mask, 0)])
    att = rm.softmax(ctx, masked, -1)
    out = rm.matmul(ctx, att, vv)
    lse = np.log(np.sum(np.exp(masked.data.data.reshape(-1, T).astype(np.float64)), -1))
    tape.backward(out, O, orc(do))
    return out.data.data, lse, qv.grad.data, kv.grad.data, vv.grad.data


@pytest.mark.parametrize("BH,T,D,cap", [(2, 64, 32, 30.0), (3, 100, 64, 0.0), (2, 129, 64, 30.0), (1, 256, 128, 30.0), (2, 1, 32, 0.0),
                                        (3, 130, 16, 30.0), (2, 70, 8, 0.0), (2, 97, 48, 2.0), (1, 200, 96, 30.0)])      # (the last four: sizes between the kernels')
def test_flash_attention_f32_vs_materialised(B, BH, T, D, cap):
    q, k, v, do = (rs.randn(BH, T, D).astype(np.float32) for _ in range(4))
    scale = 1 / math.sqrt(D)
    want_o, want_lse, dq, dk, dv = _oracle_attention(q, k, v, do, scale, cap)
    Q, K, V = dev(B, q), dev(B, k), dev(B, v)
    r = B.flashAttention(Q, K, V, T, scale, cap)
    assert r["output"].shape == (BH, T, D) and r["lse"].shape == (BH, T)
    assert_close(r["output"].data, want_o, what="flash.O")
    assert_close(r["lse"].data, want_lse, what="flash.LSE")
    g = B.flashAttentionBackward(Q, K, V, r["output"], dev(B, do), r["lse"], T, scale, cap)
    # dS = P*(dP - delta) cancels exactly when a row sees a single key: floor the bound at the size of its terms
    term = float(np.abs(np.einsum("bqd,bkd->bqk", do, v)).max() * max(np.abs(k).max(), np.abs(q).max()) * scale)
    assert_close(g["dQ"].data, dq, what="flash.dQ", scale=term if T < 4 else 0.0)
    assert_close(g["dK"].data, dk, what="flash.dK", scale=term if T < 4 else 0.0)
    assert_close(g["dV"].data, dv, what="flash.dV")


def test_adamw_vs_oracle_and_reference_gradscale_identity(B, golden):
    n = 100003
    p0, g = rs.randn(n).astype(np.float32), rs.randn(n).astype(np.float32)
    p, m, v = dev(B, p0), dev(B, np.zeros(n, np.float32)), dev(B, np.zeros(n, np.float32))
    po, mo, vo = orc(p0), np.zeros(n, np.float32), np.zeros(n, np.float32)
    b1p = b2p = 1.0
    for _ in range(3):
        b1p *= 0.9; b2p *= 0.95
        B.adamwStep(p, dev(B, g), m, v, 3e-4, 0.9, 0.95, 1e-8, 0.1, 1 - b1p, 1 - b2p, 0.5)
        ref.adamw_step(po, orc(g), mo, vo, 3e-4, 0.9, 0.95, 1e-8, 0.1, 1 - b1p, 1 - b2p, 0.5)
    assert_close(p.data, po.data, rel=1e-6, what="adamw.p")
    assert_close(m.data, mo, what="adamw.m")
    assert_close(v.data, vo, what="adamw.v")
    c = golden["optimizer.test.ts"]["adamw_gradscale"]      # optimizer.test.ts:23-45 on the device

    def run(prescale):
        pp, gg = dev(B, np.array(c["p"], np.float32)), np.array(c["g"], np.float32)
        gs = c["gradScale"]
        if prescale:
            gg, gs = gg * np.float32(gs), 1.0
        B.adamwStep(pp, dev(B, gg), dev(B, np.zeros(4, np.float32)), dev(B, np.zeros(4, np.float32)), c["lr"], c["beta1"], c["beta2"],
                    c["eps"], c["weightDecay"], 1 - c["beta1"], 1 - c["beta2"], gs)
        return pp.data
    assert np.max(np.abs(run(False) - run(True))) < 1e-7


def test_clip_coefficient_on_the_device_and_its_use_by_adamw(B):
    """ah_clip_coef against the trainer's rule (trainer.ts:1650-1656: norm = sqrt(sum of squares) x |gradScale|; the
    coefficient is clip / norm above the clip value, 1 at or below it, and clipping is off at clip <= 0), and an AdamW step
    that takes the coefficient from the device against the same step with the coefficient folded into gradScale on the host."""
    import ctypes as C
    import math
    from alpha2_amd import TensorData, _ffi as ffi
    out = B.zeros((2,))
    for sumsq, scale, clip in ((16.0, 0.5, 1.0), (16.0, -0.5, 1.0), (0.25, 1.0, 1.0), (1.0, 1.0, 1.0), (9.0, 1.0, 0.0), (0.0, 1.0, 1.0)):
        ss = TensorData((1,), "f32", np.array([sumsq], np.float32))
        ffi.check(B.lib.ah_clip_coef(B._ptr(ss), scale, clip, B._ptr(out)))
        B._dirty(out)
        norm = math.sqrt(sumsq) * abs(scale)
        want = clip / norm if clip > 0 and norm > clip else 1.0
        assert abs(float(out.data[0]) - want) <= 2e-7 * want and abs(float(out.data[1]) - norm) <= 2e-7 * max(norm, 1.0), (sumsq, scale, clip, out.data)
    assert B.lib.ah_clip_coef(0, 1.0, 1.0, B._ptr(out)) != 0 and b"null operand" in B.lib.ah_last_error()
    n = 4099
    p0, g = rs.randn(n).astype(np.float32), rs.randn(n).astype(np.float32)
    ssq = TensorData((1,), "f32", np.array([float((g.astype(np.float64) ** 2).sum())], np.float32))
    ffi.check(B.lib.ah_clip_coef(B._ptr(ssq), 0.5, 1.0, B._ptr(out)))
    B._dirty(out)
    coef = float(out.data[0])
    assert coef < 1.0
    h = ffi.AhAdamW(3e-4, 0.9, 0.95, 1e-8, 0.1, 0.1, 0.05, 0.5)
    pa, ma, va = dev(B, p0), dev(B, np.zeros(n, np.float32)), dev(B, np.zeros(n, np.float32))
    gt = dev(B, g)
    ffi.check(B.lib.ah_adamw(B._ptr(pa), B._ptr(gt), B._ptr(ma), B._ptr(va), n, C.byref(h), 0, B._ptr(out), 0))
    for t in (pa, ma, va):
        B._dirty(t)
    pb, mb, vb = dev(B, p0), dev(B, np.zeros(n, np.float32)), dev(B, np.zeros(n, np.float32))
    B.adamwStep(pb, dev(B, g), mb, vb, 3e-4, 0.9, 0.95, 1e-8, 0.1, 0.1, 0.05, float(np.float32(0.5) * np.float32(coef)))
    assert_close(pa.data, pb.data, rel=1e-6, what="adamw with the device coefficient: p")
    assert_close(ma.data, mb.data, rel=1e-6, what="adamw with the device coefficient: m")
    assert_close(va.data, vb.data, rel=1e-6, what="adamw with the device coefficient: v")


def test_graph_capture_replays_match_eager(B):
    import ctypes as C
    from alpha2_amd import _ffi as ffi
    lib = B.lib
    x = dev(B, rs.randn(512, 256).astype(np.float32)); w = dev(B, rs.randn(128, 256).astype(np.float32))
    acc = B.zeros((512, 128))
    B._ptr(x), B._ptr(w)

    def body():
        y = B.matmulTransposed(x, w)
        z = B.gelu(y)
        B.addInplace(acc, z)
        for t in (y, z):
            B.releaseGpuTensor(t)
    body()                                   # eager warm-up fills the pool
    B.syncGpu()
    ffi.check(lib.ah_graph_begin())
    body()
    gid = C.c_uint64()
    ffi.check(lib.ah_graph_end(C.byref(gid)))
    want = O.gelu(O.matmul(orc(x.data.reshape(512, 256)), O.transpose(orc(w.data.reshape(128, 256)), 0, 1))).data
    for i in range(2, 6):                    # replays interleaved with eager work and syncs
        ffi.check(lib.ah_graph_launch(gid.value))
        tmp = B.scale(acc, 1.0 / i)          # eager op between replays
        B.syncGpu()
        assert_close(tmp.data, want, what=f"replay {i}")
        B.releaseGpuTensor(tmp)
    ffi.check(lib.ah_graph_destroy(gid.value))


def _bf16_round(x):
    """round-to-nearest-even to bf16, returned as f32 values and as raw u16 bits"""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    bits = u.astype(np.uint16)
    return (bits.astype(np.uint32) << 16).view(np.float32).reshape(np.shape(x)), bits.reshape(np.shape(x))


def _raw_gemm(B, layout, a, b, m, n, k, in_dtype, out_dtype, epi=0, aux=None, c_init=None):
    """ah_gemm through the C ABI on raw buffers; returns C (f32 values) and aux-out if the epilogue writes one."""
    import ctypes as C
    from alpha2_amd import TensorData, _ffi as ffi

    def up(arr, store):
        if store == ffi.BF16:
            t = TensorData(arr.shape, "f16", _bf16_round(arr)[1])      # 2-byte container for the raw bits
        else:
            t = TensorData(arr.shape, "f32", arr)
        return t, B._ptr(t)
    ta, pa = up(a, in_dtype)
    tb, pb = up(b, in_dtype)
    cinit = np.zeros((m, n), np.float32) if c_init is None else c_init
    tc, pc = up(cinit, out_dtype)
    paux = 0
    if aux is not None:
        taux, paux = up(aux, out_dtype)                               # what an epilogue reads has the type of C
    elif epi in (ffi.EPI_GELU, ffi.EPI_GELU_GRAD):
        taux, paux = up(np.zeros((m, n), np.float32), out_dtype)
    lda = a.shape[1]
    ldb = b.shape[1]
    g = ffi.AhGemm(layout, in_dtype, out_dtype, epi, m, n, k, lda, ldb, n, 1, 0, 0, 0, pa, pb, pc, paux)
    ffi.check(B.lib.ah_gemm(C.byref(g)))

    def down(t, store):
        B._dirty(t)
        raw = t.data
        return (raw.astype(np.uint32) << 16).view(np.float32) if store == ffi.BF16 else raw
    out = down(tc, out_dtype).reshape(m, n)
    aux_out = down(taux, out_dtype).reshape(m, n) if epi in (ffi.EPI_GELU, ffi.EPI_GELU_GRAD) else None
    return out, aux_out


@pytest.mark.parametrize("m,n", [(256, 192), (37, 20), (5, 3)])
def test_gemm_over_an_empty_contraction(B, m, n):
    """k = 0: the product is all zeros (cpu_ref.ts:166-258 sums no terms) and the epilogue applies to that, for bf16 operands in
    every layout (leading dimensions at their minimum, 0 columns or 0 rows of operand) as for f32 ones: NONE writes zeros
    over what was there, ACCUM leaves C, RESIDUAL copies the residual, GELU gives gelu(0) = 0 with a zero pre-activation."""
    import ctypes as C
    from alpha2_amd import TensorData, _ffi as ffi
    c0, res = rs.randn(m, n).astype(np.float32), rs.randn(m, n).astype(np.float32)
    for in_dtype in (ffi.BF16, ffi.F32):
        for layout in (ffi.GEMM_NN, ffi.GEMM_NT, ffi.GEMM_TN):
            dummy = TensorData((64,), "f32", np.ones(64, np.float32))          # never read: the operands have no elements
            lda = {ffi.GEMM_NN: 0, ffi.GEMM_NT: 0, ffi.GEMM_TN: m}[layout]
            ldb = {ffi.GEMM_NN: n, ffi.GEMM_NT: 0, ffi.GEMM_TN: n}[layout]
            cases = [(ffi.F32, ffi.EPI_NONE, None, np.zeros((m, n), np.float32)), (ffi.F32, ffi.EPI_ACCUM, None, c0), (ffi.F32, ffi.EPI_RESIDUAL, res, res)]
            if in_dtype == ffi.BF16:
                cases += [(ffi.BF16, ffi.EPI_NONE, None, np.zeros((m, n), np.float32)), (ffi.BF16, ffi.EPI_RESIDUAL, res, _bf16_round(res)[0]),
                          (ffi.BF16, ffi.EPI_GELU, np.ones((m, n), np.float32), np.zeros((m, n), np.float32))]
            for out_dtype, epi, aux, want in cases:
                store = lambda arr: (TensorData(arr.shape, "f16", _bf16_round(arr)[1]) if out_dtype == ffi.BF16 else TensorData(arr.shape, "f32", arr.copy()))
                tc = store(c0)
                taux = store(aux) if aux is not None else None
                g = ffi.AhGemm(layout, in_dtype, out_dtype, epi, m, n, 0, lda, ldb, n, 1, 0, 0, 0, B._ptr(dummy), B._ptr(dummy), B._ptr(tc),
                               B._ptr(taux) if taux is not None else 0)
                ffi.check(B.lib.ah_gemm(C.byref(g)))
                B._dirty(tc)
                got = ((tc.data.astype(np.uint32) << 16).view(np.float32) if out_dtype == ffi.BF16 else tc.data).reshape(m, n)
                exp = _bf16_round(want)[0] if out_dtype == ffi.BF16 else want
                assert np.array_equal(got, exp), (in_dtype, layout, out_dtype, epi)
                if epi == ffi.EPI_GELU:
                    B._dirty(taux)
                    assert not np.any(taux.data), "pre-activation of an empty product"


@pytest.mark.parametrize("in_bf16,out_bf16", [(False, False), (True, False), (True, True)])
@pytest.mark.parametrize("M,N,K", [(128, 128, 64), (256, 384, 96), (300, 200, 72), (1024, 768, 256)])
def test_gemm_layouts_epilogues_dtypes(B, in_bf16, out_bf16, M, N, K):
    from alpha2_amd import _ffi as ffi
    idt, odt = (ffi.BF16 if in_bf16 else ffi.F32), (ffi.BF16 if out_bf16 else ffi.F32)
    a, b = rs.randn(M, K).astype(np.float32), rs.randn(N, K).astype(np.float32)
    if in_bf16:
        a, b = _bf16_round(a)[0], _bf16_round(b)[0]
    want = O.matmul(orc(a), O.transpose(orc(b), 0, 1)).data.reshape(M, N)
    rel = 1e-4 if not out_bf16 else 2.0 ** -7            # a bf16 result carries 8 significant bits

    def cmp(got, ref_, what):
        assert_close(got, ref_, rel=rel, what=what)
    cmp(_raw_gemm(B, ffi.GEMM_NT, a, b, M, N, K, idt, odt)[0], want, "NT")
    cmp(_raw_gemm(B, ffi.GEMM_NN, a, np.ascontiguousarray(b.T), M, N, K, idt, odt)[0], want, "NN")
    cmp(_raw_gemm(B, ffi.GEMM_TN, np.ascontiguousarray(a.T), np.ascontiguousarray(b.T), M, N, K, idt, odt)[0], want, "TN")
    # provided combinations: ACCUM / RESIDUAL write f32 (RESIDUAL also bf16 from bf16 operands); GELU / GELU_BWD write the operand type
    if not out_bf16:
        c0 = rs.randn(M, N).astype(np.float32)
        cmp(_raw_gemm(B, ffi.GEMM_NT, a, b, M, N, K, idt, odt, ffi.EPI_ACCUM, c_init=c0)[0], want + c0, "ACCUM")
        cmp(_raw_gemm(B, ffi.GEMM_TN, np.ascontiguousarray(a.T), np.ascontiguousarray(b.T), M, N, K, idt, odt, ffi.EPI_ACCUM, c_init=c0)[0],
            want + c0, "TN ACCUM")
        res = rs.randn(M, N).astype(np.float32)
        cmp(_raw_gemm(B, ffi.GEMM_NT, a, b, M, N, K, idt, odt, ffi.EPI_RESIDUAL, aux=res)[0], want + res, "RESIDUAL")
    if in_bf16 and out_bf16:                                 # a residual stream kept in bf16: aux and C both bf16
        res = _bf16_round(rs.randn(M, N).astype(np.float32))[0]
        cmp(_raw_gemm(B, ffi.GEMM_NT, a, b, M, N, K, idt, odt, ffi.EPI_RESIDUAL, aux=res)[0], want + res, "RESIDUAL bf16")
    if in_bf16 == out_bf16:
        got, pre = _raw_gemm(B, ffi.GEMM_NT, a, b, M, N, K, idt, odt, ffi.EPI_GELU)
        cmp(pre, want, "GELU.pre")
        cmp(got, O.gelu(orc(want)).data.reshape(M, N), "GELU")
        pre_act = rs.randn(M, N).astype(np.float32)
        if out_bf16:
            pre_act = _bf16_round(pre_act)[0]
        gb = ref.gelu_backward(orc(pre_act), orc(want), fused=True).data.reshape(M, N)
        cmp(_raw_gemm(B, ffi.GEMM_NN, a, np.ascontiguousarray(b.T), M, N, K, idt, odt, ffi.EPI_GELU_BWD, aux=pre_act)[0], gb, "GELU_BWD")
        # the same pair with the derivative saved by the forward product: C = gelu(acc), aux = gelu'(acc); then C = acc * aux
        got, dsaved = _raw_gemm(B, ffi.GEMM_NT, a, b, M, N, K, idt, odt, ffi.EPI_GELU_GRAD)
        cmp(got, O.gelu(orc(want)).data.reshape(M, N), "GELU_GRAD.value")
        ones = np.ones((M, N), np.float32)
        cmp(dsaved, ref.gelu_backward(orc(want), orc(ones), fused=True).data.reshape(M, N), "GELU_GRAD.derivative")
        cmp(_raw_gemm(B, ffi.GEMM_NN, a, np.ascontiguousarray(b.T), M, N, K, idt, odt, ffi.EPI_MUL_AUX, aux=pre_act)[0], want * pre_act, "MUL_AUX")
    else:
        import ctypes as C
        g = ffi.AhGemm(ffi.GEMM_NT, idt, odt, ffi.EPI_GELU, M, N, K, K, K, N, 1, 0, 0, 0, 1 << 20, 1 << 20, 1 << 20, 1 << 20)
        assert B.lib.ah_gemm(C.byref(g)) == 5 and b"not provided" in B.lib.ah_last_error()


def test_gemm_bf16_split_k_weight_gradient(B):
    """dW = G^T X with a long token axis and few output tiles takes the split-K path (slices of the token axis into a
    workspace, summed in a fixed order by a second kernel)."""
    from alpha2_amd import _ffi as ffi
    Kc, M, N = 4096, 256, 128
    g_, x = _bf16_round(rs.randn(Kc, M).astype(np.float32) * 0.1)[0], _bf16_round(rs.randn(Kc, N).astype(np.float32))[0]
    want = O.matmul(O.transpose(orc(g_), 0, 1), orc(x)).data.reshape(M, N)
    assert_close(_raw_gemm(B, ffi.GEMM_TN, g_, x, M, N, Kc, ffi.BF16, ffi.F32)[0], want, what="split-K NONE")
    c0 = rs.randn(M, N).astype(np.float32)
    assert_close(_raw_gemm(B, ffi.GEMM_TN, g_, x, M, N, Kc, ffi.BF16, ffi.F32, ffi.EPI_ACCUM, c_init=c0)[0], want + c0, what="split-K ACCUM")


@pytest.fixture(params=[0, 1], ids=["pair", "onepass"])
def bwd_variant(request, B):
    """Both arrangements of the bf16 backward pass: a dQ and a dK/dV kernel, or one pass over the scores."""
    B.flashBackwardVariant = request.param
    yield request.param
    B.flashBackwardVariant = 0


@pytest.mark.parametrize("BH,T,D,cap", [(2, 64, 32, 30.0), (3, 100, 64, 0.0), (2, 129, 64, 30.0), (2, 320, 64, 30.0), (1, 256, 128, 30.0), (2, 1, 64, 0.0),
                                        (3, 700, 64, 30.0), (2, 513, 32, 0.0),
                                        (3, 200, 16, 30.0), (2, 70, 8, 0.0), (3, 130, 48, 0.0), (2, 96, 80, 30.0), (1, 150, 120, 2.0)])
def test_flash_attention_bf16_vs_materialised(B, bwd_variant, BH, T, D, cap):
    """bf16 operands, fp32 accumulation.  Inputs are bf16-exact so the oracle sees the same numbers; the kernel rounds P and
    dS to bf16 before the second product and its outputs to bf16, so the bar is bf16 resolution (2^-7 of the tensor scale).
    T = 700 and 513 give the one-pass kernel several 256-key blocks with a ragged last one.  Head sizes 16, 8, 48, 80 and 120 run
    the kernels of the next size up (32, 64, 128) with the missing features read as zeros and never stored: the tensors here
    are exactly [BH, T, D], so a store past a row's end would land in the next row and show."""
    rc = np.random.RandomState(1000 * BH + 7 * T + D)              # the case's own stream: the data do not depend on which tests ran before
    q, k, v, do = (_bf16_round(rc.randn(BH, T, D).astype(np.float32))[0] for _ in range(4))
    scale = 1 / math.sqrt(D)
    want_o, want_lse, dq, dk, dv = _oracle_attention(q, k, v, do, scale, cap)
    Q, K, V, dO = (B.castStore(dev(B, x), "bf16") for x in (q, k, v, do))
    r = B.flashAttention(Q, K, V, T, scale, cap)
    assert r["output"].store == "bf16"
    rel = 2.0 ** -6
    # O = sum_j p_j v_j with every p_j rounded to bf16 (relative error <= 2^-9): the error of an entry is at most
    # 2^-9 sum_j p_j |v_j| <= 2^-9 max|v| whatever the entry's own size, and over long rows the entries themselves average
    # out towards 0, so that -- not the rms of O -- is the floor of the bound (rel x scale = 2^-9 max|v|)
    assert_close(r["output"].data, want_o, rel=rel, what="flash16.O", scale=float(np.abs(v).max()) / 8)
    assert_close(r["lse"].data, want_lse, rel=1e-4, what="flash16.LSE")
    g = B.flashAttentionBackward(Q, K, V, r["output"], dO, r["lse"], T, scale, cap)
    term = float(np.abs(np.einsum("bqd,bkd->bqk", do, v)).max() * max(np.abs(k).max(), np.abs(q).max()) * scale)
    # sums of bf16-rounded products: a few entries in a thousand may sit a little outside the element-wise bound
    def loose(x):                                                   # (on a small tensor "a few in a thousand" is at least 16 entries)
        return dict(outlier_frac=max(2e-3, 16 / x.size), outlier_abs=0.1 * float(np.sqrt(np.mean(np.square(x)))) + 1e-6)
    if T < 4:
        assert_close(g["dQ"].data, dq, rel=rel, what="flash16.dQ", scale=term)
        assert_close(g["dK"].data, dk, rel=rel, what="flash16.dK", scale=term)
    else:
        assert_close(g["dQ"].data, dq, rel=rel, what="flash16.dQ", **loose(dq))
        assert_close(g["dK"].data, dk, rel=rel, what="flash16.dK", **loose(dk))
    assert_close(g["dV"].data, dv, rel=rel, what="flash16.dV", **loose(dv))


@pytest.mark.parametrize("M,N,K,tile", [(4000, 4072, 64, 4), (4000, 4072, 192, 4), (4000, 4072, 512, 4), (16376, 760, 128, 3), (8192, 1536, 320, 3),
                                           (4000, 4072, 2048, 4), (16384, 768, 2112, 3), (8192, 1024, 320, 2), (8184, 1016, 128, 2),
                                           (8192, 1024, 2112, 2)])
def test_gemm_bf16_large_tiles_direct_to_lds_kernel(B, M, N, K, tile):
    """Outputs with at least one 256x256 tile per CU take the kernel fed by global->LDS loads; edges in M and N, odd and
    even k-tile counts, every layout and epilogue.  At this size the check is a float64 numpy product of the same
    bf16-exact operands (the C oracle covers the small shapes above); fp32 accumulation of exact products."""
    from alpha2_amd import _ffi as ffi
    # ragged edges with N % 8 == 0 and M % 8 == 0 (needed by the k-major layouts); `tile` = expected column tile / 64:
    # 256 x 256 tiles, or 256 x 192 / 256 x 128 where those fill whole rounds of CUs better (N = 760, 1536 / N = 1024)
    a, b = _bf16_round(rs.randn(M, K).astype(np.float32))[0], _bf16_round(rs.randn(N, K).astype(np.float32))[0]
    want = a.astype(np.float64) @ b.astype(np.float64).T
    at, bt = np.ascontiguousarray(a.T), np.ascontiguousarray(b.T)

    got = _raw_gemm(B, ffi.GEMM_NT, a, b, M, N, K, ffi.BF16, ffi.F32)[0]
    if B.getDeviceInfo()["computeUnits"] == 256:
        name = B.lastGemmKernel()[0]
        assert name.startswith("k_gemm_bf16_dma<") and f", {tile}, " in name, name
    assert_close(got, want, rel=1e-4, what="NT f32")
    assert_close(_raw_gemm(B, ffi.GEMM_NT, a, b, M, N, K, ffi.BF16, ffi.BF16)[0], want, rel=2.0 ** -7, what="NT bf16")
    assert_close(_raw_gemm(B, ffi.GEMM_NN, a, bt, M, N, K, ffi.BF16, ffi.F32)[0], want, rel=1e-4, what="NN")
    assert_close(_raw_gemm(B, ffi.GEMM_TN, at, bt, M, N, K, ffi.BF16, ffi.F32)[0], want, rel=1e-4, what="TN")
    c0 = rs.randn(M, N).astype(np.float32)
    assert_close(_raw_gemm(B, ffi.GEMM_TN, at, bt, M, N, K, ffi.BF16, ffi.F32, ffi.EPI_ACCUM, c_init=c0)[0], want + c0, rel=1e-4, what="TN ACCUM")
    r16 = _bf16_round(c0 * 8)[0]
    assert_close(_raw_gemm(B, ffi.GEMM_NT, a, b, M, N, K, ffi.BF16, ffi.BF16, ffi.EPI_RESIDUAL, aux=r16)[0], want + r16, rel=2.0 ** -7, what="NT RESIDUAL bf16")
    assert_close(_raw_gemm(B, ffi.GEMM_NT, a, b, M, N, K, ffi.BF16, ffi.F32, ffi.EPI_RESIDUAL, aux=c0)[0], want + c0, rel=1e-4, what="RESIDUAL")
    got, pre = _raw_gemm(B, ffi.GEMM_NT, a, b, M, N, K, ffi.BF16, ffi.BF16, ffi.EPI_GELU)
    assert_close(pre, want, rel=2.0 ** -7, what="GELU.pre")
    w32 = want.astype(np.float32)
    assert_close(got, O.gelu(orc(w32)).data.reshape(M, N), rel=2.0 ** -7, what="GELU")
    pre_act = _bf16_round(rs.randn(M, N).astype(np.float32))[0]
    gb = ref.gelu_backward(orc(pre_act), orc(w32), fused=True).data.reshape(M, N)
    assert_close(_raw_gemm(B, ffi.GEMM_NN, a, bt, M, N, K, ffi.BF16, ffi.BF16, ffi.EPI_GELU_BWD, aux=pre_act)[0], gb, rel=2.0 ** -7, what="GELU_BWD")
    got, dsaved = _raw_gemm(B, ffi.GEMM_NT, a, b, M, N, K, ffi.BF16, ffi.BF16, ffi.EPI_GELU_GRAD)
    assert_close(got, O.gelu(orc(w32)).data.reshape(M, N), rel=2.0 ** -7, what="GELU_GRAD.value")
    assert_close(dsaved, ref.gelu_backward(orc(w32), orc(np.ones((M, N), np.float32)), fused=True).data.reshape(M, N), rel=2.0 ** -7, what="GELU_GRAD.derivative")
    assert_close(_raw_gemm(B, ffi.GEMM_NN, a, bt, M, N, K, ffi.BF16, ffi.BF16, ffi.EPI_MUL_AUX, aux=pre_act)[0], want * pre_act, rel=2.0 ** -7, what="MUL_AUX")


def test_gemm_grouped_matches_separate_products(B):
    """One grouped launch over problems of different sizes (ragged tile edges, NONE then ACCUM) against float64 numpy
    products of the same bf16-exact operands; descriptor errors are reported, not launched."""
    import ctypes as C
    from alpha2_amd import TensorData, _ffi as ffi
    K = 640
    shapes = [(768, 768), (264, 520), (2304, 768), (8, 8), (1000, 256)]
    keep, descs, wants, outs = [], [], [], []
    for m, n in shapes:
        gy, x = _bf16_round(rs.randn(K, m).astype(np.float32))[0], _bf16_round(rs.randn(K, n).astype(np.float32))[0]
        tg, tx = TensorData(gy.shape, "f16", _bf16_round(gy)[1]), TensorData(x.shape, "f16", _bf16_round(x)[1])
        out = B.zeros((m, n))
        keep += [tg, tx]
        outs.append(out)
        wants.append(gy.astype(np.float64).T @ x.astype(np.float64))
        descs.append(ffi.AhGemm(ffi.GEMM_TN, ffi.BF16, ffi.F32, ffi.EPI_NONE, m, n, K, m, n, n, 1, 0, 0, 0, B._ptr(tg), B._ptr(tx), B._ptr(out), 0))
    arr = (ffi.AhGemm * len(descs))(*descs)
    plan = C.c_uint64()
    ffi.check(B.lib.ah_gemm_grouped_plan(arr, len(descs), C.byref(plan)))
    ffi.check(B.lib.ah_gemm_grouped_run(plan.value, ffi.EPI_NONE))
    assert B.lastGemmKernel()[0].startswith("k_gemm_bf16_dma_grouped<true, true")
    assert B.lastGemmKernel()[1] == 2                     # 47 tiles: less than half a round, so every problem is cut in two along k
    for out, want, (m, n) in zip(outs, wants, shapes):
        B._dirty(out)
        assert_close(out.data.reshape(m, n), want, rel=1e-4, what=f"grouped NONE {m}x{n}")
    ffi.check(B.lib.ah_gemm_grouped_run(plan.value, ffi.EPI_ACCUM))
    assert B.lastGemmKernel()[1] == 2
    for out, want, (m, n) in zip(outs, wants, shapes):
        B._dirty(out)
        assert_close(out.data.reshape(m, n), 2 * want, rel=1e-4, what=f"grouped ACCUM {m}x{n}")
    assert B.lib.ah_gemm_grouped_run(plan.value, ffi.EPI_GELU) != 0 and b"not provided" in B.lib.ah_last_error()
    ffi.check(B.lib.ah_gemm_grouped_destroy(plan.value))
    assert B.lib.ah_gemm_grouped_run(plan.value, ffi.EPI_NONE) != 0 and b"unknown plan" in B.lib.ah_last_error()
    bad = (ffi.AhGemm * 1)(ffi.AhGemm(ffi.GEMM_TN, ffi.BF16, ffi.F32, ffi.EPI_NONE, 64, 64, 100, 64, 64, 64, 1, 0, 0, 0, 1 << 20, 1 << 20, 1 << 20, 0))
    assert B.lib.ah_gemm_grouped_plan(bad, 1, C.byref(plan)) != 0 and b"multiple of 64" in B.lib.ah_last_error()


@pytest.mark.parametrize("shapes,K", [
    ([(768, 768), (264, 520), (2304, 768), (8, 8), (1000, 256)], 640),      # ragged edges in both directions, every problem cut in two along k
    ([(4096, 4096), (768, 768), (1280, 1792)], 256),                         # the last round is cut, the first problem is not
    ([(3072, 3072), (768, 768)], 128),                                       # no cut
])
def test_gemm_grouped_sum_of_squares_of_what_it_stores(B, shapes, K):
    """ah_gemm_grouped_run_sumsq leaves the same matrices as ah_gemm_grouped_run, bit for bit, and adds the sum of their
    squares (after ACCUM: of the accumulated values) to the number it is given; the first problem's C is a column block
    of a wider matrix, whose other columns are neither counted nor touched.  The same run twice gives the same number."""
    import ctypes as C
    from alpha2_amd import TensorData, _ffi as ffi
    keep, descs, outs, lds = [], [], [], []
    for i, (m, n) in enumerate(shapes):
        gy, x = _bf16_round(rs.randn(K, m).astype(np.float32))[0], _bf16_round(rs.randn(K, n).astype(np.float32))[0]
        tg, tx = TensorData(gy.shape, "f16", _bf16_round(gy)[1]), TensorData(x.shape, "f16", _bf16_round(x)[1])
        ldc = n + 8 if i == 0 else n
        out = TensorData((m, ldc), "f32", np.full(m * ldc, 7.0, np.float32))
        keep += [tg, tx]
        outs.append(out)
        lds.append(ldc)
        descs.append(ffi.AhGemm(ffi.GEMM_TN, ffi.BF16, ffi.F32, ffi.EPI_NONE, m, n, K, m, n, ldc, 1, 0, 0, 0, B._ptr(tg), B._ptr(tx), B._ptr(out), 0))
    arr = (ffi.AhGemm * len(descs))(*descs)
    plan = C.c_uint64()
    ffi.check(B.lib.ah_gemm_grouped_plan(arr, len(descs), C.byref(plan)))

    def read():
        got = []
        for out, (m, n), ldc in zip(outs, shapes, lds):
            B._dirty(out)
            full = out.data.reshape(m, ldc).copy()
            assert np.all(full[:, n:] == 7.0), "columns outside C were written"
            got.append(full[:, :n])
        return got
    ffi.check(B.lib.ah_gemm_grouped_run(plan.value, ffi.EPI_NONE))
    plain = read()
    ffi.check(B.lib.ah_gemm_grouped_run(plan.value, ffi.EPI_ACCUM))
    plain2 = read()
    for epi, want_c in ((ffi.EPI_NONE, plain), (ffi.EPI_ACCUM, plain2)):
        numbers = []
        for rep in range(2):
            if epi == ffi.EPI_ACCUM:                                          # back to the state the accumulating run started from
                ffi.check(B.lib.ah_gemm_grouped_run(plan.value, ffi.EPI_NONE))
            acc = TensorData((1,), "f32", np.array([3.0], np.float32))
            ffi.check(B.lib.ah_gemm_grouped_run_sumsq(plan.value, epi, B._ptr(acc)))
            assert B.lastGemmKernel()[0].endswith(", true>")
            got = read()
            for g_, w_, (m, n) in zip(got, want_c, shapes):
                assert np.array_equal(g_, w_), f"{m}x{n}: the matrices differ from ah_gemm_grouped_run's"
            B._dirty(acc)
            numbers.append(float(acc.data[0]))
            want = 3.0 + sum(float((g_.astype(np.float64) ** 2).sum()) for g_ in got)
            assert abs(numbers[-1] - want) <= 1e-5 * want, (epi, numbers[-1], want)
        assert numbers[0] == numbers[1]
    bf = B.zeros((64, 64))
    tb = TensorData((64, 64), "f16", np.zeros(64 * 64, np.uint16))
    d16 = (ffi.AhGemm * 1)(ffi.AhGemm(ffi.GEMM_TN, ffi.BF16, ffi.BF16, ffi.EPI_NONE, 64, 64, 64, 64, 64, 64, 1, 0, 0, 0, B._ptr(tb), B._ptr(tb), B._ptr(tb), 0))
    p16 = C.c_uint64()
    ffi.check(B.lib.ah_gemm_grouped_plan(d16, 1, C.byref(p16)))
    assert B.lib.ah_gemm_grouped_run_sumsq(p16.value, ffi.EPI_NONE, B._ptr(bf)) != 0 and b"f32 outputs" in B.lib.ah_last_error()
    assert B.lib.ah_gemm_grouped_run_sumsq(plan.value, ffi.EPI_NONE, 0) != 0
    ffi.check(B.lib.ah_gemm_grouped_destroy(p16.value))
    ffi.check(B.lib.ah_gemm_grouped_destroy(plan.value))


@pytest.mark.parametrize("shapes,K,cut", [
    ([(4096, 4096), (768, 768), (1280, 1792)], 256, True),       # 256 + 9 + 35 tiles: the last round (44) is cut, the first problem is not
    ([(2048, 2048), (1280, 1792)], 320, False),                  # 64 + 35 tiles, k not a multiple of 128: nothing to cut
    ([(3072, 3072), (768, 768)], 128, False),                    # 144 + 9 tiles: more than half a round, cutting would not pay
])
def test_gemm_grouped_last_round_cut_in_two_along_k(B, shapes, K, cut):
    """The problems that make up a short last round of the launch are computed as two k-halves and joined; the others
    are not touched, and neither are plans where the cut does not apply.  Checked against float64 products; a second run
    of the same plan must give bit-identical results (the join adds the halves in a fixed order)."""
    import ctypes as C
    from alpha2_amd import TensorData, _ffi as ffi
    keep, descs, wants, outs = [], [], [], []
    for m, n in shapes:
        gy, x = _bf16_round(rs.randn(K, m).astype(np.float32))[0], _bf16_round(rs.randn(K, n).astype(np.float32))[0]
        tg, tx = TensorData(gy.shape, "f16", _bf16_round(gy)[1]), TensorData(x.shape, "f16", _bf16_round(x)[1])
        out = B.zeros((m, n))
        keep += [tg, tx]
        outs.append(out)
        wants.append(gy.astype(np.float64).T @ x.astype(np.float64))
        descs.append(ffi.AhGemm(ffi.GEMM_TN, ffi.BF16, ffi.F32, ffi.EPI_NONE, m, n, K, m, n, n, 1, 0, 0, 0, B._ptr(tg), B._ptr(tx), B._ptr(out), 0))
    arr = (ffi.AhGemm * len(descs))(*descs)
    plan = C.c_uint64()
    ffi.check(B.lib.ah_gemm_grouped_plan(arr, len(descs), C.byref(plan)))
    first = []
    for run in range(2):
        ffi.check(B.lib.ah_gemm_grouped_run(plan.value, ffi.EPI_NONE))
        assert B.lastGemmKernel()[1] == (2 if cut else 1)
        for i, (out, want, (m, n)) in enumerate(zip(outs, wants, shapes)):
            B._dirty(out)
            got = out.data.reshape(m, n).copy()
            assert_close(got, want, rel=1e-4, what=f"run {run} {m}x{n}")
            if run == 0:
                first.append(got)
            else:
                assert np.array_equal(got, first[i]), f"{m}x{n}: the second run differs from the first"
    for run in (2, 3):                                    # accumulating runs: their second halves rely on the join leaving the workspace zero
        ffi.check(B.lib.ah_gemm_grouped_run(plan.value, ffi.EPI_ACCUM))
        for out, want, (m, n) in zip(outs, wants, shapes):
            B._dirty(out)
            assert_close(out.data.reshape(m, n), run * want, rel=1e-4, what=f"ACCUM {m}x{n}")
    # the same problems at other addresses (operands swapped in from fresh tensors, results into fresh tensors): the plan's
    # tables are rewritten in place; a list of other shapes is refused
    outs2, descs2 = [], []
    for d, (m, n) in zip(descs, shapes):
        src_g = TensorData((K, m), "f16", np.zeros(K * m, np.uint16))
        src_x = TensorData((K, n), "f16", np.zeros(K * n, np.uint16))
        ffi.check(B.lib.ah_copy(B._ptr(src_g), d.a, K * m * 2))
        ffi.check(B.lib.ah_copy(B._ptr(src_x), d.b, K * n * 2))
        out = B.zeros((m, n))
        keep += [src_g, src_x]
        outs2.append(out)
        descs2.append(ffi.AhGemm(ffi.GEMM_TN, ffi.BF16, ffi.F32, ffi.EPI_NONE, m, n, K, m, n, n, 1, 0, 0, 0, B._ptr(src_g), B._ptr(src_x), B._ptr(out), 0))
    arr2 = (ffi.AhGemm * len(descs2))(*descs2)
    ffi.check(B.lib.ah_gemm_grouped_update(plan.value, arr2, len(descs2)))
    ffi.check(B.lib.ah_gemm_grouped_run(plan.value, ffi.EPI_NONE))
    for i, (out, (m, n)) in enumerate(zip(outs2, shapes)):
        B._dirty(out)
        assert np.array_equal(out.data.reshape(m, n), first[i]), f"{m}x{n}: after the update"
    for out, want, (m, n) in zip(outs, wants, shapes):    # the old results were not touched by the run after the update
        B._dirty(out)
        assert_close(out.data.reshape(m, n), 3 * want, rel=1e-4, what=f"old C {m}x{n}")
    other = (ffi.AhGemm * len(descs2))(*descs2)
    other[0].k = K + 64
    assert B.lib.ah_gemm_grouped_update(plan.value, other, len(descs2)) != 0 and b"shapes the plan was made for" in B.lib.ah_last_error()
    assert B.lib.ah_gemm_grouped_update(plan.value, arr2, len(descs2) - 1) != 0
    ffi.check(B.lib.ah_gemm_grouped_destroy(plan.value))
    assert B.lib.ah_gemm_grouped_update(plan.value, arr2, len(descs2)) != 0 and b"unknown plan" in B.lib.ah_last_error()


# ---------------------------------------------------------------------------------------------- parity at the benchmark sizes
def _gauss_bf16(shape, seed, std):
    g = np.random.default_rng(seed)
    x = g.standard_normal(shape, dtype=np.float32) * np.float32(std)
    return _bf16_round(x)[0]


@pytest.mark.parametrize("N", [768, 2304, 3072, 50304])
@pytest.mark.parametrize("in_dtype", ["bf16", "f32"])
def test_gemm_microbench_shapes_forward_and_both_backward(B, N, in_dtype):
    """C = A B^T, dA = G B, dB = G^T A at M = 16384 (B*T), K = 768, N as in the GEMM microbenchmark; operands
    N(0,1)*0.02, as f32 (fp32 MFMA) and rounded to bf16 (bf16 MFMA, fp32 accumulate).  The full products are too large for
    the CPU oracle, so a sample of output rows is read back and checked against float64 numpy products of the same operands."""
    import ctypes as C
    from alpha2_amd import _ffi as ffi
    M, K = 16384, 768
    lib = B.lib
    idt = ffi.BF16 if in_dtype == "bf16" else ffi.F32

    def bits_of(shape, seed):           # the operand as the device stores it, and nothing else kept on the host
        x = np.random.default_rng(seed).standard_normal(shape, dtype=np.float32)
        x *= np.float32(0.02)
        if in_dtype == "f32":
            return x
        u = x.view(np.uint32)
        u += np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))          # round to nearest even
        return (u >> np.uint32(16)).astype(np.uint16)

    def f64(bits):
        if bits.dtype == np.float32:
            return bits.astype(np.float64)
        return (bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)

    def up(bits):
        p = C.c_uint64()
        ffi.check(lib.ah_alloc(bits.nbytes, C.byref(p)))
        ffi.check(lib.ah_upload(p.value, bits.ctypes.data_as(C.c_void_p), bits.nbytes))
        return p.value

    def rows_of(ptr, rows, ncols):
        out = np.empty((len(rows), ncols), np.float32)
        for i, r in enumerate(rows):
            ffi.check(lib.ah_download(out[i].ctypes.data_as(C.c_void_p), ptr + int(r) * ncols * 4, ncols * 4))
        return out
    a, b, g_ = bits_of((M, K), 2), bits_of((N, K), 3), bits_of((M, N), 4)
    pa, pb, pg = up(a), up(b), up(g_)
    pick = np.random.default_rng(5)
    rows_m, rows_n = np.sort(pick.choice(M, 24, replace=False)), np.sort(pick.choice(N, 24, replace=False))
    out = C.c_uint64()
    ffi.check(lib.ah_alloc(max(M * N, N * K, M * K) * 4, C.byref(out)))
    run = lambda layout, pa_, pb_, m, n, k, lda, ldb: ffi.check(lib.ah_gemm(C.byref(
        ffi.AhGemm(layout, idt, ffi.F32, ffi.EPI_NONE, m, n, k, lda, ldb, n, 1, 0, 0, 0, pa_, pb_, out.value, 0))))
    run(ffi.GEMM_NT, pa, pb, M, N, K, K, K)
    assert_close(rows_of(out.value, rows_m, N), f64(a[rows_m]) @ f64(b).T, rel=1e-4, what=f"C rows N={N}")
    run(ffi.GEMM_NN, pg, pb, M, K, N, N, K)                                   # dA = G [M,N] x B [N,K]
    assert_close(rows_of(out.value, rows_m, K), f64(g_[rows_m]) @ f64(b), rel=1e-4, what=f"dA rows N={N}")
    run(ffi.GEMM_TN, pg, pa, N, K, M, N, K)                                   # dB = G^T [N,M] x A [M,K]
    assert_close(rows_of(out.value, rows_n, K), f64(np.ascontiguousarray(g_[:, rows_n])).T @ f64(a), rel=1e-4, what=f"dB rows N={N}")
    for p in (pa, pb, pg, out.value):
        lib.ah_free(p)


@pytest.mark.parametrize("M,Cc", [(16384, 768), (4096, 768), (8192, 1024)])
def test_gemm_with_an_operand_in_planes_equals_the_product_around_copies(B, M, Cc):
    """ah_gemm_planes: the fused qkv projection writing q, k, v as three contiguous [M, C] matrices (what sliceQkv,
    ops.ts:816-840, makes of the [M, 3C] product) and the input gradient read from dq, dk, dv lying apart (what three
    scatterSlice results added up, ops.ts:826-834, would hold as one [M, 3C] matrix): bit for bit the ordinary products
    of the same operands, which are checked against float64 on sampled rows."""
    import ctypes as C
    from alpha2_amd import _ffi as ffi
    lib = B.lib
    rng = np.random.default_rng(11)

    def bits(shape, std):
        x = (rng.standard_normal(shape, dtype=np.float32) * np.float32(std)).view(np.uint32)
        x += np.uint32(0x7FFF) + ((x >> np.uint32(16)) & np.uint32(1))
        return (x >> np.uint32(16)).astype(np.uint16)
    f64 = lambda u: (u.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    live = []

    def up(u):
        p = C.c_uint64()
        ffi.check(lib.ah_alloc(max(u.nbytes, 16), C.byref(p)))
        ffi.check(lib.ah_upload(p.value, u.ctypes.data_as(C.c_void_p), u.nbytes))
        live.append(p.value)
        return p.value

    def down(ptr, shape):
        out = np.empty(shape, np.uint16)
        ffi.check(lib.ah_download(out.ctypes.data_as(C.c_void_p), ptr, out.nbytes))
        return out
    x, w, g = bits((M, Cc), 1.0), bits((3 * Cc, Cc), 0.02), bits((M, 3 * Cc), 0.5)
    px, pw, pg = up(x), up(w), up(g)
    pg_planes = up(np.ascontiguousarray(g.reshape(M, 3, Cc).transpose(1, 0, 2)))            # [3][M][C]
    c1, c2 = up(np.zeros((M, 3 * Cc), np.uint16)), up(np.full((3, M, Cc), 0x7FC0, np.uint16))
    d1, d2 = up(np.zeros((M, Cc), np.uint16)), up(np.full((M, Cc), 0x7FC0, np.uint16))
    BF = ffi.BF16
    # forward: [M, C] x [3C, C]^T
    fwd = ffi.AhGemm(ffi.GEMM_NT, BF, BF, ffi.EPI_NONE, M, 3 * Cc, Cc, Cc, Cc, 3 * Cc, 1, 0, 0, 0, px, pw, c1, 0)
    ffi.check(lib.ah_gemm(C.byref(fwd)))
    fwd.ldc, fwd.c = Cc, c2
    ffi.check(lib.ah_gemm_planes(C.byref(fwd), Cc, M * Cc, 0, 0, 1))                          # asked first, nothing launched
    assert (down(c2, (8,)) == 0x7FC0).all()
    ffi.check(lib.ah_gemm_planes(C.byref(fwd), Cc, M * Cc, 0, 0, 0))
    assert B.lastGemmKernel()[0].startswith("k_gemm_bf16_dma_planes<false, false")
    whole, planes = down(c1, (M, 3 * Cc)), down(c2, (3, M, Cc))
    for p in range(3):
        assert np.array_equal(planes[p], whole[:, p * Cc:(p + 1) * Cc]), p
    rows = np.sort(rng.choice(M, 16, replace=False))
    assert_close(f64(whole[rows]), f64(x[rows]) @ f64(w).T, rel=1e-2, what="qkv rows")         # (bf16 result: half an ulp is 2^-9)
    # input gradient: [M, 3C] x [3C, C]
    bwd = ffi.AhGemm(ffi.GEMM_NN, BF, BF, ffi.EPI_NONE, M, Cc, 3 * Cc, 3 * Cc, Cc, Cc, 1, 0, 0, 0, pg, pw, d1, 0)
    ffi.check(lib.ah_gemm(C.byref(bwd)))
    bwd.lda, bwd.a, bwd.c = Cc, pg_planes, d2
    ffi.check(lib.ah_gemm_planes(C.byref(bwd), 0, 0, Cc, M * Cc, 0))
    assert B.lastGemmKernel()[0].startswith("k_gemm_bf16_dma_planes<false, true")
    whole, planes = down(d1, (M, Cc)), down(d2, (M, Cc))
    assert np.array_equal(whole, planes)
    assert_close(f64(planes[rows]), f64(g[rows]) @ f64(w), rel=1e-2, what="dx rows")
    # what it does not take is refused with a reason and nothing is launched
    small = ffi.AhGemm(ffi.GEMM_NT, BF, BF, ffi.EPI_NONE, 128, 3 * Cc, Cc, Cc, Cc, Cc, 1, 0, 0, 0, px, pw, c2, 0)
    assert lib.ah_gemm_planes(C.byref(small), Cc, 128 * Cc, 0, 0, 1) == 5
    f32out = ffi.AhGemm(ffi.GEMM_NT, BF, ffi.F32, ffi.EPI_NONE, M, 3 * Cc, Cc, Cc, Cc, Cc, 1, 0, 0, 0, px, pw, c2, 0)
    assert lib.ah_gemm_planes(C.byref(f32out), Cc, M * Cc, 0, 0, 0) == 5
    ragged = ffi.AhGemm(ffi.GEMM_NT, BF, BF, ffi.EPI_NONE, M, 3 * Cc, Cc, Cc, Cc, Cc, 1, 0, 0, 0, px, pw, c2, 0)
    assert lib.ah_gemm_planes(C.byref(ragged), Cc - 64, M * Cc, 0, 0, 0) == 2
    assert lib.ah_gemm_planes(C.byref(ragged), Cc, M * Cc - 8, 0, 0, 0) == 2 and b"overlap" in lib.ah_last_error()
    for p in live:
        lib.ah_free(p)


@pytest.mark.parametrize("BH,T,D", [(20, 384, 64), (60, 2048, 128)])
@pytest.mark.parametrize("store", ["bf16", "f32"])
def test_flash_attention_heads_are_independent_of_how_blocks_are_dealt_out(B, store, BH, T, D):
    """The kernels decode (head, sequence block) from the linear workgroup id so that a head's blocks share one XCD and an
    XCD runs the longest blocks of a group of its heads first; heads past the last multiple of 8 keep the natural order.
    One call over all heads must equal, bit for bit, one call per head (where the mapping is the identity).  20 heads x 3
    blocks: one group of 2 heads per XCD and 4 heads left over; 60 heads x 16 blocks at head size 128: 7 heads per XCD in
    groups of 6 + 1 (bf16) or 3 + 3 + 1 (f32), 4 left over."""
    scale, cap = float(1.0 / np.sqrt(D)), 30.0
    q, k, v, do = (_gauss_bf16((BH, T, D), 60 + i, 1.0) for i in range(4))
    put = (lambda x: B.castStore(dev(B, x), "bf16")) if store == "bf16" else (lambda x: dev(B, x))
    r = B.flashAttention(put(q), put(k), put(v), T, scale, cap)
    g = B.flashAttentionBackward(put(q), put(k), put(v), r["output"], put(do), r["lse"], T, scale, cap)
    whole = [np.asarray(t.data).reshape(BH, T, -1).copy() for t in (r["output"], g["dQ"], g["dK"], g["dV"])] + [np.asarray(r["lse"].data).reshape(BH, T).copy()]
    for h in range(BH):
        one = lambda x: put(x[h:h + 1])
        r1 = B.flashAttention(one(q), one(k), one(v), T, scale, cap)
        g1 = B.flashAttentionBackward(one(q), one(k), one(v), r1["output"], one(do), r1["lse"], T, scale, cap)
        single = [np.asarray(t.data).reshape(T, -1) for t in (r1["output"], g1["dQ"], g1["dK"], g1["dV"])] + [np.asarray(r1["lse"].data).reshape(T)]
        for a, b_, what in zip(whole, single, ("O", "dQ", "dK", "dV", "LSE")):
            assert np.array_equal(a[h], b_), (h, what)


@pytest.mark.parametrize("T", [256, 1024, 2048])
@pytest.mark.parametrize("cap", [0.0, 30.0])
def test_flash_attention_microbench_shapes(B, bwd_variant, T, cap):
    """B = 16, H = 12, head_dim 64, bf16 in / fp32 accumulate, scale 1/8, as in the attention microbenchmark.  The kernels
    run on all 192 heads; three of them (first, a middle one, last) are checked against the oracle's materialised chain."""
    BH, D, scale = 192, 64, 0.125
    q, k, v, do = (_gauss_bf16((BH, T, D), 30 + i, 1.0) for i in range(4))
    Q, K, V, dO = (B.castStore(dev(B, x), "bf16") for x in (q, k, v, do))
    r = B.flashAttention(Q, K, V, T, scale, cap)
    g = B.flashAttentionBackward(Q, K, V, r["output"], dO, r["lse"], T, scale, cap)
    heads = [0, 77, 191]
    want_o, want_lse, dq, dk, dv = _oracle_attention(q[heads], k[heads], v[heads], do[heads], scale, cap)
    rel = 2.0 ** -6

    def loose(x):
        return dict(outlier_frac=2e-3, outlier_abs=0.1 * float(np.sqrt(np.mean(np.square(x)))) + 1e-6)
    sel = lambda t: np.asarray(t.data).reshape(BH, T, -1)[heads]
    # sums of bf16-rounded probabilities: a few entries in a hundred thousand sit a little outside the element-wise bound
    assert_close(sel(r["output"]), want_o.reshape(3, T, D), rel=rel, what="O", **loose(want_o))
    assert_close(np.asarray(r["lse"].data).reshape(BH, T)[heads], want_lse.reshape(3, T), rel=1e-4, what="LSE")
    assert_close(sel(g["dQ"]), dq.reshape(3, T, D), rel=rel, what="dQ", **loose(dq))
    assert_close(sel(g["dK"]), dk.reshape(3, T, D), rel=rel, what="dK", **loose(dk))
    assert_close(sel(g["dV"]), dv.reshape(3, T, D), rel=rel, what="dV", **loose(dv))


@pytest.mark.parametrize("K", [128, 192])      # every problem cut in two along k (the joining kernel sums) / none cut (the epilogue sums)
def test_gemm_grouped_sum_of_squares_is_not_finite_when_a_product_is_not(B, K):
    """The trainer skips a step whose gradient norm is not finite (trainer.ts:1248,1495-1522): an Inf or a NaN that a weight-gradient
    product stores must reach the sum its launch takes, also from the last row of a ragged tile."""
    import ctypes as C
    import math
    from alpha2_amd import TensorData, _ffi as ffi
    for bad in (np.inf, np.nan):
        keep, descs = [], []
        for m, n, poison in ((256, 256, False), (264, 520, True), (512, 256, False)):
            gy, x = _bf16_round(rs.randn(K, m).astype(np.float32))[0], _bf16_round(rs.randn(K, n).astype(np.float32))[0]
            if poison:
                gy[5, m - 1] = bad                                            # reaches row m - 1 of C, in the ragged edge tile
            tg, tx = TensorData(gy.shape, "f16", _bf16_round(gy)[1]), TensorData(x.shape, "f16", _bf16_round(x)[1])
            out = B.zeros((m, n))
            keep += [tg, tx, out]
            descs.append(ffi.AhGemm(ffi.GEMM_TN, ffi.BF16, ffi.F32, ffi.EPI_NONE, m, n, K, m, n, n, 1, 0, 0, 0, B._ptr(tg), B._ptr(tx), B._ptr(out), 0))
        arr = (ffi.AhGemm * len(descs))(*descs)
        plan = C.c_uint64()
        ffi.check(B.lib.ah_gemm_grouped_plan(arr, len(descs), C.byref(plan)))
        acc = TensorData((1,), "f32", np.array([0.0], np.float32))
        ffi.check(B.lib.ah_gemm_grouped_run_sumsq(plan.value, ffi.EPI_NONE, B._ptr(acc)))
        assert B.lastGemmKernel()[1] == (2 if K % 128 == 0 else 1)
        B._dirty(acc)
        assert not math.isfinite(float(acc.data[0])), (bad, float(acc.data[0]))
        ffi.check(B.lib.ah_gemm_grouped_destroy(plan.value))


def test_mfma_probe_runs_and_refuses_sizes_outside_its_range(B):
    """The measurement aid launches and finishes (every wave runs a counted loop), reports the flops of its launch, and
    refuses iteration counts and wave counts beyond its stated range."""
    import ctypes as C
    from alpha2_amd import _ffi as ffi
    fl = C.c_double()
    for random_ops in (0, 1):
        ffi.check(B.lib.ah_probe_mfma_bf16(2, 50, random_ops, C.byref(fl)))
    ffi.check(B.lib.ah_sync())
    info = ffi.AhDeviceInfo()
    ffi.check(B.lib.ah_device_info(C.byref(info)))
    assert fl.value == info.compute_units * 2 * 4 * 50 * 8 * 2.0 * 32 * 32 * 16
    assert B.lib.ah_probe_mfma_bf16(5, 50, 1, None) != 0 and b"1-4 waves" in B.lib.ah_last_error()
    assert B.lib.ah_probe_mfma_bf16(1, 200001, 1, None) != 0


def test_issue_probe_runs_and_refuses_sizes_outside_its_range(B):
    """The issue-rate aid launches and finishes for every kind of group (every wave runs a counted loop), reports the groups
    issued per SIMD, and refuses kinds, wave counts and iteration counts beyond its stated range."""
    import ctypes as C
    from alpha2_amd import _ffi as ffi
    n = C.c_double()
    for kind in range(6):
        for waves in ((1, 4) if kind < 3 else (1, 2)):
            ffi.check(B.lib.ah_probe_issue(kind, waves, 20, C.byref(n)))
            assert n.value == 20 * 32 * waves
    ffi.check(B.lib.ah_sync())
    assert B.lib.ah_probe_issue(6, 1, 20, None) != 0 and b"kind 0-5" in B.lib.ah_last_error()
    assert B.lib.ah_probe_issue(3, 3, 20, None) != 0
    assert B.lib.ah_probe_issue(0, 5, 20, None) != 0
    assert B.lib.ah_probe_issue(0, 1, 200001, None) != 0


def test_the_extras_the_trainer_calls_on_a_gpu_backend(B):
    """resetStepOps / gpuOpsThisStep and purgeBufferPools, which the reference trainer calls when the backend has them
    (trainer.ts:1003-1032,1915,1956): the launch counter restarts and counts, and purging the pool frees every cached block
    without touching live tensors."""
    x = dev(B, rs.randn(1000).astype(np.float32))
    B.resetStepOps()
    assert B.gpuOpsThisStep == 0
    tmp = [B.scale(x, float(i)) for i in range(1, 6)]
    assert B.gpuOpsThisStep >= 5
    want = [t.data.copy() for t in tmp]
    keep = tmp.pop()
    for t in tmp:
        B.releaseGpuTensor(t)
    B.syncGpu()
    assert B.gpuMemStats()["bufferPoolEntries"] >= 4
    live = B.gpuMemStats()["liveAllocs"]
    B.purgeBufferPools()
    st = B.gpuMemStats()
    assert st["bufferPoolEntries"] == 0 and st["bufferPoolBytes"] == 0 and st["liveAllocs"] == live
    B._dirty(keep)
    assert np.array_equal(keep.data, want[-1])                  # a live tensor is where it was
    assert_close(B.scale(x, 2.0).data, 2 * x.data, what="an op after the purge")
