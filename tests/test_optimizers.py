"""Lion, Adafactor and SGD (packages/train/src/optimizers.ts:236-603): the oracle restatement against closed forms and the
reference's own test properties (packages/tests/src/optimizer.test.ts), then the device kernels against the oracle."""
import math

import numpy as np
import pytest

from oracle import ref_model as M
from oracle.ref import TD


class _Var:
    def __init__(self, data, grad):
        self.data, self.grad = data, grad


def _entries(p, g, shape=None):
    shape = shape or (p.size,)
    return [("w", _Var(TD(shape, "f32", p), TD(shape, "f32", g)))]


# ---------------------------------------------------------------------------------------------- oracle: closed forms

def test_lion_first_step_is_a_sign_step_with_decoupled_decay():
    """With zero momentum the interpolated update is (1 - beta1) g, so the first step moves every weight by exactly lr
    against the sign of its gradient after shrinking it by (1 - lr wd), and the momentum becomes (1 - beta2) g."""
    p0 = np.array([1.0, -2.0, 0.5, 3.0, 0.25], dtype=np.float32)
    g = np.array([0.4, -0.2, 0.8, -0.5, 0.0], dtype=np.float32)
    p = p0.copy()
    opt = M.Lion(lr=1e-2, beta1=0.9, beta2=0.99, weightDecay=0.1)
    opt.stepParamEntries(_entries(p, g))
    want = p0.astype(np.float64) * (1 - 1e-2 * 0.1) - 1e-2 * np.array([1, -1, 1, -1, 0])
    np.testing.assert_allclose(p, want, rtol=0, atol=1e-7)
    np.testing.assert_allclose(opt.m["w"], 0.01 * g.astype(np.float64), rtol=1e-6)
    assert opt.state_dict()["step"] == 1 and list(opt.state_dict()["buffers"]) == ["w.m"]


def test_lion_second_step_uses_the_momentum_not_the_gradient_alone():
    """A small gradient of opposite sign must not flip the direction while beta1 m still dominates."""
    p = np.array([0.0], dtype=np.float32)
    opt = M.Lion(lr=1.0, beta1=0.9, beta2=0.5, weightDecay=0.0)
    opt.stepParamEntries(_entries(p, np.array([1.0], dtype=np.float32)))          # p = -1, m = 0.5
    opt.stepParamEntries(_entries(p, np.array([-0.1], dtype=np.float32)))         # update = 0.45 - 0.01 > 0: p = -2
    assert p[0] == -2.0 and abs(opt.m["w"][0] - (0.25 - 0.05)) < 1e-7


def test_adafactor_rank_one_gradient_gives_a_pure_sign_step():
    """For g = a b^T the factored second moment reproduces g^2 exactly, every update entry has magnitude
    1 / sqrt(1 - beta2), so its RMS is that too and clipping at 1 scales the step to exactly lr * sign(g)."""
    a = np.array([0.5, -2.0, 1.5, 0.25], dtype=np.float64)
    b = np.array([1.0, -0.5, 3.0], dtype=np.float64)
    g = np.outer(a, b).astype(np.float32)
    p0 = np.linspace(-1, 1, 12).astype(np.float32).reshape(4, 3)
    p = p0.copy()
    opt = M.Adafactor(lr=1e-2, beta2=0.999, eps=1e-30, clipThreshold=1.0, weightDecay=0.0)
    opt.stepParamEntries(_entries(p, g, (4, 3)))
    np.testing.assert_allclose(p, p0 - 1e-2 * np.sign(g), rtol=0, atol=2e-7)
    assert list(opt.state_dict()["buffers"]) == ["w.vr", "w.vc"]
    np.testing.assert_allclose(opt.vr["w"], 0.001 * (a * a) * np.mean(b * b), rtol=1e-6)
    np.testing.assert_allclose(opt.vc["w"], 0.001 * (b * b) * np.mean(a * a), rtol=1e-6)


def test_adafactor_unfactored_branch_and_clip_disabled():
    """A 1-D parameter keeps a full second moment; with clipping off the first step is lr * g / sqrt((1 - beta2) g^2),
    i.e. lr * sign(g) / sqrt(1 - beta2), after the decoupled decay."""
    g = np.array([0.3, -0.7, 2.0], dtype=np.float32)
    p0 = np.array([1.0, 2.0, -3.0], dtype=np.float32)
    p = p0.copy()
    opt = M.Adafactor(lr=1e-3, beta2=0.99, eps=1e-30, clipThreshold=0.0, weightDecay=0.5)
    opt.stepParamEntries(_entries(p, g))
    want = p0.astype(np.float64) * (1 - 1e-3 * 0.5) - 1e-3 * np.sign(g) / math.sqrt(0.01)
    np.testing.assert_allclose(p, want, rtol=0, atol=3e-7)
    assert list(opt.state_dict()["buffers"]) == ["w.v"]


def test_sgd_known_answer():
    p = np.array([2.0, -1.0, 0.75], dtype=np.float32)
    M.SGD(0.1).stepParamEntries(_entries(p, np.array([0.5, 0.25, -1.0], dtype=np.float32)), 0.25)
    np.testing.assert_allclose(p, [2.0 - 0.0125, -1.0 - 0.00625, 0.75 + 0.025], rtol=0, atol=1e-7)


@pytest.mark.parametrize("make", [lambda: M.Lion(lr=1e-4, beta1=0.9, beta2=0.99, weightDecay=0.01),
                                  lambda: M.Adafactor(lr=1e-3, beta2=0.999, eps=1e-30, clipThreshold=1e9, weightDecay=0.01),
                                  lambda: M.SGD(0.1)])
def test_grad_scale_equals_prescaled_gradients(make):
    """optimizer.test.ts:47-198: stepping with gradScale s equals stepping on gradients multiplied by s beforehand."""
    p0 = np.array([1.0, -2.0, 0.5, 3.0, -1.0, 2.0], dtype=np.float32)
    g = np.array([0.4, -0.2, 0.8, -0.5, 0.1, 0.3], dtype=np.float32)
    s = 0.25                                                    # a power of two: the pre-scaling itself is exact
    pa, pb = p0.copy(), p0.copy()
    make().stepParamEntries(_entries(pa, g, (2, 3)), s)
    make().stepParamEntries(_entries(pb, (g * np.float32(s)).astype(np.float32), (2, 3)))
    assert np.max(np.abs(pa - pb)) < 1e-8


# ---------------------------------------------------------------------------------------------- device kernels vs the oracle

@pytest.fixture(scope="module")
def B():
    from alpha2_amd import HipBackend
    return HipBackend(0)


def _dev_entries(B, p, g, shape):
    from alpha2_amd import TensorData
    return [("w", _Var(TensorData(shape, "f32", p.copy()), TensorData(shape, "f32", g.copy())))]


@pytest.mark.gpu
@pytest.mark.parametrize("n", [1, 5, 1000, 70001])
def test_lion_and_sgd_kernels_reproduce_the_host_loops_bit_for_bit(B, n):
    from alpha2_amd.optimizers import Lion, SGD
    rs = np.random.RandomState(n)
    p0, steps = rs.randn(n).astype(np.float32), [rs.randn(n).astype(np.float32) * 10.0 ** rs.randint(-6, 2) for _ in range(3)]
    steps[1][: n // 2] = 0.0                                    # sign(0) = 0 entries
    want = p0.copy()
    ora, dev = M.Lion(lr=3e-3, beta1=0.9, beta2=0.95, weightDecay=0.1), Lion(B, lr=3e-3, beta1=0.9, beta2=0.95, weightDecay=0.1)
    ent = _dev_entries(B, p0, steps[0], (n,))
    for k, g in enumerate(steps):
        scale = 1.0 if k == 0 else 0.37
        ora.stepParamEntries(_entries(want, g), scale)
        ent[0][1].grad = type(ent[0][1].data)((n,), "f32", g.copy())
        dev.stepParamEntries(ent, scale)
        assert np.array_equal(ent[0][1].data.data, want), f"step {k}"
    assert np.array_equal(dev.stateDict()["buffers"]["w.m"].data, ora.m["w"])
    want2, ent2 = p0.copy(), _dev_entries(B, p0, steps[2], (n,))
    M.SGD(0.05).stepParamEntries(_entries(want2, steps[2]), 0.5)
    SGD(B, 0.05).stepParamEntries(ent2, 0.5)
    assert np.array_equal(ent2[0][1].data.data, want2)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(2, 3), (1, 7), (33, 65), (768, 96), (5,), (3, 4, 5), (4097,)])
def test_adafactor_kernels_match_the_host_loops(B, shape):
    """Both branches, three steps with state carried over, decay and clipping active.  The kernels sum in double like the
    reference but block-wise instead of left to right, so the comparison allows one f32 rounding (1e-6 relative)."""
    from alpha2_amd import TensorData
    from alpha2_amd.optimizers import Adafactor
    n = int(np.prod(shape))
    rs = np.random.RandomState(n)
    p0 = rs.randn(n).astype(np.float32)
    cfg = dict(lr=1e-2, beta2=0.99, eps=1e-30, clipThreshold=1.0, weightDecay=0.05)
    ora, dev = M.Adafactor(**cfg), Adafactor(B, **cfg)
    want = p0.copy().reshape(shape)
    ent = _dev_entries(B, p0, p0, shape)
    for k in range(3):
        g = (rs.randn(n) * (0.1 + k)).astype(np.float32)
        ora.stepParamEntries([("w", _Var(TD(shape, "f32", want), TD(shape, "f32", g)))], 0.5 if k == 1 else 1.0)
        ent[0][1].grad = TensorData(shape, "f32", g.copy())
        dev.stepParamEntries(ent, 0.5 if k == 1 else 1.0)
        got = np.asarray(ent[0][1].data.data).reshape(shape)
        np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-7, err_msg=f"step {k}")
    od, dd = ora.state_dict()["buffers"], dev.stateDict()["buffers"]
    assert list(od) == list(dd)
    for key in od:
        np.testing.assert_allclose(dd[key].data, od[key].data, rtol=1e-6, atol=0)


def test_adafactor_with_a_gradient_that_is_not_finite_poisons_the_whole_tensor():
    """Math.max(1, rms / clip) is NaN when the update's RMS is (optimizers.ts:465-466,498-499), and the step scale with it:
    one NaN or infinite gradient entry makes every parameter of the tensor NaN, in both branches (Python's max would keep 1)."""
    for shape in ((6,), (2, 3)):
        p = np.arange(1, 7, dtype=np.float32)
        g = np.array([0.1, -0.2, np.nan, 0.3, 0.4, -0.5], dtype=np.float32)
        M.Adafactor(lr=1e-2, beta2=0.99, eps=1e-30, clipThreshold=1.0, weightDecay=0.0).stepParamEntries(_entries(p, g, shape))
        assert np.isnan(p).all(), (shape, p)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(12,), (3, 4)])
def test_optimizer_kernels_on_gradients_at_the_ends_of_the_range(B, shape):
    """Infinite, NaN, denormal and largest-finite gradient entries through two steps of each optimizer: the device gives what the
    host loops give, NaN for NaN (sign(NaN), Math.max with a NaN) included."""
    from alpha2_amd import TensorData
    from alpha2_amd.optimizers import Adafactor, Lion, SGD
    p0 = np.array([1.0, -2.0, 0.5, 3.0, 0.0, -0.0, 1e-30, 1e30, 7.0, -7.0, 2.0, 2.0], np.float32)
    g0 = np.array([np.inf, -np.inf, np.nan, 0.0, -0.0, 1e-45, 3.4e38, -3.4e38, 1e-20, -1e-20, 1.0, -1.0], np.float32)
    makers = (("lion", lambda: M.Lion(lr=3e-3, beta1=0.9, beta2=0.95, weightDecay=0.1), lambda: Lion(B, lr=3e-3, beta1=0.9, beta2=0.95, weightDecay=0.1)),
              ("sgd", lambda: M.SGD(0.05), lambda: SGD(B, 0.05)),
              ("adafactor", lambda: M.Adafactor(lr=1e-2, beta2=0.99, eps=1e-30, clipThreshold=1.0, weightDecay=0.05),
               lambda: Adafactor(B, lr=1e-2, beta2=0.99, eps=1e-30, clipThreshold=1.0, weightDecay=0.05)))
    for name, mk_o, mk_d in makers:
        for g in (g0, np.where(np.isfinite(g0), g0, 1.0).astype(np.float32)):
            want, o, d = p0.copy(), mk_o(), mk_d()
            ent = _dev_entries(B, p0, g, shape)
            for k in range(2):
                o.stepParamEntries(_entries(want, g, shape), 0.5)
                ent[0][1].grad = TensorData(shape, "f32", g.copy())
                d.stepParamEntries(ent, 0.5)
            got = np.asarray(ent[0][1].data.data).reshape(-1)
            assert np.array_equal(np.isnan(got), np.isnan(want)), (name, got, want)
            ok = ~np.isnan(want)
            np.testing.assert_allclose(got[ok], want[ok], rtol=2e-6, atol=1e-37, err_msg=name)


@pytest.mark.gpu
def test_optimizer_registry_and_state_round_trip(B):
    from alpha2_amd import TensorData
    from alpha2_amd.optimizers import createOptimizerRegistry
    reg = createOptimizerRegistry(B)
    assert sorted(reg) == ["adafactor", "adamw", "lion", "sgd"]                 # optimizers.ts:596-603
    rs = np.random.RandomState(3)
    for name in ("lion", "adafactor"):
        a, b = reg[name](), reg[name]()
        ent = _dev_entries(B, rs.randn(12).astype(np.float32), rs.randn(12).astype(np.float32), (3, 4))
        a.stepParamEntries(ent)
        b.loadStateDict(a.stateDict())
        sa, sb = a.stateDict(), b.stateDict()
        assert sa["step"] == sb["step"] == 1 and list(sa["buffers"]) == list(sb["buffers"])
        # resuming from the copied state continues identically (entry form and map form, optimizer.test.ts:95-232)
        ent_b = _dev_entries(B, np.asarray(ent[0][1].data.data), np.asarray(ent[0][1].grad.data), (3, 4))
        a.stepParamEntries(ent, 0.45)
        b.step({"w": ent_b[0][1].data}, {"w": ent_b[0][1].grad}, 0.45)
        assert np.array_equal(ent[0][1].data.data, ent_b[0][1].data.data)
