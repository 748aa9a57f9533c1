"""Step plans (ah_step_begin / ah_step_end): the generic tape-driven trainer issues the same Backend calls every step;
the library records them once as hipGraph segments and replays them.  Replayed steps must give exactly what eager
execution gives (the same kernels in the same order: bit-identical), and a step that deviates from the plan must fall back
to eager execution with the right results."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

CFG = dict(vocabSize=96, blockSize=32, nLayer=2, nEmbd=64, nHead=2)


@pytest.fixture()
def B():
    from alpha2_amd import HipBackend
    b = HipBackend(0)
    b.resetStepPlan()
    yield b
    b.enableStepGraphs(False)
    b.resetStepPlan()


def _trainer(B, accum=1, **kw):
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig, Trainer
    return Trainer(B, ModelConfig(**dict(CFG, **kw)), TrainConfig(iters=12, gradAccumSteps=accum), seed=3)


def _run(B, graphs, steps=8, accum=1, batch_of=None, **kw):
    from alpha2_amd.train import syntheticBatch
    tr = _trainer(B, accum, **kw)
    B.enableStepGraphs(graphs)
    out, hows = [], []
    for s in range(steps):
        bs = batch_of(s) if batch_of else [syntheticBatch(40 + accum * s + m, 4, 32, 96) for m in range(accum)]
        r = tr.step(bs)
        out.append((r.loss, r.gradNorm, r.clipCoef, r.lr))
        hows.append(B.lastStepHow if graphs else "eager")
    B.enableStepGraphs(False)
    params = {n: v.data.data.copy() for n, v in tr.entries}
    return out, hows, params


@pytest.mark.parametrize("accum", [1, 2])
def test_replayed_steps_are_bit_identical_to_eager_steps(B, accum):
    before = B.stepStats()
    eager, _, pe = _run(B, False, accum=accum)
    graph, hows, pg = _run(B, True, accum=accum)
    after = B.stepStats()
    assert graph == eager, (graph, eager)
    for n in pe:
        assert np.array_equal(pe[n], pg[n]), n
    # flush() ends step s and opens the plan for step s+1: step 0 runs before the first flush (eager, parameters are
    # uploaded and moments created), step 1 is recorded, every later step is replayed
    assert after["recorded"] - before["recorded"] == 1, (before, after, hows, B.lastStepNote)
    assert after["replayed"] - before["replayed"] >= 5 and after["fellBack"] == before["fellBack"], (before, after, B.lastStepNote)


def test_a_step_that_deviates_falls_back_and_the_plan_is_recorded_again(B):
    """Step 4 uses a batch of another size: other grids, so the replay stops at the first launch that differs, the step
    finishes eagerly with the right numbers, and the following steps record and replay a new plan."""
    from alpha2_amd.train import syntheticBatch

    def batch_of(s):
        return [syntheticBatch(70 + s, 2 if s == 4 else 4, 32, 96)]
    before = B.stepStats()
    eager, _, pe = _run(B, False, steps=9, batch_of=batch_of)
    graph, hows, pg = _run(B, True, steps=9, batch_of=batch_of)
    after = B.stepStats()
    assert graph == eager
    for n in pe:
        assert np.array_equal(pe[n], pg[n]), n
    assert after["fellBack"] - before["fellBack"] >= 1 and after["recorded"] - before["recorded"] >= 2
    assert after["replayed"] - before["replayed"] >= 3


def test_resetting_the_plan_makes_the_next_bracketed_step_record_again(B):
    """resetStepPlan forgets the recorded plan: refused while a step is open, and after it the next bracketed step is recorded
    anew and the following ones replay it - with the numbers of eager execution all along."""
    from alpha2_amd._ffi import AlphaHipError
    from alpha2_amd.train import syntheticBatch
    eager, _, _ = _run(B, False, steps=9)
    tr = _trainer(B)
    got = []

    def go(lo, hi):
        for s in range(lo, hi):
            r = tr.step([syntheticBatch(40 + s, 4, 32, 96)])
            got.append((r.loss, r.gradNorm, r.clipCoef, r.lr))
    B.enableStepGraphs(True)
    go(0, 4)
    with pytest.raises(AlphaHipError, match="while a step is open"):
        B.resetStepPlan()
    B.enableStepGraphs(False)
    a = B.stepStats()
    B.resetStepPlan()
    B.enableStepGraphs(True)
    go(4, 9)
    B.enableStepGraphs(False)
    b = B.stepStats()
    assert b["recorded"] - a["recorded"] == 1 and b["replayed"] - a["replayed"] >= 2 and b["fellBack"] == a["fellBack"], (a, b, B.lastStepNote)
    assert got == eager


def test_per_step_scalars_and_dropout_seeds_follow_the_caller(B):
    """Learning rate, bias corrections, the clip coefficient and the dropout seed change every step: they are kernel
    arguments, rewritten in the graph nodes, not frozen at recording time."""
    eager, _, pe = _run(B, False, dropout=0.1)
    graph, hows, pg = _run(B, True, dropout=0.1)
    assert graph == eager
    assert len({x[3] for x in graph}) > 3                       # the schedule moved
    for n in pe:
        assert np.array_equal(pe[n], pg[n]), n


def test_a_kick_is_a_boundary_of_the_plan(B):
    """ah_step_kick launches what has been issued so far as a segment of its own: the same results as without it, expected at
    the same place on replay (a step that kicks elsewhere falls back), and a no-op outside a step or with nothing issued."""
    from alpha2_amd import TensorData
    from alpha2_amd._ffi import check
    x = TensorData((4096,), "f32", np.arange(4096, dtype=np.float32))
    assert B.lib.ah_step_kick() == 0                                 # outside a step
    B._ptr(x)                                                        # (uploaded before the plan, so every step issues the same calls)

    def step(kick_after):
        t = x
        check(B.lib.ah_step_kick())                                  # nothing issued yet
        for i in range(6):
            t = B.scale(t, 1.5)
            if i == kick_after:
                check(B.lib.ah_step_kick())
        return t

    B.enableStepGraphs(True)
    B.flush()
    want = x.data * np.float32(1.5) ** 6
    hows = []
    for kick_after in (2, 2, 2, 4, 2, 2):
        got = step(kick_after).data.copy()
        B.flush()
        hows.append(B.lastStepHow)
        assert np.array_equal(got, want), kick_after               # (every product is exact in f32)
    B.enableStepGraphs(False)
    assert hows[0] == "recorded" and hows[1] == hows[2] == "replayed", hows
    assert hows[3] == "fell-back" and hows[4] == "recorded" and hows[5] == "replayed", (hows, B.lastStepNote)


def test_an_early_read_back_waits_for_its_own_copy_only(B):
    """ah_download_begin / ah_download_end: the value is the one the tensor held when the copy was queued, whatever is issued
    (and overwrites the tensor) afterwards; a ticket whose slot has been taken by sixteen newer ones is refused; inside a step
    plan the pair gives the same values on recorded and replayed steps."""
    import ctypes as C
    from alpha2_amd import TensorData
    from alpha2_amd._ffi import check
    lib = B.lib
    x = TensorData((64,), "f32", np.arange(64, dtype=np.float32))
    p = B._ptr(x)

    def begin(ptr, nbytes):
        tk = C.c_uint64(0)
        check(lib.ah_download_begin(ptr, nbytes, C.byref(tk)))
        return tk.value

    def end(tk, n):
        out = np.empty(n, np.float32)
        rc = lib.ah_download_end(tk, out.ctypes.data_as(C.c_void_p), out.nbytes)
        return rc, out

    tk = begin(p + 16, 32)
    B.scaleInplace(x, 3.0)                                          # queued behind the copy: must not show in it
    big = B.scale(TensorData((1 << 22,), "f32", np.ones(1 << 22, np.float32)), 2.0)
    rc, got = end(tk, 8)
    assert rc == 0 and np.array_equal(got, np.arange(4, 12, dtype=np.float32))
    assert np.array_equal(x.data, 3 * np.arange(64, dtype=np.float32)) and float(big.data[5]) == 2.0
    old = begin(p, 4)
    for _ in range(16):
        last = begin(p, 4)
    assert end(old, 1)[0] != 0                                      # sixteen newer tickets took its slot
    rc, got = end(last, 1)
    assert rc == 0 and got[0] == 0.0
    assert lib.ah_download_end(last, got.ctypes.data_as(C.c_void_p), 8) != 0      # another size than was copied

    B.enableStepGraphs(True)
    B.flush()
    vals, hows = [], []
    for s in range(4):
        t = B.scale(x, float(s + 1))
        tk = begin(B._ptr(t) + 4, 4)
        t2 = B.scale(t, 10.0)
        rc, got = end(tk, 1)
        vals.append((rc, float(got[0]), float(t2.data[1])))
        B.flush()
        hows.append(B.lastStepHow)
    B.enableStepGraphs(False)
    assert vals == [(0, 3.0 * (s + 1), 30.0 * (s + 1)) for s in range(4)], vals
    assert hows[0] == "recorded" and hows[-1] == "replayed", hows
