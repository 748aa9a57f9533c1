"""The fast-mode (bf16 operands, fp32 accumulate / master weights) hand-scheduled step against the CPU oracle, and
its hipGraph replay against eager execution.  Bars from the task statement: step loss within 2e-2 relative of the
fp32 reference path; bf16-level agreement of gradients (direction and norm)."""
import math

import numpy as np
import pytest

from oracle import ref_model as rm

pytestmark = pytest.mark.gpu

CFG = dict(vocabSize=256, blockSize=64, nLayer=2, nEmbd=128, nHead=4)


@pytest.fixture(scope="module")
def B():
    from alpha2_amd import HipBackend
    return HipBackend(0)


def _make(B, tc_kw, use_graph, seed=0, batch=4, attention="heads", **kw):
    from alpha2_amd.fused import FusedTrainer
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig
    return FusedTrainer(B, ModelConfig(**CFG, attention=attention), TrainConfig(**tc_kw), batch, seed=seed, use_graph=use_graph, **kw)


# "heads": multi-head attention (the oracle's CPU branch, gpt.ts:255-279); "reference-flash": the slabs an unchanged gpt.ts
# hands to flashAttention (gpt.ts:247-254), which the fused step wires without moving data (ah_gemm_planes)
ATTENTION = ["heads", "reference-flash"]


@pytest.mark.parametrize("attention", ATTENTION)
def test_fused_step_gradients_and_update_match_oracle(B, attention):
    from alpha2_amd.train import syntheticBatch
    ft = _make(B, dict(iters=1), use_graph=False, attention=attention)
    assert ft.slabs == (attention == "reference-flash")
    orc = rm.Trainer(rm.ModelConfig(**CFG, attention=attention), rm.TrainConfig(iters=1), seed=0)
    for name, v in orc.entries:
        assert np.array_equal(ft.param(name), v.data.data), name          # same initial parameters, bit for bit
    ft.set_batch(*syntheticBatch(1, 4, 64, 256))
    ob = rm.synthetic_batch(1, 4, 64, 256)
    # oracle gradients before its optimizer step
    _, oloss = rm.gptForward(orc.cfg, orc.params, orc.B, orc.tape, ob[0], ob[1], True)
    orc.tape.backward(oloss, orc.B)
    ograds = {n: v.grad.data.copy() for n, v in orc.entries}
    orc.tape.clear()
    for _, v in orc.entries:
        v.grad = None
    o = orc.step([ob])
    ft.step()
    st = ft.history(0, 1)[0]
    assert abs(st.loss - o.loss) <= 2e-2 * abs(o.loss), (st.loss, o.loss)
    assert abs(st.gradNorm - o.gradNorm) <= 3e-2 * o.gradNorm, (st.gradNorm, o.gradNorm)
    assert abs(st.clipCoef - o.clipCoef) <= 3e-2
    for name, g in ograds.items():
        got = ft.grad(name).astype(np.float64)
        w = g.astype(np.float64)
        cos = float(got @ w / (np.linalg.norm(got) * np.linalg.norm(w) + 1e-300))
        assert cos > 0.995, (name, cos)
        assert abs(np.linalg.norm(got) / np.linalg.norm(w) - 1) < 3e-2, name
    for name, v in orc.entries:                                           # after AdamW: every entry moved by at most lr
        d = ft.param(name) - v.data.data
        assert np.max(np.abs(d)) <= 2 * 3e-4 * 1.001 + 1e-7, name
        assert np.sqrt(np.mean(d * d)) <= 0.35 * 3e-4, name               # and mostly in the same direction as the oracle


@pytest.mark.parametrize("attention", ATTENTION)
def test_fused_loss_parity_over_steps_graph_replay(B, attention):
    from alpha2_amd.train import syntheticBatch
    steps = 50
    tc = dict(iters=steps)
    ft = _make(B, tc, use_graph=True, seed=3, attention=attention)
    eager = _make(B, tc, use_graph=False, seed=3, attention=attention)
    orc = rm.Trainer(rm.ModelConfig(**CFG, attention=attention), rm.TrainConfig(iters=steps), seed=3)
    ids = [ft.add_batch(*syntheticBatch(50 + s, 4, 64, 256)) for s in range(steps)]
    for s in range(steps):
        eager.add_batch(*syntheticBatch(50 + s, 4, 64, 256))
    olosses = []
    for s in range(steps):
        ft.step(ids[s])
        eager.step(s)
        olosses.append(orc.step([rm.synthetic_batch(50 + s, 4, 64, 256)]))
    hg, he = ft.history(0, steps), eager.history(0, steps)
    for s in range(steps):
        assert abs(hg[s].loss - olosses[s].loss) <= 2e-2 * abs(olosses[s].loss), (s, hg[s].loss, olosses[s].loss)
        assert abs(hg[s].lr - olosses[s].lr) < 1e-12
        # every replay of the captured step equals the eager step (atomics in the embedding scatter-add aside)
        assert abs(hg[s].loss - he[s].loss) <= 1e-4 * abs(he[s].loss), (s, hg[s].loss, he[s].loss)
        assert abs(hg[s].gradNorm - he[s].gradNorm) <= 1e-3 * he[s].gradNorm
    assert all(math.isfinite(h.loss) for h in hg)
    ft.close(), eager.close()


@pytest.mark.parametrize("attention", ATTENTION)
def test_fused_step_with_head_size_16_tracks_the_oracle(B, attention):
    """nEmbd 128 with 8 heads, as in the reference's small domains (packages/core/src/domains.ts:30-31): the attention kernels of
    size 32 run with half their features read as zeros; 10 steps against the oracle, both wirings."""
    from alpha2_amd.fused import FusedTrainer
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig, syntheticBatch
    cfg = dict(CFG, nHead=8, attention=attention)
    ft = FusedTrainer(B, ModelConfig(**cfg), TrainConfig(iters=10), 4, seed=2)
    orc = rm.Trainer(rm.ModelConfig(**cfg), rm.TrainConfig(iters=10), seed=2)
    for s in range(10):
        ft.step(ft.add_batch(*syntheticBatch(20 + s, 4, 64, 256)))
        o = orc.step([rm.synthetic_batch(20 + s, 4, 64, 256)])
        h = ft.history(s, 1)[0]
        assert abs(h.loss - o.loss) <= 2e-2 * abs(o.loss), (s, h.loss, o.loss)
        assert abs(h.gradNorm - o.gradNorm) <= 3e-2 * o.gradNorm, (s, h.gradNorm, o.gradNorm)
    ft.close()


@pytest.mark.parametrize("accum,stream", [(1, "bf16"), (2, "bf16"), (2, "f32")])
def test_fused_step_with_dropout_matches_oracle(B, accum, stream):
    """dropout 0.25 in the two residualDropoutAdd of every block (gpt.ts:281,332) on the reference's flash-branch wiring: masks
    from DropoutRng's counter hash (ops.ts:25-82), reseeded per step and micro-step (trainer.ts:1169,1202), made on the fly from
    a seed in device memory, so a replayed graph draws new masks every step.  Against the oracle: gradients of the first step,
    then the loss of 12 steps; graph replay = eager."""
    from alpha2_amd.fused import FusedTrainer
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig, syntheticBatch
    cfg = dict(CFG, attention="reference-flash", dropout=0.25)
    steps = 12
    tc = dict(iters=steps, gradAccumSteps=accum, seed=77)
    mk = lambda graph: FusedTrainer(B, ModelConfig(**cfg), TrainConfig(**tc), 4, seed=6, use_graph=graph, accum=accum, stream=stream)
    ft, eager = mk(True), mk(False)
    orc = rm.Trainer(rm.ModelConfig(**cfg), rm.TrainConfig(**tc), seed=6)
    nodrop = rm.Trainer(rm.ModelConfig(**dict(cfg, dropout=0.0)), rm.TrainConfig(**tc), seed=6)
    differs = 0
    for s in range(steps):
        seeds = [900 + accum * s + m for m in range(accum)]
        ids = [ft.add_batch(*syntheticBatch(sd, 4, 64, 256)) for sd in seeds]
        ide = [eager.add_batch(*syntheticBatch(sd, 4, 64, 256)) for sd in seeds]
        ft.step(ids if accum > 1 else ids[0])
        eager.step(ide if accum > 1 else ide[0])
        ob = [rm.synthetic_batch(sd, 4, 64, 256) for sd in seeds]
        o, o0 = orc.step(ob), nodrop.step(ob)
        hg, he = ft.history(s, 1)[0], eager.history(s, 1)[0]
        assert abs(hg.loss - o.loss) <= 2e-2 * abs(o.loss), (s, hg.loss, o.loss)
        assert abs(hg.gradNorm - o.gradNorm) <= 4e-2 * o.gradNorm, (s, hg.gradNorm, o.gradNorm)
        assert hg.loss == he.loss and hg.gradNorm == he.gradNorm, (s, hg, he)
        differs += abs(o.loss - o0.loss) > 1e-3 * abs(o0.loss)
    assert differs >= 3                                   # the masks matter at this size: the comparison is not vacuous
    ft.close(), eager.close()


def test_fused_dropout_gradients_match_oracle_and_other_wirings_are_refused(B):
    from alpha2_amd.fused import FusedTrainer
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig, syntheticBatch
    cfg = dict(CFG, attention="reference-flash", dropout=0.2)
    with pytest.raises(ValueError, match="reference-flash"):
        FusedTrainer(B, ModelConfig(**dict(cfg, attention="heads")), TrainConfig(iters=1), 4)
    ft = FusedTrainer(B, ModelConfig(**cfg), TrainConfig(iters=1, seed=5), 4, seed=1, use_graph=False)
    orc = rm.Trainer(rm.ModelConfig(**cfg), rm.TrainConfig(iters=1, seed=5), seed=1)
    ft.set_batch(*syntheticBatch(3, 4, 64, 256))
    ob = rm.synthetic_batch(3, 4, 64, 256)
    orc.dropoutRng.reset(5 + 0 * 1000 + 0, 0)             # the masks of step 0, micro-step 0 (trainer.ts:1169,1202)
    _, oloss = rm.gptForward(orc.cfg, orc.params, orc.B, orc.tape, ob[0], ob[1], True, dropoutRng=orc.dropoutRng)
    orc.tape.backward(oloss, orc.B)
    ograds = {n: v.grad.data.copy() for n, v in orc.entries}
    ft.step()
    st = ft.history(0, 1)[0]
    assert abs(st.loss - float(oloss.data.data[0])) <= 2e-2 * abs(float(oloss.data.data[0]))
    for name, g in ograds.items():
        got, w = ft.grad(name).astype(np.float64), g.astype(np.float64)
        cos = float(got @ w / (np.linalg.norm(got) * np.linalg.norm(w) + 1e-300))
        assert cos > 0.995 and abs(np.linalg.norm(got) / np.linalg.norm(w) - 1) < 3e-2, (name, cos)
    ft.close()


@pytest.mark.parametrize("attention", ATTENTION)
def test_fused_gradient_accumulation_matches_oracle(B, attention):
    """Two micro-batches per optimizer step: summed gradients scaled once, reported loss = mean of the micro losses
    (trainer.ts:1164-1273); graph replay and eager execution agree."""
    from alpha2_amd.fused import FusedTrainer
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig, syntheticBatch
    steps, K = 6, 2
    tc = dict(iters=steps, gradAccumSteps=K)
    mk = lambda graph: FusedTrainer(B, ModelConfig(**CFG, attention=attention), TrainConfig(**tc), 4, seed=5, use_graph=graph, accum=K)
    ft, eager = mk(True), mk(False)
    orc = rm.Trainer(rm.ModelConfig(**CFG, attention=attention), rm.TrainConfig(iters=steps, gradAccumSteps=K), seed=5)
    for s in range(steps):
        seeds = [300 + K * s + m for m in range(K)]
        ids = [ft.add_batch(*syntheticBatch(sd, 4, 64, 256)) for sd in seeds]
        ide = [eager.add_batch(*syntheticBatch(sd, 4, 64, 256)) for sd in seeds]
        ft.step(ids)
        eager.step(ide)
        o = orc.step([rm.synthetic_batch(sd, 4, 64, 256) for sd in seeds])
        hg, he = ft.history(s, 1)[0], eager.history(s, 1)[0]
        assert abs(hg.loss - o.loss) <= 2e-2 * abs(o.loss), (s, hg.loss, o.loss)
        assert abs(hg.gradNorm - o.gradNorm) <= 3e-2 * o.gradNorm, (s, hg.gradNorm, o.gradNorm)
        assert abs(hg.loss - he.loss) <= 1e-4 * abs(he.loss) and abs(hg.gradNorm - he.gradNorm) <= 1e-3 * he.gradNorm
    with pytest.raises(ValueError, match="one per micro-step"):
        ft.step([0])
    ft.close(), eager.close()


@pytest.mark.parametrize("dropout", [0.0, 0.2])
@pytest.mark.parametrize("K,P", [(2, 2), (4, 2), (4, 4)])
def test_micro_steps_run_several_to_a_pass_give_the_numbers_of_one_at_a_time(B, K, P, dropout):
    """`micro_per_pass`: the K micro-steps of a step (trainer.ts:1164-1273) run P at a time as one pass over P micro-batches.  The
    reported loss (mean of the micro-step losses), the gradient norm and the update must be those of the oracle's K separate
    micro-steps -- with dropout too, every micro-batch of a pass drawing the masks of its own micro-step (trainer.ts:1202) --
    and those of the same trainer running them one at a time."""
    from alpha2_amd.fused import FusedTrainer
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig, syntheticBatch
    cfg = dict(CFG, attention="reference-flash", dropout=dropout)
    steps = 5
    tc = dict(iters=steps, gradAccumSteps=K, seed=21)
    mk = lambda per, graph: FusedTrainer(B, ModelConfig(**cfg), TrainConfig(**tc), 4, seed=8, use_graph=graph, accum=K, micro_per_pass=per)
    merged, eager, single = mk(P, True), mk(P, False), mk(1, True)
    assert (merged.batch, merged.accum, merged.micro_steps) == (4 * P, K // P, K)
    orc = rm.Trainer(rm.ModelConfig(**cfg), rm.TrainConfig(**tc), seed=8)
    for s in range(steps):
        seeds = [500 + K * s + m for m in range(K)]
        ids = [[t.add_batch(*syntheticBatch(sd, 4, 64, 256)) for sd in seeds] for t in (merged, eager, single)]
        for t, i in zip((merged, eager, single), ids):
            t.step(i)
        o = orc.step([rm.synthetic_batch(sd, 4, 64, 256) for sd in seeds])
        hm, he, h1 = (t.history(s, 1)[0] for t in (merged, eager, single))
        assert abs(hm.loss - o.loss) <= 2e-2 * abs(o.loss) and abs(hm.gradNorm - o.gradNorm) <= 4e-2 * o.gradNorm, (s, hm, o.loss, o.gradNorm)
        assert abs(hm.loss - h1.loss) <= 2e-3 * abs(h1.loss) and abs(hm.gradNorm - h1.gradNorm) <= 1e-2 * h1.gradNorm, (s, hm, h1)
        assert hm.loss == he.loss and hm.gradNorm == he.gradNorm, (s, hm, he)
    for name in ("wte", "layer.1.attn.wqkv", "layer.0.mlp.fc2", "lmHead"):
        assert np.max(np.abs(merged.param(name) - single.param(name))) <= 2.5 * steps * 3e-4, name      # (AdamW moves an entry by about lr per step)
    with pytest.raises(ValueError, match="one per micro-step"):
        merged.step([0] * (K - 1))
    with pytest.raises(ValueError, match="must divide"):
        FusedTrainer(B, ModelConfig(**cfg), TrainConfig(**tc), 4, accum=K, micro_per_pass=3)
    merged.close(), eager.close(), single.close()


def test_fused_checkpoint_resume(B, tmp_path):
    """The fast path writes and reads the same file format; a resumed run (graph captured after the load) follows the
    uninterrupted one, and the generic trainer accepts the file too."""
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig, Trainer, syntheticBatch
    tc = dict(iters=8)
    a = _make(B, tc, use_graph=True, seed=6)
    ids = [a.add_batch(*syntheticBatch(700 + s, 4, 64, 256)) for s in range(8)]
    for s in range(4):
        a.step(ids[s])
    path = str(tmp_path / "fused.alph")
    a.saveCheckpoint(path)
    at_save = a.param("layer.1.mlp.fc1")
    b = _make(B, tc, use_graph=True, seed=11)
    idb = [b.add_batch(*syntheticBatch(700 + s, 4, 64, 256)) for s in range(8)]
    st = b.loadCheckpoint(path)
    assert st["step"] == 4 and b.stepIdx == 4
    for s in range(4, 8):
        a.step(ids[s])
        b.step(idb[s])
    ha, hb = a.history(4, 4), b.history(4, 4)
    for x, y in zip(ha, hb):
        assert abs(x.loss - y.loss) <= 1e-4 * abs(x.loss) and abs(x.lr - y.lr) < 1e-15, (x, y)
    g = Trainer(B, ModelConfig(**CFG), TrainConfig(**tc), seed=0)
    g.loadCheckpoint(path)
    assert g.stepIdx == 4 and g.optimizer._step == 4
    assert np.array_equal(dict(g.entries)["layer.1.mlp.fc1"].data.data, at_save)       # bit-for-bit what was saved
    assert not np.array_equal(a.param("layer.1.mlp.fc1"), at_save)                     # (training has moved on since)
    a.close(), b.close()


def test_fused_resume_with_dropout_draws_the_masks_of_the_uninterrupted_run(B, tmp_path):
    """The masks of a step depend on its index (trainer.ts:1169: seed + 1000 step): a run resumed at step 3 must drop what the
    uninterrupted run drops from step 3 on."""
    from alpha2_amd.fused import FusedTrainer
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig, syntheticBatch
    cfg = ModelConfig(**CFG, attention="reference-flash", dropout=0.2)
    mk = lambda seed: FusedTrainer(B, cfg, TrainConfig(iters=6, seed=9), 4, seed=seed, use_graph=True)
    a = mk(6)
    ids = [a.add_batch(*syntheticBatch(800 + s, 4, 64, 256)) for s in range(6)]
    for s in range(3):
        a.step(ids[s])
    path = str(tmp_path / "drop.alph")
    a.saveCheckpoint(path)
    b = mk(11)
    idb = [b.add_batch(*syntheticBatch(800 + s, 4, 64, 256)) for s in range(6)]
    assert b.loadCheckpoint(path)["step"] == 3
    for s in range(3, 6):
        a.step(ids[s])
        b.step(idb[s])
    for x, y in zip(a.history(3, 3), b.history(3, 3)):
        assert abs(x.loss - y.loss) <= 1e-4 * abs(x.loss) and abs(x.gradNorm - y.gradNorm) <= 1e-3 * x.gradNorm, (x, y)
    a.close(), b.close()


def test_fused_step_with_a_non_finite_gradient_is_skipped_on_the_device(B):
    """The reference trainer skips the optimizer call when the loss or the gradient norm is not finite
    (trainer.ts:1248-1262,1495-1522).  The fast path takes that decision on the device: parameters, moments, the bf16
    shadow and the running bias corrections stay as they were, the skip shows in history(), and the next clean step equals
    the step a run without the incident takes."""
    import ctypes as C
    from alpha2_amd.train import syntheticBatch
    tc = dict(iters=6)
    a, b = _make(B, tc, use_graph=False, seed=8), _make(B, tc, use_graph=False, seed=8)
    for t in (a, b):
        t.set_batch(*syntheticBatch(900, 4, 64, 256))
        t.step()
    before = {n: a.param(n) for n in ("wte", "layer.0.mlp.fc1", "lnF.weight")}
    m_before = a.stateDict()["buffers"]["layer.0.mlp.fc1.m"].data.copy()
    # poison: run forward/backward, then put an Inf into the gradient arena before the optimizer part (as a micro-step that is
    # not the last: the norm is then taken by the optimizer part, over the arena as it finds it)
    a._write_hyper()
    a._forward_backward(True, 0, last_micro=False)
    inf = np.array([np.inf], np.float32)
    ffi_check = __import__("alpha2_amd._ffi", fromlist=["check"]).check
    ffi_check(B.lib.ah_upload(a.g("layer.0.mlp.fc1") + 40, inf.ctypes.data_as(C.c_void_p), 4))
    a._optimizer()
    i = a.stepIdx % a.loss_hist_cap
    ffi_check(B.lib.ah_copy(a.loss_hist + i * 4, a.loss, 4))
    ffi_check(B.lib.ah_copy(a.norm_hist + i * 16, a.clip, 16))
    a.stepIdx += 1
    h = a.history(1, 1)[0]
    assert h.skipped and not math.isfinite(h.gradNorm) and math.isnan(h.clipCoef)
    for n, v in before.items():
        assert np.array_equal(a.param(n), v), n
    assert np.array_equal(a.stateDict()["buffers"]["layer.0.mlp.fc1.m"].data, m_before)
    # the next clean step of `a` (schedule index 2) against `b` stepping the same batch at the same schedule index
    b.stepIdx = 2
    a.step(), b.step()
    ha, hb = a.history(2, 1)[0], b.history(2, 1)[0]
    assert not ha.skipped and abs(ha.loss - hb.loss) <= 1e-6 * abs(hb.loss)
    for n in before:
        assert np.allclose(a.param(n), b.param(n), rtol=0, atol=1e-7), n          # same bias corrections: beta powers did not advance
    a.close(), b.close()


def test_set_batch_reuses_the_resident_slot(B):
    from alpha2_amd.train import syntheticBatch
    ft = _make(B, dict(iters=4), use_graph=False, seed=1)
    ft.set_batch(*syntheticBatch(1, 4, 64, 256))
    live = B.gpuMemStats()["liveAllocs"]
    for s in range(5):
        ft.set_batch(*syntheticBatch(2 + s, 4, 64, 256))
    assert B.gpuMemStats()["liveAllocs"] == live
    i = ft.add_batch(*syntheticBatch(9, 4, 64, 256))
    assert B.gpuMemStats()["liveAllocs"] == live + 3                  # tokens, targets, sorted-position index
    ft.drop_batches()
    assert B.gpuMemStats()["liveAllocs"] == live and i == 0
    ft.close()


def test_fused_step_is_bit_identical_from_run_to_run(B):
    """Every sum of the step has a fixed order (split-K and grouped GEMM joins, LayerNorm column sums, the embedding
    scatter-add over positions sorted by id, the gradient norm): two runs from the same seed give the same bits, and the
    replayed graph gives the bits of eager execution."""
    from alpha2_amd.train import syntheticBatch
    runs = []
    for graph in (False, False, True):
        ft = _make(B, dict(iters=4), use_graph=graph, seed=9)
        ids = [ft.add_batch(*syntheticBatch(400 + s, 4, 64, 256)) for s in range(4)]
        for s in range(4):
            ft.step(ids[s])
        h = ft.history(0, 4)
        runs.append(([(x.loss, x.gradNorm) for x in h], {n: ft.param(n) for n in ("wte", "wpe", "layer.0.attn.wqkv", "lnF.weight")},
                     ft.grad("wte")))
        ft.close()
    for other in runs[1:]:
        assert other[0] == runs[0][0]
        assert np.array_equal(other[2], runs[0][2])
        for n, v in runs[0][1].items():
            assert np.array_equal(other[1][n], v), n


@pytest.mark.parametrize("graph", [False, True])
def test_sorting_the_ids_inside_the_step_gives_the_same_bits(B, graph):
    """index_in_step: the scatter-add index of the token embedding's gradient is built in every step, on the side stream
    beside the forward pass (a fork and a join of the captured graph), instead of once when the batch is stored: same index,
    so the same bits, with two micro-steps as well."""
    from alpha2_amd.fused import FusedTrainer
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig, syntheticBatch
    runs = []
    for in_step in (False, True):
        ft = FusedTrainer(B, ModelConfig(**CFG), TrainConfig(iters=4, gradAccumSteps=2), 4, seed=9, use_graph=graph, accum=2, index_in_step=in_step)
        ids = [ft.add_batch(*syntheticBatch(400 + s, 4, 64, 256)) for s in range(6)]
        for s in range(3):
            ft.step([ids[2 * s], ids[2 * s + 1]])
        runs.append(([(x.loss, x.gradNorm) for x in ft.history(0, 3)], ft.param("wte"), ft.grad("wte")))
        ft.close()
    assert runs[0][0] == runs[1][0] and np.array_equal(runs[0][1], runs[1][1]) and np.array_equal(runs[0][2], runs[1][2])


@pytest.mark.parametrize("graph", [False, True])
@pytest.mark.parametrize("accum", [1, 2])
def test_gradient_norm_from_the_weight_gradient_epilogue(B, graph, accum):
    """By default the grouped weight-gradient launch of the last micro-step squares and sums what it stores, and only the
    other gradients are read again for the norm.  Against a trainer that reads the whole gradient arena: the gradients are
    the same bits, the norm agrees to f32 rounding (another order of the same sum), the parameters after four steps to a
    rounding of the clip coefficient; and the reported norm is the norm of the arena the step left."""
    import ctypes as C
    from alpha2_amd import TensorData, _ffi as ffi
    from alpha2_amd.fused import FusedTrainer
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig, syntheticBatch
    mk = lambda fold: FusedTrainer(B, ModelConfig(**CFG), TrainConfig(iters=6, gradAccumSteps=accum), 4, seed=0, use_graph=graph,
                                   accum=accum, norm_in_epilogue=fold)
    one, two = mk(True), mk(False)
    assert one._norm_in_epilogue and not two._norm_in_epilogue
    batches = [syntheticBatch(3 + m, 4, 64, 256) for m in range(accum)]
    i1, i2 = [one.add_batch(*b) for b in batches], [two.add_batch(*b) for b in batches]
    for s in range(4):
        one.step(i1 if accum > 1 else i1[0])
        two.step(i2 if accum > 1 else i2[0])
        if s == 0:
            for name in ("wte", "wpe", "lmHead", "layer.0.attn.wqkv", "layer.1.mlp.fc2", "layer.1.ln1.weight", "lnF.bias"):
                assert np.array_equal(one.grad(name), two.grad(name)), name
    for a, b in zip(one.history(0, 4), two.history(0, 4)):
        assert abs(a.loss - b.loss) <= 1e-6 * abs(b.loss) and abs(a.gradNorm - b.gradNorm) <= 1e-5 * b.gradNorm, (a, b)
    assert one.history(0, 1)[0].loss == two.history(0, 1)[0].loss
    for name in ("wte", "lmHead", "layer.0.attn.wqkv", "layer.1.mlp.fc2", "layer.1.ln1.weight"):
        assert np.allclose(one.param(name), two.param(name), rtol=0, atol=1e-6), name
    arena = TensorData((1,), "f32", np.zeros(1, np.float32))
    ffi.check(B.lib.ah_sum_sq(one.G, one.nparam, B._ptr(arena)))
    B._dirty(arena)
    want = math.sqrt(float(arena.data[0])) / accum
    got = one.history(3, 1)[0].gradNorm
    assert abs(got - want) <= 1e-5 * want, (got, want)
    one.close(), two.close()


@pytest.mark.parametrize("graph", [False, True])
@pytest.mark.parametrize("accum", [1, 2])
def test_weight_gradients_on_the_side_stream_give_the_same_step(B, graph, accum):
    """dw_groups = 2 launches the weight-gradient GEMMs of the upper layer beside the backward kernels of the lower one on
    a second stream; every product keeps its own kernel configuration, so the step must not change by a bit."""
    from alpha2_amd.fused import FusedTrainer
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig, syntheticBatch
    mk = lambda groups: FusedTrainer(B, ModelConfig(**CFG), TrainConfig(iters=6, gradAccumSteps=accum), 4, seed=0, use_graph=graph,
                                     accum=accum, dw_groups=groups, norm_in_epilogue=False)      # (both sum the norm over the arena)
    one, two = mk(1), mk(2)
    batches = [syntheticBatch(3 + m, 4, 64, 256) for m in range(accum)]
    i1, i2 = [one.add_batch(*b) for b in batches], [two.add_batch(*b) for b in batches]
    for _ in range(4):
        one.step(i1 if accum > 1 else i1[0])
        two.step(i2 if accum > 1 else i2[0])
    h1, h2 = one.history(0, 4), two.history(0, 4)
    for a, b in zip(h1, h2):
        assert a.loss == b.loss and a.gradNorm == b.gradNorm, (a, b)
    for name in ("wte", "lmHead", "layer.0.attn.wqkv", "layer.1.mlp.fc2", "layer.1.ln1.weight"):
        assert np.array_equal(one.param(name), two.param(name)), name
    one.close(), two.close()


@pytest.mark.parametrize("act", ["silu", "relu", "swiglu", "universal", "kan_spline"])
@pytest.mark.parametrize("accum", [1, 2])
def test_fused_step_with_the_other_mlp_activations_matches_oracle(B, act, accum):
    """gpt.ts:286-321: the MLP variants in the hand-scheduled bf16 step (pre-activation saved in bf16, one element-wise pass
    each way; swiglu's gate and up weights as one stacked operand).  Loss, gradient norm, every gradient's direction and size,
    and the parameters after the update against the fp32 oracle, with and without accumulation over two micro-batches."""
    from alpha2_amd.fused import FusedTrainer
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig, syntheticBatch
    cfg = dict(CFG, ffnActivation=act)
    ft = FusedTrainer(B, ModelConfig(**cfg), TrainConfig(iters=3, gradAccumSteps=accum), 4, seed=0, use_graph=True, accum=accum)
    orc = rm.Trainer(rm.ModelConfig(**cfg), rm.TrainConfig(iters=3, gradAccumSteps=accum), seed=0)
    for name, v in orc.entries:
        assert np.array_equal(ft.param(name), v.data.data), name
    idx = [ft.add_batch(*syntheticBatch(1 + m, 4, 64, 256)) for m in range(accum)]
    obs = [rm.synthetic_batch(1 + m, 4, 64, 256) for m in range(accum)]
    # oracle gradients (sum over micro-batches, as the gradient arena holds them before the 1 / accum scale) before its optimizer step
    for ob in obs:
        _, oloss = rm.gptForward(orc.cfg, orc.params, orc.B, orc.tape, ob[0], ob[1], True)
        orc.tape.backward(oloss, orc.B)
        orc.tape.clear()
    ograds = {n: v.grad.data.copy() for n, v in orc.entries}
    for _, v in orc.entries:
        v.grad = None
    for s in range(3):
        o = orc.step(obs)
        ft.step(idx if accum > 1 else idx[0])
        st = ft.history(s, s + 1)[0]
        assert abs(st.loss - o.loss) <= 2e-2 * abs(o.loss), (s, st.loss, o.loss)
        assert abs(st.gradNorm - o.gradNorm) <= 3e-2 * o.gradNorm, (s, st.gradNorm, o.gradNorm)
        if s == 0:
            for name, g in ograds.items():
                got, w = ft.grad(name).astype(np.float64), g.astype(np.float64)
                cos = float(got @ w / (np.linalg.norm(got) * np.linalg.norm(w) + 1e-300))
                assert cos > 0.995, (name, cos)
                assert abs(np.linalg.norm(got) / np.linalg.norm(w) - 1) < 3e-2, name
    for name, v in orc.entries:                                           # three AdamW steps: every entry within 3 lr of the oracle's
        assert np.max(np.abs(ft.param(name) - v.data.data)) <= 3 * 2 * 3e-4 * 1.001 + 1e-6, name
    ft.close()


def test_fused_step_with_a_bf16_residual_stream_tracks_the_oracle(B):
    """stream = "bf16" (the default): the residual stream and its gradient in bf16 like every other activation; stream = "f32"
    keeps them in f32.  Both against the fp32 oracle at the bf16 bars (loss 2e-2 relative over 50 steps, gradient direction and
    size), and against each other."""
    from alpha2_amd.fused import FusedTrainer
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig, syntheticBatch
    steps = 50
    tc = dict(iters=steps, lr=1e-3)
    f16 = FusedTrainer(B, ModelConfig(**CFG), TrainConfig(**tc), 4, seed=0, use_graph=True, stream="bf16")
    f32 = FusedTrainer(B, ModelConfig(**CFG), TrainConfig(**tc), 4, seed=0, use_graph=True, stream="f32")
    orc = rm.Trainer(rm.ModelConfig(**CFG), rm.TrainConfig(**tc), seed=0)
    ob = rm.synthetic_batch(1, 4, 64, 256)
    _, oloss = rm.gptForward(orc.cfg, orc.params, orc.B, orc.tape, ob[0], ob[1], True)
    orc.tape.backward(oloss, orc.B)
    ograds = {n: v.grad.data.copy() for n, v in orc.entries}
    orc.tape.clear()
    for _, v in orc.entries:
        v.grad = None
    i16, i32 = f16.add_batch(*syntheticBatch(1, 4, 64, 256)), f32.add_batch(*syntheticBatch(1, 4, 64, 256))
    worst = worst_pair = 0.0
    for s in range(steps):
        o = orc.step([ob])
        f16.step(i16), f32.step(i32)
        a, b = f16.history(s, s + 1)[0], f32.history(s, s + 1)[0]
        worst = max(worst, abs(a.loss - o.loss) / abs(o.loss), abs(b.loss - o.loss) / abs(o.loss))
        worst_pair = max(worst_pair, abs(a.loss - b.loss) / abs(b.loss))
        if s == 0:
            for ft in (f16, f32):
                for name, g in ograds.items():
                    got, w = ft.grad(name).astype(np.float64), g.astype(np.float64)
                    cos = float(got @ w / (np.linalg.norm(got) * np.linalg.norm(w) + 1e-300))
                    assert cos > 0.995, (ft.stream, name, cos)
                    assert abs(np.linalg.norm(got) / np.linalg.norm(w) - 1) < 3e-2, (ft.stream, name)
    assert worst <= 2e-2, worst
    assert worst_pair <= 1e-2, worst_pair
    f16.close(), f32.close()


@pytest.mark.parametrize("stream", ["bf16", "f32"])
def test_fused_step_on_a_ragged_shape(B, stream):
    """72 tokens per batch (3 x 24: not a multiple of the 64-token k-tile, so every weight gradient is a general GEMM instead of
    the grouped launch; a context shorter than an attention tile), head size 64, a vocabulary that is not a multiple of 64:
    the edge paths of the same step against the oracle."""
    from alpha2_amd.fused import FusedTrainer
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig, syntheticBatch
    cfg = dict(vocabSize=264, blockSize=24, nLayer=2, nEmbd=128, nHead=2)
    ft = FusedTrainer(B, ModelConfig(**cfg), TrainConfig(iters=3), 3, seed=0, use_graph=True, stream=stream)
    orc = rm.Trainer(rm.ModelConfig(**cfg), rm.TrainConfig(iters=3), seed=0)
    ob = rm.synthetic_batch(2, 3, 24, 264)
    _, oloss = rm.gptForward(orc.cfg, orc.params, orc.B, orc.tape, ob[0], ob[1], True)
    orc.tape.backward(oloss, orc.B)
    ograds = {n: v.grad.data.copy() for n, v in orc.entries}
    orc.tape.clear()
    for _, v in orc.entries:
        v.grad = None
    i = ft.add_batch(*syntheticBatch(2, 3, 24, 264))
    for s in range(3):
        o = orc.step([ob])
        ft.step(i)
        st = ft.history(s, s + 1)[0]
        assert abs(st.loss - o.loss) <= 2e-2 * abs(o.loss), (s, st.loss, o.loss)
        assert abs(st.gradNorm - o.gradNorm) <= 3e-2 * o.gradNorm, (s, st.gradNorm, o.gradNorm)
        if s == 0:
            for name, g in ograds.items():
                got, w = ft.grad(name).astype(np.float64), g.astype(np.float64)
                cos = float(got @ w / (np.linalg.norm(got) * np.linalg.norm(w) + 1e-300))
                assert cos > 0.995, (name, cos)
    ft.close()
