"""Model-level parity on the GPU: the HipBackend-driven forward / backward / AdamW step against the CPU oracle's
restatement of the reference trainer, on identical seeded parameters and token batches (fp32 parity mode)."""
import gc
import math

import numpy as np
import pytest

from oracle import ref
from oracle import ref_model as rm
from tests.util import assert_close

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def B():
    from alpha2_amd import HipBackend
    return HipBackend(0)


def _both(B, cfg_kw, tc_kw, seed=0):
    from alpha2_amd.model import ModelConfig
    from alpha2_amd.train import TrainConfig, Trainer
    dev = Trainer(B, ModelConfig(**cfg_kw), TrainConfig(**tc_kw), seed=seed)
    # the oracle knows the two branches of gpt.ts:246-280; "unfused" is the product's op-by-op form of the heads branch
    okw = dict(cfg_kw, attention="reference-flash" if cfg_kw.get("attention") == "reference-flash" else "heads")
    orc = rm.Trainer(rm.ModelConfig(**okw),
                     rm.TrainConfig(**{k: v for k, v in tc_kw.items() if k in rm.TrainConfig.__dataclass_fields__}), seed=seed)
    for (n1, v1), (n2, v2) in zip(dev.entries, orc.entries):        # same names, same order, same initial values
        assert n1 == n2 and np.array_equal(v1.data.data, v2.data.data), n1
    return dev, orc


@pytest.mark.parametrize("attention,heads", [("heads", 2), ("unfused", 4), ("heads", 4), ("heads", 8)])
def test_forward_backward_grads_match_oracle(B, attention, heads):
    """Head sizes 32, 16 (unfused), 16 and 8 through the fused kernel (the reference's small domains have 128 / 8 and 64 / 4:
    packages/core/src/domains.ts): the kernels of size 32 with the missing features read as zeros."""
    from alpha2_amd.autograd import Tape
    from alpha2_amd.model import gptForward
    from alpha2_amd.train import syntheticBatch
    cfg = dict(vocabSize=61, blockSize=24, nLayer=2, nEmbd=64, nHead=heads, attention=attention)
    dev, orc = _both(B, cfg, dict(iters=1))
    inp, tgt = syntheticBatch(3, 3, 24, 61)
    oi, ot = rm.synthetic_batch(3, 3, 24, 61)
    assert np.array_equal(inp.data, oi.data) and np.array_equal(tgt.data, ot.data)       # token ids: bit exact
    tape = Tape()
    r = gptForward(dev.cfg, dev.params, B, tape, inp, tgt, True)
    otape = rm.Tape()
    ologits, oloss = rm.gptForward(orc.cfg, orc.params, orc.B, otape, oi, ot, True)
    assert_close(r["logits"].data.data, ologits.data.data, what="logits")
    assert_close(r["loss"].data.data, oloss.data.data, what="loss")
    tape.backward(r["loss"], B)
    otape.backward(oloss, orc.B)
    for (n, v), (_, ov) in zip(dev.entries, orc.entries):
        assert_close(v.grad.data, ov.grad.data, what=f"grad {n}")


@pytest.mark.parametrize("act", ["swiglu", "universal", "kan_spline", "silu", "relu", "composed"])
def test_custom_activation_models_match_oracle(B, act):
    from alpha2_amd.autograd import Tape
    from alpha2_amd.model import gptForward
    from alpha2_amd.train import syntheticBatch
    cfg = dict(vocabSize=40, blockSize=16, nLayer=1, nEmbd=64, nHead=2, ffnActivation=act)
    if act == "composed":           # the expression tree of the oracle's own pin (every node type and basis, an unknown basis name)
        from tests.test_oracle_model import COMPOSED_GRAPH
        cfg["activationGraph"] = COMPOSED_GRAPH
    dev, orc = _both(B, cfg, dict(iters=1), seed=5)
    rs = np.random.RandomState(1)
    for (n, v), (_, ov) in zip(dev.entries, orc.entries):           # generic gates / coefficients
        d = (rs.randn(v.data.size) * 0.05).astype(np.float32)
        v.data.data = v.data.data + d
        ov.data.data += d
    inp, tgt = syntheticBatch(9, 2, 16, 40)
    oi, ot = rm.synthetic_batch(9, 2, 16, 40)
    tape, otape = Tape(), rm.Tape()
    r = gptForward(dev.cfg, dev.params, B, tape, inp, tgt, True)
    _, oloss = rm.gptForward(orc.cfg, orc.params, orc.B, otape, oi, ot, True)
    assert_close(r["loss"].data.data, oloss.data.data, what="loss")
    tape.backward(r["loss"], B, B.releaseGpuTensor)
    otape.backward(oloss, orc.B)
    for (n, v), (_, ov) in zip(dev.entries, orc.entries):
        assert_close(v.grad.data, ov.grad.data, what=f"grad {n}")


def test_tiny_char_gpt_one_step_matches_oracle(B):
    """The reference's CPU-runnable configuration: vocab 256, d 128, 4 layers, 4 heads, B=8 x T=128, AdamW 3e-4,
    betas (0.9, 0.95), wd 0.1, clip 1.0, seed 0 parameters, seed 1 tokens."""
    from alpha2_amd.train import syntheticBatch
    cfg = dict(vocabSize=256, blockSize=128, nLayer=4, nEmbd=128, nHead=4)
    dev, orc = _both(B, cfg, dict(iters=1))
    r = dev.step([syntheticBatch(1, 8, 128, 256)])
    o = orc.step([rm.synthetic_batch(1, 8, 128, 256)])
    assert abs(r.loss - o.loss) <= 1e-4 * abs(o.loss)
    assert abs(r.gradNorm - o.gradNorm) <= 1e-4 * o.gradNorm
    assert abs(r.clipCoef - o.clipCoef) <= 1e-4 and r.lr == o.lr
    assert abs(o.loss - math.log(256)) < 0.1
    for (n, v), (_, ov) in zip(dev.entries, orc.entries):
        # step 1 of Adam moves every entry by lr*g/(|g|+eps): entries whose gradient cancels to ~eps are ill-conditioned
        assert_close(v.data.data, ov.data.data, rel=1e-5, what=f"param {n} after step", outlier_frac=max(1e-3, 2.5 / v.data.size),
                     outlier_abs=0.1 * 3e-4)
        m, mo = dev.optimizer._m[n].data, orc.opt.m[n]
        assert_close(m, mo, what=f"adam m {n}")
    del o
    gc.collect()
    st = B.gpuMemStats()
    assert st["liveAllocs"] >= 3 * len(dev.entries)              # params + m + v are resident ...


def test_loss_parity_over_steps_with_accumulation(B):
    """Step loss within 1e-3 relative over a 50-step run (10 warm-up steps, cosine decay, clip, 2 micro-batches)."""
    from alpha2_amd.train import syntheticBatch
    cfg = dict(vocabSize=96, blockSize=32, nLayer=2, nEmbd=64, nHead=2)
    tc = dict(iters=50, gradAccumSteps=2)
    dev, orc = _both(B, cfg, tc, seed=2)
    live = None
    for s in range(50):
        db = [syntheticBatch(100 + 2 * s + i, 4, 32, 96) for i in range(2)]
        ob = [rm.synthetic_batch(100 + 2 * s + i, 4, 32, 96) for i in range(2)]
        r, o = dev.step(db), orc.step(ob)
        assert abs(r.loss - o.loss) <= 1e-3 * abs(o.loss), (s, r.loss, o.loss)
        assert abs(r.gradNorm - o.gradNorm) <= 1e-3 * o.gradNorm and abs(r.lr - o.lr) < 1e-15
        gc.collect()                                       # tensors of earlier tests may still be awaiting collection
        n = B.gpuMemStats()["liveAllocs"]
        if s >= 1:
            assert n <= live, "live allocations must not grow from step to step"
        live = n
    assert math.isfinite(r.loss)          # random batches at warm-up learning rates: the loss stays near log(vocab)


@pytest.mark.parametrize("optimizer,lr", [("lion", 1e-4), ("adafactor", 1e-3), ("sgd", 1e-2)])
def test_training_steps_with_the_other_optimizers_match_oracle(B, optimizer, lr):
    """Ten trainer steps (warm-up, clip folded into gradScale) with each optimizer of the reference's registry besides AdamW
    (apps/cli/src/resolve.ts:25-36): loss within 1e-3 relative, final parameters close."""
    from alpha2_amd.train import syntheticBatch
    cfg = dict(vocabSize=96, blockSize=32, nLayer=2, nEmbd=64, nHead=2)
    dev, orc = _both(B, cfg, dict(iters=10, lr=lr, optimizer=optimizer), seed=5)
    assert dev.optimizer.name == optimizer
    for s in range(10):
        r, o = dev.step([syntheticBatch(300 + s, 4, 32, 96)]), orc.step([rm.synthetic_batch(300 + s, 4, 32, 96)])
        assert abs(r.loss - o.loss) <= 1e-3 * abs(o.loss), (s, r.loss, o.loss)
    for (n1, v1), (_, v2) in zip(dev.entries, orc.entries):
        # Lion moves every weight by +-lr per step: a gradient entry whose sign differs within fp32 noise shifts it by 2 lr
        tol = 2.5 * lr * 10 if optimizer == "lion" else 0.0
        assert_close(v1.data.data, v2.data.data, rel=2e-3, what=n1, outlier_frac=0.02 if optimizer == "lion" else 0.0, outlier_abs=tol)


def test_activation_checkpointing_matches_plain(B):
    from alpha2_amd.autograd import Tape
    from alpha2_amd.model import ModelConfig, collectParamEntries, gptForward, initGPT
    from alpha2_amd.rng import SeededRng
    from alpha2_amd.train import syntheticBatch
    cfg = ModelConfig(vocabSize=50, blockSize=16, nLayer=2, nEmbd=64, nHead=2)
    out = []
    for ck in (False, True):
        params = initGPT(cfg, B, SeededRng(4))
        tape = Tape()
        inp, tgt = syntheticBatch(8, 2, 16, 50)
        r = gptForward(cfg, params, B, tape, inp, tgt, True, ck, False, None, B.releaseGpuTensor)
        loss = float(r["loss"].data.data[0])
        tape.backward(r["loss"], B, B.releaseGpuTensor)
        out.append((loss, [v.grad.data.copy() for _, v in collectParamEntries(params)]))
    assert abs(out[0][0] - out[1][0]) < 1e-6
    for a, b in zip(out[0][1], out[1][1]):
        assert_close(b, a, rel=1e-5)


@pytest.mark.parametrize("kw", [dict(), dict(softCap=0.0), dict(nHead=4, ffnActivation="swiglu", softCap=2.0),
                                dict(nEmbd=128, nHead=4, softCap=2.0), dict(nEmbd=96, nHead=8, softCap=30.0)])      # (head sizes 32, 32, 16, 32 and 12: the last has no fused kernel)
def test_reference_flash_branch_matches_its_oracle(B, kw):
    """What an unchanged gpt.ts runs on a backend that offers flashAttention (gpt.ts:247-254: [B, T, C] re-read as
    [B*H, T, D] slabs without a head transpose, flashAttention per slab, transpose (1, 2) back) against the oracle's
    restatement of that branch: logits, loss and every gradient at the fp32 bar, with the attention weights made large
    enough that the wiring of slabs matters; it is not the cpu_ref function (checked against the heads branch)."""
    from alpha2_amd.autograd import Tape
    from alpha2_amd.model import gptForward
    from alpha2_amd.train import syntheticBatch
    cfg = dict(dict(vocabSize=61, blockSize=24, nLayer=2, nEmbd=64, nHead=2, attention="reference-flash"), **kw)
    dev, orc = _both(B, cfg, dict(iters=1), seed=4)
    for (n, v), (_, ov) in zip(dev.entries, orc.entries):
        if n.endswith("attn.wqkv"):
            v.data.data = v.data.data * 20
            ov.data.data *= 20
    inp, tgt = syntheticBatch(3, 3, 24, 61)
    oi, ot = rm.synthetic_batch(3, 3, 24, 61)
    tape, otape = Tape(), rm.Tape()
    r = gptForward(dev.cfg, dev.params, B, tape, inp, tgt, True)
    ologits, oloss = rm.gptForward(orc.cfg, orc.params, orc.B, otape, oi, ot, True)
    assert_close(r["logits"].data.data, ologits.data.data, what="logits")
    assert_close(r["loss"].data.data, oloss.data.data, what="loss")
    tape.backward(r["loss"], B)
    otape.backward(oloss, orc.B)
    for (n, v), (_, ov) in zip(dev.entries, orc.entries):
        assert_close(v.grad.data, ov.grad.data, what=f"grad {n}")
    hcfg = rm.ModelConfig(**dict(cfg, attention="heads", softCap=cfg.get("softCap") or 30.0))
    _, hloss = rm.gptForward(hcfg, orc.params, orc.B, rm.Tape(), oi, ot, True)
    assert abs(float(hloss.data.data[0]) - float(oloss.data.data[0])) > 1e-4


def test_reference_flash_branch_training_steps_with_dropout_match_oracle(B):
    """The same branch through the trainer: 6 steps with two micro-steps and dropout 0.1, which in this branch has two
    sites per layer (the residual branches; no dropout on the attention weights, gpt.ts:247-254 against :276)."""
    from alpha2_amd.train import syntheticBatch
    cfg = dict(vocabSize=96, blockSize=32, nLayer=2, nEmbd=64, nHead=2, dropout=0.1, attention="reference-flash")
    dev, orc = _both(B, cfg, dict(iters=6, gradAccumSteps=2, seed=7), seed=2)
    for s in range(6):
        bs = [syntheticBatch(300 + 2 * s + m, 4, 32, 96) for m in range(2)]
        obs = [rm.synthetic_batch(300 + 2 * s + m, 4, 32, 96) for m in range(2)]
        r, o = dev.step(bs), orc.step(obs)
        assert abs(r.loss - o.loss) <= 1e-3 * abs(o.loss), (s, r.loss, o.loss)
        assert abs(r.gradNorm - o.gradNorm) <= 1e-3 * o.gradNorm, (s, r.gradNorm, o.gradNorm)
    assert (dev.dropoutRng.counter, orc.dropoutRng.counter) == (4, 4)


@pytest.mark.parametrize("N,Bt,T,packed", [(5000, 8, 128, False), (129, 2, 128, False), (1000, 4, 64, True), (10, 3, 7, True),
                                            (5, 2, 12, True), (70000, 16, 1024, False)])
def test_dataloader_batches_are_bit_exact(B, N, Bt, T, packed):
    """Device-assembled batches equal the oracle's slice-by-slice loader, batch after batch (integer data: bit-exact)."""
    from alpha2_amd.rng import SeededRng
    from alpha2_amd.train import DataLoader
    tok = (np.arange(N, dtype=np.int64) * 7919 % 50304).astype(np.int32)
    dev = DataLoader(B, tok, SeededRng(5), Bt, T, packed)
    orc = rm.DataLoader(tok, ref.SeededRng(5), Bt, T, packed)
    held = []
    for i in range(5):
        x, y = dev.nextBatch()
        xo, yo = orc.next_batch()
        assert x.shape == (Bt, T) and x.dtype == "i32"
        assert np.array_equal(x.data, xo.data) and np.array_equal(y.data, yo.data), i
        held.append((x, xo.data.copy()))
        if len(held) >= 2:        # the ring keeps the previous batch valid for one more call
            px, pxo = held[-2]
            assert np.array_equal(px.data, pxo)
    assert dev.stepsPerEpoch == N // (Bt * T)


@pytest.mark.parametrize("accum", [1, 2])
def test_trainer_driven_by_the_dataloader_matches_oracle(B, accum):
    """The training loop as the reference runs it: every micro-step takes loader.nextBatch(), and the trainer releases
    the batch tensors it consumed (trainer.ts:1190,1267-1272), so each ring slot is written again after a release."""
    from alpha2_amd.rng import SeededRng
    from alpha2_amd.train import DataLoader
    cfg = dict(vocabSize=96, blockSize=32, nLayer=2, nEmbd=64, nHead=2)
    dev, orc = _both(B, cfg, dict(iters=6, gradAccumSteps=accum), seed=3)
    tok = (np.arange(5000, dtype=np.int64) * 7919 % 96).astype(np.int32)
    dl, odl = DataLoader(B, tok, SeededRng(8), 4, 32), rm.DataLoader(tok, ref.SeededRng(8), 4, 32)
    for s in range(6):
        r = dev.step([dl.nextBatch() for _ in range(accum)])
        o = orc.step([odl.next_batch() for _ in range(accum)])
        assert abs(r.loss - o.loss) <= 1e-3 * abs(o.loss), (s, r.loss, o.loss)
        assert abs(r.gradNorm - o.gradNorm) <= 1e-3 * o.gradNorm, (s, r.gradNorm, o.gradNorm)


def test_training_steps_with_dropout_match_oracle(B):
    """dropout = 0.1: masks at the three sites of every layer (attention weights, both residual branches) come from the
    reference's counter hash, re-seeded with seed + step * 1000 + microStep before every forward (trainer.ts:1169,1202;
    ops.ts:25-82); the device masks are bit-equal to the CPU path's, so losses agree as tightly as without dropout."""
    from alpha2_amd.train import syntheticBatch
    cfg = dict(vocabSize=96, blockSize=32, nLayer=2, nEmbd=64, nHead=2, dropout=0.1)
    dev, orc = _both(B, cfg, dict(iters=4, gradAccumSteps=2, seed=7), seed=2)
    nodrop, _ = _both(B, dict(cfg, dropout=0.0), dict(iters=4, gradAccumSteps=2, seed=7), seed=2)
    for s in range(4):
        bs = [syntheticBatch(300 + 2 * s + m, 4, 32, 96) for m in range(2)]
        obs = [rm.synthetic_batch(300 + 2 * s + m, 4, 32, 96) for m in range(2)]
        r, o = dev.step(bs), orc.step(obs)
        assert abs(r.loss - o.loss) <= 1e-3 * abs(o.loss), (s, r.loss, o.loss)
        assert abs(r.gradNorm - o.gradNorm) <= 1e-3 * o.gradNorm, (s, r.gradNorm, o.gradNorm)
        if s == 0:
            r0 = nodrop.step([syntheticBatch(300 + m, 4, 32, 96) for m in range(2)])
            assert abs(r0.loss - r.loss) > 1e-4 * abs(r.loss)                  # dropout really is on
    for (n, v), (_, ov) in zip(dev.entries, orc.entries):
        assert_close(v.data.data, ov.data.data, rel=1e-3, what=f"param {n} after 4 steps", outlier_frac=max(2e-3, 2.5 / v.data.size),
                     outlier_abs=4 * 0.1 * 3e-4)


def test_dataloader_rejects_a_corpus_not_longer_than_the_block(B):
    from alpha2_amd.rng import SeededRng
    from alpha2_amd.train import DataLoader
    with pytest.raises(IndexError, match="must exceed block size"):
        DataLoader(B, np.arange(16, dtype=np.int32), SeededRng(0), 2, 16).nextBatch()


def test_checkpoint_resume_matches_uninterrupted_run_and_loads_in_the_oracle(B, tmp_path):
    """Save after 3 steps in the reference's file format, resume in a fresh trainer: the next steps follow the
    uninterrupted run; the same file restores the CPU oracle, which then tracks the device trainer."""
    from alpha2_amd.train import syntheticBatch
    cfg = dict(vocabSize=96, blockSize=32, nLayer=2, nEmbd=64, nHead=2)
    a, orc = _both(B, cfg, dict(iters=6), seed=4)
    for s in range(3):
        a.step([syntheticBatch(500 + s, 4, 32, 96)])
    path = str(tmp_path / "ckpt.alph")
    a.saveCheckpoint(path, configHash="cafe")
    b, _ = _both(B, cfg, dict(iters=6), seed=9)               # different initial weights: everything must come from the file
    st = b.loadCheckpoint(path)
    assert st["configHash"] == "cafe" and st["step"] == 3 and st["modelConfig"]["nEmbd"] == 64
    ost = rm.checkpoint_load_bytes(open(path, "rb").read())
    rm.restore_params(orc.entries, ost["params"])
    orc.opt.load_state_dict(ost["optimizerState"])
    orc.step_idx = ost["step"]
    for s in range(3, 6):
        ra, rb = a.step([syntheticBatch(500 + s, 4, 32, 96)]), b.step([syntheticBatch(500 + s, 4, 32, 96)])
        ro = orc.step([rm.synthetic_batch(500 + s, 4, 32, 96)])
        assert abs(ra.loss - rb.loss) <= 1e-5 * abs(ra.loss) and ra.lr == rb.lr, (s, ra.loss, rb.loss)
        assert abs(rb.loss - ro.loss) <= 1e-3 * abs(ro.loss), (s, rb.loss, ro.loss)
