"""Pins the oracle's model-level restatement (RNG stream, init order, full forward/backward, trainer
step arithmetic) against independent computations: a big-int Python xorshift, PyTorch float64
autograd of the same network, and closed forms.  No GPU."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import ref
from oracle import ref_model as rm


def _py_rng_stream(seed, n):
    """Independent restatement of the int32 xorshift in arbitrary-precision ints
    (packages/core/src/rng.ts:13-50)."""
    M = 0xFFFFFFFF

    def i32(x):
        x &= M
        return x - (1 << 32) if x >> 31 else x
    s0, s1 = i32(seed), i32(seed ^ 0xDEADBEEF)
    out = []
    for i in range(n + 20):
        a, b = s0 & M, s1 & M
        s0 = i32(b)
        a ^= (a << 23) & M
        a ^= a >> 17
        a ^= b
        a ^= b >> 26
        s1 = i32(a)
        if i >= 20:
            out.append(((s0 + s1) & M) / 4294967296.0)
    return out


def test_rng_integer_stream_bit_exact():
    for seed in (0, 1, 42, 123, -7, 2**31 - 1):
        r = ref.SeededRng(seed)
        got = [r.next() for _ in range(500)]
        assert got == _py_rng_stream(seed, 500)
        assert all(0 <= v < 1 for v in got)
    assert ref.SeededRng(1).next() != ref.SeededRng(2).next()      # rng.test.ts:32-38


def test_rng_gauss_polar_with_spare():
    r = ref.SeededRng(42)
    u = iter(_py_rng_stream(42, 4000))
    want = []
    while len(want) < 1000:
        while True:
            a, b = next(u) * 2 - 1, next(u) * 2 - 1
            s = a * a + b * b
            if not (s >= 1 or s == 0):
                break
        m = math.sqrt(-2.0 * math.log(s) / s)
        want += [a * m, b * m]
    got = [r.nextGauss() for _ in range(1000)]
    assert np.allclose(got, want, rtol=1e-15, atol=0)
    assert abs(np.mean([ref.SeededRng(42).nextGauss() for _ in range(1)])) < 10
    r2 = ref.SeededRng(42)
    assert abs(sum(r2.nextGauss() for _ in range(10000)) / 10000) < 0.1   # rng.test.ts:24-30


def test_init_order_and_std():
    cfg = rm.ModelConfig(vocabSize=11, blockSize=5, nLayer=2, nEmbd=8, nHead=2)
    p = rm.initGPT(cfg, ref.CpuRef(), ref.SeededRng(0))
    r = ref.SeededRng(0)
    C_, Fd, L = 8, 32, 2
    draws = lambda n, std: r.fill_gauss(n, std)
    assert np.array_equal(p["wte"].data.data, draws(11 * C_, 0.02))
    assert np.array_equal(p["wpe"].data.data, draws(5 * C_, 0.02))
    for l in p["layers"]:   # mlp is built before the attention weights (gpt.ts:89-144)
        assert np.array_equal(l["mlp"]["fc1"].data.data, draws(Fd * C_, 0.02))
        assert np.array_equal(l["mlp"]["fc2"].data.data, draws(C_ * Fd, 0.02 / math.sqrt(2 * L)))
        assert np.array_equal(l["attn"]["wqkv"].data.data, draws(3 * C_ * C_, 0.02))
        assert np.array_equal(l["attn"]["wo"].data.data, draws(C_ * C_, 0.02 / math.sqrt(2 * L)))
        assert np.all(l["ln1"]["weight"].data.data == 1) and np.all(l["ln2"]["bias"].data.data == 0)
    assert np.array_equal(p["lmHead"].data.data, draws(11 * C_, 0.02))
    names = [n for n, _ in rm.collectParamEntries(p)]
    assert names[:5] == ["wte", "wpe", "lmHead", "lnF.weight", "lnF.bias"]
    assert names[5:13] == [f"layer.0.{s}" for s in ("ln1.weight", "ln1.bias", "attn.wqkv", "attn.wo", "ln2.weight",
                                                   "ln2.bias", "mlp.fc1", "mlp.fc2")]
    assert "lmHead" not in rm.no_decay_names(2) and "wte" in rm.no_decay_names(2)


# A composed activation (packages/model/src/gpt.ts:170-192) that uses every node type, every basis, a repeated sub-tree
# and an unknown basis name (which the reference evaluates as gelu) ...
COMPOSED_GRAPH = {"type": "add",
                  "left": {"type": "scale", "factor": 0.5, "child": {"type": "mul", "left": {"type": "basis", "op": "silu"},
                                                                     "right": {"type": "basis", "op": "square"}}},
                  "right": {"type": "add",
                            "left": {"type": "mul", "left": {"type": "basis", "op": "relu"}, "right": {"type": "basis", "op": "gelu"}},
                            "right": {"type": "add", "left": {"type": "scale", "factor": -0.3, "child": {"type": "basis", "op": "identity"}},
                                      "right": {"type": "scale", "factor": 0.25, "child": {"type": "basis", "op": "softsign"}}}}}


def _composed_closed_form(h):
    """... and the function it denotes, written out by hand."""
    g = lambda t: F.gelu(t, approximate="tanh")
    return 0.5 * (F.silu(h) * (h * h)) + (F.relu(h) * g(h) + (-0.3 * h + 0.25 * g(h)))


def _torch_forward(cfg, P, tokens, targets, cap=30.0, masks=None, flash=False):
    """The same network in PyTorch float64 (library ops; independent of the oracle's loops).  `masks`: per layer the
    dropout masks of the attention weights and of the two residual branches, in the order the model draws them."""
    Bt, T = tokens.shape
    H, Cc = cfg.nHead, cfg.nEmbd
    D = Cc // H
    x = P["wte"][tokens] + P["wpe"][torch.arange(T)][None]
    mask = torch.triu(torch.ones(T, T, dtype=torch.bool), 1)
    for i in range(cfg.nLayer):
        g = lambda s: P[f"layer.{i}.{s}"]
        h = F.layer_norm(x, (Cc,), g("ln1.weight"), g("ln1.bias"), 1e-5)
        qkv = h.reshape(Bt * T, Cc) @ g("attn.wqkv").T
        if flash:
            # gpt.ts:247-254: the three [B*T, C] matrices re-read as [B*H, T, D] slabs as they lie in memory (no head
            # transpose), causal soft-capped attention per slab (library routine; no dropout on the weights in this
            # branch), then [B, H, T, D] -> transpose(1, 2) -> [B*T, C]
            q, k, v = [t.contiguous().reshape(Bt * H, T, D) for t in qkv.split(Cc, dim=1)]
            bias = torch.zeros(T, T, dtype=torch.float64).masked_fill(mask, float("-inf"))
            s = (q @ k.transpose(1, 2)) / math.sqrt(D)
            s = (cap * torch.tanh(s / cap) if cap > 0 else s) + bias       # a cap of 0 switches it off (interfaces.ts:127-135)
            a = (torch.softmax(s, -1) @ v).reshape(Bt, H, T, D)
            if cap == 0:        # plain causal attention: the library's fused routine must agree
                assert torch.allclose(a, F.scaled_dot_product_attention(q, k, v, is_causal=True).reshape(Bt, H, T, D), atol=1e-9)
        else:
            q, k, v = [t.reshape(Bt, T, H, D).transpose(1, 2) for t in qkv.split(Cc, dim=1)]
            s = (q @ k.transpose(2, 3)) / math.sqrt(D)
            s = cap * torch.tanh(s / cap)
            s = s.masked_fill(mask, -1e9)
            w = torch.softmax(s, -1)
            if masks is not None:
                w = w * masks[i][0].reshape(w.shape)
            a = w @ v
        proj = (a.transpose(1, 2).reshape(Bt * T, Cc) @ g("attn.wo").T).reshape(Bt, T, Cc)
        x = x + (proj * masks[i][1].reshape(proj.shape) if masks is not None else proj)
        h = F.layer_norm(x, (Cc,), g("ln2.weight"), g("ln2.bias"), 1e-5).reshape(Bt * T, Cc)
        act = cfg.ffnActivation
        if act == "swiglu":
            hh = F.silu(h @ g("mlp.fc_gate").T) * (h @ g("mlp.fc_up").T)
            m = hh @ g("mlp.fc_proj").T
        else:
            pre = h @ g("mlp.fc1").T
            if act == "gelu":
                hh = F.gelu(pre, approximate="tanh")
            elif act == "silu":
                hh = F.silu(pre)
            elif act == "relu":
                hh = F.relu(pre)
            elif act == "universal":
                hh = F.silu(pre) * g("mlp.act_gate") + pre * g("mlp.act_skip")
            elif act == "composed":
                hh = _composed_closed_form(pre)
            else:
                hh = (F.silu(pre) * g("mlp.kan_c0") + F.relu(pre) * g("mlp.kan_c1") + F.gelu(pre, approximate="tanh") * g("mlp.kan_c2")
                      + pre * g("mlp.kan_c3") + pre * pre * g("mlp.kan_c4"))
            m = hh @ g("mlp.fc2").T
        m = m.reshape(Bt, T, Cc)
        x = x + (m * masks[i][2].reshape(m.shape) if masks is not None else m)
    x = F.layer_norm(x, (Cc,), P["lnF.weight"], P["lnF.bias"], 1e-5)
    logits = x.reshape(Bt * T, Cc) @ P["lmHead"].T
    return logits, F.cross_entropy(logits, targets.reshape(-1))


def _check_model(act, seed, dropout=0.0, attention="heads", cap=None):
    cfg = rm.ModelConfig(vocabSize=29, blockSize=12, nLayer=2, nEmbd=16, nHead=4, ffnActivation=act, dropout=dropout,
                         activationGraph=COMPOSED_GRAPH if act == "composed" else None, attention=attention, softCap=cap)
    flash = attention == "reference-flash"
    Bm = ref.CpuRef()
    params = rm.initGPT(cfg, Bm, ref.SeededRng(seed))
    entries = rm.collectParamEntries(params)
    rs = np.random.RandomState(seed)
    for _, v in entries:       # perturb so LN weights/biases and gates are generic
        v.data.data += (rs.randn(v.data.data.size) * 0.05).astype(np.float32)
    inp, tgt = rm.synthetic_batch(seed + 1, 3, 12, 29)
    tape = rm.Tape()
    masks = None
    drng = None
    if dropout:
        # DropoutRng (ops.ts:25-82): one mask per dropout site, the counter advancing by one each; per layer the sites are
        # the attention weights [B, H, T, T], the attention branch [B, T, C], the MLP branch [B, T, C] (gpt.ts:276,281,332)
        from tests.util import py_dropout_mask
        drng = rm.DropoutRng(77)
        sizes = [3 * 4 * 12 * 12, 3 * 12 * 16, 3 * 12 * 16]
        if flash:       # no dropout on the attention weights in this branch: two sites per layer, the counter follows
            masks = [[None] + [torch.tensor(py_dropout_mask(77, 2 * l + j, dropout, range(n)).astype(np.float64))
                               for j, n in enumerate(sizes[1:])] for l in range(cfg.nLayer)]
        else:
            masks = [[torch.tensor(py_dropout_mask(77, 3 * l + j, dropout, range(n)).astype(np.float64)) for j, n in enumerate(sizes)]
                     for l in range(cfg.nLayer)]
    logits, loss = rm.gptForward(cfg, params, Bm, tape, inp, tgt, True, drng)
    tape.backward(loss, Bm)
    P = {n: torch.tensor(v.data.data.astype(np.float64)).reshape(v.data.shape).requires_grad_() for n, v in entries}
    tl, tloss = _torch_forward(cfg, P, torch.tensor(inp.data.astype(np.int64)).reshape(3, 12),
                               torch.tensor(tgt.data.astype(np.int64)).reshape(3, 12), masks=masks, flash=flash,
                               cap=30.0 if cap is None else cap)      # gpt.ts:244: config.softCap ?? 30
    tloss.backward()
    assert abs(float(loss.data.data[0]) - tloss.item()) < 2e-6
    assert np.max(np.abs(logits.data.data - tl.detach().numpy().reshape(-1))) < 2e-6
    for n, v in entries:
        want = P[n].grad.numpy().reshape(-1)
        got = v.grad.data.astype(np.float64)
        assert np.max(np.abs(got - want)) <= 2e-6 * (1 + np.max(np.abs(want))), n


def test_full_model_forward_backward_vs_torch_f64_gelu():
    _check_model("gelu", 0)


def test_full_model_forward_backward_vs_torch_f64_custom_activations():
    for act in ("swiglu", "universal", "kan_spline", "silu", "relu"):
        _check_model(act, 3)


def test_full_model_forward_backward_vs_torch_f64_composed_activation():
    _check_model("composed", 4)


def test_full_model_forward_backward_vs_torch_f64_with_dropout():
    """Dropout 0.2 at the three sites of every layer, masks from the independently restated hash."""
    _check_model("gelu", 6, dropout=0.2)


@pytest.mark.parametrize("cap,mag", [(30.0, 1.0), (0.0, 1.0), (2.0, 6.0)])
def test_flash_attention_contract_vs_torch_f64(cap, mag):
    """The oracle's closed forms for Backend.flashAttention / flashAttentionBackward (interfaces.ts:127-135) against PyTorch
    float64 autograd through the materialised definition, incl. scores far into the cap's flat part (where the composed
    clamped-exponential form of ops.ts:329-340 overflows its f32 denominator and is NOT what the fused op computes), and
    against torch's own fused causal attention when the cap is off."""
    rs = np.random.RandomState(5)
    BH, T, D = 3, 19, 8
    q, k, v, do = (rs.randn(BH, T, D).astype(np.float32) * mag for _ in range(4))
    scl = 1 / math.sqrt(D)
    out, lse, _, _ = rm.flash_attention_forward(q, k, v, scl, cap)
    dq, dk, dv = rm.flash_attention_backward(q, k, v, do, scl, cap)
    Q, K, V = (torch.tensor(x.astype(np.float64)).requires_grad_() for x in (q, k, v))
    s = (Q @ K.transpose(1, 2)) * scl
    if cap > 0:
        s = cap * torch.tanh(s / cap)
    s = s.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), float("-inf"))
    o = torch.softmax(s, -1) @ V
    o.backward(torch.tensor(do.astype(np.float64)))
    assert np.max(np.abs(out - o.detach().numpy())) < 1e-12 and np.max(np.abs(lse - torch.logsumexp(s, -1).detach().numpy())) < 1e-12
    for got, want in ((dq, Q.grad), (dk, K.grad), (dv, V.grad)):
        assert np.max(np.abs(got - want.numpy())) < 1e-10 * (1 + float(want.abs().max()))
    if cap == 0:
        assert torch.allclose(o, F.scaled_dot_product_attention(Q, K, V, is_causal=True), atol=1e-12)
    # recorded on the tape (ops.ts:741-770): f32 in and out
    tape = rm.Tape()
    ctx = rm.Ctx(tape, ref.CpuRef())
    qv, kv, vv = (rm.Variable(ref.TD((BH, T, D), "f32", x.reshape(-1).copy()), True) for x in (q, k, v))
    ov = rm.flashAttention(ctx, qv, kv, vv, T, scl, cap)
    tape.backward(ov, ref.CpuRef(), ref.TD((BH, T, D), "f32", do.reshape(-1).copy()))
    assert ov.data.data.dtype == np.float32 and np.array_equal(ov.data.data, out.astype(np.float32).reshape(-1))
    assert np.array_equal(qv.grad.data, dq.astype(np.float32).reshape(-1)) and np.array_equal(vv.grad.data, dv.astype(np.float32).reshape(-1))


def test_flash_branch_of_the_block_vs_torch_f64():
    """gpt.ts:247-254, the branch an unchanged model takes on a backend with flashAttention: slabs cut from [B, T, C]
    without a head transpose.  It is a different function from the heads branch (checked), with the default cap, with a cap
    low enough to bend the scores, with the cap switched off (where torch's fused attention routine is compared too), and
    with dropout (two sites per layer here)."""
    _check_model("gelu", 0, attention="reference-flash")
    _check_model("gelu", 1, attention="reference-flash", cap=0.7)
    _check_model("swiglu", 2, attention="reference-flash", cap=0.0)
    _check_model("gelu", 6, dropout=0.2, attention="reference-flash")
    losses = []
    for att in ("heads", "reference-flash"):
        cfg = rm.ModelConfig(vocabSize=29, blockSize=12, nLayer=2, nEmbd=16, nHead=4, attention=att)
        Bm = ref.CpuRef()
        params = rm.initGPT(cfg, Bm, ref.SeededRng(0))
        for _, v in rm.collectParamEntries(params):
            v.data.data *= 8
        inp, tgt = rm.synthetic_batch(1, 3, 12, 29)
        losses.append(float(rm.gptForward(cfg, params, Bm, rm.Tape(), inp, tgt)[1].data.data[0]))
    assert abs(losses[0] - losses[1]) > 1e-4


def test_dropout_is_off_when_not_training_and_masks_follow_the_step_seed():
    cfg = rm.ModelConfig(vocabSize=29, blockSize=12, nLayer=1, nEmbd=16, nHead=4, dropout=0.3)
    Bm = ref.CpuRef()
    params = rm.initGPT(cfg, Bm, ref.SeededRng(0))
    inp, tgt = rm.synthetic_batch(1, 2, 12, 29)
    ev = [rm.gptForward(cfg, params, Bm, rm.Tape(), inp, tgt, False, rm.DropoutRng(s))[1].data.data[0] for s in (1, 2)]
    assert ev[0] == ev[1]                                                      # ops.ts:575,624: identity unless training
    tr = [rm.gptForward(cfg, params, Bm, rm.Tape(), inp, tgt, True, rm.DropoutRng(s))[1].data.data[0] for s in (1, 1, 2)]
    assert tr[0] == tr[1] and tr[0] != tr[2] and tr[0] != ev[0]
    # trainer.ts:1169,1202: the stream is re-seeded with seed + step * 1000 + microStep before every forward
    t = rm.Trainer(cfg, rm.TrainConfig(iters=3, seed=5), seed=0)
    t.step([(inp, tgt), (inp, tgt)])
    assert (t.dropoutRng.seed, t.dropoutRng.counter) == (5 + 0 * 1000 + 1, 3)
    t.step([(inp, tgt), (inp, tgt)])
    assert (t.dropoutRng.seed, t.dropoutRng.counter) == (5 + 1 * 1000 + 1, 3)


def test_lr_schedule_closed_form():
    tc = rm.TrainConfig(iters=50, lr=3e-4)
    assert abs(rm.lr_at(tc, 0) - (3e-5 + 2.7e-4 * 1 / 10)) < 1e-18            # warm-up = min(2000, 50//5) = 10
    assert abs(rm.lr_at(tc, 9) - 3e-4) < 1e-18
    assert abs(rm.lr_at(tc, 30) - (3e-5 + 2.7e-4 * 0.5 * (1 + math.cos(math.pi * 20 / 40)))) < 1e-18
    assert abs(rm.lr_at(rm.TrainConfig(iters=1, lr=3e-4), 0) - 3e-4) < 1e-18  # no warm-up at iters=1


def test_trainer_step_clip_identity_and_initial_loss():
    cfg = rm.ModelConfig(vocabSize=64, blockSize=16, nLayer=2, nEmbd=32, nHead=4)
    tr = rm.Trainer(cfg, rm.TrainConfig(iters=1), seed=0)
    before = {n: v.data.data.copy() for n, v in tr.entries}
    r = tr.step([rm.synthetic_batch(1, 2, 16, 64)])
    assert abs(r.loss - math.log(64)) < 0.05                # uniform prediction at std-0.02 init
    assert r.gradNorm > 1.0 and abs(r.clipCoef * r.gradNorm - 1.0) < 1e-12      # post-clip norm == clip
    # step 1 from m=v=0: |dp| <= lr * (1 + wd*|p|); sign(dp) = -sign(g) for no-decay tensors
    for n, v in tr.entries:
        d = v.data.data - before[n]
        assert np.all(np.abs(d) <= 3e-4 * (1 + 0.1 * np.abs(before[n])) + 2e-8), n


def test_grad_accumulation_scales_by_one_over_k():
    cfg = rm.ModelConfig(vocabSize=32, blockSize=8, nLayer=1, nEmbd=16, nHead=2)
    b1, b2 = rm.synthetic_batch(5, 2, 8, 32), rm.synthetic_batch(6, 2, 8, 32)
    tr = rm.Trainer(cfg, rm.TrainConfig(iters=1, gradClip=0.0), seed=1)
    r = tr.step([b1, b2])
    tr1 = rm.Trainer(cfg, rm.TrainConfig(iters=1, gradClip=0.0), seed=1)
    l1 = tr1.forward_backward(*b1); l2 = tr1.forward_backward(*b2)
    assert abs(r.loss - (l1 + l2) / 2) < 1e-6              # gpu-perf.test.ts:303-321: sum(loss_i)/K
    sq = sum(ref.sum_sq(v.grad) for _, v in tr1.entries)
    assert abs(r.gradNorm - math.sqrt(sq) * 0.5) < 1e-9


# ---------------------------------------------------------------------------------------------- DataLoader (data.ts:94-167)
def _naive_windows(tok, starts, T):
    """Element-by-element definition: inputs[b,t] = tok[(s+t) % N], targets[b,t] = tok[(s+t+1) % N]."""
    N = len(tok)
    inp = np.array([[tok[(s + t) % N] for t in range(T)] for s in starts], np.int32)
    tgt = np.array([[tok[(s + t + 1) % N] for t in range(T)] for s in starts], np.int32)
    return inp, tgt


def test_dataloader_random_windows_follow_the_rng_stream():
    tok = (np.arange(1000) * 7919 % 503).astype(np.int32)
    dl = rm.DataLoader(tok, ref.SeededRng(11), 4, 16)
    probe = ref.SeededRng(11)
    for _ in range(3):
        x, y = dl.next_batch()
        starts = [int(np.floor(probe.next() * (1000 - 16))) for _ in range(4)]      # data.ts:105,111
        assert all(0 <= s < 1000 - 16 for s in starts)
        inp, tgt = _naive_windows(tok, starts, 16)
        assert np.array_equal(x.data.reshape(4, 16), inp) and np.array_equal(y.data.reshape(4, 16), tgt)
        assert np.array_equal(x.data.reshape(4, 16)[:, 1:], y.data.reshape(4, 16)[:, :-1])     # targets = inputs shifted by one


def test_dataloader_needs_more_tokens_than_the_block():
    with pytest.raises(IndexError):
        rm.DataLoader(np.arange(16, dtype=np.int32), ref.SeededRng(0), 2, 16).next_batch()      # data.ts:97-101
    rm.DataLoader(np.arange(17, dtype=np.int32), ref.SeededRng(0), 2, 16).next_batch()


@pytest.mark.parametrize("N,Bt,T", [(103, 4, 8), (64, 4, 16), (10, 3, 7), (5, 2, 12), (9, 2, 1)])
def test_dataloader_packed_cursors_cover_the_corpus_and_wrap(N, Bt, T):
    tok = (np.arange(N) * 31 % 97).astype(np.int32)
    dl = rm.DataLoader(tok, ref.SeededRng(0), Bt, T, packed=True)
    cursors = [b * (N // Bt) for b in range(Bt)]                                    # data.ts:37-45
    seen = np.zeros(N, np.int64)
    for _ in range(2 * N):
        x, y = dl.next_batch()
        inp, tgt = _naive_windows(tok, cursors, T)
        assert np.array_equal(x.data.reshape(Bt, T), inp) and np.array_equal(y.data.reshape(Bt, T), tgt)
        for c in cursors:
            for t in range(T):
                seen[(c + t) % N] += 1
        cursors = [(c + T) % N for c in cursors]
        assert dl.cursors == cursors
    # every cursor has advanced 2*N*T positions = 2*T whole passes: each token was served equally often
    assert seen.min() == seen.max() == 2 * T * Bt
