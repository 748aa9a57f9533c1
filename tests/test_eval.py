"""evaluate() (packages/train/src/eval.ts:15-61): the oracle restatement pinned by closed forms, the device path against it."""
import math

import numpy as np
import pytest

from oracle import ref
from oracle import ref_model as rm

CFG = dict(vocabSize=64, blockSize=16, nLayer=1, nEmbd=32, nHead=2)
TEXT = "".join(chr(32 + (i * 7 + i // 5) % 60) for i in range(900))


class CharTok:
    """A tokenizer in the sense of packages/core/src/interfaces.ts:17-23: code point - 32."""
    name, vocabSize = "char", 64

    def encode(self, text):
        return np.array([min(63, max(0, ord(c) - 32)) for c in text], dtype=np.int32)


def test_oracle_evaluate_closed_forms():
    O = ref.CpuRef()
    cfg = rm.ModelConfig(**CFG)
    params = rm.initGPT(cfg, O, ref.SeededRng(3))
    tokens = CharTok().encode(TEXT)
    # all logits equal (zero output projection): every batch loss is ln V whatever the batch, perplexity = V
    params["lmHead"].data.data[:] = 0.0
    loss, ppl = rm.evaluate(cfg, params, O, tokens, ref.SeededRng(5), 4, 3)
    assert abs(loss - math.log(64)) < 1e-6 and abs(ppl - 64) < 1e-3
    # general case: the mean of the losses of the batches the same rng stream produces, in that order
    params = rm.initGPT(cfg, O, ref.SeededRng(3))
    loss, ppl = rm.evaluate(cfg, params, O, tokens, ref.SeededRng(5), 4, 3)
    loader, manual = rm.DataLoader(tokens, ref.SeededRng(5), 4, 16), []
    for _ in range(3):
        x, y = loader.next_batch()
        manual.append(float(rm.gptForward(cfg, params, O, rm.Tape(), x, y)[1].data.data[0]))
    assert abs(loss - sum(manual) / 3) < 1e-12 and ppl == math.exp(loss)
    assert len(set(manual)) == 3                                    # three different batches were drawn


def test_text_helpers(tmp_path):
    from alpha2_amd import data
    p = tmp_path / "t.txt"
    p.write_text(TEXT, encoding="utf-8")
    assert data.loadText(str(p)) == TEXT
    tok = CharTok()
    assert np.array_equal(data.encodeText(TEXT, tok), tok.encode(TEXT))
    old = data.FROM_TEXT_CHUNK_CHARS
    try:                                                            # pieces are encoded separately and concatenated
        data.FROM_TEXT_CHUNK_CHARS = 100
        assert np.array_equal(data.encodeText(TEXT, tok), tok.encode(TEXT))
    finally:
        data.FROM_TEXT_CHUNK_CHARS = old
    big = tmp_path / "big.bin"
    with open(big, "wb") as f:
        f.truncate(data.MAX_STRING_BYTES + 1)
    with pytest.raises(ValueError, match="too large"):
        data.loadText(str(big))


@pytest.mark.gpu
def test_device_evaluate_matches_oracle(tmp_path):
    from alpha2_amd import HipBackend
    from alpha2_amd.eval import evaluate
    from alpha2_amd.model import ModelConfig, initGPT
    from alpha2_amd.rng import SeededRng
    B = HipBackend(0)
    p = tmp_path / "val.txt"
    p.write_text(TEXT, encoding="utf-8")
    cfg = ModelConfig(**CFG)
    params = initGPT(cfg, B, SeededRng(3))
    live0 = B.gpuMemStats()["liveAllocs"]
    r = evaluate(cfg, params, B, CharTok(), SeededRng(5), str(p), 4, 9)
    O = ref.CpuRef()
    ocfg = rm.ModelConfig(**CFG)
    oloss, oppl = rm.evaluate(ocfg, rm.initGPT(ocfg, O, ref.SeededRng(3)), O, CharTok().encode(TEXT), ref.SeededRng(5), 4, 9)
    assert r.nBatches == 9
    assert abs(r.loss - oloss) <= 1e-4 * abs(oloss), (r.loss, oloss)
    assert abs(r.perplexity - oppl) <= 2e-4 * oppl
    r2 = evaluate(cfg, params, B, CharTok(), SeededRng(5), str(p), 4, 9)
    assert r2.loss == r.loss                                          # same rng seed, same batches, same result
    assert B.gpuMemStats()["liveAllocs"] <= live0 + 40                # nothing accumulates per batch (parameters upload lazily)
