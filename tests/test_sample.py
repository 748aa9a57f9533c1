"""sample() (packages/train/src/sample.ts): the selection rules on hand-worked distributions with scripted rng draws (these
pin the oracle and the product's host logic alike), then generated sequences on the device against the oracle's."""
import math

import numpy as np
import pytest

from oracle import ref_model as M


class ScriptedRng:
    """Returns the given numbers as successive next() values."""
    def __init__(self, *draws):
        self.draws, self.used = list(draws), 0

    def next(self):
        self.used += 1
        return self.draws.pop(0)


def _both(fn):
    """Run a check against the oracle's selection and the product's."""
    from alpha2_amd.sample import selectToken
    fn(M.select_token)
    fn(selectToken)


def _logits_for(probs):
    return np.log(np.asarray(probs, dtype=np.float64)).astype(np.float32)


def test_greedy_takes_the_first_maximum_and_draws_nothing():
    def check(select):
        rng = ScriptedRng()
        assert select(np.array([0.1, 2.0, -1.0, 2.0, 0.5], dtype=np.float32), rng, 0.0, 40, 1.0) == 1
        assert rng.used == 0
    _both(check)


def test_full_softmax_inverts_the_cumulative_distribution():
    """p = (0.1, 0.2, 0.3, 0.4): cumulative 0.1, 0.3, 0.6, 1.0; a draw r picks the first index with r < cumulative."""
    def check(select):
        for r, want in ((0.0, 0), (0.0999, 0), (0.1001, 1), (0.2999, 1), (0.31, 2), (0.5999, 2), (0.61, 3), (0.9999, 3)):
            rng = ScriptedRng(r)
            assert select(_logits_for([0.1, 0.2, 0.3, 0.4]), rng, 1.0, 0, 1.0) == want, r
            assert rng.used == 1
    _both(check)


def test_top_k_keeps_ties_with_the_kth_value_and_renormalises():
    """logits (3, 1, 2, 2, 0), k = 2: the threshold is the second largest value, 2, and BOTH entries equal to it stay.
    Remaining weights e^3 : e^2 : e^2 -> probabilities (0.5761, 0, 0.2119, 0.2119, 0)."""
    def check(select):
        z = math.e ** 3 + 2 * math.e ** 2
        p0, p2 = math.e ** 3 / z, math.e ** 2 / z
        for r, want in ((p0 - 1e-4, 0), (p0 + 1e-4, 2), (p0 + p2 - 1e-4, 2), (p0 + p2 + 1e-4, 3), (0.9999, 3)):
            assert select(np.array([3, 1, 2, 2, 0], dtype=np.float32), ScriptedRng(r), 1.0, 2, 1.0) == want, r
    _both(check)


def test_nucleus_keeps_the_smallest_prefix_reaching_the_mass_and_samples_inside_it():
    """p = (0.5, 0.3, 0.15, 0.05), top-p 0.7: sorted prefix 0.5 + 0.3 = 0.8 >= 0.7 -> two tokens kept, mass 0.8; the draw
    is scaled by that mass (r * 0.8 < 0.5 picks token 0).  Given out of order to exercise the sort."""
    def check(select):
        probs = [0.15, 0.5, 0.05, 0.3]                       # sorted: index 1 (0.5), 3 (0.3), 0 (0.15), 2 (0.05)
        for r, want in ((0.0, 1), (0.62, 1), (0.63, 3), (0.999, 3)):          # boundary at 0.5 / 0.8 = 0.625
            rng = ScriptedRng(r)
            assert select(_logits_for(probs), rng, 1.0, 0, 0.7) == want, r
            assert rng.used == 1
        # a mass that the first token alone reaches keeps exactly one token whatever the draw
        assert select(_logits_for(probs), ScriptedRng(0.999), 1.0, 0, 0.4) == 1
    _both(check)


def test_top_k_then_nucleus_compose():
    """Top-k first removes all but (0.5, 0.3) [+ nothing tied]; the nucleus then works on the renormalised pair:
    0.625, 0.375 -> top-p 0.6 keeps only the first."""
    def check(select):
        assert select(_logits_for([0.15, 0.5, 0.05, 0.3]), ScriptedRng(0.99), 1.0, 2, 0.6) == 1
        assert select(_logits_for([0.15, 0.5, 0.05, 0.3]), ScriptedRng(0.99), 1.0, 2, 0.7) == 3
    _both(check)


def test_product_and_oracle_selection_agree_on_random_rows():
    from alpha2_amd.sample import selectToken
    from oracle.ref import SeededRng
    rs = np.random.RandomState(0)
    for trial in range(200):
        V = int(rs.randint(2, 60))
        row = (rs.randn(V) * rs.choice([0.5, 2.0, 8.0])).astype(np.float32)
        if trial % 3 == 0:
            row[rs.randint(0, V, size=V // 3)] = row[0]                      # ties
        temp = float(rs.choice([0.0, 0.7, 1.0, 1.3]))
        if temp > 0:
            row = (row.astype(np.float64) / temp).astype(np.float32)
        topk, topp = int(rs.choice([0, 1, 3, 40])), float(rs.choice([1.0, 0.9, 0.5, 0.05]))
        a = M.select_token(row.copy(), SeededRng(trial), temp, topk, topp)
        b = selectToken(row.copy(), SeededRng(trial), temp, topk, topp)
        assert a == b, (trial, V, temp, topk, topp)


# ---------------------------------------------------------------------------------------------- on the device

@pytest.fixture(scope="module")
def B():
    from alpha2_amd import HipBackend
    return HipBackend(0)


@pytest.mark.gpu
@pytest.mark.parametrize("temperature,topk,topp", [(0.0, 0, 1.0), (0.8, 40, 1.0), (1.0, 5, 0.9), (1.2, 0, 0.6)])
def test_generated_tokens_match_the_oracle(B, temperature, topk, topp):
    """Same parameters (bit-equal initialisation), same prompt, same rng seed: the device forward differs from the CPU
    one by fp32 rounding only, which moves a choice only when a draw lands within ~1e-6 of a boundary."""
    from alpha2_amd.model import ModelConfig, initGPT
    from alpha2_amd.rng import SeededRng
    from alpha2_amd.sample import SampleConfig, sampleTokens
    from oracle.ref import CpuRef, SeededRng as ORng
    kw = dict(vocabSize=80, blockSize=24, nLayer=2, nEmbd=64, nHead=2)
    params = initGPT(ModelConfig(**kw), B, SeededRng(7))
    oparams = M.initGPT(M.ModelConfig(**kw), CpuRef(), ORng(7))
    prompt = [3, 17, 42, 5]
    sampleTokens(ModelConfig(**kw), params, B, SeededRng(1), prompt, SampleConfig(steps=2, temperature=0.0, topk=0), B.releaseGpuTensor, B.syncGpu)
    live0 = B.gpuMemStats()["liveAllocs"]                                # parameters are resident now
    got = sampleTokens(ModelConfig(**kw), params, B, SeededRng(11), prompt, SampleConfig(steps=30, temperature=temperature, topk=topk, topp=topp),
                       B.releaseGpuTensor, B.syncGpu)
    want = M.sample_tokens(M.ModelConfig(**kw), oparams, CpuRef(), ORng(11), prompt, 30, temperature, topk, topp)
    assert got.dtype == np.int32 and got.size == 24                      # prompt 4 + generation stops at blockSize
    assert np.array_equal(got, want)
    assert np.array_equal(got[:4], prompt)
    # per-step tensors were released (sample.ts:72-79); a position-index tensor per context length stays cached
    assert B.gpuMemStats()["liveAllocs"] <= live0 + 24


@pytest.mark.gpu
def test_sample_wraps_encode_and_decode(B):
    from alpha2_amd.model import ModelConfig, initGPT
    from alpha2_amd.rng import SeededRng
    from alpha2_amd.sample import SampleConfig, sample
    cfg = ModelConfig(vocabSize=30, blockSize=16, nLayer=1, nEmbd=32, nHead=2)
    params = initGPT(cfg, B, SeededRng(1))
    text = sample(cfg, params, B, SeededRng(2), lambda s: np.array([ord(c) - 97 for c in s], dtype=np.int32),
                  lambda t: "".join(chr(97 + int(x) % 26) for x in t), "abc", SampleConfig(steps=5, temperature=0.0, topk=0), B.releaseGpuTensor)
    assert text.startswith("abc") and len(text) == 8
