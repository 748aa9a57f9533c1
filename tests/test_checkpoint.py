"""The reference's checkpoint container (packages/train/src/checkpoint.ts): byte layout pinned by a hand-assembled file that
follows the layout comment at checkpoint.ts:6-11; oracle and product writers/readers against it and against each other.
No checkpoint file ships with the reference, so there is no reference-written fixture: parity with a file produced by the
reference itself is unpinned beyond this layout."""
import json
import struct

import numpy as np
import pytest

from oracle import ref_model as rm
from oracle.ref import TD


def _tiny_state(mod):
    """mod = namespace providing the tensor type for optimizer buffers."""
    w = np.array([1.5, -2.25, 0.125, 3.0, -0.5, 7.0], np.float32)
    b = np.array([0.0, -1.0], np.float32)
    bufs = {"w.m": mod((6,), "f32", w * 0.1), "w.v": mod((6,), "f32", w * w), "b.m": mod((2,), "f32", b), "b.v": mod((2,), "f32", b * b)}
    return {"modelConfig": {"vocabSize": 4, "nLayer": 1}, "configHash": "abc123", "rngState": 42, "step": 7,
            "params": {"w": {"shape": [2, 3], "data": w}, "b": {"shape": [2], "data": b}},
            "optimizerState": {"step": 7, "buffers": bufs}}


def _hand_assembled():
    """Bytes written field by field from the documented layout, independent of both implementations."""
    w = np.array([1.5, -2.25, 0.125, 3.0, -0.5, 7.0], "<f4")
    b = np.array([0.0, -1.0], "<f4")
    tensors = [{"name": "p.w", "shape": [2, 3], "elements": 6}, {"name": "p.b", "shape": [2], "elements": 2},
               {"name": "o.w.m", "shape": [6], "elements": 6}, {"name": "o.w.v", "shape": [6], "elements": 6},
               {"name": "o.b.m", "shape": [2], "elements": 2}, {"name": "o.b.v", "shape": [2], "elements": 2}]
    header = ('{"modelConfig":{"vocabSize":4,"nLayer":1},"configHash":"abc123","rngState":42,"step":7,"optimizerStep":7,"tensors":'
              + json.dumps(tensors, separators=(",", ":")) + "}").encode()
    payload = w.tobytes() + b.tobytes() + (w * np.float32(0.1)).astype("<f4").tobytes() + (w * w).tobytes() + b.tobytes() + (b * b).tobytes()
    return b"ALPH" + struct.pack("<I", len(header)) + header + payload


def _check_loaded(st):
    assert st["step"] == 7 and st["rngState"] == 42 and st["configHash"] == "abc123" and st["modelConfig"] == {"vocabSize": 4, "nLayer": 1}
    assert st["optimizerState"]["step"] == 7
    assert list(st["params"]) == ["w", "b"] and st["params"]["w"]["shape"] == [2, 3]
    assert np.array_equal(np.asarray(st["params"]["w"]["data"]), np.array([1.5, -2.25, 0.125, 3.0, -0.5, 7.0], np.float32))
    assert list(st["optimizerState"]["buffers"]) == ["w.m", "w.v", "b.m", "b.v"]
    assert np.array_equal(np.asarray(st["optimizerState"]["buffers"]["w.v"].data), np.array([2.25, 5.0625, 0.015625, 9.0, 0.25, 49.0], np.float32))


def test_oracle_writer_and_reader_follow_the_documented_layout():
    want = _hand_assembled()
    assert rm.checkpoint_save_bytes(_tiny_state(TD)) == want
    assert want[:4] == b"ALPH" and struct.unpack_from("<I", want, 4)[0] == want.index(b"}]}") + 3 - 8
    _check_loaded(rm.checkpoint_load_bytes(want))


def test_product_file_checkpoint_matches_oracle_bytes_and_round_trips(tmp_path):
    from alpha2_amd.backend import TensorData
    from alpha2_amd.checkpoint import CheckpointError, FileCheckpoint
    p = tmp_path / "run" / "ckpt.bin"            # the directory is created on save (checkpoint.ts:68-70)
    FileCheckpoint().save(str(p), _tiny_state(TensorData))
    assert p.read_bytes() == _hand_assembled() == rm.checkpoint_save_bytes(_tiny_state(TD))
    _check_loaded(FileCheckpoint().load(str(p)))
    _check_loaded(rm.checkpoint_load_bytes(p.read_bytes()))
    with pytest.raises(CheckpointError, match="Failed to load checkpoint"):
        FileCheckpoint().load(str(tmp_path / "missing.bin"))
    (tmp_path / "cut.bin").write_bytes(_hand_assembled()[:-5])
    with pytest.raises(CheckpointError):
        FileCheckpoint().load(str(tmp_path / "cut.bin"))


def test_optional_header_members_and_legacy_json(tmp_path):
    from alpha2_amd.backend import TensorData
    from alpha2_amd.checkpoint import FileCheckpoint
    st = _tiny_state(TensorData)
    st["tokenizerArtifacts"] = {"type": "char", "vocab": ["a", "b"]}
    st["symbioActivationGraph"] = {"op": "gelu"}
    FileCheckpoint().save(str(tmp_path / "a.bin"), st)
    raw = (tmp_path / "a.bin").read_bytes()
    hdr = json.loads(raw[8:8 + struct.unpack_from("<I", raw, 4)[0]])
    assert list(hdr) == ["modelConfig", "configHash", "rngState", "step", "tokenizerArtifacts", "optimizerStep", "symbioActivationGraph", "tensors"]
    back = FileCheckpoint().load(str(tmp_path / "a.bin"))
    assert back["tokenizerArtifacts"] == st["tokenizerArtifacts"] and back["symbioActivationGraph"] == {"op": "gelu"}
    # legacy JSON form (checkpoint.ts:168-189): plain arrays, optimizer buffers as {shape, data}
    legacy = {"modelConfig": {"nLayer": 1}, "params": {"w": {"shape": [2], "data": [1.0, 2.0]}}, "rngState": 3, "configHash": "h", "step": 5,
              "optimizerState": {"step": 5, "buffers": {"w.m": {"shape": [2], "data": [0.5, 0.25]}}}}
    (tmp_path / "l.json").write_text(json.dumps(legacy))
    for st2 in (FileCheckpoint().load(str(tmp_path / "l.json")), rm.checkpoint_load_bytes(json.dumps(legacy).encode())):
        assert st2["step"] == 5 and st2["optimizerState"]["step"] == 5
        assert np.array_equal(np.asarray(st2["optimizerState"]["buffers"]["w.m"].data), np.array([0.5, 0.25], np.float32))
        assert st2["params"]["w"]["data"] == [1.0, 2.0]


def test_restore_params_concatenates_separate_qkv_of_old_checkpoints():
    cfg = rm.ModelConfig(vocabSize=16, blockSize=8, nLayer=1, nEmbd=8, nHead=2)
    tr = rm.Trainer(cfg, rm.TrainConfig(iters=1), seed=0)
    saved = {n: {"shape": list(v.data.shape), "data": np.full(v.data.data.size, 0.5, np.float32)} for n, v in tr.entries if not n.endswith("wqkv")}
    for i, w in enumerate(("wq", "wk", "wv")):
        saved[f"layer.0.attn.{w}"] = {"shape": [8, 8], "data": np.full(64, float(i + 1), np.float32)}
    rm.restore_params(tr.entries, saved)
    got = dict(tr.entries)["layer.0.attn.wqkv"].data.data
    assert np.array_equal(got, np.repeat(np.array([1, 2, 3], np.float32), 64))
    assert np.all(dict(tr.entries)["wte"].data.data == 0.5)


def test_oracle_resume_continues_bit_for_bit():
    """Save after 3 steps, resume in a fresh trainer: the next steps equal the uninterrupted run exactly (the beta powers are
    rebuilt as pow(beta, step), optimizers.ts:214-215, which differs from the running product by at most rounding: bound it)."""
    cfg = rm.ModelConfig(vocabSize=32, blockSize=16, nLayer=1, nEmbd=16, nHead=2)
    mk = lambda: rm.Trainer(cfg, rm.TrainConfig(iters=6), seed=1)
    a = mk()
    batches = [rm.synthetic_batch(100 + s, 2, 16, 32) for s in range(6)]
    for s in range(3):
        a.step([batches[s]])
    raw = rm.checkpoint_save_bytes({"modelConfig": {}, "configHash": "", "rngState": 0, "step": a.step_idx,
                                    "params": {n: {"shape": list(v.data.shape), "data": v.data.data.copy()} for n, v in a.entries},
                                    "optimizerState": a.opt.state_dict()})
    b = mk()
    st = rm.checkpoint_load_bytes(raw)
    rm.restore_params(b.entries, st["params"])
    b.opt.load_state_dict(st["optimizerState"])
    b.step_idx = st["step"]
    for s in range(3, 6):
        ra, rb = a.step([batches[s]]), b.step([batches[s]])
        assert abs(ra.loss - rb.loss) <= 1e-6 * abs(ra.loss) and ra.lr == rb.lr, (s, ra.loss, rb.loss)
