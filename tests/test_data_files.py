"""Token cache files and corpus splitting (packages/train/src/data.ts:179-397).  The cache layout (big-endian float64 mtime,
little-endian int32 tokens) is pinned by a hand-assembled file; the reference ships no cache fixture."""
import os
import struct

import numpy as np

from alpha2_amd import data as D


class ByteTok:
    name, vocabSize = "byte", 256

    def __init__(self):
        self.calls = 0

    def encode(self, text):
        self.calls += 1
        return np.frombuffer(text.encode("utf-8"), dtype=np.uint8).astype(np.int32)


def test_token_cache_layout_and_invalidation(tmp_path):
    src = tmp_path / "corpus.txt"
    src.write_bytes(b"hello\nworld\n")
    tok = ByteTok()
    t1 = D.loadOrCacheTokens(str(src), tok)
    assert tok.calls == 1 and t1.dtype == np.int32 and bytes(t1.astype(np.uint8)) == b"hello\nworld\n"
    cache = tmp_path / "corpus.txt.byte-256.tokens"                       # <data>.<name>-<vocab>.tokens
    raw = cache.read_bytes()
    mtime_ms = os.stat(src).st_mtime_ns / 1e6
    assert raw == struct.pack(">d", mtime_ms) + np.frombuffer(b"hello\nworld\n", np.uint8).astype("<i4").tobytes()
    t2 = D.loadOrCacheTokens(str(src), tok)                               # served from the cache: no second encode
    assert tok.calls == 1 and np.array_equal(t1, t2)
    os.utime(src, ns=(os.stat(src).st_atime_ns, os.stat(src).st_mtime_ns + 5_000_000))      # source touched 5 ms later
    D.loadOrCacheTokens(str(src), tok)
    assert tok.calls == 2
    # a hand-written cache is read back exactly; a truncated tail is ignored
    D.writeTokenCache(str(tmp_path / "x.tokens"), 1234.5, [1, -2, 70000])
    hand = struct.pack(">d", 1234.5) + struct.pack("<3i", 1, -2, 70000)
    assert (tmp_path / "x.tokens").read_bytes() == hand
    (tmp_path / "y.tokens").write_bytes(hand + b"\x01\x02")
    m, t = D.readTokenCache(str(tmp_path / "y.tokens"))
    assert m == 1234.5 and t.tolist() == [1, -2, 70000]
    rng = D.loadOrCacheTokens(str(src), tok, (6, 12))
    assert bytes(rng.astype(np.uint8)) == b"world\n" and (tmp_path / "corpus.txt.byte-256.6-12.tokens").exists()


def test_chunked_tokenisation_cuts_at_newlines(tmp_path, monkeypatch):
    monkeypatch.setattr(D, "MAX_STRING_BYTES", 64)
    monkeypatch.setattr(D, "CHUNK_BYTES", 50)
    lines = [("line %03d " % i) * 2 + "\n" for i in range(20)]            # 19-byte lines
    src = tmp_path / "big.txt"
    src.write_text("".join(lines))
    seen = []

    class Tok(ByteTok):
        def encode(self, text):
            seen.append(text)
            return super().encode(text)
    out = D.loadAndTokenize(str(src), Tok())
    assert bytes(out.astype(np.uint8)).decode() == "".join(lines)          # nothing lost or duplicated
    assert len(seen) > 1 and all(s.endswith("\n") for s in seen)           # every chunk ends on a line boundary
    part = D.loadAndTokenize(str(src), Tok(), (19, 19 * 5))
    assert bytes(part.astype(np.uint8)).decode() == "".join(lines[1:5])


def test_split_byte_lands_after_the_nearest_newline(tmp_path):
    src = tmp_path / "c.txt"
    body = b"".join(b"x" * 9 + b"\n" for _ in range(100))                 # newline at every 10th byte
    src.write_bytes(body)
    assert D.getSplitByte(str(src), 0.899) == 900                          # byte 899 is a newline: found at once, the split is the byte after
    assert D.getSplitByte(str(src), 0.9) == 910                            # from byte 900 the next newline forward is byte 909
    src.write_bytes(b"a" * 50 + b"\n" + b"b" * 49)                         # only newline lies before the split point
    assert D.getSplitByte(str(src), 0.9) == 51
    src.write_bytes(b"z" * 100)
    assert D.getSplitByte(str(src), 0.5) == 50                             # no newline in the window: the raw split
    assert D.splitText("abcdefghij", 0.75) == ("abcdefg", "hij")
