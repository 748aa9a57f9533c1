"""Token files either side of the DataLoader (packages/train/src/data.ts:179-397): chunked tokenisation of large text
files, the `.tokens` cache next to the corpus, and the newline-aligned train/validation split.

`.tokens` cache (data.ts:297-358): 8 bytes big-endian float64 = mtime of the source file in milliseconds, then the tokens as
little-endian int32.  File name `<data>.<tokenizer.name>-<vocabSize>[.<startByte>-<endByte>].tokens`; a cache is used when
its stored mtime is within 1 ms of the source's.  A tokenizer is any object with `name`, `vocabSize` and
`encode(text) -> int32 array` (packages/core/src/interfaces.ts:17-23); tokenizers themselves are not part of this package.
"""
from __future__ import annotations

import os
import struct
from typing import Optional, Tuple

import numpy as np

MAX_STRING_BYTES = 30 * 1024 * 1024          # data.ts:180
CHUNK_BYTES = 10 * 1024 * 1024               # data.ts:238


def loadText(path: str) -> str:
    """data.ts:182-193: the whole file as one string; files above 30 MB are refused (tokenise those with loadAndTokenize)."""
    size = os.stat(path).st_size
    if size > MAX_STRING_BYTES:
        raise ValueError(f"File is {size / 1024 / 1024:.0f}MB — too large for a single string. "
                         "Use loadAndTokenize() for data loading.")
    with open(path, "r", encoding="utf-8", errors="replace") as f:
        return f.read()


FROM_TEXT_CHUNK_CHARS = 5_000_000            # data.ts:64


def encodeText(text: str, tokenizer) -> np.ndarray:
    """The tokenisation step of DataLoader.fromText (data.ts:61-87): at once up to 5 M characters, else in 5 M-character
    pieces whose token arrays are concatenated."""
    if len(text) <= FROM_TEXT_CHUNK_CHARS:
        return np.asarray(tokenizer.encode(text), dtype=np.int32)
    parts = [np.asarray(tokenizer.encode(text[i:i + FROM_TEXT_CHUNK_CHARS]), dtype=np.int32) for i in range(0, len(text), FROM_TEXT_CHUNK_CHARS)]
    return np.concatenate(parts)


def loadAndTokenize(path: str, tokenizer, range_: Optional[Tuple[int, int]] = None) -> np.ndarray:
    """data.ts:228-290: whole range at once up to 30 MB, else 10 MB chunks cut at the last newline."""
    size = os.stat(path).st_size
    start, end = range_ if range_ is not None else (0, size)
    total = end - start
    with open(path, "rb") as f:
        if total <= MAX_STRING_BYTES:
            f.seek(start)
            return np.asarray(tokenizer.encode(f.read(total).decode("utf-8", "replace")), dtype=np.int32)
        chunks, pos = [], start
        while pos < end:
            f.seek(pos)
            buf = f.read(min(CHUNK_BYTES, end - pos))
            cut = len(buf)
            if pos + len(buf) < end:
                nl = buf.rfind(b"\n", 0, cut)
                if nl > 0:
                    cut = nl + 1
            chunks.append(np.asarray(tokenizer.encode(buf[:cut].decode("utf-8", "replace")), dtype=np.int32))
            pos += cut
    return np.concatenate(chunks) if chunks else np.zeros(0, np.int32)


def tokenCachePath(dataPath: str, tokenizer, range_: Optional[Tuple[int, int]] = None) -> str:
    suffix = f".{range_[0]}-{range_[1]}" if range_ is not None else ""
    return f"{dataPath}.{tokenizer.name}-{tokenizer.vocabSize}{suffix}.tokens"


def readTokenCache(cacheFile: str) -> Tuple[float, np.ndarray]:
    """(source mtime in ms, tokens).  A trailing partial int32 is ignored, as `tokenBytes / 4` truncates in the reference."""
    with open(cacheFile, "rb") as f:
        raw = f.read()
    if len(raw) < 8:
        raise ValueError(f"{cacheFile}: shorter than its 8-byte header")
    (mtime,) = struct.unpack(">d", raw[:8])
    n = (len(raw) - 8) // 4
    return mtime, np.frombuffer(raw, dtype="<i4", count=n, offset=8).astype(np.int32)


def writeTokenCache(cacheFile: str, mtimeMs: float, tokens) -> None:
    with open(cacheFile, "wb") as f:
        f.write(struct.pack(">d", float(mtimeMs)))
        f.write(np.ascontiguousarray(tokens, dtype="<i4").tobytes())


def loadOrCacheTokens(dataPath: str, tokenizer, range_: Optional[Tuple[int, int]] = None) -> np.ndarray:
    """data.ts:297-358."""
    cacheFile = tokenCachePath(dataPath, tokenizer, range_)
    src_mtime = os.stat(dataPath).st_mtime_ns / 1e6
    try:
        if os.stat(cacheFile).st_size > 8:
            cached_mtime, tokens = readTokenCache(cacheFile)
            if abs(cached_mtime - src_mtime) < 1:
                return tokens
    except OSError:
        pass                                      # no cache: tokenize
    tokens = loadAndTokenize(dataPath, tokenizer, range_)
    try:
        writeTokenCache(cacheFile, src_mtime, tokens)
    except OSError:
        pass                                      # the reference only warns (data.ts:353-355)
    return tokens


def getSplitByte(path: str, trainRatio: float = 0.9) -> int:
    """data.ts:364-388: the byte after the newline nearest to size * ratio (searching forward first) within +-4096 bytes."""
    size = os.stat(path).st_size
    approx = int(size * trainRatio)               # Math.floor for non-negative values
    window = 4096
    start = max(0, approx - window)
    with open(path, "rb") as f:
        f.seek(start)
        buf = f.read(min(window * 2, size - start))
    target = approx - start
    for i in range(target, len(buf)):
        if buf[i] == 0x0A:
            return start + i + 1
    for i in range(target - 1, -1, -1):
        if buf[i] == 0x0A:
            return start + i + 1
    return approx


def splitText(text: str, trainRatio: float = 0.9) -> Tuple[str, str]:
    """data.ts:391-397."""
    i = int(len(text) * trainRatio)
    return text[:i], text[i:]
