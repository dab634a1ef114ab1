"""Lossless container for the reference's golden ``.block4`` files.

A ``.block4`` file is raw little-endian int32 quadruples.  The four columns are
smooth, so each is stored as its first difference and the whole is xz-packed:
23 MB of golden data becomes ~50 KB.  ``decode`` returns the exact bytes of the
original file; ``MANIFEST.json`` holds their SHA-256 so the round trip is
checked, not assumed.
"""
from __future__ import annotations

import hashlib
import json
import lzma
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
BLOCK4_DIR = HERE / "block4"
MANIFEST = BLOCK4_DIR / "MANIFEST.json"


def encode(raw: bytes) -> bytes:
    a = np.frombuffer(raw, dtype="<i4").reshape(-1, 4)
    cols = [np.diff(a[:, i], prepend=np.int32(0)).astype("<i4") for i in range(4)]
    return lzma.compress(np.concatenate(cols).tobytes(), preset=9)


def decode(packed: bytes) -> bytes:
    flat = np.frombuffer(lzma.decompress(packed), dtype="<i4")
    cols = flat.reshape(4, -1)
    a = np.cumsum(cols, axis=1, dtype=np.int32).T
    return np.ascontiguousarray(a, dtype="<i4").tobytes()


def manifest() -> dict:
    return json.loads(MANIFEST.read_text())


def names():
    return sorted(manifest())


def load(name: str) -> np.ndarray:
    """Golden metadata of one graph as int32 [B, 4], verified against its hash."""
    entry = manifest()[name]
    raw = decode((BLOCK4_DIR / entry["file"]).read_bytes())
    if hashlib.sha256(raw).hexdigest() != entry["sha256"] or len(raw) != entry["bytes"]:
        raise RuntimeError(f"golden fixture {name} does not decode to the recorded bytes")
    return np.frombuffer(raw, dtype="<i4").reshape(-1, 4)
