"""Writes tests/golden/block4/*.xz and MANIFEST.json from the reference's own
golden outputs (block_level_meta/*.block4 in the upstream tree).

Run once in the build container, where the upstream tree is mounted:
    python tests/golden/make_block4_fixtures.py /root/reference
Only data files are read; no reference code is imported or executed.
"""
import hashlib
import json
import sys
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parent))
import block4_codec as codec  # noqa: E402


def main(ref_root: str) -> None:
    src = Path(ref_root) / "block_level_meta"
    codec.BLOCK4_DIR.mkdir(parents=True, exist_ok=True)
    man = {}
    for f in sorted(src.glob("*.block4")):
        raw = f.read_bytes()
        packed = codec.encode(raw)
        assert codec.decode(packed) == raw
        out = codec.BLOCK4_DIR / (f.stem + ".block4.dxz")
        out.write_bytes(packed)
        man[f.stem] = {"file": out.name, "bytes": len(raw), "blocks": len(raw) // 16,
                       "sha256": hashlib.sha256(raw).hexdigest()}
        print(f.stem, len(raw), "->", len(packed))
    codec.MANIFEST.write_text(json.dumps(man, indent=1, sort_keys=True) + "\n")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
