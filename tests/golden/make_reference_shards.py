"""Write a reference-made MFQ1 shard set (and the single-file form of the same records) as a fixture.

The reference's own writer -- mfq.formats.shards.write_blob_record_shards with a FileHeader, imported IN THE BUILD
CONTAINER ONLY from /root/reference -- lays seeded byte blobs out as one unsharded file, as shards by tensor count
and as shards by size.  The fixture (tests/golden/reference_shards.npz) holds the input records and every file the
reference wrote, byte for byte; tests check that this package's writer produces the same bytes and that both of its
readers recover the records from them.  Data only; the reference itself never travels.

    python tests/golden/make_reference_shards.py
"""
import sys
import tempfile
from dataclasses import dataclass
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
sys.path.insert(0, "/root/reference")
from mfq.formats.header import FileHeader  # noqa: E402
from mfq.formats.shards import write_blob_record_shards  # noqa: E402


@dataclass
class Rec:
    name: str
    dtype: str
    nbytes: int
    path: Path
    offset: int = 0


rng = np.random.default_rng(2024)
specs = [("blk.0.attn_q.weight", "NINT4", 700), ("__mfq_asset__/config.json", "BLOB", 41), ("blk.0.attn_k.weight", "NINT3", 300),
         ("blk.0.ffn_gate.weight", "NVQ3J-512", 900), ("blk.0.ffn_up.weight", "NVQ3J-512", 900),
         ("blk.0.ffn_down.weight", "NEPQ1-S", 1200), ("blk.0.ffn_gate_up_exps.weight", "NINTM", 1500),
         ("output.weight", "NINT8-0", 64)]
out = {"names": np.array([s[0] for s in specs]), "dtypes": np.array([s[1] for s in specs])}
with tempfile.TemporaryDirectory() as tmp:
    tmp = Path(tmp)
    records = []
    for i, (name, dtype, n) in enumerate(specs):
        blob = rng.integers(0, 256, size=n, dtype=np.uint8).tobytes()
        if dtype == "BLOB":
            blob = b'{"architectures":["Tiny"],"hidden":64}   '[:n]
        p = tmp / f"blob{i}.bin"
        p.write_bytes(blob)
        records.append(Rec(name, dtype, n, p))
        out[f"blob{i}"] = np.frombuffer(blob, dtype=np.uint8)
    header = FileHeader(version=2, model_arch="tiny-arch", extra={"general.name": "tiny", "block_count": 1})
    out["extra_keys"] = np.array(list(header.extra))
    for label, kw in (("single", {}), ("by_count", {"split_max_tensors": 3}), ("by_size", {"split_max_size": 2000})):
        d = tmp / label
        d.mkdir()
        paths = write_blob_record_shards(d / "model.mfq", header, records, **kw)
        out[f"{label}_files"] = np.array([p.name for p in paths])
        for p in paths:
            out[f"{label}/{p.name}"] = np.frombuffer(p.read_bytes(), dtype=np.uint8)
np.savez_compressed(HERE / "reference_shards.npz", **out)
print("wrote", HERE / "reference_shards.npz", {k: v for k, v in out.items() if k.endswith("_files")})
