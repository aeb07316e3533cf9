"""Extract the lattice / ternary grids the reference vendors as literals into raw
binary data files, WITHOUT importing the reference: its source files are read as
text, the hex / base85 literals are decoded, and each table's SHA-256 is checked
against the hash the reference itself pins (mfq/formats/nvq.py:95-99,
mfq/formats/nvq1_l.py:75, mfq/formats/nvq1_s.py:131).

The tables are data (llama.cpp's kgrid_2bit_256 / kgrid_256 / kgrid_512 /
iq1s_grid, and the reference's NVQ1-S synthetic banks); the .bin files written
under tyloquant_amd/data/ are what the synthetic payload producers and the tests
load.  Run only in the build container (it needs /root/reference).

    python tests/golden/extract_reference_tables.py
"""
from __future__ import annotations

import base64
import hashlib
import re
from pathlib import Path

REF = Path("/root/reference/mfq/formats")
OUT = Path(__file__).resolve().parents[2] / "tyloquant_amd" / "data"

EXPECTED = {
    "e8_256": "915952ebc4af8ddba8113583ca1316fc818843f7b825bbf1a25ae1c39bf0e16d",
    "d4_256": "c9678803c61b2210fbd8cbbb3f965a835409cd7d88a04d086d236261bd221d11",
    "d4_512": "353274c58dd7d8dc5ee960dc8fc54ff9164eaf2b49206b841cd49415cf393f81",
    "iq1s_2048": "e9ffebfc997ad6023063a667c0bf4eedd8ebf7f56b3da399cbc7d1b1f7ea52c6",
    "nvq1s_banks": "beb341195ce650979d2640b6a494652047d8a371ea0af66183fc5c9f38a5a37e",
}


def _literal(text: str, name: str) -> str:
    m = re.search(name + r'\s*=\s*"""(.*?)"""', text, re.S)
    if not m:
        raise SystemExit(f"literal {name} not found")
    return "".join(m.group(1).split())


def main() -> None:
    OUT.mkdir(parents=True, exist_ok=True)
    nvq = (REF / "nvq.py").read_text()
    raw = {
        "e8_256": bytes.fromhex(_literal(nvq, "_E8_256_HEX")),
        "d4_256": bytes.fromhex(_literal(nvq, "_D4_256_HEX")),
        "d4_512": bytes.fromhex(_literal(nvq, "_D4_512_HEX")),
        "iq1s_2048": base64.b85decode(
            _literal((REF / "nvq1_l.py").read_text(), "_IQ1S_GRID_B85").encode()),
        "nvq1s_banks": base64.b85decode(
            _literal((REF / "nvq1_s.py").read_text(), "_NVQ1_S_SYNTHETIC_BANKS_B85").encode()),
    }
    for name, data in raw.items():
        digest = hashlib.sha256(data).hexdigest()
        if digest != EXPECTED[name]:
            raise SystemExit(f"{name}: sha256 {digest} != {EXPECTED[name]}")
        (OUT / f"{name}.bin").write_bytes(data)
        print(f"{name}: {len(data)} bytes sha256 ok")


if __name__ == "__main__":
    main()
