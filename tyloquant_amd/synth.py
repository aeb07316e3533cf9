"""Seeded synthetic payloads of the BASELINE configurations (there is no network for real checkpoints).

NINT tensors come from the NINT quantizer on N(0, sigma) weights; NVQ / NEPQ tensors are drawn directly
in the packed domain, as the reference's own fixtures do (tests/test_nvq3j512_cpp_runtime.py:58-75,
tests/mixed_family_fixtures.py:55-153).  Large tensors quantize a `slab_rows` slab and tile it over the
rows, which leaves the value distribution and every byte count unchanged.
"""
from __future__ import annotations

import math
from pathlib import Path

import numpy as np

from . import formats as F
from .quantize import nint_quantize

_DATA = Path(__file__).resolve().parent / "data"

# expert-wise production profiles: bits -> (bits, groupsize, sub_bits)
MOE_PROFILES = {2: (2, 16, 5), 3: (3, 24, 5), 4: (4, 24, 6), 5: (5, 28, 7)}


def activations(rng, M, K, outlier_frac=0.0, outlier_scale=20.0) -> np.ndarray:
    """N(0,1) rows; a fraction of the K channels (chosen once) is scaled up (BASELINE config 2)."""
    x = rng.standard_normal((M, K)).astype(np.float32)
    n = math.ceil(outlier_frac * K) if outlier_frac > 0 else 0
    if n:
        x[:, rng.choice(K, size=n, replace=False)] *= outlier_scale
    return x


def nint_linear_blob(seed, out, K, bits, gs, sub_bits, sigma=0.02, slab_rows=None):
    """(dtype, blob) of an [out, K] NINT tensor quantized from N(0, sigma) weights."""
    rng = np.random.default_rng(seed)
    rows = out if slab_rows is None else min(out, slab_rows)
    W = (rng.standard_normal((rows, K)) * sigma).astype(np.float32)
    r = nint_quantize(W, bits, gs, sub_bits)
    if rows < out:
        reps = -(-out // rows)
        for k in ("ns", "nm", "ss", "sm", "q"):
            r[k] = np.concatenate([r[k]] * reps, axis=0)[:out]
    return f"NINT{bits}", F.nint_blob(bits, sub_bits, gs, K, r["ns"], r["nm"], r["ss"], r["sm"], r["q"])


def d4_512_banks(banks=2) -> np.ndarray:
    raw = np.frombuffer((_DATA / "d4_512.bin").read_bytes(), dtype="<u2")
    digits = (raw[:, None] >> (3 * np.arange(4, dtype=np.uint16))[None, :]) & 7
    grid = (2 * digits + 1).astype(np.int16) * 8
    return np.stack([np.roll(grid, 7 * b, axis=0) for b in range(banks)]).astype(np.int8)


def nvq3j512_blob(seed, out, K, banks=2):
    """NVQ3J-512: D4_512 * 8 and a rolled copy as banks, scale LUT linspace(0.45, 1.55), anchors
    U(0.002, 0.02) * 0.02, random state / index / sign streams."""
    rng = np.random.default_rng(seed)
    ng, nvec, nsign = math.ceil(K / 24), math.ceil(K / 4), math.ceil(K / 8)
    blob = F.nvq_jsc_blob(
        "d4_512", K, rng.uniform(0.002, 0.02, out).astype(np.float32) * 0.02, np.linspace(0.45, 1.55, 16, dtype=np.float32),
        np.arange(16) % banks, d4_512_banks(banks), rng.integers(0, 16, (out, ng), dtype=np.uint8),
        rng.integers(0, 512, (out, nvec), dtype=np.uint16), rng.integers(0, 128, (out, nsign), dtype=np.uint8))
    return "NVQ3J-512", blob


def nepq1_blob(seed, label, out, K, banks=16, experts=1):
    rng = np.random.default_rng(seed)
    pid = F.NEPQ_PROFILE[label]
    sb, ib, ab, tb = F.NEPQ_BITS[pid]
    iq1s = np.frombuffer((_DATA / "iq1s_2048.bin").read_bytes(), dtype="<u2")
    tables = []
    for _ in range(banks):
        if label == "NEPQ1-L":
            tables.append(rng.permutation(iq1s).astype("<u2").tobytes())
        else:
            tables.append(rng.permutation(iq1s)[:512].astype("<u2").tobytes()
                          + rng.permutation(iq1s)[:512].astype("<u2").tobytes())
    tables = np.frombuffer(b"".join(tables), dtype=np.uint8).reshape(banks, tb)
    ng, nvec = math.ceil(K / 24), K // 8
    nsuper = math.ceil(ng / 4)
    shape = (experts, out, K)
    blob = F.nepq_blob(label, shape, tables, rng.uniform(0.0005, 0.005, (experts, out)).astype(np.float32),
                       rng.integers(0, 1 << sb, (experts, out, ng), dtype=np.uint8),
                       rng.integers(0, 1 << ib, (experts, out, nvec), dtype=np.uint16),
                       rng.integers(0, 2, (experts, out, ng), dtype=np.uint8),
                       rng.integers(0, banks, (experts, out, nsuper), dtype=np.uint8))
    return label, blob
