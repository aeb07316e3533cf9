"""Seeded synthetic payloads of the BASELINE configurations (there is no network for real checkpoints).

NINT tensors come from the NINT quantizer on N(0, sigma) weights; NVQ / NEPQ tensors are drawn directly
in the packed domain, as the reference's own fixtures do (tests/test_nvq3j512_cpp_runtime.py:58-75,
tests/mixed_family_fixtures.py:55-153).  Large tensors quantize a `slab_rows` slab and tile it over the
rows, which leaves the value distribution and every byte count unchanged.
"""
from __future__ import annotations

import math
import struct
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


def nintm_quantized_blob(seed, n_experts, out_per_expert, K, expert_bits, sigma=0.02, slab_rows=1024):
    """(blob, pools) of an expert-wise NINTM tensor of the BASELINE config-4 kind: expert e at MOE_PROFILES[expert_bits[e]].

    One slab of N(0, sigma) weights per precision goes through the expert-wise quantizer (nint_quantize_expertwise on a
    [precisions, slab_rows, K] tensor); each cohort of the result is then tiled over its experts -- every stream of a
    NINT payload is the slab's stream repeated, because a slab ends on a byte boundary of every stream -- so that byte
    counts, value distribution and cohort order are those of quantizing the full tensor, at the cost of repeated rows.
    `pools` = [(expert_ids, NINT payload of the cohort)], in the container's order."""
    from .quantize import nint_quantize_expertwise
    expert_bits = [int(b) for b in expert_bits]
    order = list(dict.fromkeys(expert_bits))           # precisions in order of first appearance, as the quantizer groups
    rows = min(out_per_expert, slab_rows)
    if out_per_expert % rows or rows % 8:
        raise ValueError("the slab must divide the expert's rows and end on a byte boundary of every stream")
    rng = np.random.default_rng(seed)
    W = (rng.standard_normal((len(order), rows, K)) * sigma).astype(np.float32)
    small, _ = nint_quantize_expertwise(W, [MOE_PROFILES[b] for b in order])
    pools = []
    for (_, dtype, r), b in zip(small, order):
        ids = np.asarray([e for e, v in enumerate(expert_bits) if v == b], dtype=np.int32)
        reps = len(ids) * (out_per_expert // rows)
        out = reps * rows
        bits, gs, sb = MOE_PROFILES[b]
        ng = r["q"].shape[1]
        head = F._NINT_HDR.pack(bits, sb, gs, 0, K) + struct.pack("<I", 2) + struct.pack("<2q", out, K) + \
            struct.pack("<II", out, ng)
        parts = [np.ascontiguousarray(r["ns"], dtype=np.float16).tobytes(), np.ascontiguousarray(r["nm"], dtype=np.float16).tobytes(),
                 F.pack_bitstream(r["ss"], sb), F.pack_bitstream(r["sm"], sb), F.pack_bitstream(r["q"], bits)]
        pools.append((ids, dtype, b"".join([head] + [p * reps for p in parts])))
    return F.nintm_blob(n_experts, out_per_expert, K, pools), [(ids, payload) for ids, _, payload in pools]


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


def nvq2j_blob(seed, out, K, banks=4):
    """NVQ2J: 8-dimensional vectors out of `banks` 256-entry tables of random int8 magnitudes in [0, 7] (the reference
    learns them from the E8 grid; a matmul's time does not depend on their values), scale LUT linspace(0.45, 1.55),
    random state / index / sign streams (stream layout of mfq/quantize/nvq_jsc.py:1053-1079)."""
    rng = np.random.default_rng(seed)
    ng, nvec = math.ceil(K / 24), math.ceil(K / 8)
    blob = F.nvq_jsc_blob(
        "e8_256", K, rng.uniform(0.002, 0.02, out).astype(np.float32) * 0.02, np.linspace(0.45, 1.55, 16, dtype=np.float32),
        np.arange(16) % banks, rng.integers(0, 8, (banks, 256, 8), dtype=np.int8), rng.integers(0, 16, (out, ng), dtype=np.uint8),
        rng.integers(0, 256, (out, nvec), dtype=np.uint16), rng.integers(0, 128, (out, nvec), dtype=np.uint8))
    return "NVQ2J", blob


def nint8_zero_blob(seed, out, K):
    """(dtype, blob) of an [out, K] NINT8-0 tensor drawn in the packed domain: 34-byte blocks of an fp16 scale
    U(1, 3) * 1e-4 and 32 int8 codes in [-127, 127] (block layout of mfq/formats/nint8_zero.py:84-124)."""
    rng = np.random.default_rng(seed)
    ng = K // 32
    blocks = np.zeros((out, ng), dtype=np.dtype([("d", "<f2"), ("q", "i1", (32,))]))
    blocks["d"] = rng.uniform(1e-4, 3e-4, (out, ng)).astype(np.float16)
    blocks["q"] = rng.integers(-127, 128, (out, ng, 32), dtype=np.int8)
    import struct
    head = F._N8Z_HDR.pack(b"NI80", 0, K, 2) + struct.pack("<2q", out, K) + struct.pack("<II", out, ng)
    return "NINT8-0", head + blocks.tobytes()


def mx_blob(seed, dtype, out, K, lo=118, hi=132):
    """(dtype, blob) of an [out, K] MXFP4 / MXFP8 tensor drawn in the packed domain: random value bytes without the E4M3FN
    NaN codes, E8M0 block scales within a few octaves of one (container of mfq/formats/mx.py:120-151)."""
    rng = np.random.default_rng(seed)
    storage, scale = F.mx_shapes(dtype, out, K)
    values = rng.integers(0, 256, storage, dtype=np.uint8)
    if dtype == "MXFP8":
        values[(values & 0x7F) == 0x7F] = 0x38
    return dtype, F.write_mx(dtype, out, K, values, rng.integers(lo, hi, scale, dtype=np.uint8))


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


# ---- timing-only weights -------------------------------------------------------------------------
# Tensors too large to push through the CPU quantizer for a benchmark (hundreds of experts, whole
# linear stacks) are drawn directly in the device layout: uniformly random code / sub-scale bytes and
# constant anchors.  Every byte pattern is a valid payload, the kernels do the same work as on real
# weights, and byte counts are those of the format; the values mean nothing, so these are for
# throughput runs only -- parity is tested on quantized and packed-domain fixtures.
def random_nint_weight(seed, out, K, bits, gs, sub_bits, device="cuda", anchor=1e-6):
    import ctypes as C

    import torch

    from . import _lib as L
    from .runtime import NintWeight

    desc = L.NintDesc()
    L.check(L.lib().mfq_hip_nint_plan(bits, sub_bits, gs, out, K, C.byref(desc)))
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    total = int(desc.total_bytes)
    data = torch.empty(total, dtype=torch.uint8, device=device)
    body = int(desc.anchors_off)
    # int32 draws fill four bytes at a time (the body is a whole number of dwords)
    data[:body].view(torch.int32).random_(-2 ** 31, 2 ** 31 - 1, generator=g)
    data[body:].view(torch.float32).fill_(anchor)
    return NintWeight(desc, data, (out, K))


def random_nint_moe(seed, n_experts, out_per_expert, K, expert_bits, device="cuda"):
    """NintMoeWeight whose expert e has bit width expert_bits[e] (cohorts by MOE_PROFILES)."""
    from .runtime_moe import NintMoeWeight

    expert_bits = np.asarray(expert_bits)
    pools, ids = [], []
    for b in sorted(set(int(v) for v in expert_bits)):
        members = np.nonzero(expert_bits == b)[0].astype(np.int32)
        bits, gs, sb = MOE_PROFILES[b]
        pools.append(random_nint_weight(seed * 16 + b, len(members) * out_per_expert, K, bits, gs, sb, device))
        ids.append(members)
    return NintMoeWeight(n_experts, out_per_expert, K, pools, ids, device)


def tile_rows(w, out):
    """Timing-only: an [out, K] NVQ / dense NEPQ weight whose rows repeat those of the smaller weight `w`
    (built from a real packed payload).  Device layout = row-block bodies | tables | fp32 anchors."""
    import copy
    import ctypes as C

    import torch

    from . import _lib as L

    small = w.desc
    rows = small.out if hasattr(small, "out") else small.rows
    if rows % 16 or out % rows:
        raise ValueError("tile_rows needs a source of a multiple of 16 rows that divides the target")
    if isinstance(small, L.NvqDesc):
        big = L.NvqDesc()
        L.check(L.lib().mfq_hip_nvq_plan(small.index_bits, small.banks, out, small.neuron_len, C.byref(big)))
    else:
        big = L.NepqDesc()
        L.check(L.lib().mfq_hip_nepq_plan(small.profile, small.banks, out, small.neuron_len, C.byref(big)))
    reps = out // rows
    data = torch.empty(int(big.total_bytes), dtype=torch.uint8, device=w.data.device)
    data[: big.tables_off] = w.data[: small.tables_off].repeat(reps)
    ntab = small.anchors_off - small.tables_off
    data[big.tables_off: big.tables_off + ntab] = w.data[small.tables_off: small.anchors_off]
    data[big.anchors_off:] = w.data[small.anchors_off:].repeat(reps)
    t = copy.copy(w)
    t.desc, t.data = big, data
    t.out = out
    if hasattr(t, "out_per_expert"):
        t.out_per_expert = out
    t._ws = type(w._ws)()
    return t
