"""Packed-domain random tensors for the tests (oracle dataclasses), in the style of the reference's own
fixtures (tests/test_nvq3j512_cpp_runtime.py:58-75, tests/mixed_family_fixtures.py:55-153)."""
import math

import numpy as np

from oracle import mfq_oracle as O


def nint_random(rng, out, K, bits, gs, sb):
    ng = -(-K // gs)
    return O.NintTensor(bits, gs, sb, (out, K), 0, K,
                        rng.integers(0, 1 << bits, (out, ng, gs), dtype=np.uint8),
                        O._f16_round(rng.uniform(1e-4, 2e-3, out)), O._f16_round(rng.uniform(1e-3, 2e-2, out)),
                        rng.integers(0, 1 << sb, (out, ng), dtype=np.uint8),
                        rng.integers(0, 1 << sb, (out, ng), dtype=np.uint8))


def nvq_jsc_random(rng, out, K, codebook="d4_512", banks=2):
    grid = O.nvq_grid(codebook).astype(np.int16) * 8
    cbs = np.stack([np.roll(grid, b * 7, axis=0) for b in range(banks)]).astype(np.int8)
    ib = O._NVQ_INDEX_BITS[codebook]
    ng, nvec, nsign = math.ceil(K / 24), math.ceil(K / 4), math.ceil(K / 8)
    return O.NvqJscTensor(codebook, (out, K), K, O._f16_round(rng.uniform(0.002, 0.02, out)),
                          O._f16_round(np.linspace(0.45, 1.55, 16)), (np.arange(16) % banks).astype(np.uint8),
                          rng.integers(0, 16, (out, ng), dtype=np.uint8),
                          rng.integers(0, 1 << ib, (out, nvec)).astype(np.uint16),
                          rng.integers(0, 128, (out, nsign), dtype=np.uint8), cbs)


def nvq_plain_random(rng, out, K):
    ng, nvec, nsign = math.ceil(K / 24), math.ceil(K / 4), math.ceil(K / 8)
    return O.NvqTensor("d4_256", (out, K), K, O._f16_round(rng.uniform(0.0002, 0.002, out)),
                       rng.integers(0, 16, (out, ng), dtype=np.uint8),
                       rng.integers(0, 256, (out, nvec)).astype(np.uint16),
                       rng.integers(0, 128, (out, nsign), dtype=np.uint8))


def nepq_random(rng, label, E, out, K, banks):
    _, sb, ib, ab, tb = O.NEPQ_SPECS[label]
    iq1s = np.frombuffer((O._DATA / "iq1s_2048.bin").read_bytes(), dtype="<u2")
    tables = []
    for b in range(banks):
        if label == "NEPQ1-L":
            tables.append(rng.permutation(iq1s).astype("<u2").tobytes())
        else:
            tables.append(rng.permutation(iq1s)[:512].astype("<u2").tobytes()
                          + rng.permutation(iq1s)[:512].astype("<u2").tobytes())
    tables = np.frombuffer(b"".join(tables), dtype=np.uint8).reshape(banks, tb)
    ng, nvec = math.ceil(K / 24), K // 8
    nsuper = math.ceil(ng / 4)
    return O.NepqTensor(label, (E, out, K), O._f16_round(rng.uniform(0.0005, 0.005, (E, out))),
                        rng.integers(0, 1 << sb, (E, out, ng), dtype=np.uint8),
                        rng.integers(0, 1 << ib, (E, out, nvec)).astype(np.uint16),
                        rng.integers(0, 2, (E, out, ng), dtype=np.uint8),
                        rng.integers(0, banks, (E, out, nsuper), dtype=np.uint8), tables)


MOE_PROFILES = {2: (2, 16, 5), 3: (3, 24, 5), 4: (4, 24, 6), 5: (5, 28, 7), 6: (6, 24, 6), 8: (8, 24, 8)}


def moe_random(rng, E, out, K, bits_per_expert, quantize=False):
    """NINTM tensor with one cohort per distinct bit width."""
    pools = []
    for bits in sorted(set(int(b) for b in bits_per_expert)):
        ids = np.flatnonzero(np.asarray(bits_per_expert) == bits).astype(np.int32)
        b, gs, sb = MOE_PROFILES[bits]
        if quantize:
            W = (rng.standard_normal((len(ids) * out, K)) * 0.02).astype(np.float32)
            t = O.quantize_nint(W, b, gs, sb)
        else:
            t = nint_random(rng, len(ids) * out, K, b, gs, sb)
        pools.append(O.MoePool(ids, f"NINT{bits}", t))
    return O.NintMoeTensor((E, out, K), pools)
