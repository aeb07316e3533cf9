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
    """Random streams for a JSC tensor of any codebook: the built-in grids where the format has one, else random
    magnitudes (the 1024- and 4096-entry codebooks travel in the payload anyway)."""
    ib, vs = O._NVQ_INDEX_BITS[codebook], O.nvq_vector_size(codebook)
    if codebook in ("e8_256", "d4_256", "d4_512"):
        grid = O.nvq_grid(codebook).astype(np.int16) * 8
    else:
        grid = np.random.default_rng(ib * 100 + vs).integers(0, 128, (1 << ib, vs)).astype(np.int16)
    cbs = np.stack([np.roll(grid, b * 7, axis=0) for b in range(banks)]).astype(np.int8)
    ng, nvec, nsign = math.ceil(K / 24), math.ceil(K / vs), math.ceil(K / 8)
    return O.NvqJscTensor(codebook, (out, K), K, O._f16_round(rng.uniform(0.002, 0.02, out)),
                          O._f16_round(np.linspace(0.45, 1.55, 16)), (np.arange(16) % banks).astype(np.uint8),
                          rng.integers(0, 16, (out, ng), dtype=np.uint8),
                          rng.integers(0, 1 << ib, (out, nvec)).astype(np.uint16),
                          rng.integers(0, 128, (out, nsign), dtype=np.uint8), cbs)


def nvq_plain_e8_random(rng, out, K, sign_mode="even"):
    """Plain NVQ2: the built-in 256-entry E8 grid, integer relative scales, parity or index-parity signs."""
    ng, nvec, nsign = math.ceil(K / 24), math.ceil(K / 8), math.ceil(K / 8)
    return O.NvqTensor("e8_256", (out, K), K, O._f16_round(rng.uniform(0.0002, 0.002, out)),
                       rng.integers(0, 16, (out, ng), dtype=np.uint8),
                       rng.integers(0, 256, (out, nvec)).astype(np.uint16),
                       rng.integers(0, 128, (out, nsign), dtype=np.uint8), sign_mode=sign_mode)


def nvq_plain_random(rng, out, K):
    ng, nvec, nsign = math.ceil(K / 24), math.ceil(K / 4), math.ceil(K / 8)
    return O.NvqTensor("d4_256", (out, K), K, O._f16_round(rng.uniform(0.0002, 0.002, out)),
                       rng.integers(0, 16, (out, ng), dtype=np.uint8),
                       rng.integers(0, 256, (out, nvec)).astype(np.uint16),
                       rng.integers(0, 128, (out, nsign), dtype=np.uint8))


def nvq1_random(rng, label, out, K, state_bits=3, custom=False):
    """NVQ1-L (state_bits 3 or 4; custom: a permuted grid travels in the blob, else the built-in one) / NVQ1-S."""
    ng = math.ceil(K / 24)
    if label == "NVQ1-L":
        nvec, entries = math.ceil(K / 8), 2048
        cb = rng.permutation(O.iq1s_grid()) if custom else None
    else:
        nvec, entries, state_bits = K // 8, 512, 4
        cb = np.stack([rng.permutation(O.iq1s_grid())[:512], rng.permutation(O.iq1s_grid())[:512]]) if custom else None
    return O.Nvq1Tensor(label, (out, K), 0, K, state_bits, O._f16_round(rng.uniform(0.002, 0.02, out)),
                        rng.integers(0, 1 << state_bits, (out, ng), dtype=np.uint8),
                        rng.integers(0, entries, (out, nvec)).astype(np.uint16),
                        rng.integers(0, 2, (out, ng), dtype=np.uint8), cb)


def npq0_random(rng, label, out, K):
    sp = O.LOWBIT_SPECS[label]
    S, E2 = sp["states"], sp["second"]
    ng, nvec = math.ceil(K / 24), K // 8
    return O.Npq0Tensor(label, (out, K), 0, K, O._f16_round(rng.uniform(0.0002, 0.002, out)),
                        O._f16_round(rng.uniform(0.25, 2.0, S)), rng.integers(0, S, (out, ng), dtype=np.uint8),
                        rng.integers(0, 1 << sp["index_bits"], (out, nvec), dtype=np.uint8),
                        rng.integers(-127, 128, (S, 8, 4)).astype(np.int8), rng.integers(-127, 128, (S, E2, 4)).astype(np.int8))


def nepq_random(rng, label, E, out, K, banks):
    _, sb, ib, ab, tb = O.NEPQ_SPECS[label]
    iq1s = np.frombuffer((O._DATA / "iq1s_2048.bin").read_bytes(), dtype="<u2")
    tables = []
    for b in range(banks):
        if label.startswith("NEPQ0"):       # an NPQ0 table: header with the fp16 scale LUT, then the int8 sub-codebooks
            sp = O.LOWBIT_SPECS["NPQ0" + label[5:]]
            S, E2 = sp["states"], sp["second"]
            head = bytearray(64)
            head[0:6] = bytes([sp["table_version"], S, 3, sp["index_bits"] - 3, 24, 8])
            head[8:8 + 2 * S] = O._f16_round(rng.uniform(0.25, 2.0, S)).astype("<f2").tobytes()
            tables.append(bytes(head) + rng.integers(-127, 128, S * 32 + S * E2 * 4).astype(np.int8).tobytes())
        elif label == "NEPQ1-L":
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
                        rng.integers(0, 2, (E, out, ng), dtype=np.uint8) if ab else np.zeros(0, dtype=np.uint8),
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


# ---- full-size payloads drawn in the packed domain ---------------------------------------------------
# Every bit pattern of the three NINT streams is a valid payload, so a tensor too large for the numpy quantizer
# is the blob header + fp16 anchors + random stream bytes; the anchors are chosen so that the dequantized weights
# are roughly zero-mean with standard deviation `sigma` (min anchor = scale anchor * (2^bits - 1) / 2).
def _random_bytes(rng, n):
    return rng.integers(0, 1 << 64, (n + 7) // 8, dtype=np.uint64, endpoint=False).view(np.uint8)[:n]


def nint_packed_blob(rng, out, K, bits, gs, sb, sigma=0.02):
    import struct
    ng = -(-K // gs)
    ls, lq = (1 << sb) - 1, (1 << bits) - 1
    var = lambda n: ((n + 1) ** 2 - 1) / 12.0          # variance of a uniform draw from 0..n
    c = lq / 2.0
    v_ssq = (var(ls) + (ls / 2) ** 2) * (var(lq) + c * c) - (ls / 2 * c) ** 2
    unit = math.sqrt(v_ssq + c * c * var(ls))
    ns = (rng.uniform(0.7, 1.3, out) * sigma / unit).astype(np.float16)
    nm = (ns.astype(np.float32) * c).astype(np.float16)
    sub = (out * ng * sb + 7) // 8
    head = O._NINT_HDR.pack(bits, sb, gs, 0, K) + struct.pack("<I", 2) + struct.pack("<2q", out, K) + \
        struct.pack("<II", out, ng)
    streams = _random_bytes(rng, 2 * sub + (out * ng * gs * bits + 7) // 8)
    return b"".join([head, ns.tobytes(), nm.tobytes(), streams.tobytes()])


def nint_blob_rows(blob, row0, nrows):
    """Rows [row0, row0 + nrows) of a NINT blob as an oracle tensor (row0 a multiple of 8, so that every stream is
    byte-aligned there), decoded with the oracle's own bit-stream reader."""
    import struct
    assert row0 % 8 == 0
    bits, sb, gs, axis, K = O._NINT_HDR.unpack_from(blob, 0)
    off = O._NINT_HDR.size
    ndim = struct.unpack_from("<I", blob, off)[0]
    off += 4 + 8 * ndim
    out, ng = struct.unpack_from("<II", blob, off)
    off += 8
    ns = np.frombuffer(blob, dtype=np.float16, count=nrows, offset=off + 2 * row0).astype(np.float32)
    nm = np.frombuffer(blob, dtype=np.float16, count=nrows, offset=off + 2 * out + 2 * row0).astype(np.float32)
    off += 4 * out
    sub = (out * ng * sb + 7) // 8
    ss, _ = O.unpack_bits(blob, off + row0 * ng * sb // 8, nrows * ng, sb)
    sm, _ = O.unpack_bits(blob, off + sub + row0 * ng * sb // 8, nrows * ng, sb)
    q, _ = O.unpack_bits(blob, off + 2 * sub + row0 * ng * gs * bits // 8, nrows * ng * gs, bits)
    return O.NintTensor(bits, gs, sb, (nrows, K), axis, K, q.reshape(nrows, ng, gs), ns, nm, ss.reshape(nrows, ng),
                        sm.reshape(nrows, ng))


def nintm_packed_blob(rng, E, out, K, bits_per_expert, sigma=0.02):
    """NIM2 container with one packed-domain cohort per distinct bit width; returns (blob, [(ids, pool_blob)])."""
    parts = [O._NIM_HDR.pack(b"NIM2", E, out, K, len(set(int(b) for b in bits_per_expert)))]
    pools = []
    for bits in sorted(set(int(b) for b in bits_per_expert)):
        ids = np.flatnonzero(np.asarray(bits_per_expert) == bits).astype(np.int32)
        b, gs, sb = MOE_PROFILES[bits]
        pb = nint_packed_blob(rng, len(ids) * out, K, b, gs, sb, sigma)
        db = f"NINT{bits}".encode("ascii")
        parts += [O._NIM_POOL.pack(ids.size, len(db), len(pb), 0), ids.tobytes(), db, pb]
        pools.append((ids, pb))
    return b"".join(parts), pools


def mx_random(rng, dtype, rows, cols, lo=118, hi=132):
    """An MXFP4 / MXFP8 tensor of random codes without NaNs (E4M3FN 0x7f / 0xff, scale byte 255), the block scales within
    a few octaves of one."""
    storage, scale = O.mx_shapes(dtype, (rows, cols))
    values = rng.integers(0, 256, storage, dtype=np.uint8)
    if dtype == "MXFP8":
        values[(values & 0x7F) == 0x7F] = 0x38
    return O.MxTensor(dtype, (rows, cols), values, rng.integers(lo, hi, scale, dtype=np.uint8))

