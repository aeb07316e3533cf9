"""MFQ payload writers and header parsers for the packed-weight matmul path.

Host-side mirror of the reference's payload layer (mfq/formats/io.py, nvq.py, nepq.py):
the writers produce byte-identical blobs for the same packed-domain arrays, and the
parsers validate a blob and locate its body so the device-side repack kernels can read
the bit streams in place.  No dequantization happens here: that is the GPU's job.
"""
from __future__ import annotations

import math
import struct
from dataclasses import dataclass, field

import numpy as np

# ---------------------------------------------------------------------------------------
# bit streams (little-endian, value i at bit i*bits; mfq/formats/io.py:144-162)
# ---------------------------------------------------------------------------------------


def pack_bitstream(values, bits: int) -> bytes:
    v = np.ascontiguousarray(values).reshape(-1)
    if bits == 0 or v.size == 0:
        return b""
    if bits == 8:
        return v.astype(np.uint8).tobytes()
    if np.any(v < 0) or np.any(v >= (1 << bits)):
        raise ValueError(f"value exceeds {bits}-bit packed width")
    if bits == 4:
        u = v.astype(np.uint8)
        if u.size % 2:
            u = np.concatenate([u, np.zeros(1, np.uint8)])
        return (u[0::2] | (u[1::2] << 4)).astype(np.uint8).tobytes()
    parts = []
    chunk = 1 << 22  # a multiple of 8 values, so every chunk ends on a byte boundary
    for lo in range(0, v.size, chunk):
        u = v[lo: lo + chunk].astype("<u2")
        rows = np.unpackbits(u.view(np.uint8).reshape(-1, 2), axis=1, bitorder="little")[:, :bits]
        parts.append(np.packbits(rows.reshape(-1), bitorder="little").tobytes())
    return b"".join(parts)


def unpack_bitstream(blob, off: int, count: int, bits: int) -> np.ndarray:
    """Inverse of pack_bitstream (mfq/formats/io.py:165-188); returns uint8 (bits <= 8) or uint16 values."""
    if bits == 0 or count == 0:
        return np.empty(0, dtype=np.uint8)
    nbytes = (count * bits + 7) // 8
    if off + nbytes > len(blob):
        raise ValueError("truncated bit stream")
    packed = np.frombuffer(blob, dtype=np.uint8, count=nbytes, offset=off)
    if bits == 8:
        return packed.copy()
    rows = np.unpackbits(packed, bitorder="little")[: count * bits].reshape(count, bits)
    if bits <= 8:
        return np.packbits(rows, axis=1, bitorder="little").reshape(-1)
    lo = np.packbits(rows[:, :8], axis=1, bitorder="little").reshape(-1).astype(np.uint16)
    hi = np.packbits(rows[:, 8:], axis=1, bitorder="little").reshape(-1).astype(np.uint16)
    return lo | (hi << 8)


# ---------------------------------------------------------------------------------------
# NINT (mfq/formats/io.py:191-248)
# ---------------------------------------------------------------------------------------
_NINT_HDR = struct.Struct("<BBiii")


@dataclass
class NintHeader:
    bits: int
    sub_bits: int
    gs: int
    axis: int
    neuron_len: int
    shape: tuple
    out: int
    ng: int
    body_off: int      # offset of ns f16[out] inside the blob
    body_bytes: int
    legacy: bool       # one byte per value tail (mfq/formats/io.py:223-232)


def nint_blob(bits, sub_bits, gs, neuron_len, ns, nm, ss, sm, q, shape=None, axis=0) -> bytes:
    q = np.asarray(q)
    out, ng, gs_ = q.shape
    if gs_ != gs or ng != math.ceil(neuron_len / gs):
        raise ValueError("NINT q must be [out, ceil(K/gs), gs]")
    shape = tuple(shape) if shape is not None else (out, neuron_len)
    return b"".join([
        _NINT_HDR.pack(bits, sub_bits, gs, axis, neuron_len), struct.pack("<I", len(shape)),
        struct.pack(f"<{len(shape)}q", *shape), struct.pack("<II", out, ng),
        np.ascontiguousarray(ns, dtype=np.float16).tobytes(), np.ascontiguousarray(nm, dtype=np.float16).tobytes(),
        pack_bitstream(ss, sub_bits), pack_bitstream(sm, sub_bits), pack_bitstream(q, bits)])


def parse_nint(blob) -> NintHeader:
    if len(blob) < _NINT_HDR.size + 4:
        raise ValueError("truncated NINT header")
    bits, sub_bits, gs, axis, neuron_len = _NINT_HDR.unpack_from(blob, 0)
    off = _NINT_HDR.size
    ndim, = struct.unpack_from("<I", blob, off)
    off += 4
    if ndim > 8 or len(blob) < off + 8 * ndim + 8:
        raise ValueError("truncated NINT header")
    shape = struct.unpack_from(f"<{ndim}q", blob, off)
    off += 8 * ndim
    out, ng = struct.unpack_from("<II", blob, off)
    off += 8
    if not (1 <= bits <= 8 and 1 <= sub_bits <= 8 and gs > 0 and neuron_len > 0 and out > 0):
        raise ValueError(f"unsupported NINT spec bits={bits} sub_bits={sub_bits} gs={gs}")
    if ng != math.ceil(neuron_len / gs):
        raise ValueError("NINT header group count does not match neuron_len")
    subs, qn = out * ng, out * ng * gs
    packed = 4 * out + ((subs * sub_bits + 7) // 8) * 2 + (qn * bits + 7) // 8
    old = 4 * out + 2 * subs + qn
    remaining = len(blob) - off
    if remaining == old and remaining != packed:
        legacy = True
    elif remaining == packed:
        legacy = False
    else:
        raise ValueError(f"invalid NINT blob tail: remaining={remaining - 4 * out}, "
                         f"packed={packed - 4 * out}, old={old - 4 * out}")
    return NintHeader(bits, sub_bits, gs, axis, neuron_len, tuple(shape), out, ng, off, remaining, legacy)


# NINT8-0 (GGML Q8_0 blocks): "<4siiI" ("NI80", axis, neuron_len, ndim) + shape i64[ndim] + out u32 + ng u32 + blocks
# (mfq/formats/nint8_zero.py:20-23, 166-205; cpp_runtime/mfq_decode.cpp:1601-1650)
_N8Z_HDR = struct.Struct("<4siiI")


@dataclass
class Nint8zHeader:
    axis: int
    neuron_len: int
    shape: tuple
    out: int
    ng: int
    body_off: int
    body_bytes: int


def parse_nint8_zero(blob) -> Nint8zHeader:
    if len(blob) < _N8Z_HDR.size:
        raise ValueError("truncated NINT8-0 header")
    magic, axis, neuron_len, ndim = _N8Z_HDR.unpack_from(blob, 0)
    if magic != b"NI80":
        raise ValueError(f"invalid NINT8-0 magic: {magic!r}")
    if ndim == 0:
        raise ValueError("NINT8-0 tensor rank cannot be zero")
    off = _N8Z_HDR.size
    if ndim > 8 or off + 8 * ndim + 8 > len(blob):
        raise ValueError("truncated NINT8-0 shape")
    shape = struct.unpack_from(f"<{ndim}q", blob, off)
    off += 8 * ndim
    out, ng = struct.unpack_from("<II", blob, off)
    off += 8
    if not 0 <= axis < ndim:
        raise ValueError("NINT8-0 axis is outside the tensor rank")
    if neuron_len <= 0 or neuron_len % 32:
        raise ValueError("NINT8-0 neuron_len must be a positive multiple of 32")
    if len(blob) - off != out * ng * 34:
        raise ValueError(f"invalid NINT8-0 block bytes: got {len(blob) - off}, expected {out * ng * 34}")
    if out <= 0 or shape[axis] != out or ng != neuron_len // 32 or math.prod(shape) != out * neuron_len:
        raise ValueError("NINT8-0 dimensions disagree with the logical shape")
    return Nint8zHeader(axis, neuron_len, tuple(shape), out, ng, off, len(blob) - off)


def nint_arrays(blob) -> dict:
    """Packed-domain arrays of a NINT blob (the unpack half of mfq/formats/io.py:206-248)."""
    h = parse_nint(blob)
    out, ng, gs = h.out, h.ng, h.gs
    off = h.body_off
    ns = np.frombuffer(blob, dtype=np.float16, count=out, offset=off).astype(np.float32)
    nm = np.frombuffer(blob, dtype=np.float16, count=out, offset=off + 2 * out).astype(np.float32)
    off += 4 * out
    sb, qb = (8, 8) if h.legacy else (h.sub_bits, h.bits)
    ss = unpack_bitstream(blob, off, out * ng, sb).reshape(out, ng)
    off += (out * ng * sb + 7) // 8
    sm = unpack_bitstream(blob, off, out * ng, sb).reshape(out, ng)
    off += (out * ng * sb + 7) // 8
    q = unpack_bitstream(blob, off, out * ng * gs, qb).reshape(out, ng, gs)
    return {"bits": h.bits, "sub_bits": h.sub_bits, "gs": gs, "neuron_len": h.neuron_len, "ns": ns, "nm": nm,
            "ss": ss, "sm": sm, "q": q}


def nint_concat_rows(blobs) -> bytes:
    """One NINT blob holding the neurons of several tensors of the same spec one after the other: the
    concatenated weight of a projection group (NintLinearGroup, cpp_runtime/mfq_decode.cpp:8618-8660)."""
    parts = [nint_arrays(b) for b in blobs]
    a = parts[0]
    for p in parts[1:]:
        if (p["bits"], p["sub_bits"], p["gs"], p["neuron_len"]) != (a["bits"], a["sub_bits"], a["gs"], a["neuron_len"]):
            raise ValueError("grouped NINT projections must share bits, sub_bits, groupsize and neuron length")
    cat = {k: np.concatenate([p[k] for p in parts], axis=0) for k in ("ns", "nm", "ss", "sm", "q")}
    return nint_blob(a["bits"], a["sub_bits"], a["gs"], a["neuron_len"], cat["ns"], cat["nm"], cat["ss"], cat["sm"],
                     cat["q"])


# ---------------------------------------------------------------------------------------
# NVQ (mfq/formats/nvq.py:586-820)
# ---------------------------------------------------------------------------------------
_NVQ_HDR = struct.Struct("<4sBBHiiI")
NVQ_CODEBOOK_ID = {"e8_256": 1, "d4_256": 2, "d4_512": 3, "e8_1024": 4, "e8_4096": 5, "d4_1024": 6}
NVQ_ID_CODEBOOK = {v: k for k, v in NVQ_CODEBOOK_ID.items()}
NVQ_INDEX_BITS = {"e8_256": 8, "e8_1024": 10, "e8_4096": 12, "d4_256": 8, "d4_512": 9, "d4_1024": 10}
NVQ_JSC_DTYPE = {"e8_256": "NVQ2J", "e8_1024": "NVQ2J-L", "e8_4096": "NVQ2J-XL", "d4_256": "NVQ3J",
                 "d4_512": "NVQ3J-512", "d4_1024": "NVQ3J-L"}


@dataclass
class NvqHeader:
    codebook: str
    index_bits: int
    vector_size: int
    jsc: bool
    banks: int
    out: int
    neuron_len: int
    ng: int
    nvec: int
    nsign: int
    body_off: int     # JSC: offset of the 64-byte JSC header; plain: offset of the anchors
    body_bytes: int
    gs: int = 24
    sub_bits: int = 4
    sign_mode: str = "even"

    @property
    def dtype(self) -> str:
        return NVQ_JSC_DTYPE[self.codebook] if self.jsc else {"e8_256": "NVQ2", "d4_256": "NVQ3"}[self.codebook]


def jsc_tables(scale_lut, bank_for_state, codebooks) -> bytes:
    """64-byte JSC header + raw int8 banks (mfq/formats/nvq.py:446-483)."""
    cb = np.ascontiguousarray(codebooks)
    if cb.ndim != 3 or cb.shape[0] not in (1, 2, 4) or np.any(cb < 0) or np.any(cb > 127):
        raise ValueError("NVQ-JSC deployment codebooks must be integers in [0,127] with banks in {1,2,4}")
    banks, _, vs = cb.shape
    lut = np.asarray(scale_lut, dtype=np.float32).reshape(-1)
    bfs = np.asarray(bank_for_state).reshape(-1)
    if lut.shape != (16,) or bfs.shape != (16,) or np.any(bfs >= banks) or np.any(lut < 0):
        raise ValueError("NVQ-JSC tables must hold 16 states")
    hdr = bytearray(64)
    hdr[0:3] = bytes([1, banks, 16])
    st = np.arange(16)
    a_scale = st.astype(np.float32) if banks == 1 else (
        (st // banks + 1).astype(np.float32) if vs == 4 else (15.0 * (st // banks + 1) / (16 // banks)).astype(np.float32))
    if np.array_equal(lut, a_scale) and np.array_equal(bfs, st % banks):
        hdr[3] = 1
    hdr[4:36] = lut.astype("<f2").tobytes()
    hdr[36:52] = bfs.astype(np.uint8).tobytes()
    return bytes(hdr) + cb.astype(np.int8).tobytes()


def nvq_jsc_blob(codebook, neuron_len, ns, scale_lut, bank_for_state, codebooks, state, indices, signs) -> bytes:
    out = int(np.asarray(ns).size)
    ib = NVQ_INDEX_BITS[codebook]
    return b"".join([
        _NVQ_HDR.pack(b"NVQ1", NVQ_CODEBOOK_ID[codebook] | 0x20, 4, 24, 0, neuron_len, 2),
        struct.pack("<2q", out, neuron_len), struct.pack("<I", out),
        jsc_tables(scale_lut, bank_for_state, codebooks),
        np.ascontiguousarray(ns, dtype=np.float16).tobytes(),
        pack_bitstream(state, 4), pack_bitstream(indices, ib), pack_bitstream(signs, 7)])


def nvq_plain_blob(codebook, neuron_len, ns, sub_scale, indices, signs, gs=24, sub_bits=4) -> bytes:
    out = int(np.asarray(ns).size)
    return b"".join([
        _NVQ_HDR.pack(b"NVQ1", NVQ_CODEBOOK_ID[codebook], sub_bits, gs, 0, neuron_len, 2),
        struct.pack("<2q", out, neuron_len), struct.pack("<I", out),
        np.ascontiguousarray(ns, dtype=np.float16).tobytes(),
        pack_bitstream(sub_scale, sub_bits), pack_bitstream(indices, NVQ_INDEX_BITS[codebook]),
        pack_bitstream(signs, 7)])


def parse_nvq(blob) -> NvqHeader:
    if len(blob) < _NVQ_HDR.size:
        raise ValueError("truncated NVQ header")
    magic, enc, sub_bits, gs, axis, neuron_len, ndim = _NVQ_HDR.unpack_from(blob, 0)
    if magic not in (b"NVQ1", b"NIQ1"):
        raise ValueError(f"invalid NVQ magic: {magic!r}")
    cid = enc & 0x1F
    if cid not in NVQ_ID_CODEBOOK:
        raise ValueError(f"unknown NVQ codebook id: {cid}")
    codebook = NVQ_ID_CODEBOOK[cid]
    jsc, custom = bool(enc & 0x20), bool(enc & 0x40)
    sign_mode = "index_parity" if enc & 0x80 else "even"
    off = _NVQ_HDR.size + 8 * ndim
    out, = struct.unpack_from("<I", blob, off)
    off += 4
    vs, ib = (8 if codebook.startswith("e8") else 4), NVQ_INDEX_BITS[codebook]
    ng, nvec, nsign = math.ceil(neuron_len / gs), math.ceil(neuron_len / vs), math.ceil(neuron_len / 8)
    streams = 2 * out + (out * ng * sub_bits + 7) // 8 + (out * nvec * ib + 7) // 8 + (out * nsign * 7 + 7) // 8
    banks = 0
    if jsc:
        if custom or sign_mode != "even" or gs != 24 or sub_bits != 4:
            raise ValueError("invalid NVQ-JSC profile flags")
        if len(blob) < off + 64:
            raise ValueError("truncated NVQ-JSC metadata header")
        version, banks, states, mode = blob[off], blob[off + 1], blob[off + 2], blob[off + 3]
        if version != 1 or banks not in (1, 2, 4) or states != 16 or mode not in (0, 1) or any(blob[off + 52: off + 64]):
            raise ValueError("invalid NVQ-JSC metadata")
        if any(b >= banks for b in blob[off + 36: off + 52]):
            raise ValueError("invalid NVQ-JSC state-to-bank map")
        expect = 64 + banks * (1 << ib) * vs + streams
    else:
        if custom:
            raise ValueError("custom-codebook NVQ blobs are outside this runtime's scope")
        expect = streams
    if len(blob) - off != expect:
        raise ValueError(f"invalid NVQ blob tail: consumed={off + expect}, size={len(blob)}")
    return NvqHeader(codebook, ib, vs, jsc, banks, out, neuron_len, ng, nvec, nsign, off, expect, gs, sub_bits, sign_mode)


# ---------------------------------------------------------------------------------------
# NEPQ (mfq/formats/nepq.py:209-474)
# ---------------------------------------------------------------------------------------
_NEPQ_HDR = struct.Struct("<4sBBBBIIIIIQ")
NEPQ_PROFILE = {"NEPQ0-S": 0, "NEPQ0-L": 1, "NEPQ1-S": 2, "NEPQ1-L": 3}
NEPQ_LABEL = {v: k for k, v in NEPQ_PROFILE.items()}
#               profile: (state_bits, index_bits, aux_bits, table_bytes)
NEPQ_BITS = {2: (4, 9, 1, 2048), 3: (3, 11, 1, 4096)}


@dataclass
class NepqHeader:
    label: str
    profile: int
    n_experts: int
    out_per_expert: int
    neuron_len: int
    banks: int
    rotation_block: int
    rotation_seed: int
    ng: int
    nvec: int
    nsuper: int
    body_off: int
    body_bytes: int


def nepq_blob(label, shape, tables, ns, state, indices, aux, bank_ids, rotation_block=0, rotation_seed=0) -> bytes:
    pid = NEPQ_PROFILE[label]
    sb, ib, ab, tb = NEPQ_BITS[pid]
    E, out, K = shape
    tables = np.ascontiguousarray(tables, dtype=np.uint8)
    if tables.ndim != 2 or tables.shape[1] != tb:
        raise ValueError(f"{label} bank must contain {tb} bytes")
    return b"".join([
        _NEPQ_HDR.pack(b"NEP1", 1, pid, 4, 1 if rotation_block else 0, E, out, K, tables.shape[0],
                       rotation_block, rotation_seed),
        tables.tobytes(), np.ascontiguousarray(ns, dtype="<f2").tobytes(), pack_bitstream(state, sb),
        pack_bitstream(indices, ib), pack_bitstream(aux, ab), np.ascontiguousarray(bank_ids, dtype=np.uint8).tobytes()])


def parse_nepq(blob) -> NepqHeader:
    if len(blob) < _NEPQ_HDR.size:
        raise ValueError("truncated NEPQ header")
    magic, ver, pid, gps, flags, E, out, K, banks, rblock, rseed = _NEPQ_HDR.unpack_from(blob, 0)
    if magic != b"NEP1" or ver != 1:
        raise ValueError("invalid or unsupported NEPQ header")
    if pid not in NEPQ_LABEL or gps != 4:
        raise ValueError("unsupported NEPQ super-group profile")
    if flags & ~1 or bool(flags & 1) != bool(rblock):
        raise ValueError("inconsistent NEPQ rotation flag")
    if E <= 0 or out <= 0 or K <= 0 or K % 8 or not 1 <= banks <= 256:
        raise ValueError("NEPQ shape dimensions must be positive, K divisible by 8, banks in [1,256]")
    if pid not in NEPQ_BITS:
        raise NotImplementedError(f"{NEPQ_LABEL[pid]} is not on the accelerated path")
    sb, ib, ab, tb = NEPQ_BITS[pid]
    rows = E * out
    ng, nvec = math.ceil(K / 24), K // 8
    nsuper = math.ceil(ng / 4)
    expect = banks * tb + 2 * rows + (rows * ng * sb + 7) // 8 + (rows * nvec * ib + 7) // 8 + \
        (rows * ng * ab + 7) // 8 + rows * nsuper
    if len(blob) - _NEPQ_HDR.size != expect:
        raise ValueError(f"invalid NEPQ tail: consumed={_NEPQ_HDR.size + expect}, size={len(blob)}")
    return NepqHeader(NEPQ_LABEL[pid], pid, E, out, K, banks, rblock, rseed, ng, nvec, nsuper, _NEPQ_HDR.size, expect)


# ---------------------------------------------------------------------------------------
# NINTM / NIM2 container (mfq/formats/io.py:251-446)
# ---------------------------------------------------------------------------------------
_NIM_HDR = struct.Struct("<4sIIII")
_NIM_POOL = struct.Struct("<IIQQ")


@dataclass
class NintmPool:
    expert_ids: np.ndarray
    dtype: str
    payload_off: int
    payload_bytes: int
    runtime_off: int
    runtime_bytes: int


@dataclass
class NintmHeader:
    n_experts: int
    out_per_expert: int
    neuron_len: int
    pools: list = field(default_factory=list)


def nintm_blob(n_experts, out_per_expert, neuron_len, pools) -> bytes:
    """pools: iterable of (expert_ids, dtype string, payload bytes)."""
    pools = list(pools)
    parts = [_NIM_HDR.pack(b"NIM2", n_experts, out_per_expert, neuron_len, len(pools))]
    for ids, dtype, payload in pools:
        ids = np.ascontiguousarray(ids, dtype=np.int32).reshape(-1)
        db = dtype.encode("ascii")
        if not db or len(db) > 32:
            raise ValueError(f"invalid NINTM cohort dtype: {dtype!r}")
        parts += [_NIM_POOL.pack(ids.size, len(db), len(payload), 0), ids.tobytes(), db, payload]
    return b"".join(parts)


def parse_nintm(blob) -> NintmHeader:
    if len(blob) < _NIM_HDR.size:
        raise ValueError("truncated NINTM header")
    magic, E, out, K, npools = _NIM_HDR.unpack_from(blob, 0)
    if magic != b"NIM2":
        raise ValueError(f"invalid NINTM magic: {magic!r}")
    if npools == 0 or npools > E:
        raise ValueError("invalid NINTM pool count")
    off = _NIM_HDR.size
    hdr = NintmHeader(E, out, K)
    owners = np.full(E, -1, dtype=np.int32)
    for pi in range(npools):
        if off + _NIM_POOL.size > len(blob):
            raise ValueError("truncated NINTM v2 pool header")
        n_ids, dlen, plen, rlen = _NIM_POOL.unpack_from(blob, off)
        off += _NIM_POOL.size
        if n_ids == 0 or dlen == 0 or dlen > 32:
            raise ValueError("invalid NINTM v2 pool metadata")
        end = off + 4 * n_ids + dlen + rlen + plen
        if end > len(blob):
            raise ValueError("truncated NINTM v2 pool payload")
        ids = np.frombuffer(blob, dtype=np.int32, count=n_ids, offset=off).copy()
        off += 4 * n_ids
        try:
            dtype = bytes(blob[off: off + dlen]).decode("ascii")
        except UnicodeDecodeError as exc:
            raise ValueError("NINTM cohort dtype must be ASCII") from exc
        off += dlen
        if np.any(ids < 0) or np.any(ids >= E):
            raise ValueError(f"NINTM pool {pi} contains an invalid expert id")
        if np.unique(ids).size != ids.size:
            raise ValueError(f"NINTM pool {pi} repeats an expert id")
        if np.any(owners[ids] >= 0):
            raise ValueError("an expert belongs to multiple NINTM pools")
        owners[ids] = pi
        hdr.pools.append(NintmPool(ids, dtype, off + rlen, plen, off, rlen))
        off = end
    if off != len(blob):
        raise ValueError(f"invalid NINTM tail: {len(blob) - off} extra bytes")
    missing = np.flatnonzero(owners < 0)
    if missing.size:
        raise ValueError(f"NINTM pools do not cover experts {missing[:16].tolist()}")
    return hdr


# ---------------------------------------------------------------------------------------
# MFQ1 container (mfq/formats/io.py:646-685): header, directory, blobs back to back
# ---------------------------------------------------------------------------------------
def write_mfq(path, tensors: dict, model_arch: str = "synthetic", version: int = 1) -> None:
    """tensors: name -> (dtype string, blob bytes)."""
    with open(path, "wb") as f:
        a = model_arch.encode()
        f.write(b"MFQ1" + struct.pack("<I", version) + struct.pack("<I", len(a)) + a)
        if version >= 2:
            f.write(struct.pack("<I", 0))
        f.write(struct.pack("<I", len(tensors)))
        for name, (dtype, blob) in tensors.items():
            nb, db = name.encode(), dtype.encode()
            f.write(struct.pack("<I", len(nb)) + nb + struct.pack("<I", len(db)) + db + struct.pack("<Q", len(blob)))
        for _, (_, blob) in tensors.items():
            f.write(blob)


def read_mfq_directory(data) -> dict:
    """name -> (dtype, offset, nbytes) of an MFQ1 file image."""
    if data[:4] != b"MFQ1":
        raise ValueError("invalid MFQ magic")
    version, = struct.unpack_from("<I", data, 4)
    off = 8
    n, = struct.unpack_from("<I", data, off)
    off += 4 + n
    if version >= 2:
        ne, = struct.unpack_from("<I", data, off)
        off += 4
        for _ in range(2 * ne):
            n, = struct.unpack_from("<I", data, off)
            off += 4 + n
    nt, = struct.unpack_from("<I", data, off)
    off += 4
    recs = []
    for _ in range(nt):
        n, = struct.unpack_from("<I", data, off)
        name = bytes(data[off + 4: off + 4 + n]).decode()
        off += 4 + n
        n, = struct.unpack_from("<I", data, off)
        dtype = bytes(data[off + 4: off + 4 + n]).decode()
        off += 4 + n
        ln, = struct.unpack_from("<Q", data, off)
        off += 8
        recs.append((name, dtype, ln))
    out = {}
    for name, dtype, ln in recs:
        if name in out:
            raise ValueError(f"duplicate MFQ tensor record: {name}")
        if off + ln > len(data):
            raise ValueError(f"truncated MFQ blob for {name}")
        out[name] = (dtype, off, ln)
        off += ln
    if off != len(data):       # mfq/formats/io.py:826-827
        raise ValueError(f"MFQ file length mismatch: records end={off}, file size={len(data)}")
    return out
