"""MFQ payload writers and header parsers for the packed-weight matmul path.

Host-side mirror of the reference's payload layer (mfq/formats/io.py, nvq.py, nepq.py):
the writers produce byte-identical blobs for the same packed-domain arrays, and the
parsers validate a blob and locate its body so the device-side repack kernels can read
the bit streams in place.  No dequantization happens here: that is the GPU's job.
"""
from __future__ import annotations

import json
import math
import os
import re
import struct
from dataclasses import dataclass, field
from pathlib import Path

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


# ---------------------------------------------------------------------------
# The 1-bit families: NVQ1-L / NVQ1-S / NPQ0-L / NPQ0-S (mfq/formats/nvq1_l.py, nvq1_s.py, npq0_l.py, npq0_s.py)
# ---------------------------------------------------------------------------
# dtype: magic, header byte (None: profile 1 or 2), state bits (None: in the header), index bits, table bytes in the blob
LOWBIT_FORMATS = {
    "NVQ1-L": (b"NQ1L", None, None, 11),
    "NVQ1-S": (b"NQ1S", 1, 4, 9),
    "NPQ0-L": (b"NPQL", 1, 3, 7),
    "NPQ0-S": (b"NPQS", 2, 2, 6),
}
_NPQ0_TABLES = {"NPQ0-L": (1, 8, 16), "NPQ0-S": (2, 4, 8)}   # table version, states, second sub-codebook entries


# OCP MX payloads (mfq/formats/mx.py:20-182): "MXT1", version, kind (4 | 8), reserved, logical / storage / scale shapes,
# then the value bytes and the E8M0 scale bytes.
MX_KINDS = {"MXFP4": 4, "MXFP8": 8}
_MX_HEADER = struct.Struct("<4sBBHQQQQQQ")


@dataclass
class MxHeader:
    dtype: str
    kind: int
    rows: int
    cols: int
    values_off: int
    values_bytes: int
    scales_off: int
    scales_bytes: int


def is_mx_dtype(dtype: str) -> bool:
    return dtype in MX_KINDS


def mx_shapes(dtype: str, rows: int, cols: int):
    """(storage shape, scale shape) with the reference's geometry checks and messages (validate_mx_shapes,
    mfq/formats/mx.py:65-117)."""
    if dtype not in MX_KINDS:
        raise ValueError(f"unsupported MX dtype: {dtype}")
    if rows <= 0 or cols <= 0:
        raise ValueError(f"invalid MX logical shape: {(rows, cols)}")
    if dtype == "MXFP4":
        if cols % 32:
            raise ValueError("MXFP4 columns must be divisible by 32")
        return (rows, cols // 2), (rows, cols // 32)
    if cols % 128:
        raise ValueError("MXFP8 columns must be divisible by 128")
    return (rows, cols), ((rows + 127) // 128, cols // 128)


def parse_mx(dtype: str, blob) -> MxHeader:
    """parse_mx_layout (mfq/formats/mx.py:154-173; C++ unpack_mxfp8 / unpack_mxfp4, cpp_runtime/mfq_decode.cpp:1832-1918)."""
    mv = memoryview(blob)
    if len(mv) < _MX_HEADER.size:
        raise ValueError("truncated MFQ MX tensor header")
    magic, version, kind, reserved, *dims = _MX_HEADER.unpack_from(mv)
    if magic != b"MXT1" or version != 1 or kind != MX_KINDS.get(dtype) or reserved:
        raise ValueError(f"invalid {dtype} payload header: magic={magic!r}, version={version}, kind={kind}")
    rows, cols = int(dims[0]), int(dims[1])
    storage, scale = mx_shapes(dtype, rows, cols)
    if (int(dims[2]), int(dims[3])) != storage:
        raise ValueError(f"{dtype} storage shape {(int(dims[2]), int(dims[3]))} != {storage}")
    if (int(dims[4]), int(dims[5])) != scale:
        raise ValueError(f"{dtype} scale shape {(int(dims[4]), int(dims[5]))} != {scale}")
    nv, ns = storage[0] * storage[1], scale[0] * scale[1]
    if len(mv) != _MX_HEADER.size + nv + ns:
        raise ValueError(f"{dtype} payload size {len(mv)} != {_MX_HEADER.size + nv + ns}")
    return MxHeader(dtype, kind, rows, cols, _MX_HEADER.size, nv, _MX_HEADER.size + nv, ns)


def write_mx(dtype: str, rows: int, cols: int, values, scales) -> bytes:
    """pack_mx (mfq/formats/mx.py:120-151) from the two byte matrices."""
    storage, scale = mx_shapes(dtype, rows, cols)
    values, scales = np.ascontiguousarray(values, dtype=np.uint8), np.ascontiguousarray(scales, dtype=np.uint8)
    if values.shape != storage:
        raise ValueError(f"{dtype} storage shape {values.shape} != {storage}")
    if scales.shape != scale:
        raise ValueError(f"{dtype} scale shape {scales.shape} != {scale}")
    return _MX_HEADER.pack(b"MXT1", 1, MX_KINDS[dtype], 0, rows, cols, *storage, *scale) + values.tobytes() + scales.tobytes()


@dataclass
class LowbitHeader:
    dtype: str
    state_bits: int
    out: int
    neuron_len: int
    body_off: int      # tables (if the blob has them), fp16 anchors, streams
    body_bytes: int
    table_bytes: int


def is_lowbit_dtype(dtype: str) -> bool:
    return dtype in LOWBIT_FORMATS


def lowbit_stream_bytes(dtype: str, out: int, neuron_len: int, state_bits: int) -> int:
    """anchors + state / scale stream + index stream (+ delta-sign stream), every stream packed across the tensor
    (mfq/formats/nvq1_l.py:157-169, nvq1_s.py:188-199, npq0_l.py:228-238, npq0_s.py:226-236)."""
    ib = LOWBIT_FORMATS[dtype][3]
    ng = -(-neuron_len // 24)
    nvec = -(-neuron_len // 8) if dtype == "NVQ1-L" else neuron_len // 8
    n = 2 * out + (out * ng * state_bits + 7) // 8 + (out * nvec * ib + 7) // 8
    return n + ((out * ng + 7) // 8 if dtype.startswith("NVQ1") else 0)


def parse_lowbit(dtype: str, blob) -> LowbitHeader:
    """Header, shape and table checks of unpack_nvq1_l / unpack_nvq1_s / unpack_npq0_l / unpack_npq0_s (and of the C++
    loader, cpp_runtime/mfq_decode.cpp:3800-3910), with their messages."""
    magic, ver_want, sbits_want, _ = LOWBIT_FORMATS[dtype]
    if len(blob) < _NVQ_HDR.size:
        raise ValueError(f"truncated {dtype} header")
    m, ver, sbits, gs, axis, neuron_len, ndim = _NVQ_HDR.unpack_from(blob, 0)
    if m != magic:
        raise ValueError(f"invalid {dtype} magic: {m!r}")
    if dtype == "NVQ1-L":
        if ver not in (1, 2):
            raise ValueError(f"unsupported NVQ1-L profile: {ver}")
        if gs != 24 or sbits not in (3, 4):
            raise ValueError("unsupported NVQ1-L profile")
    elif ver != ver_want or sbits != sbits_want or gs != 24:
        raise ValueError(f"unsupported {dtype} stream profile")
    if ndim <= 0 or neuron_len <= 0 or (dtype != "NVQ1-L" and neuron_len % 8):
        raise ValueError(f"invalid {dtype} dimensions")
    off = _NVQ_HDR.size
    if off + 8 * ndim + 4 > len(blob):
        raise ValueError(f"truncated {dtype} shape")
    shape = struct.unpack_from(f"<{ndim}q", blob, off)
    off += 8 * ndim
    out = struct.unpack_from("<I", blob, off)[0]
    off += 4
    if out <= 0 or int(np.prod(shape)) != out * neuron_len:
        raise ValueError(f"{dtype} shape does not match neuron dimensions")
    if dtype == "NVQ1-L":
        table = 4096 if ver == 2 else 0
    elif dtype == "NVQ1-S":
        table = 2048
    else:
        tv, states, second = _NPQ0_TABLES[dtype]
        table = 64 + states * 32 + states * second * 4
        if off + table > len(blob):
            raise ValueError(f"truncated {dtype} product tables")
        head = bytes(blob[off:off + 64])
        if tuple(head[:6]) != (tv, states, 3, LOWBIT_FORMATS[dtype][3] - 3, 24, 8):
            raise ValueError(f"unsupported {dtype} table profile")
        if any(head[6:8]) or any(head[8 + 2 * states:64]):
            raise ValueError(f"invalid {dtype} reserved table bytes")
        lut = np.frombuffer(head, dtype="<f2", count=states, offset=8).astype(np.float32)
        if not np.isfinite(lut).all() or np.any(lut < 0) or float(lut.max()) <= 0:
            raise ValueError(f"{dtype} scale LUT must be finite and non-negative")
    if table and dtype.startswith("NVQ1"):
        if off + table > len(blob):
            raise ValueError(f"truncated {dtype} codebook")
        enc = np.frombuffer(blob, dtype="<u2", count=table // 2, offset=off)
        if np.any(((enc[:, None] >> (2 * np.arange(8, dtype=np.uint16))[None, :]) & 3) > 2):
            raise ValueError(f"packed {dtype} codebook contains a non-ternary digit")
    expect = table + lowbit_stream_bytes(dtype, out, neuron_len, sbits)
    if len(blob) - off != expect:
        raise ValueError(f"invalid {dtype} blob tail: remaining={len(blob) - off}, expected={expect}")
    return LowbitHeader(dtype, sbits, out, neuron_len, off, expect, table)


def _slice_bits(buf, byte_off: int, bit0: int, nbits: int) -> bytes:
    """Bits [bit0, bit0 + nbits) of the little-endian bit stream that starts at byte_off, as a stream of its own."""
    b0, b1 = bit0 // 8, (bit0 + nbits + 7) // 8
    bits = np.unpackbits(np.frombuffer(buf, dtype=np.uint8, count=b1 - b0, offset=byte_off + b0), bitorder="little")
    return np.packbits(bits[bit0 - 8 * b0: bit0 - 8 * b0 + nbits], bitorder="little").tobytes()


def split_rows(dtype: str, blob, parts: int) -> list[bytes]:
    """Cut an NVQ-family, 1-bit-family or NINT8-0 tensor of parts * n neurons into `parts` blobs of n neurons each (the experts of a
    NINTM cohort, cpp_runtime/mfq_decode.cpp:4800-5360): same header flags and tables, the anchors and the rows' share
    of every tensor-wide bit stream re-packed from bit 0."""
    blob = bytes(blob)
    if dtype == "NINT8-0":                  # [rows, K] along axis 0: a row is its ng blocks of 34 bytes, back to back
        h = parse_nint8_zero(blob)
        if h.axis != 0 or len(h.shape) != 2:
            raise ValueError("NINT8-0 cohorts are [rows, K] tensors quantized along axis 0")
        if parts <= 0 or h.out % parts:
            raise ValueError(f"{dtype}: {h.out} neurons do not split into {parts} equal parts")
        n, row = h.out // parts, h.ng * 34
        head = _N8Z_HDR.pack(b"NI80", 0, h.neuron_len, 2) + struct.pack("<2q", n, h.neuron_len) + struct.pack("<II", n, h.ng)
        return [head + blob[h.body_off + i * n * row: h.body_off + (i + 1) * n * row] for i in range(parts)]
    if is_lowbit_dtype(dtype):
        h = parse_lowbit(dtype, blob)
        ib = LOWBIT_FORMATS[dtype][3]
        ng = -(-h.neuron_len // 24)
        nvec = -(-h.neuron_len // 8) if dtype == "NVQ1-L" else h.neuron_len // 8
        per_row = [h.state_bits * ng, ib * nvec] + ([ng] if dtype.startswith("NVQ1") else [])
        tables, out, K = h.table_bytes, h.out, h.neuron_len
    else:
        h = parse_nvq(blob)
        per_row = [h.sub_bits * h.ng, h.index_bits * h.nvec, 7 * h.nsign]
        tables = 64 + h.banks * (1 << h.index_bits) * h.vector_size if h.jsc else 0
        out, K = h.out, h.neuron_len
    if parts <= 0 or out % parts:
        raise ValueError(f"{dtype}: {out} neurons do not split into {parts} equal parts")
    n = out // parts
    head8 = blob[:8]                                         # magic, flags / version, state bits, groupsize
    anchors_off = h.body_off + tables
    stream_off, off = [], anchors_off + 2 * out
    for bits in per_row:
        stream_off.append(off)
        off += (out * bits + 7) // 8
    res = []
    for i in range(parts):
        piece = [head8, struct.pack("<iiI", 0, K, 2), struct.pack("<2q", n, K), struct.pack("<I", n),
                 blob[h.body_off:h.body_off + tables], blob[anchors_off + 2 * i * n: anchors_off + 2 * (i + 1) * n]]
        piece += [_slice_bits(blob, so, i * n * bits, n * bits) for so, bits in zip(stream_off, per_row)]
        res.append(b"".join(piece))
    return res


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
    if ndim > 8 or len(blob) < _NVQ_HDR.size + 8 * ndim + 4:
        raise ValueError("truncated NVQ header")
    off = _NVQ_HDR.size + 8 * ndim
    out, = struct.unpack_from("<I", blob, off)
    off += 4
    if gs <= 0 or neuron_len <= 0 or out <= 0 or not 1 <= sub_bits <= 8:
        raise ValueError("NVQ dimensions must be positive (groupsize, neuron_len, rows) and sub_bits in [1,8]")
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
NEPQ_BITS = {0: (2, 6, 0, 320), 1: (3, 7, 0, 832), 2: (4, 9, 1, 2048), 3: (3, 11, 1, 4096)}


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
    if pid < 2:     # NEPQ0: every table of the pool is an NPQ0 table (mfq/formats/nepq.py:270-290)
        base = "NPQ0-S" if pid == 0 else "NPQ0-L"
        tv, states, second = _NPQ0_TABLES[base]
        for bnk in range(banks):
            head = bytes(blob[_NEPQ_HDR.size + bnk * tb: _NEPQ_HDR.size + bnk * tb + 64])
            if tuple(head[:6]) != (tv, states, 3, ib - 3, 24, 8):
                raise ValueError(f"unsupported {NEPQ_LABEL[pid]} table profile")
            if any(head[6:8]) or any(head[8 + 2 * states:64]):
                raise ValueError(f"invalid {NEPQ_LABEL[pid]} reserved table bytes")
            lut = np.frombuffer(head, dtype="<f2", count=states, offset=8).astype(np.float32)
            if not np.isfinite(lut).all() or np.any(lut < 0) or float(lut.max()) <= 0:
                raise ValueError(f"{NEPQ_LABEL[pid]} scale LUT must be finite and non-negative")
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


def parse_nintm(blob, allow_partial: bool = False) -> NintmHeader:
    """allow_partial: also take an expert delta (an NINTMD overlay record: magic NID2, the same layout, pools for some
    experts only -- unpack_nint_moe_impl, cpp_runtime/mfq_decode.cpp:2367-2477)."""
    if len(blob) < _NIM_HDR.size:
        raise ValueError("truncated NINTM header")
    magic, E, out, K, npools = _NIM_HDR.unpack_from(blob, 0)
    if magic == b"NID2" and not allow_partial:
        raise ValueError("NINTM delta cannot be loaded as a full tensor")
    if magic not in (b"NIM2", b"NID2"):
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
    if missing.size and not allow_partial:
        raise ValueError(f"NINTM pools do not cover experts {missing[:16].tolist()}")
    return hdr


# ---------------------------------------------------------------------------------------
# MFQ1 container (mfq/formats/io.py:646-965, mfq/formats/shards.py): header, directory, blobs back to back; one file or a
# shard set <stem>-NNNNN-of-NNNNN.mfq whose headers carry split.* metadata
# ---------------------------------------------------------------------------------------
ASSET_PREFIX = "__mfq_asset__/"        # runtime assets: container metadata, first shard only (mfq/formats/assets.py:17)
SPLIT_NO, SPLIT_COUNT, SPLIT_TENSORS, SPLIT_RECORDS = "split.no", "split.count", "split.tensors.count", "split.records.count"
_SHARD_RE = re.compile(r"^(?P<stem>.+)-(?P<index>[0-9]{5})-of-(?P<count>[0-9]{5})\.mfq$")


def _mfq_head(records, model_arch: str, version: int, extra: dict | None) -> bytes:
    """Header and record table: magic, version, architecture, (version >= 2) metadata as key / JSON text pairs, then
    per record name, dtype string and byte length (mfq/formats/shards.py:205-236)."""
    extra = dict(extra or {})
    if extra and version < 2:
        version = 2
    a = model_arch.encode()
    out = [b"MFQ1", struct.pack("<I", version), struct.pack("<I", len(a)), a]
    if version >= 2:
        out.append(struct.pack("<I", len(extra)))
        for key, value in extra.items():
            kb, vb = str(key).encode(), json.dumps(value).encode()
            out += [struct.pack("<I", len(kb)), kb, struct.pack("<I", len(vb)), vb]
    out.append(struct.pack("<I", len(records)))
    for name, dtype, nbytes in records:
        nb, db = name.encode(), dtype.encode()
        out += [struct.pack("<I", len(nb)), nb, struct.pack("<I", len(db)), db, struct.pack("<Q", nbytes)]
    return b"".join(out)


def write_mfq(path, tensors: dict, model_arch: str = "synthetic", version: int = 1, extra: dict | None = None) -> None:
    """tensors: name -> (dtype string, blob bytes); extra: metadata of a version 2 header (values are stored as JSON)."""
    with open(path, "wb") as f:
        f.write(_mfq_head([(n, d, len(b)) for n, (d, b) in tensors.items()], model_arch, version, extra))
        for _, (_, blob) in tensors.items():
            f.write(blob)


def format_shard_path(path, index: int, count: int) -> Path:
    """<stem>-00001-of-00004.mfq, 1-based (format_shard_path, mfq/formats/shards.py:46-53)."""
    source = Path(path)
    if not 1 <= index <= count <= 99999:
        raise ValueError(f"invalid MFQ shard index/count: {index}/{count}")
    stem = source.name[:-4] if source.name.lower().endswith(".mfq") else source.name
    return source.with_name(f"{stem}-{index:05d}-of-{count:05d}.mfq")


def parse_shard_path(path):
    """(base path, 1-based index, count) of a shard file name, or None (parse_shard_path, shards.py:56-68)."""
    source = Path(path)
    m = _SHARD_RE.fullmatch(source.name)
    if m is None:
        return None
    count, index = int(m.group("count")), int(m.group("index"))
    if count < 1 or index < 1 or index > count:
        raise ValueError(f"invalid MFQ shard file name: {source}")
    return source.with_name(f"{m.group('stem')}.mfq"), index, count


def plan_shards(sizes, split_max_size: int = 0, split_max_tensors: int = 0):
    """Records -> shards by the reference's rule (plan_record_shards, shards.py:133-173): `sizes` is [(name, nbytes)] in
    file order; a tensor opens a new shard when adding it to a non-empty shard would pass split_max_size, or when the
    shard already holds split_max_tensors tensors; runtime assets all go to the front of the first shard.  Returns the
    list of shards, each a list of names."""
    if split_max_size < 0 or split_max_tensors < 0:
        raise ValueError("MFQ shard limits must be non-negative")
    if split_max_size and split_max_tensors:
        raise ValueError("--split-max-size and --split-max-tensors are mutually exclusive")
    if not split_max_size and not split_max_tensors:
        return [[n for n, _ in sizes]]
    assets = [n for n, _ in sizes if n.startswith(ASSET_PREFIX)]
    shards, payload, count = [[]], [0], [0]
    for name, nbytes in sizes:
        if name.startswith(ASSET_PREFIX):
            continue
        over_size = bool(split_max_size and count[-1] > 0 and payload[-1] + int(nbytes) > split_max_size)
        over_count = bool(split_max_tensors and count[-1] >= split_max_tensors)
        if over_size or over_count:
            shards.append([]); payload.append(0); count.append(0)
        shards[-1].append(name)
        payload[-1] += int(nbytes)
        count[-1] += 1
    shards[0][0:0] = assets
    return shards


def write_mfq_shards(path, tensors: dict, model_arch: str = "synthetic", version: int = 2, extra: dict | None = None,
                     split_max_size: int = 0, split_max_tensors: int = 0) -> list:
    """The shard set of `tensors` next to `path` (write_blob_record_shards, shards.py:254-336): every shard is an MFQ1
    file of version >= 2 whose metadata holds split.no / split.count and the totals of tensors and records; the model's
    own metadata stays in the first shard only.  Without a limit: the single file `path`.  Returns the paths written."""
    plan = plan_shards([(n, len(b)) for n, (_, b) in tensors.items()], split_max_size, split_max_tensors)
    if not (split_max_size or split_max_tensors):
        write_mfq(path, tensors, model_arch, version, extra)
        return [Path(path)]
    n_tensors = sum(not n.startswith(ASSET_PREFIX) for n in tensors)
    paths = []
    for no, names in enumerate(plan):
        meta = {k: v for k, v in (extra or {}).items() if not k.startswith("split.")} if no == 0 else {}
        meta.update({SPLIT_NO: no, SPLIT_COUNT: len(plan), SPLIT_TENSORS: n_tensors, SPLIT_RECORDS: len(tensors)})
        dest = format_shard_path(path, no + 1, len(plan))
        write_mfq(dest, {n: tensors[n] for n in names}, model_arch, max(2, version), meta)
        paths.append(dest)
    return paths


def read_mfq_header(data):
    """(version, architecture, metadata {key: decoded JSON value}, [(name, dtype, nbytes)], offset of the first blob)."""
    if len(data) < 12 or bytes(data[:4]) != b"MFQ1":
        raise ValueError("invalid MFQ magic")
    version, = struct.unpack_from("<I", data, 4)
    pos = [8]

    def text():
        if pos[0] + 4 > len(data):
            raise ValueError("truncated MFQ header")
        n, = struct.unpack_from("<I", data, pos[0])
        if n > len(data) - pos[0] - 4:
            raise ValueError("truncated MFQ header")
        v = bytes(data[pos[0] + 4: pos[0] + 4 + n]).decode()
        pos[0] += 4 + n
        return v

    arch = text()
    extra = {}
    if version >= 2:
        ne, = struct.unpack_from("<I", data, pos[0])
        pos[0] += 4
        for _ in range(ne):
            key, value = text(), text()
            if key in extra:
                raise ValueError(f"duplicate MFQ metadata key: {key}")
            extra[key] = json.loads(value)
    if pos[0] + 4 > len(data):
        raise ValueError("truncated MFQ header")
    nt, = struct.unpack_from("<I", data, pos[0])
    pos[0] += 4
    recs = []
    for _ in range(nt):
        name, dtype = text(), text()
        if pos[0] + 8 > len(data):
            raise ValueError("truncated MFQ directory")
        ln, = struct.unpack_from("<Q", data, pos[0])
        pos[0] += 8
        recs.append((name, dtype, ln))
    return version, arch, extra, recs, pos[0]


def read_mfq_directory(data) -> dict:
    """name -> (dtype, offset, nbytes) of an MFQ1 file image."""
    _, _, _, recs, off = read_mfq_header(data)
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


def _split_values(extra: dict):
    """(split.no, split.count, tensors total or None, records total or None) (split_values, shards.py:96-113)."""
    no, count = int(extra.get(SPLIT_NO, 0)), int(extra.get(SPLIT_COUNT, 1))
    if count < 1 or count > 99999:
        raise ValueError(f"invalid {SPLIT_COUNT}: {count}")
    if no < 0 or no >= count:
        raise ValueError(f"invalid {SPLIT_NO}: {no}")
    t, r = extra.get(SPLIT_TENSORS), extra.get(SPLIT_RECORDS)
    return no, count, None if t is None else int(t), None if r is None else int(r)


@dataclass
class MfqRecord:
    name: str
    dtype: str
    source: int      # index into MfqStore.paths
    offset: int
    nbytes: int


class MfqStore:
    """One MFQ1 file or shard set as one lazy record table over read-only memory maps (open_mmap,
    mfq/formats/io.py:834-965; MfqFile, cpp_runtime/mfq_decode.cpp:1294-1527).  `path` may be any shard of a set.
    blob(name) is a zero-copy view into the map.  tensor_overlay: an unsharded MFQ1 file whose records replace records
    of the same name (each must exist); expert_overlay: NINTMD records over NINTM records, kept in expert_overlays.
    None takes MFQ_TENSOR_OVERLAY / MFQ_EXPERT_OVERLAY from the environment, as the reference does; "" takes none."""

    def __init__(self, path, tensor_overlay: str | None = None, expert_overlay: str | None = None):
        self.paths, self._files, self._maps = [], [], []
        self.records: dict[str, MfqRecord] = {}
        self.tensor_overlays: dict[str, MfqRecord] = {}
        self.expert_overlays: dict[str, MfqRecord] = {}
        try:
            self._open(Path(path), tensor_overlay, expert_overlay)
        except Exception:
            self.close()
            raise

    def _map(self, path: Path):
        """Maps one file; returns (source index, version, architecture, metadata, {name: MfqRecord})."""
        import mmap
        if not path.is_file():
            raise FileNotFoundError(f"cannot open MFQ file: {path}")
        f = open(path, "rb")
        self._files.append(f)
        m = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ)
        self._maps.append(m)
        self.paths.append(path)
        src = len(self._maps) - 1
        view = memoryview(m)
        try:
            version, arch, extra, recs, off = read_mfq_header(view)
            out = {}
            for name, dtype, ln in recs:
                if name in out:
                    raise ValueError(f"duplicate MFQ tensor record: {name}: {path}")
                if ln > len(view) - off:
                    raise ValueError(f"truncated MFQ blob for {name}: {path}")
                out[name] = MfqRecord(name, dtype, src, off, ln)
                off += ln
            if off != len(view):
                raise ValueError(f"MFQ file length mismatch: records end={off}, file size={len(view)}: {path}")
        finally:
            view.release()
        return src, version, arch, extra, out

    def _open(self, requested: Path, tensor_overlay, expert_overlay):
        _, version, arch, extra, first = self._map(requested)
        split_no, split_count, want_tensors, want_records = _split_values(extra)
        parsed = parse_shard_path(requested)
        self.version, self.model_arch, self.extra = version, arch, extra
        if split_count == 1:
            if parsed is not None and parsed[2] != 1:
                raise ValueError(f"MFQ filename claims multiple shards but metadata does not: {requested}")
            self.records = first
        else:
            if parsed is None:
                raise ValueError(f"sharded MFQ path lacks -00001-of-00000 suffix: {requested}")
            if parsed[1] - 1 != split_no or parsed[2] != split_count:
                raise ValueError(f"MFQ shard filename/metadata mismatch: {requested}")
            paths = [format_shard_path(parsed[0], i, split_count) for i in range(1, split_count + 1)]
            for p in paths:
                if not p.is_file():
                    raise FileNotFoundError(f"missing MFQ shard: {p}")
            self.close()                                    # start over in shard order
            for i, p in enumerate(paths):
                _, v, a, ex, recs = self._map(p)
                no, count, t, r = _split_values(ex)
                if no != i or count != split_count:
                    raise ValueError(f"MFQ shard metadata mismatch: expected {i}/{split_count}, got {no}/{count}: {p}")
                if v != version or a != arch:
                    raise ValueError(f"MFQ shard architecture/version mismatch: {p}")
                if want_tensors is None:
                    want_tensors = t
                elif t is not None and t != want_tensors:
                    raise ValueError(f"MFQ shard tensor count mismatch: {p}")
                if want_records is None:
                    want_records = r
                elif r is not None and r != want_records:
                    raise ValueError(f"MFQ shard record count mismatch: {p}")
                if i == 0:
                    self.extra = ex                         # model metadata lives in the first shard
                for name, rec in recs.items():
                    if name in self.records:
                        raise ValueError(f"duplicate MFQ tensor across shards: {name}")
                    self.records[name] = rec
            if want_records is not None and len(self.records) != want_records:
                raise ValueError(f"MFQ shard record total mismatch: {len(self.records)} != {want_records}")
            if want_tensors is not None and self.tensor_count() != want_tensors:
                raise ValueError(f"MFQ shard tensor total mismatch: {self.tensor_count()} != {want_tensors}")
        self.n_shards = len(self.paths)
        if tensor_overlay is None:
            tensor_overlay = os.environ.get("MFQ_TENSOR_OVERLAY", "")
        if expert_overlay is None:
            expert_overlay = os.environ.get("MFQ_EXPERT_OVERLAY", "")
        if tensor_overlay:
            _, _, _, ex, recs = self._map(Path(tensor_overlay))
            if _split_values(ex)[1] != 1:
                raise ValueError("sharded MFQ tensor overlays are not supported")
            for name, rec in recs.items():
                if name not in self.records:
                    raise ValueError(f"tensor overlay replaces an unknown record: {name}")
                self.records[name] = rec
                self.tensor_overlays[name] = rec
        if expert_overlay:
            _, _, _, ex, recs = self._map(Path(expert_overlay))
            if _split_values(ex)[1] != 1:
                raise ValueError("sharded MFQ expert overlays are not supported")
            for name, rec in recs.items():
                if rec.dtype != "NINTMD" or name not in self.records or self.records[name].dtype != "NINTM":
                    raise ValueError(f"invalid expert overlay record: {name}")
                self.expert_overlays[name] = rec

    def tensor_count(self) -> int:
        return sum(not n.startswith(ASSET_PREFIX) for n in self.records)

    def __contains__(self, name) -> bool:
        return name in self.records

    def names(self):
        return list(self.records)

    def record(self, name) -> MfqRecord:
        if name not in self.records:
            raise KeyError(f"missing tensor: {name}")
        return self.records[name]

    def blob(self, name) -> memoryview:
        """The record's bytes as a read-only view into the file map (no copy); valid until close()."""
        r = self.record(name)
        return memoryview(self._maps[r.source])[r.offset: r.offset + r.nbytes]

    def expert_overlay_blob(self, name):
        """The NINTMD record an expert overlay holds for NINTM tensor `name` (read_expert_overlay,
        cpp_runtime/mfq_decode.cpp:1513-1521) as a view into its file map, or None when there is none: what
        NintMoeWeight.from_blob takes as `expert_overlay`."""
        r = self.expert_overlays.get(name)
        return None if r is None else memoryview(self._maps[r.source])[r.offset: r.offset + r.nbytes]

    def asset_text(self, name) -> str:
        r = self.record(name)
        if r.dtype != "BLOB":
            raise ValueError(f"MFQ runtime asset has non-BLOB dtype: {name}")
        return bytes(self.blob(name)).decode()

    def close(self):
        for m in self._maps:
            try:
                m.close()
            except BufferError:          # a blob view is still alive: the map goes with its last view
                pass
        for f in self._files:
            f.close()
        self.paths, self._files, self._maps, self.records = [], [], [], {}

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
