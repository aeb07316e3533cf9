"""CPU oracle for the MFQ packed-weight matmul path  --  TEST INFRASTRUCTURE ONLY.

This module restates, in plain numpy, the reference's CPU algorithm for the hot
path: the MFQ payload codecs, the CPU dequantizers, the fp32
dequant-then-matmul linear, and the MoE routing / grouped-matmul reference loop.
Nothing in the shipped product imports it: only tests/, __graft_entry__.smoke()
and bench.py's cpu_baseline leg may.  It never touches a GPU.

Each function cites the reference file:line it follows (paths relative to the
reference tree).  Parity status of each function:

  pinned (closed form / reference constants / brute force, see tests/test_oracle_*.py)
    pack_bits / unpack_bits        mfq/formats/io.py:144-188, mfq/formats/nvq.py:556-581
    pack_nint / unpack_nint        mfq/formats/io.py:191-248
    dequantize_nint                mfq/quantize/nint_quant.py:896-908
    pack_nvq_jsc / unpack_nvq      mfq/formats/nvq.py:586-820
    dequantize_nvq_jsc             mfq/quantize/nvq_jsc.py:1053-1079
    dequantize_nvq                 mfq/quantize/nvq_quant.py:591-626
    pack_nepq / unpack_nepq        mfq/formats/nepq.py:368-474
    dequantize_nepq (NEPQ1-S/L)    mfq/formats/nepq.py:492-544
    pack_nint_moe / unpack_nint_moe  mfq/formats/io.py:251-446
    dequantize_expertwise          mfq/quantize/expert_nint.py:605-615
    linear_forward                 mfq/runtime/linear.py:37-42
    moe_topk                       mfq/kernels/cuda/moe.cu:124-263
    build_expert_map               mfq/kernels/cuda/moe.cu:472-542
    moe_grouped_matmul / moe_ffn   tests/test_moe_kernels_cuda.py:58-68, cpp_runtime/mfq_decode.cpp:3394-3416
    mfq_file_write / mfq_file_read mfq/formats/io.py:646-685
    pack_nint8_zero / unpack_nint8_zero / dequantize_nint8_zero / quantize_nint8_zero
                                   mfq/formats/nint8_zero.py:107-218 (the GGML Q8_0 rule: closed form)
    moe_swiglu / moe_geglu / input_mul   mfq/kernels/cuda/glu.cuh:5-16, cpp_runtime/mfq_decode.cpp:8395-8417

  additionally pinned by reference-written blobs and reference-dequantized values
  (tests/golden/reference_blobs.npz, made by tests/golden/make_reference_blobs.py; tests/test_reference_blobs.py)
    pack_nint / unpack_nint / dequantize_nint, pack_nvq_jsc / pack_nvq_plain / unpack_nvq / dequantize_nvq_jsc /
    dequantize_nvq (incl. the index-parity sign rule on e8_256), pack_nepq / unpack_nepq / dequantize_nepq,
    pack_nint_moe / unpack_nint_moe / dequantize_expertwise

  pinned by reference-written blobs and reference-dequantized values of the 1-bit families
  (tests/golden/reference_lowbit.npz, made by tests/golden/make_reference_lowbit.py; tests/test_reference_lowbit.py)
    pack_nvq1 / unpack_nvq1        mfq/formats/nvq1_l.py:234-345, nvq1_s.py:262-347
    dequantize_nvq1                mfq/quantize/nvq1_l_quant.py:384-414, nvq1_s_quant.py:142-174
    pack_npq0 / unpack_npq0        mfq/formats/npq0_l.py:112-185, 326-415, npq0_s.py:110-183, 320-406
    dequantize_npq0                mfq/quantize/npq0_l.py:766-790, npq0_s.py:812-836
    pack_nepq / unpack_nepq / dequantize_nepq on NEPQ0-S / NEPQ0-L   mfq/formats/nepq.py:95-116, 368-474, 492-521

  pinned by a reference-written blob (tests/golden/reference_mx.npz, made by tests/golden/make_reference_mx.py), by
  torch's own float8_e4m3fn conversion over all 256 codes, and by closed forms (tests/test_oracle_mx.py)
    pack_mx / unpack_mx            mfq/formats/mx.py:65-182
    dequantize_mx                  cpp_runtime/mfq_decode.cpp:1920-1947 (MXFP4), 8810-8840 and
                                   mfq/kernels/cuda/mx_matmul.cu:17-47, 222-240 (MXFP8: E4M3FN x E8M0 per 128 x 128 block)

  pinned by golden vectors written from the reference's own numpy quantizer
  (tests/golden/nint_quant_vectors.npz, made by tests/golden/make_nint_quant_vectors.py)
    make_qkx2 / quantize_nint      mfq/formats/nint.py:119-174, mfq/quantize/nint_quant.py:745-893
    (weight-only branch, importance=None)
"""
from __future__ import annotations

import math
import struct
from dataclasses import dataclass, field
from pathlib import Path

import numpy as np

_DATA = Path(__file__).resolve().parents[1] / "tyloquant_amd" / "data"


# ---------------------------------------------------------------------------
# bit streams  (mfq/formats/io.py:144-188; mfq/formats/nvq.py:556-581;
#               mfq/formats/nepq.py:217-255)
# ---------------------------------------------------------------------------
def pack_bits(values, bits: int) -> bytes:
    """Little-endian bit stream: value i occupies bits [i*bits, (i+1)*bits)."""
    v = np.ascontiguousarray(values).reshape(-1).astype(np.uint32)
    if bits == 0:
        return b""
    if bits == 8:
        return v.astype(np.uint8).tobytes()
    # 8 values fill exactly `bits` bytes: value i of such a run is OR-ed in at bit i * bits (bits <= 16, so it
    # touches at most the three bytes from byte (i * bits) // 8)
    n = v.size
    n8 = (n + 7) // 8
    vv = np.zeros(n8 * 8, dtype=np.uint32)
    vv[:n] = v & ((1 << bits) - 1)
    vv = vv.reshape(n8, 8)
    by = np.zeros((n8, bits + 2), dtype=np.uint32)
    for i in range(8):
        k, sh = (i * bits) // 8, (i * bits) % 8
        w = vv[:, i] << sh
        by[:, k] |= w & 0xFF
        by[:, k + 1] |= (w >> 8) & 0xFF
        by[:, k + 2] |= (w >> 16) & 0xFF
    return by[:, :bits].astype(np.uint8).reshape(-1)[: (n * bits + 7) // 8].tobytes()


def unpack_bits(blob, off: int, count: int, bits: int):
    if bits == 0 or count == 0:
        return np.empty(0, dtype=np.uint8), off + ((count * bits + 7) // 8 if bits else 0)
    nbytes = (count * bits + 7) // 8
    if off + nbytes > len(blob):
        raise ValueError("truncated bit stream")
    packed = np.frombuffer(blob, dtype=np.uint8, count=nbytes, offset=off)
    # 8 values occupy exactly `bits` bytes; value i of such a run starts at bit i * bits, i.e. inside the three
    # bytes from byte (i * bits) // 8 (bits <= 16).  Same stream definition as one bit at a time, a few bytes of
    # scratch per value.
    n8 = (count + 7) // 8
    by = np.zeros((n8, bits + 2), dtype=np.uint32)
    flat = np.zeros(n8 * bits, dtype=np.uint8)
    flat[:nbytes] = packed
    by[:, :bits] = flat.reshape(n8, bits)
    out = np.empty((n8, 8), dtype=np.uint8 if bits <= 8 else np.uint16)
    for i in range(8):
        k, sh = (i * bits) // 8, (i * bits) % 8
        out[:, i] = ((by[:, k] | (by[:, k + 1] << 8) | (by[:, k + 2] << 16)) >> sh) & ((1 << bits) - 1)
    return out.reshape(-1)[:count], off + nbytes


def _f16_round(x):
    return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)


# ---------------------------------------------------------------------------
# NINT  (mfq/formats/nint.py, mfq/quantize/nint_quant.py, mfq/formats/io.py:191-248)
# ---------------------------------------------------------------------------
@dataclass
class NintTensor:
    bits: int
    groupsize: int
    sub_bits: int
    shape: tuple
    axis: int
    neuron_len: int
    q: np.ndarray             # (out, ng, gs) uint8
    neuron_scale: np.ndarray  # (out,) f32 (f16-representable)
    neuron_min: np.ndarray    # (out,) f32
    sub_scale: np.ndarray     # (out, ng) uint8
    sub_min: np.ndarray       # (out, ng) uint8

    @property
    def out(self):
        return self.q.shape[0]

    @property
    def ng(self):
        return self.q.shape[1]


_NINT_HDR = struct.Struct("<BBiii")


def nint_payload_nbytes(out, neuron_len, bits, gs, sub_bits):
    """Compact payload bytes without the blob header (mfq/formats/io.py:191-203)."""
    ng = -(-neuron_len // gs)
    return 4 * out + 2 * ((out * ng * sub_bits + 7) // 8) + (out * ng * gs * bits + 7) // 8


def pack_nint(t: NintTensor) -> bytes:
    """mfq/formats/io.py:191-203."""
    out, ng, _ = t.q.shape
    parts = [_NINT_HDR.pack(t.bits, t.sub_bits, t.groupsize, t.axis, t.neuron_len),
             struct.pack("<I", len(t.shape)), struct.pack(f"<{len(t.shape)}q", *t.shape),
             struct.pack("<II", out, ng),
             np.ascontiguousarray(t.neuron_scale, dtype=np.float16).tobytes(),
             np.ascontiguousarray(t.neuron_min, dtype=np.float16).tobytes(),
             pack_bits(t.sub_scale, t.sub_bits), pack_bits(t.sub_min, t.sub_bits),
             pack_bits(t.q, t.bits)]
    return b"".join(parts)


def unpack_nint(blob) -> NintTensor:
    """mfq/formats/io.py:206-248 (bit-stream tail and the legacy one-byte-per-value tail)."""
    blob = bytes(blob)
    bits, sub_bits, gs, axis, neuron_len = _NINT_HDR.unpack_from(blob, 0)
    off = _NINT_HDR.size
    ndim = struct.unpack_from("<I", blob, off)[0]
    off += 4
    shape = struct.unpack_from(f"<{ndim}q", blob, off)
    off += 8 * ndim
    out, ng = struct.unpack_from("<II", blob, off)
    off += 8
    ns = np.frombuffer(blob, dtype=np.float16, count=out, offset=off).astype(np.float32)
    off += 2 * out
    nm = np.frombuffer(blob, dtype=np.float16, count=out, offset=off).astype(np.float32)
    off += 2 * out
    sub_count, q_count = out * ng, out * ng * gs
    packed_tail = ((sub_count * sub_bits + 7) // 8) * 2 + (q_count * bits + 7) // 8
    old_tail = sub_count * 2 + q_count
    remaining = len(blob) - off
    if remaining == old_tail and bits <= 8 and sub_bits <= 8:
        ss = np.frombuffer(blob, dtype=np.uint8, count=sub_count, offset=off).copy()
        off += sub_count
        sm = np.frombuffer(blob, dtype=np.uint8, count=sub_count, offset=off).copy()
        off += sub_count
        q = np.frombuffer(blob, dtype=np.uint8, count=q_count, offset=off).copy()
    else:
        if remaining != packed_tail:
            raise ValueError(f"invalid NINT blob tail: remaining={remaining}, packed={packed_tail}, old={old_tail}")
        ss, off = unpack_bits(blob, off, sub_count, sub_bits)
        sm, off = unpack_bits(blob, off, sub_count, sub_bits)
        q, off = unpack_bits(blob, off, q_count, bits)
    return NintTensor(bits, gs, sub_bits, tuple(shape), axis, neuron_len,
                      q.reshape(out, ng, gs), ns, nm, ss.reshape(out, ng), sm.reshape(out, ng))


def dequantize_nint(t: NintTensor) -> np.ndarray:
    """mfq/quantize/nint_quant.py:896-908: four separate fp32 roundings, no FMA."""
    out, ng, gs = t.q.shape
    q = t.q.astype(np.float32)
    d_eff = t.neuron_scale.astype(np.float32)[:, None] * t.sub_scale.astype(np.float32)
    m_eff = t.neuron_min.astype(np.float32)[:, None] * t.sub_min.astype(np.float32)
    recon = d_eff[..., None] * q - m_eff[..., None]
    return np.ascontiguousarray(recon.reshape(out, ng * gs)[:, : t.neuron_len])


def make_qkx2(x, w, nmax=15):
    """mfq/formats/nint.py:119-174 (weighted LS search of (scale, zp) per group)."""
    nmax = int(nmax)
    rmin, rdelta, nstep = (-1.0, 0.1, 20) if nmax <= 15 else (-0.5, 0.1, 15)
    mn = np.minimum(x.min(-1), 0.0)
    mx = x.max(-1)
    sum_w = w.sum(-1)
    sum_x = (w * x).sum(-1)
    degen = (mx == mn) | (sum_w <= 0)
    rng = np.where(degen, 1.0, mx - mn)
    iscale0 = nmax / rng
    scale0 = 1.0 / iscale0
    L0 = np.clip(np.rint(iscale0[..., None] * (x - mn[..., None])), 0, nmax).astype(np.int32)
    diff = scale0[..., None] * L0 + mn[..., None] - x
    best_err = (w * diff * diff).sum(-1)
    best_scale = scale0.copy()
    best_min = mn.copy()
    for is_ in range(nstep + 1):
        iscale = (rmin + rdelta * is_ + nmax) / rng
        Laux = np.clip(np.rint(iscale[..., None] * (x - mn[..., None])), 0, nmax).astype(np.int32)
        Laf = Laux.astype(np.float32)
        sl = (w * Laf).sum(-1)
        sl2 = (w * Laf * Laf).sum(-1)
        sxl = (w * Laf * x).sum(-1)
        D = sum_w * sl2 - sl * sl
        valid = D > 0
        Ds = np.where(valid, D, 1.0)
        ts = (sum_w * sxl - sum_x * sl) / Ds
        tm = (sl2 * sum_x - sl * sxl) / Ds
        pos = tm > 0
        sl2s = np.where(sl2 > 0, sl2, 1.0)
        ts = np.where(pos, sxl / sl2s, ts)
        tm = np.where(pos, 0.0, tm)
        cd = ts[..., None] * Laux + tm[..., None] - x
        ce = (w * cd * cd).sum(-1)
        better = valid & (ce < best_err)
        best_err = np.where(better, ce, best_err)
        best_scale = np.where(better, ts, best_scale)
        best_min = np.where(better, tm, best_min)
    best_scale = np.where(degen, 0.0, best_scale)
    best_min = np.where(degen, np.minimum(mn, 0.0), best_min)
    return best_scale.astype(np.float32), best_min.astype(np.float32)


def quantize_nint(weight, bits=4, gs=24, sub_bits=6) -> NintTensor:
    """mfq/quantize/nint_quant.py:745-823, 883-893 (weight-only branch, axis=0, rank 2)."""
    bits, gs, sub_bits = int(bits), int(gs), int(sub_bits)   # numpy ints would promote to fp64
    W = np.asarray(weight, dtype=np.float32)
    out, neuron_len = W.shape
    nmax = (1 << bits) - 1
    K = (1 << sub_bits) - 1
    W2 = W.copy()
    pad = (-neuron_len) % gs
    if pad:
        W2 = np.concatenate([W2, np.zeros((out, pad), dtype=np.float32)], axis=1)
    ng = W2.shape[1] // gs
    grps = W2.reshape(out, ng, gs)
    sx2 = (grps * grps).sum(-1)
    av = np.sqrt(sx2 / gs)
    w = av[..., None] + np.abs(grps)
    if pad:
        w[:, -1, gs - pad:] = 0.0
    scale, zp = make_qkx2(grps, w, nmax=nmax)
    the_min = -zp
    neu_s = scale.max(-1)
    neu_m = the_min.max(-1)
    neu_d = np.where(neu_s > 0, (neu_s / K).astype(np.float16).astype(np.float32), np.float32(0.0))
    neu_dm = np.where(neu_m > 0, (neu_m / K).astype(np.float16).astype(np.float32), np.float32(0.0))
    nss = np.where(neu_s > 0, neu_s, 1.0)
    nmm = np.where(neu_m > 0, neu_m, 1.0)
    sub_scale = np.clip(np.rint(K * scale / nss[..., None]), 0, K)
    sub_min = np.clip(np.rint(K * the_min / nmm[..., None]), 0, K)
    d_eff = neu_d[:, None] * sub_scale.astype(np.float32)
    m_eff = neu_dm[:, None] * sub_min.astype(np.float32)
    de = np.where(d_eff > 0, d_eff, 1.0)
    q = np.clip(np.rint((grps + m_eff[..., None]) / de[..., None]), 0, nmax)
    return NintTensor(bits, gs, sub_bits, (out, neuron_len), 0, neuron_len, q.astype(np.uint8),
                      neu_d.astype(np.float32), neu_dm.astype(np.float32),
                      sub_scale.astype(np.uint8), sub_min.astype(np.uint8))


# ---------------------------------------------------------------------------
# NVQ  (mfq/formats/nvq.py)
# ---------------------------------------------------------------------------
_NVQ_HDR = struct.Struct("<4sBBHiiI")
_NVQ_CODEBOOK_ID = {"e8_256": 1, "d4_256": 2, "d4_512": 3, "e8_1024": 4, "e8_4096": 5, "d4_1024": 6}
_NVQ_ID_CODEBOOK = {v: k for k, v in _NVQ_CODEBOOK_ID.items()}
_NVQ_INDEX_BITS = {"e8_256": 8, "e8_1024": 10, "e8_4096": 12, "d4_256": 8, "d4_512": 9, "d4_1024": 10}


def nvq_vector_size(codebook: str) -> int:
    return 8 if codebook.startswith("e8_") else 4


def nvq_grid(name: str) -> np.ndarray:
    """Built-in magnitude grids, decoded as 2*digit+1 (mfq/formats/nvq.py:102-129)."""
    raw = np.frombuffer((_DATA / f"{name}.bin").read_bytes(), dtype="<u2")
    dims, digit_bits = (8, 2) if name.startswith("e8_") else (4, 3)
    shifts = digit_bits * np.arange(dims, dtype=np.uint16)
    digits = (raw[:, None] >> shifts[None, :]) & ((1 << digit_bits) - 1)
    return np.ascontiguousarray(2 * digits + 1, dtype=np.int8)


def nvq_payload_nbytes(codebook, out, neuron_len, gs=24, sub_bits=4):
    """mfq/formats/nvq.py:197-207 (streams + anchors, excluding tables and header)."""
    ng = math.ceil(neuron_len / gs)
    nvec = math.ceil(neuron_len / nvq_vector_size(codebook))
    nsign = math.ceil(neuron_len / 8)
    return (out * 2 + (out * ng * sub_bits + 7) // 8
            + (out * nvec * _NVQ_INDEX_BITS[codebook] + 7) // 8 + (out * nsign * 7 + 7) // 8)


@dataclass
class NvqJscTensor:
    codebook: str
    shape: tuple
    neuron_len: int
    neuron_scale: np.ndarray   # (out,) f32
    scale_lut: np.ndarray      # (16,) f32
    bank_for_state: np.ndarray # (16,) u8
    state: np.ndarray          # (out, ng) u8
    indices: np.ndarray        # (out, nvec) u16
    signs: np.ndarray          # (out, nsign) u8
    codebooks: np.ndarray      # (banks, entries, dim) i8, values 0..127
    axis: int = 0
    groupsize: int = 24
    sub_bits: int = 4


@dataclass
class NvqTensor:
    codebook: str
    shape: tuple
    neuron_len: int
    neuron_scale: np.ndarray
    sub_scale: np.ndarray      # (out, ng) u8 integer relative scale
    indices: np.ndarray
    signs: np.ndarray
    axis: int = 0
    groupsize: int = 24
    sub_bits: int = 4
    sign_mode: str = "even"
    custom_codebook: np.ndarray | None = None


def pack_jsc_tables(scale_lut, bank_for_state, codebooks) -> bytes:
    """mfq/formats/nvq.py:446-483 (64-byte header + raw int8 banks)."""
    codebooks = np.ascontiguousarray(codebooks, dtype=np.int8)
    banks = codebooks.shape[0]
    lut = np.asarray(scale_lut, dtype=np.float32).reshape(16)
    bfs = np.ascontiguousarray(bank_for_state, dtype=np.uint8).reshape(16)
    header = bytearray(64)
    header[0], header[1], header[2] = 1, banks, 16
    st = np.arange(16, dtype=np.uint8)
    a_bank = st % banks
    if banks == 1:
        a_scale = st.astype(np.float32)
    elif codebooks.shape[2] == 4:
        a_scale = (st // banks).astype(np.float32) + 1.0
    else:
        a_scale = 15.0 * ((st // banks).astype(np.float32) + 1.0) / (16 // banks)
    if np.array_equal(lut, a_scale) and np.array_equal(bfs, a_bank):
        header[3] = 1
    header[4:36] = lut.astype("<f2").tobytes()
    header[36:52] = bfs.tobytes()
    return bytes(header) + codebooks.tobytes()


def pack_nvq_jsc(t: NvqJscTensor) -> bytes:
    """mfq/formats/nvq.py:644-716."""
    out = int(t.neuron_scale.size)
    return b"".join([
        _NVQ_HDR.pack(b"NVQ1", _NVQ_CODEBOOK_ID[t.codebook] | 0x20, 4, 24, t.axis, t.neuron_len, len(t.shape)),
        struct.pack(f"<{len(t.shape)}q", *t.shape), struct.pack("<I", out),
        pack_jsc_tables(t.scale_lut, t.bank_for_state, t.codebooks),
        np.ascontiguousarray(t.neuron_scale, dtype=np.float16).tobytes(),
        pack_bits(t.state, 4), pack_bits(t.indices, _NVQ_INDEX_BITS[t.codebook]), pack_bits(t.signs, 7)])


def pack_nvq_plain(t: NvqTensor) -> bytes:
    """mfq/formats/nvq.py:603-641 (non-JSC NVQ2/NVQ3 with the built-in grid)."""
    out = int(t.neuron_scale.size)
    cid = _NVQ_CODEBOOK_ID[t.codebook] | (0x80 if t.sign_mode == "index_parity" else 0)
    return b"".join([
        _NVQ_HDR.pack(b"NVQ1", cid, t.sub_bits, t.groupsize, t.axis, t.neuron_len, len(t.shape)),
        struct.pack(f"<{len(t.shape)}q", *t.shape), struct.pack("<I", out),
        np.ascontiguousarray(t.neuron_scale, dtype=np.float16).tobytes(),
        pack_bits(t.sub_scale, t.sub_bits), pack_bits(t.indices, _NVQ_INDEX_BITS[t.codebook]),
        pack_bits(t.signs, 7)])


def unpack_nvq(blob):
    """mfq/formats/nvq.py:719-820."""
    blob = bytes(blob)
    magic, enc_id, sub_bits, gs, axis, neuron_len, ndim = _NVQ_HDR.unpack_from(blob)
    if magic not in (b"NVQ1", b"NIQ1"):
        raise ValueError(f"invalid NVQ magic: {magic!r}")
    sign_mode = "index_parity" if enc_id & 0x80 else "even"
    custom, is_jsc = bool(enc_id & 0x40), bool(enc_id & 0x20)
    cid = enc_id & ~0xE0
    if cid not in _NVQ_ID_CODEBOOK:
        raise ValueError(f"unknown NVQ codebook id: {cid}")
    codebook = _NVQ_ID_CODEBOOK[cid]
    off = _NVQ_HDR.size
    shape = struct.unpack_from(f"<{ndim}q", blob, off)
    off += 8 * ndim
    out = struct.unpack_from("<I", blob, off)[0]
    off += 4
    vs, ib = nvq_vector_size(codebook), _NVQ_INDEX_BITS[codebook]
    ng, nvec, nsign = math.ceil(neuron_len / gs), math.ceil(neuron_len / vs), math.ceil(neuron_len / 8)
    if is_jsc:
        if custom or sign_mode != "even" or gs != 24 or sub_bits != 4:
            raise ValueError("invalid NVQ-JSC profile flags")
        if len(blob) < off + 64:
            raise ValueError("truncated NVQ-JSC metadata header")
        hdr = blob[off:off + 64]
        version, banks, states, mode = hdr[0], hdr[1], hdr[2], hdr[3]
        if version != 1 or banks not in (1, 2, 4) or states != 16 or mode not in (0, 1) or any(hdr[52:64]):
            raise ValueError("invalid NVQ-JSC metadata")
        lut = np.frombuffer(hdr[4:36], dtype="<f2").astype(np.float32)
        bfs = np.frombuffer(hdr[36:52], dtype=np.uint8).copy()
        entries = 1 << ib
        cb_bytes = banks * entries * vs
        off += 64
        if len(blob) < off + cb_bytes:
            raise ValueError("truncated NVQ-JSC codebook banks")
        cbs = np.frombuffer(blob, dtype=np.int8, count=cb_bytes, offset=off).copy().reshape(banks, entries, vs)
        off += cb_bytes
        if np.any(cbs < 0) or np.any(bfs >= banks) or not np.isfinite(lut).all() or np.any(lut < 0):
            raise ValueError("invalid NVQ-JSC tables")
        if off + 2 * out > len(blob):
            raise ValueError("truncated NVQ-JSC neuron anchors")
        ns = np.frombuffer(blob, dtype=np.float16, count=out, offset=off).astype(np.float32)
        off += 2 * out
        state, off = unpack_bits(blob, off, out * ng, 4)
        idx, off = unpack_bits(blob, off, out * nvec, ib)
        sg, off = unpack_bits(blob, off, out * nsign, 7)
        if off != len(blob):
            raise ValueError(f"invalid NVQ-JSC blob tail: consumed={off}, size={len(blob)}")
        return NvqJscTensor(codebook, tuple(shape), neuron_len, ns, lut, bfs, state.reshape(out, ng),
                            idx.reshape(out, nvec).astype(np.uint16), sg.reshape(out, nsign), cbs, axis)
    cbk = None
    if custom:
        n = (1 << ib) * 2
        raw = np.frombuffer(blob, dtype="<u2", count=n // 2, offset=off)
        digit_bits = 2 if vs == 8 else 3
        shifts = (digit_bits * np.arange(vs, dtype=np.uint16))[None, :]
        cbk = (2 * ((raw[:, None] >> shifts) & ((1 << digit_bits) - 1)) + 1).astype(np.int8)
        off += n
    ns = np.frombuffer(blob, dtype=np.float16, count=out, offset=off).astype(np.float32)
    off += 2 * out
    ss, off = unpack_bits(blob, off, out * ng, sub_bits)
    idx, off = unpack_bits(blob, off, out * nvec, ib)
    sg, off = unpack_bits(blob, off, out * nsign, 7)
    if off != len(blob):
        raise ValueError(f"invalid NVQ blob tail: consumed={off}, size={len(blob)}")
    return NvqTensor(codebook, tuple(shape), neuron_len, ns, ss.reshape(out, ng),
                     idx.reshape(out, nvec).astype(np.uint16), sg.reshape(out, nsign), axis, gs, sub_bits,
                     sign_mode, cbk)


def _nvq_signs(masks, neuron_len, index_parity_bank=None):
    """Bits 0..6 from the mask, bit 7 = parity of the seven (mfq/quantize/nvq_jsc.py:1066-1071)."""
    masks = np.asarray(masks, dtype=np.uint8)
    lower = ((masks[..., None] >> np.arange(7, dtype=np.uint8)) & 1).astype(np.uint8)
    last = (lower.sum(axis=-1, keepdims=True) & 1).astype(np.uint8)
    if index_parity_bank is not None:
        last = last ^ index_parity_bank[..., None]
    negative = np.concatenate([lower, last], axis=-1)
    sign = np.where(negative != 0, -1.0, 1.0).astype(np.float32)
    return sign.reshape(masks.shape[0], -1)[:, :neuron_len]


def dequantize_nvq_jsc(t: NvqJscTensor) -> np.ndarray:
    """mfq/quantize/nvq_jsc.py:1053-1079: f32(mag) * sign * fl(anchor * lut[state])."""
    out, neuron_len = t.shape
    gs, vs = 24, nvq_vector_size(t.codebook)
    ng = math.ceil(neuron_len / gs)
    vpg = gs // vs
    idx = np.zeros((out, ng * vpg), dtype=np.uint16)
    idx[:, : t.indices.shape[1]] = t.indices
    group_bank = t.bank_for_state[t.state]
    vector_bank = np.repeat(group_bank, vpg, axis=1)
    magnitude = t.codebooks[vector_bank, idx].reshape(out, -1)[:, :neuron_len]
    sign = _nvq_signs(t.signs, neuron_len)
    group_scale = t.neuron_scale.astype(np.float32)[:, None] * t.scale_lut[t.state].astype(np.float32)
    scale = np.repeat(group_scale, gs, axis=1)[:, :neuron_len]
    return magnitude.astype(np.float32) * sign * scale


def dequantize_nvq(t: NvqTensor) -> np.ndarray:
    """mfq/quantize/nvq_quant.py:608-626: (table[idx] * sign) * (anchor * sub_scale)."""
    out = t.neuron_scale.size
    table = (t.custom_codebook if t.custom_codebook is not None else nvq_grid(t.codebook)).astype(np.float32)
    magnitude = table[t.indices].reshape(out, -1)[:, : t.neuron_len]
    bank = None
    if t.sign_mode == "index_parity":
        bank = ((np.asarray(t.indices, dtype=np.uint16) >> 7) & 1).astype(np.uint8)
    sign = _nvq_signs(t.signs, t.neuron_len, bank)
    group_scale = t.neuron_scale.astype(np.float32)[:, None] * t.sub_scale.astype(np.float32)
    scale = np.repeat(group_scale, t.groupsize, axis=1)[:, : t.neuron_len]
    return magnitude * sign * scale


# ---------------------------------------------------------------------------
# NEPQ  (mfq/formats/nepq.py): NEPQ1-S / NEPQ1-L (ternary tables) and NEPQ0-S / NEPQ0-L (the product tables of NPQ0)
# ---------------------------------------------------------------------------
_NEPQ_HDR = struct.Struct("<4sBBBBIIIIIQ")
#              label: (profile_id, state_bits, index_bits, aux_bits, table_bytes)
NEPQ_SPECS = {"NEPQ0-S": (0, 2, 6, 0, 320), "NEPQ0-L": (1, 3, 7, 0, 832),
              "NEPQ1-S": (2, 4, 9, 1, 2048), "NEPQ1-L": (3, 3, 11, 1, 4096)}
_NEPQ_BY_ID = {v[0]: k for k, v in NEPQ_SPECS.items()}


@dataclass
class NepqTensor:
    label: str
    shape: tuple              # (experts, out, K)
    neuron_scale: np.ndarray  # (E, out) f32
    state: np.ndarray         # (E, out, ng)
    indices: np.ndarray       # (E, out, nvec) u16
    aux: np.ndarray           # (E, out, ng)
    bank_ids: np.ndarray      # (E, out, nsuper) u8
    table_payloads: np.ndarray  # (banks, table_bytes) u8
    rotation_block: int = 0
    rotation_seed: int = 0


def nepq_payload_nbytes(label, n_experts, out, K, bank_count):
    """mfq/formats/nepq.py:53-75."""
    _, sb, ib, ab, tb = NEPQ_SPECS[label]
    rows = n_experts * out
    ng, nvec = math.ceil(K / 24), K // 8
    nsuper = math.ceil(ng / 4)
    pk = lambda c, b: (c * b + 7) // 8 if b else 0
    return bank_count * tb + 2 * rows + pk(rows * ng, sb) + pk(rows * nvec, ib) + pk(rows * ng, ab) + rows * nsuper


def unpack_ternary_table(payload: bytes) -> np.ndarray:
    """2 bits per digit, digit = code + 1, 8 digits per u16 (mfq/formats/nvq1_l.py:121-130)."""
    enc = np.frombuffer(payload, dtype="<u2")
    digits = (enc[:, None] >> (2 * np.arange(8, dtype=np.uint16))[None, :]) & 3
    if np.any(digits > 2):
        raise ValueError("non-ternary digit in packed table")
    return digits.astype(np.int8) - 1


def pack_ternary_table(codes: np.ndarray) -> bytes:
    d = (np.asarray(codes, dtype=np.int16) + 1).astype(np.uint16)
    return np.bitwise_or.reduce(d << (2 * np.arange(8, dtype=np.uint16))[None, :], axis=1).astype("<u2").tobytes()


def pack_nepq(t: NepqTensor) -> bytes:
    """mfq/formats/nepq.py:368-399."""
    pid, sb, ib, ab, tb = NEPQ_SPECS[t.label]
    E, out, K = t.shape
    return b"".join([
        _NEPQ_HDR.pack(b"NEP1", 1, pid, 4, 1 if t.rotation_block else 0, E, out, K,
                       int(t.table_payloads.shape[0]), int(t.rotation_block), int(t.rotation_seed)),
        np.ascontiguousarray(t.table_payloads, dtype=np.uint8).tobytes(),
        np.ascontiguousarray(t.neuron_scale, dtype="<f2").tobytes(),
        pack_bits(t.state, sb), pack_bits(t.indices, ib), pack_bits(t.aux, ab) if ab else b"",
        np.ascontiguousarray(t.bank_ids, dtype=np.uint8).tobytes()])


def unpack_nepq(blob) -> NepqTensor:
    """mfq/formats/nepq.py:402-474."""
    blob = bytes(blob)
    if len(blob) < _NEPQ_HDR.size:
        raise ValueError("truncated NEPQ header")
    magic, ver, pid, gps, flags, E, out, K, banks, rblock, rseed = _NEPQ_HDR.unpack_from(blob)
    if magic != b"NEP1" or ver != 1 or pid not in _NEPQ_BY_ID or gps != 4:
        raise ValueError("invalid or unsupported NEPQ header")
    if flags & ~1 or bool(flags & 1) != bool(rblock):
        raise ValueError("inconsistent NEPQ flags")
    if E <= 0 or out <= 0 or K <= 0 or K % 8 or not 1 <= banks <= 256:
        raise ValueError("invalid NEPQ dimensions")
    label = _NEPQ_BY_ID[pid]
    _, sb, ib, ab, tb = NEPQ_SPECS[label]
    if tb is None:
        raise NotImplementedError(f"{label} tables are outside the oracle's scope")
    rows = E * out
    ng, nvec = math.ceil(K / 24), K // 8
    nsuper = math.ceil(ng / 4)
    off = _NEPQ_HDR.size
    if off + banks * tb > len(blob):
        raise ValueError("truncated NEPQ table pool")
    tables = np.frombuffer(blob, dtype=np.uint8, count=banks * tb, offset=off).copy().reshape(banks, tb)
    off += banks * tb
    if off + 2 * rows > len(blob):
        raise ValueError("truncated NEPQ neuron anchors")
    ns = np.frombuffer(blob, dtype="<f2", count=rows, offset=off).astype(np.float32).reshape(E, out)
    off += 2 * rows
    state, off = unpack_bits(blob, off, rows * ng, sb)
    idx, off = unpack_bits(blob, off, rows * nvec, ib)
    aux, off = unpack_bits(blob, off, rows * ng, ab)
    if off + rows * nsuper > len(blob):
        raise ValueError("truncated NEPQ bank selectors")
    bank_ids = np.frombuffer(blob, dtype=np.uint8, count=rows * nsuper, offset=off).copy().reshape(E, out, nsuper)
    off += rows * nsuper
    if off != len(blob):
        raise ValueError(f"invalid NEPQ tail: consumed={off}, size={len(blob)}")
    if np.any(bank_ids >= banks):
        raise ValueError("NEPQ bank ID exceeds the table pool")
    for tbl in tables:   # table validity (mfq/formats/nepq.py:270-290)
        if label.startswith("NEPQ1"):
            unpack_ternary_table(tbl.tobytes())
        else:
            _npq0_tables(tbl.tobytes(), "NPQ0" + label[5:])
    return NepqTensor(label, (E, out, K), ns, state.reshape(E, out, ng), idx.reshape(E, out, nvec).astype(np.uint16),
                      aux.reshape(E, out, ng) if ab else np.zeros(0, dtype=np.uint8), bank_ids, tables, rblock, rseed)


def dequantize_nepq(t: NepqTensor) -> np.ndarray:
    """mfq/formats/nepq.py:492-544: fl(anchor*state) * (code + (-/+)delta), code+delta exact."""
    E, out, K = t.shape
    rows = E * out
    ng, nvec = math.ceil(K / 24), K // 8
    state = t.state.reshape(rows, ng).astype(np.uint8)
    idx = t.indices.reshape(rows, nvec).astype(np.int64)
    anchors = t.neuron_scale.reshape(rows).astype(np.float32)
    bank_ids = t.bank_ids.reshape(rows, -1)
    group_bank = np.repeat(bank_ids, 4, axis=1)[:, :ng]
    vector_bank = np.repeat(group_bank, 3, axis=1)[:, :nvec].astype(np.int64)
    aux = t.aux.reshape(rows, ng).astype(np.uint8) if NEPQ_SPECS[t.label][3] else None   # NEPQ0 stores no aux stream
    if t.label == "NEPQ1-S":
        tables = np.stack([np.stack([unpack_ternary_table(p.tobytes()[:1024]),
                                     unpack_ternary_table(p.tobytes()[1024:])]) for p in t.table_payloads])
        vector_aux = np.repeat(aux, 3, axis=1)[:, :nvec].astype(np.int64)
        code = tables[vector_bank, vector_aux, idx]
        delta = np.where(aux != 0, -0.15625, 0.15625).astype(np.float32)
    elif t.label == "NEPQ1-L":
        tables = np.stack([unpack_ternary_table(p.tobytes()) for p in t.table_payloads])
        code = tables[vector_bank, idx]
        delta = np.where(aux != 0, -0.125, 0.125).astype(np.float32)
    else:
        # the product form: the bank id of a neuron's 96 weights picks scale LUT and sub-codebooks, the group state the
        # entry of each (mfq/formats/nepq.py:509-521)
        tabs = [_npq0_tables(p.tobytes(), "NPQ0" + t.label[5:]) for p in t.table_payloads]
        lut = np.stack([x[0] for x in tabs]); first = np.stack([x[1] for x in tabs]); second = np.stack([x[2] for x in tabs])
        vector_state = np.repeat(state, 3, axis=1)[:, :nvec].astype(np.int64)
        code = np.concatenate((first[vector_bank, vector_state, idx & 7], second[vector_bank, vector_state, idx >> 3]), axis=-1)
        group_scale = anchors[:, None] * lut[group_bank.astype(np.int64), state.astype(np.int64)]
        scale = np.repeat(group_scale, 24, axis=1)[:, :K]
        return (code.reshape(rows, K).astype(np.float32) * scale).astype(np.float32).reshape(t.shape)
    group_scale = anchors[:, None] * state.astype(np.float32)
    scale = np.repeat(group_scale, 24, axis=1)[:, :K]
    bias = np.repeat(delta, 24, axis=1)[:, :K]
    result = scale * (code.reshape(rows, K).astype(np.float32) + bias)
    return result.reshape(t.shape)


# ---------------------------------------------------------------------------
# NINTM container  (mfq/formats/io.py:251-446, mfq/formats/moe.py:83-155)
# ---------------------------------------------------------------------------
@dataclass
class MoePool:
    expert_ids: np.ndarray
    dtype: str
    tensor: object


@dataclass
class NintMoeTensor:
    shape: tuple               # (experts, out_per_expert, K)
    pools: list = field(default_factory=list)


# ---------------------------------------------------------------------------
# NINT8-0 = GGML Q8_0 blocks  (mfq/formats/nint8_zero.py)
# ---------------------------------------------------------------------------
@dataclass
class Nint8ZeroTensor:
    shape: tuple
    axis: int
    scale: np.ndarray   # (out, ng) float16
    q: np.ndarray       # (out, ng, 32) int8
    neuron_len: int

    @property
    def out(self):
        return self.q.shape[0]

    @property
    def ng(self):
        return self.q.shape[1]


_N8Z_HDR = struct.Struct("<4siiI")


def quantize_nint8_zero(weight, axis=0) -> Nint8ZeroTensor:
    """The deterministic GGML Q8_0 rule per block of 32 (mfq/formats/nint8_zero.py:128-155): scale = max|x| / 127 in
    fp32 (stored as fp16), codes = round-half-away(x * (1 / scale_f32)) clipped to +-127; an all-zero block gets
    scale 0 and codes 0."""
    values = np.asarray(weight, dtype=np.float32)
    if not values.ndim or not 0 <= axis < values.ndim:
        raise ValueError("NINT8-0 axis is outside the tensor rank")
    moved = np.moveaxis(values, axis, 0)
    out = moved.shape[0]
    neuron_len = moved.size // out
    if neuron_len <= 0 or neuron_len % 32:
        raise ValueError("NINT8-0 neuron_len must be a positive multiple of 32")
    blocks = np.ascontiguousarray(moved).reshape(out, neuron_len // 32, 32)
    scale = np.max(np.abs(blocks), axis=-1, keepdims=True) / np.float32(127.0)
    inv = np.zeros_like(scale, dtype=np.float32)
    np.divide(np.float32(1.0), scale, out=inv, where=scale != 0)
    norm = blocks * inv
    q = np.clip(np.sign(norm) * np.floor(np.abs(norm) + np.float32(0.5)), -127, 127).astype(np.int8)
    return Nint8ZeroTensor(tuple(int(v) for v in values.shape), axis, scale[..., 0].astype(np.float16), q, neuron_len)


def pack_nint8_zero(t: Nint8ZeroTensor) -> bytes:
    """"<4siiI" header ("NI80", axis, neuron_len, ndim) + shape i64[ndim] + out u32 + ng u32 + 34-byte blocks
    (fp16 scale || 32 int8) in row order (mfq/formats/nint8_zero.py:84-124, 157-164)."""
    head = _N8Z_HDR.pack(b"NI80", t.axis, t.neuron_len, len(t.shape)) + struct.pack(f"<{len(t.shape)}q", *t.shape)
    head += struct.pack("<II", t.out, t.ng)
    blocks = np.empty((t.out, t.ng, 34), dtype=np.uint8)
    blocks[..., :2] = np.ascontiguousarray(t.scale.astype("<f2")).view(np.uint8).reshape(t.out, t.ng, 2)
    blocks[..., 2:] = np.ascontiguousarray(t.q).view(np.uint8)
    return head + blocks.tobytes()


def unpack_nint8_zero(blob) -> Nint8ZeroTensor:
    """mfq/formats/nint8_zero.py:166-205, with its error messages."""
    if len(blob) < _N8Z_HDR.size:
        raise ValueError("truncated NINT8-0 header")
    magic, axis, neuron_len, ndim = _N8Z_HDR.unpack_from(blob, 0)
    if magic != b"NI80":
        raise ValueError(f"invalid NINT8-0 magic: {magic!r}")
    if ndim == 0:
        raise ValueError("NINT8-0 tensor rank cannot be zero")
    off = _N8Z_HDR.size
    if off + 8 * ndim + 8 > len(blob):
        raise ValueError("truncated NINT8-0 shape")
    shape = struct.unpack_from(f"<{ndim}q", blob, off)
    off += 8 * ndim
    out, ng = struct.unpack_from("<II", blob, off)
    off += 8
    expected = out * ng * 34
    if len(blob) - off != expected:
        raise ValueError(f"invalid NINT8-0 block bytes: got {len(blob) - off}, expected {expected}")
    blocks = np.frombuffer(blob, dtype=np.uint8, count=expected, offset=off).reshape(out, ng, 34)
    scale = np.ascontiguousarray(blocks[..., :2]).view("<f2").reshape(out, ng)
    q = np.ascontiguousarray(blocks[..., 2:]).view(np.int8)
    if not 0 <= axis < ndim:
        raise ValueError("NINT8-0 axis is outside the tensor rank")
    if neuron_len <= 0 or neuron_len % 32:
        raise ValueError("NINT8-0 neuron_len must be a positive multiple of 32")
    if shape[axis] != out or ng != neuron_len // 32 or math.prod(shape) != out * neuron_len:
        raise ValueError("NINT8-0 dimensions disagree with the logical shape")
    return Nint8ZeroTensor(tuple(int(v) for v in shape), int(axis), scale, q, int(neuron_len))


def dequantize_nint8_zero(t: Nint8ZeroTensor) -> np.ndarray:
    """float32 scale * float32 code, [out, neuron_len] (mfq/formats/nint8_zero.py:208-218)."""
    return (t.scale.astype(np.float32)[..., None] * t.q.astype(np.float32)).reshape(t.out, t.neuron_len)


# ---------------------------------------------------------------------------
# The 1-bit families: NVQ1-L / NVQ1-S (8-dimensional ternary codebooks, an integer relative scale and a delta sign
# per group of 24) and NPQ0-L / NPQ0-S (two 4-dimensional int8 sub-codebooks chosen by a per-group state that also
# selects the relative scale).  One fp16 anchor per neuron; every stream is packed across the whole tensor.
# (mfq/formats/nvq1_l.py:130-330, nvq1_s.py:168-347, npq0_l.py:20-415, npq0_s.py:18-406)
# ---------------------------------------------------------------------------
_LOWBIT_HDR = struct.Struct("<4sBBHiiI")      # magic, profile / version, state bits, groupsize, axis, neuron_len, ndim
# label: magic, header byte, state bits, index bits, states, first / second sub-codebook entries, table version
LOWBIT_SPECS = {
    "NVQ1-L": dict(magic=b"NQ1L", index_bits=11, entries=2048, banks=1, delta=0.125),
    "NVQ1-S": dict(magic=b"NQ1S", version=1, state_bits=4, index_bits=9, entries=512, banks=2, delta=0.15625),
    "NPQ0-L": dict(magic=b"NPQL", version=1, state_bits=3, index_bits=7, states=8, second=16, table_version=1),
    "NPQ0-S": dict(magic=b"NPQS", version=2, state_bits=2, index_bits=6, states=4, second=8, table_version=2),
}


@dataclass
class Nvq1Tensor:
    """NVQ1-L (codebook None: the built-in IQ1_S grid, else a custom [2048, 8] ternary table; state_bits 3 or 4) and
    NVQ1-S (codebook [2, 512, 8]: the group's delta sign also selects the bank)."""
    label: str
    shape: tuple
    axis: int
    neuron_len: int
    state_bits: int
    neuron_scale: np.ndarray      # float32 [out], fp16-representable
    sub_scale: np.ndarray         # [out, ng] integers below 2^state_bits
    indices: np.ndarray           # [out, nvec]
    delta_sign: np.ndarray        # [out, ng] 0 / 1
    codebook: np.ndarray | None = None


@dataclass
class Npq0Tensor:
    label: str
    shape: tuple
    axis: int
    neuron_len: int
    neuron_scale: np.ndarray      # float32 [out]
    scale_lut: np.ndarray         # float32 [states], fp16-representable
    state: np.ndarray             # [out, ng]
    indices: np.ndarray           # [out, nvec]: first index in the low 3 bits, second above
    first_codebooks: np.ndarray   # int8 [states, 8, 4]
    second_codebooks: np.ndarray  # int8 [states, 8 or 16, 4]


def iq1s_grid() -> np.ndarray:
    """The 2048 x 8 ternary grid NVQ1-L uses when its blob carries none (mfq/formats/nvq1_l.py:78-94)."""
    return unpack_ternary_table((_DATA / "iq1s_2048.bin").read_bytes())


def nvq1s_default_banks() -> np.ndarray:
    """The [2, 512, 8] table NVQ1-S writes when a tensor brings none (mfq/formats/nvq1_s.py:126-137)."""
    raw = (_DATA / "nvq1s_banks.bin").read_bytes()
    return np.stack([unpack_ternary_table(raw[:1024]), unpack_ternary_table(raw[1024:])])


def _lowbit_counts(label, neuron_len):
    ng = -(-neuron_len // 24)
    nvec = -(-neuron_len // 8) if label == "NVQ1-L" else neuron_len // 8
    return ng, nvec


def pack_nvq1(t: Nvq1Tensor) -> bytes:
    """mfq/formats/nvq1_l.py:234-284 (profile 1: built-in grid, 2: table in the blob) and nvq1_s.py:262-290."""
    sp = LOWBIT_SPECS[t.label]
    out = t.neuron_scale.size
    if t.label == "NVQ1-L":
        head = _LOWBIT_HDR.pack(sp["magic"], 2 if t.codebook is not None else 1, t.state_bits, 24, t.axis, t.neuron_len,
                                len(t.shape))
        table = pack_ternary_table(t.codebook) if t.codebook is not None else b""
    else:
        if t.neuron_len % 8:
            raise ValueError("NVQ1-S neuron length must be divisible by 8")
        head = _LOWBIT_HDR.pack(sp["magic"], sp["version"], 4, 24, t.axis, t.neuron_len, len(t.shape))
        cb = nvq1s_default_banks() if t.codebook is None else np.asarray(t.codebook)
        table = pack_ternary_table(cb[0]) + pack_ternary_table(cb[1])
    return b"".join([head, struct.pack(f"<{len(t.shape)}q", *t.shape), struct.pack("<I", out), table,
                     np.ascontiguousarray(t.neuron_scale, dtype="<f2").tobytes(), pack_bits(t.sub_scale, t.state_bits),
                     pack_bits(t.indices, sp["index_bits"]), pack_bits(t.delta_sign, 1)])


def _lowbit_head(blob, label):
    sp = LOWBIT_SPECS[label]
    if len(blob) < _LOWBIT_HDR.size:
        raise ValueError(f"truncated {label} header")
    magic, ver, sbits, gs, axis, neuron_len, ndim = _LOWBIT_HDR.unpack_from(blob)
    if magic != sp["magic"]:
        raise ValueError(f"invalid {label} magic: {magic!r}")
    if ndim <= 0 or neuron_len <= 0 or gs != 24:
        raise ValueError(f"invalid {label} dimensions")
    off = _LOWBIT_HDR.size
    if off + 8 * ndim + 4 > len(blob):
        raise ValueError(f"truncated {label} shape")
    shape = tuple(struct.unpack_from(f"<{ndim}q", blob, off))
    off += 8 * ndim
    out = struct.unpack_from("<I", blob, off)[0]
    return ver, sbits, axis, neuron_len, shape, out, off + 4


def unpack_nvq1(blob, label) -> Nvq1Tensor:
    """mfq/formats/nvq1_l.py:287-345, nvq1_s.py:293-347."""
    sp = LOWBIT_SPECS[label]
    ver, sbits, axis, K, shape, out, off = _lowbit_head(blob, label)
    codebook = None
    if label == "NVQ1-L":
        if ver not in (1, 2):
            raise ValueError(f"unsupported NVQ1-L profile: {ver}")
        if not 1 <= sbits <= 8:
            raise ValueError("NVQ1-L sub_bits must be in [1, 8]")
        if ver == 2:
            if off + 4096 > len(blob):
                raise ValueError("truncated NVQ1-L custom codebook")
            codebook = unpack_ternary_table(bytes(blob[off:off + 4096]))
            off += 4096
    else:
        if ver != sp["version"] or sbits != 4 or K % 8:
            raise ValueError("unsupported NVQ1-S stream profile")
        if off + 2048 > len(blob):
            raise ValueError("truncated NVQ1-S codebook")
        codebook = np.stack([unpack_ternary_table(bytes(blob[off:off + 1024])),
                             unpack_ternary_table(bytes(blob[off + 1024:off + 2048]))])
        off += 2048
    ng, nvec = _lowbit_counts(label, K)
    if off + 2 * out > len(blob):
        raise ValueError(f"truncated {label} neuron anchors")
    ns = np.frombuffer(blob, dtype="<f2", count=out, offset=off).astype(np.float32)
    off += 2 * out
    sub, off = unpack_bits(blob, off, out * ng, sbits)
    idx, off = unpack_bits(blob, off, out * nvec, sp["index_bits"])
    dsg, off = unpack_bits(blob, off, out * ng, 1)
    if off != len(blob):
        raise ValueError(f"invalid {label} blob tail: consumed={off}, size={len(blob)}")
    return Nvq1Tensor(label, shape, axis, K, sbits, ns, sub.reshape(out, ng), idx.reshape(out, nvec).astype(np.uint16),
                      dsg.reshape(out, ng), codebook)


def dequantize_nvq1(t: Nvq1Tensor) -> np.ndarray:
    """w = fl(fl(anchor * sub_scale) * (code + delta)), delta = -/+ 1/8 (L) or 5/32 (S) by the group's sign bit, which
    for NVQ1-S also picks the bank of all three vectors of the group (mfq/quantize/nvq1_l_quant.py:384-414,
    nvq1_s_quant.py:142-174).  code + delta is exact in fp32."""
    sp = LOWBIT_SPECS[t.label]
    out, K = t.neuron_scale.size, t.neuron_len
    idx = np.asarray(t.indices, dtype=np.int64)
    if t.label == "NVQ1-L":
        table = iq1s_grid() if t.codebook is None else np.asarray(t.codebook, dtype=np.int8)
        code = table[idx]
    else:
        table = nvq1s_default_banks() if t.codebook is None else np.asarray(t.codebook, dtype=np.int8)
        bank = np.repeat(np.asarray(t.delta_sign, dtype=np.int64), 3, axis=1)[:, : idx.shape[1]]
        code = table[bank, idx]
    code = code.reshape(out, -1)[:, :K].astype(np.float32)
    d = np.float32(sp["delta"])
    delta = np.repeat(np.where(np.asarray(t.delta_sign) != 0, -d, d).astype(np.float32), 24, axis=1)[:, :K]
    scale = np.repeat(t.neuron_scale.astype(np.float32)[:, None] * np.asarray(t.sub_scale).astype(np.float32), 24, axis=1)[:, :K]
    return (scale * (code + delta)).astype(np.float32)


def _npq0_tables(payload: bytes, label: str):
    """One NPQ0 table: (scale LUT float32 [states], first int8 [states, 8, 4], second int8 [states, 8 or 16, 4]), with the
    header checks of unpack_npq0_l_tables / unpack_npq0_s_tables (mfq/formats/npq0_l.py:136-185, npq0_s.py:134-183)."""
    sp = LOWBIT_SPECS[label]
    S, E2 = sp["states"], sp["second"]
    if len(payload) < 64 + S * 32 + S * E2 * 4:
        raise ValueError(f"truncated {label} product tables")
    head = payload[:64]
    if tuple(head[:6]) != (sp["table_version"], S, 3, sp["index_bits"] - 3, 24, 8):
        raise ValueError(f"unsupported {label} table profile")
    if any(head[6:8]) or any(head[8 + 2 * S:64]):
        raise ValueError(f"{label} reserved table bytes must be zero")
    lut = np.frombuffer(head, dtype="<f2", count=S, offset=8).astype(np.float32)
    if not np.isfinite(lut).all() or np.any(lut < 0) or float(lut.max()) <= 0:
        raise ValueError(f"{label} scale LUT must be finite, non-negative, and nonzero")
    first = np.frombuffer(payload, dtype=np.int8, count=S * 32, offset=64).reshape(S, 8, 4).copy()
    second = np.frombuffer(payload, dtype=np.int8, count=S * E2 * 4, offset=64 + S * 32).reshape(S, E2, 4).copy()
    return lut, first, second


def pack_npq0_tables(t: Npq0Tensor) -> bytes:
    """64-byte header (version, states, first / second index bits, 24, 8; fp16 scale LUT at byte 8), then the int8
    sub-codebooks (mfq/formats/npq0_l.py:112-133, npq0_s.py:110-131)."""
    sp = LOWBIT_SPECS[t.label]
    head = bytearray(64)
    head[0:6] = bytes([sp["table_version"], sp["states"], 3, sp["index_bits"] - 3, 24, 8])
    head[8:8 + 2 * sp["states"]] = np.ascontiguousarray(t.scale_lut, dtype="<f2").tobytes()
    return bytes(head) + np.ascontiguousarray(t.first_codebooks, dtype=np.int8).tobytes() + \
        np.ascontiguousarray(t.second_codebooks, dtype=np.int8).tobytes()


def pack_npq0(t: Npq0Tensor) -> bytes:
    """mfq/formats/npq0_l.py:326-351, npq0_s.py:320-345."""
    sp = LOWBIT_SPECS[t.label]
    if t.neuron_len % 8:
        raise ValueError(f"{t.label} neuron length must be divisible by 8")
    return b"".join([_LOWBIT_HDR.pack(sp["magic"], sp["version"], sp["state_bits"], 24, t.axis, t.neuron_len, len(t.shape)),
                     struct.pack(f"<{len(t.shape)}q", *t.shape), struct.pack("<I", t.neuron_scale.size), pack_npq0_tables(t),
                     np.ascontiguousarray(t.neuron_scale, dtype="<f2").tobytes(), pack_bits(t.state, sp["state_bits"]),
                     pack_bits(t.indices, sp["index_bits"])])


def unpack_npq0(blob, label) -> Npq0Tensor:
    """mfq/formats/npq0_l.py:354-415 (tables :136-185), npq0_s.py:348-406 (tables :134-183)."""
    sp = LOWBIT_SPECS[label]
    ver, sbits, axis, K, shape, out, off = _lowbit_head(blob, label)
    if ver != sp["version"] or sbits != sp["state_bits"] or K % 8:
        raise ValueError(f"unsupported {label} stream profile")
    S, E2 = sp["states"], sp["second"]
    tb = 64 + S * 8 * 4 + S * E2 * 4
    if off + tb > len(blob):
        raise ValueError(f"truncated {label} product tables")
    head = bytes(blob[off:off + 64])
    if tuple(head[:6]) != (sp["table_version"], S, 3, sp["index_bits"] - 3, 24, 8):
        raise ValueError(f"unsupported {label} table profile")
    if any(head[6:8]) or any(head[8 + 2 * S:64]):
        raise ValueError(f"{label} reserved table bytes must be zero")
    lut = np.frombuffer(head, dtype="<f2", count=S, offset=8).astype(np.float32)
    if not np.isfinite(lut).all() or np.any(lut < 0) or float(lut.max()) <= 0:
        raise ValueError(f"{label} scale LUT must be finite, non-negative, and nonzero")
    first = np.frombuffer(blob, dtype=np.int8, count=S * 32, offset=off + 64).reshape(S, 8, 4).copy()
    second = np.frombuffer(blob, dtype=np.int8, count=S * E2 * 4, offset=off + 64 + S * 32).reshape(S, E2, 4).copy()
    off += tb
    ng, nvec = _lowbit_counts(label, K)
    if off + 2 * out > len(blob):
        raise ValueError(f"truncated {label} neuron anchors")
    ns = np.frombuffer(blob, dtype="<f2", count=out, offset=off).astype(np.float32)
    off += 2 * out
    state, off = unpack_bits(blob, off, out * ng, sbits)
    idx, off = unpack_bits(blob, off, out * nvec, sp["index_bits"])
    if off != len(blob):
        raise ValueError(f"invalid {label} blob tail: consumed={off}, size={len(blob)}")
    return Npq0Tensor(label, shape, axis, K, ns, lut, state.reshape(out, ng), idx.reshape(out, nvec), first, second)


def dequantize_npq0(t: Npq0Tensor) -> np.ndarray:
    """w = int8 code * fl(anchor * scale_lut[state]); a vector's first four weights come from first[state][index & 7],
    the last four from second[state][index >> 3] (mfq/quantize/npq0_l.py:766-790, npq0_s.py:812-836)."""
    out, K = t.neuron_scale.size, t.neuron_len
    idx = np.asarray(t.indices, dtype=np.int64)
    vs = np.repeat(np.asarray(t.state, dtype=np.int64), 3, axis=1)[:, : idx.shape[1]]
    code = np.concatenate((np.asarray(t.first_codebooks, dtype=np.int8)[vs, idx & 7],
                           np.asarray(t.second_codebooks, dtype=np.int8)[vs, idx >> 3]), axis=-1)
    scale = np.repeat(t.neuron_scale.astype(np.float32)[:, None] * np.asarray(t.scale_lut, dtype=np.float32)[np.asarray(t.state)],
                      24, axis=1)[:, :K]
    return (code.reshape(out, K).astype(np.float32) * scale).astype(np.float32)


# ---------------------------------------------------------------------------
# OCP MX payloads: MXFP4 (E2M1 nibbles, one E8M0 scale per 32 columns of a row) and MXFP8 (E4M3FN bytes, one E8M0
# scale per 128 x 128 block).  Container mfq/formats/mx.py:20-182.
# ---------------------------------------------------------------------------
MX_HEADER = struct.Struct("<4sBBHQQQQQQ")  # magic, version, kind, reserved, shape, storage shape, scale shape
MX_KINDS = {"MXFP4": 4, "MXFP8": 8}
FP4_E2M1 = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=np.float32)  # cpp_runtime/mfq_decode.cpp:1926-1928


@dataclass
class MxTensor:
    dtype: str           # "MXFP4" | "MXFP8"
    shape: tuple         # (rows, columns)
    values: np.ndarray   # uint8: [rows, columns / 2] (low nibble = even column) or [rows, columns]
    scales: np.ndarray   # uint8 E8M0: [rows, columns / 32] or [ceil(rows / 128), columns / 128]


def mx_shapes(dtype: str, shape):
    """(storage shape, scale shape) of a logical [rows, columns] matrix (validate_mx_shapes, mx.py:65-117)."""
    if dtype not in MX_KINDS:
        raise ValueError(f"unsupported MX dtype: {dtype}")
    if len(shape) != 2:
        raise ValueError("MFQ MX tensors must be rank-2 matrices")
    rows, cols = int(shape[0]), int(shape[1])
    if rows <= 0 or cols <= 0:
        raise ValueError(f"invalid MX logical shape: {tuple(shape)}")
    if dtype == "MXFP4":
        if cols % 32:
            raise ValueError("MXFP4 columns must be divisible by 32")
        return (rows, cols // 2), (rows, cols // 32)
    if cols % 128:
        raise ValueError("MXFP8 columns must be divisible by 128")
    return (rows, cols), ((rows + 127) // 128, cols // 128)


def pack_mx(t: MxTensor) -> bytes:
    """mx.py:120-151: header, value bytes, scale bytes."""
    storage, scale = mx_shapes(t.dtype, t.shape)
    values = np.ascontiguousarray(t.values, dtype=np.uint8)
    scales = np.ascontiguousarray(t.scales, dtype=np.uint8)
    if values.shape != storage:
        raise ValueError(f"{t.dtype} storage shape {values.shape} != {storage}")
    if scales.shape != scale:
        raise ValueError(f"{t.dtype} scale shape {scales.shape} != {scale}")
    head = MX_HEADER.pack(b"MXT1", 1, MX_KINDS[t.dtype], 0, *map(int, t.shape), *storage, *scale)
    return head + values.tobytes() + scales.tobytes()


def unpack_mx(dtype: str, blob) -> MxTensor:
    """mx.py:154-182."""
    blob = bytes(blob)
    if len(blob) < MX_HEADER.size:
        raise ValueError("truncated MFQ MX tensor header")
    magic, version, kind, reserved, *dims = MX_HEADER.unpack_from(blob)
    if magic != b"MXT1" or version != 1 or kind != MX_KINDS.get(dtype) or reserved:
        raise ValueError(f"invalid {dtype} payload header: magic={magic!r}, version={version}, kind={kind}")
    shape = (int(dims[0]), int(dims[1]))
    storage, scale = mx_shapes(dtype, shape)
    if (int(dims[2]), int(dims[3])) != storage:
        raise ValueError(f"{dtype} storage shape {(int(dims[2]), int(dims[3]))} != {storage}")
    if (int(dims[4]), int(dims[5])) != scale:
        raise ValueError(f"{dtype} scale shape {(int(dims[4]), int(dims[5]))} != {scale}")
    nv, ns = storage[0] * storage[1], scale[0] * scale[1]
    if len(blob) != MX_HEADER.size + nv + ns:
        raise ValueError(f"{dtype} payload size {len(blob)} != {MX_HEADER.size + nv + ns}")
    values = np.frombuffer(blob, np.uint8, nv, MX_HEADER.size).reshape(storage).copy()
    scales = np.frombuffer(blob, np.uint8, ns, MX_HEADER.size + nv).reshape(scale).copy()
    return MxTensor(dtype, shape, values, scales)


def decode_e8m0(raw) -> np.ndarray:
    """2^(raw - 127) as fp32, NaN for 255 (mx_matmul.cu:17-28; raw 0 is the subnormal 2^-127)."""
    raw = np.asarray(raw, dtype=np.uint8)
    out = np.ldexp(np.float32(1.0), np.minimum(raw, 254).astype(np.int32) - 127).astype(np.float32)
    return np.where(raw == 255, np.float32(np.nan), out)


def decode_e4m3fn(raw) -> np.ndarray:
    """mx_matmul.cu:30-47: no infinities, exponent 15 with mantissa 7 is NaN, subnormals are multiples of 2^-9."""
    raw = np.asarray(raw, dtype=np.uint8)
    e = ((raw >> 3) & 15).astype(np.int32)
    m = (raw & 7).astype(np.float32)
    mag = np.where(e == 0, m * np.float32(2.0 ** -9), np.ldexp(np.float32(1.0) + m / np.float32(8.0), e - 7)).astype(np.float32)
    mag = np.where((e == 15) & ((raw & 7) == 7), np.float32(np.nan), mag)
    return np.where(raw & 128, -mag, mag).astype(np.float32)


def dequantize_mx(t: MxTensor) -> np.ndarray:
    """fp32 [rows, columns] = element x block scale (one fp32 multiply: exact unless the product leaves fp32's range)."""
    rows, cols = t.shape
    if t.dtype == "MXFP4":
        v = np.asarray(t.values, dtype=np.uint8)
        codes = np.stack([v & 15, v >> 4], axis=-1).reshape(rows, cols)
        mag = FP4_E2M1[codes & 7]
        elem = np.where(codes & 8, -mag, mag).astype(np.float32)
        scale = np.repeat(decode_e8m0(t.scales), 32, axis=1)
    else:
        elem = decode_e4m3fn(t.values)
        scale = np.repeat(np.repeat(decode_e8m0(t.scales), 128, axis=0)[:rows], 128, axis=1)
    with np.errstate(invalid="ignore", over="ignore", under="ignore"):
        return (elem * scale).astype(np.float32)



def tensor_dtype(t) -> str:
    """Public dtype label (mfq/formats/io.py:576-640)."""
    if isinstance(t, NintTensor):
        return f"NINT{t.bits}"
    if isinstance(t, Nint8ZeroTensor):
        return "NINT8-0"
    if isinstance(t, NvqJscTensor):
        return {"e8_256": "NVQ2J", "e8_1024": "NVQ2J-L", "e8_4096": "NVQ2J-XL", "d4_256": "NVQ3J",
                "d4_512": "NVQ3J-512", "d4_1024": "NVQ3J-L"}[t.codebook]
    if isinstance(t, NvqTensor):
        return {"e8_256": "NVQ2", "d4_256": "NVQ3"}[t.codebook]
    if isinstance(t, NepqTensor):
        return t.label
    if isinstance(t, NintMoeTensor):
        return "NINTM"
    if isinstance(t, (Nvq1Tensor, Npq0Tensor)):
        return t.label
    if isinstance(t, MxTensor):
        return t.dtype
    raise TypeError(type(t))


def pack_tensor(t) -> tuple[str, bytes]:
    dt = tensor_dtype(t)
    if isinstance(t, NintTensor):
        return dt, pack_nint(t)
    if isinstance(t, Nint8ZeroTensor):
        return dt, pack_nint8_zero(t)
    if isinstance(t, NvqJscTensor):
        return dt, pack_nvq_jsc(t)
    if isinstance(t, NvqTensor):
        return dt, pack_nvq_plain(t)
    if isinstance(t, NepqTensor):
        return dt, pack_nepq(t)
    if isinstance(t, Nvq1Tensor):
        return dt, pack_nvq1(t)
    if isinstance(t, Npq0Tensor):
        return dt, pack_npq0(t)
    if isinstance(t, MxTensor):
        return dt, pack_mx(t)
    return dt, pack_nint_moe(t)


def unpack_tensor(dtype: str, blob):
    """dtype-string dispatch (mfq/formats/io.py:488-576)."""
    dtype = {"NIQ2": "NVQ2", "NIQ2J": "NVQ2J", "NIQ3": "NVQ3"}.get(dtype, dtype)
    if dtype == "NINTM":
        return unpack_nint_moe(blob)
    if dtype in NEPQ_SPECS:
        t = unpack_nepq(blob)
        if t.label != dtype:
            raise ValueError(f"MFQ dtype/blob mismatch: {dtype} contains {t.label}")
        return t
    if dtype == "NINT8-0":
        return unpack_nint8_zero(blob)
    if dtype in MX_KINDS:
        return unpack_mx(dtype, blob)
    if dtype in ("NVQ1-L", "NVQ1-S"):
        return unpack_nvq1(blob, dtype)
    if dtype in ("NPQ0-L", "NPQ0-S"):
        return unpack_npq0(blob, dtype)
    if dtype.startswith("NINT"):
        return unpack_nint(blob)
    if dtype.startswith("NVQ"):
        t = unpack_nvq(blob)
        if tensor_dtype(t) != dtype:
            raise ValueError(f"MFQ dtype/blob mismatch: {dtype} contains {tensor_dtype(t)}")
        return t
    raise ValueError(f"unsupported dtype {dtype}")


_NIM_HDR = struct.Struct("<4sIIII")
_NIM_POOL = struct.Struct("<IIQQ")


def pack_nint_moe(t: NintMoeTensor, delta: bool = False) -> bytes:
    """mfq/formats/io.py:304-336 (NIM2).  delta: the NID2 form of an expert overlay record (dtype NINTMD): the same
    layout, pools for some experts only (unpack_nint_moe_impl, cpp_runtime/mfq_decode.cpp:2367-2477)."""
    E, out, K = t.shape
    parts = [_NIM_HDR.pack(b"NID2" if delta else b"NIM2", E, out, K, len(t.pools))]
    for p in t.pools:
        ids = np.ascontiguousarray(p.expert_ids, dtype=np.int32).reshape(-1)
        dtype, payload = pack_tensor(p.tensor)
        db = dtype.encode("ascii")
        parts += [_NIM_POOL.pack(ids.size, len(db), len(payload), 0), ids.tobytes(), db, b"", payload]
    return b"".join(parts)


def unpack_nint_moe(blob, allow_partial: bool = False) -> NintMoeTensor:
    """mfq/formats/io.py:382-446 + invariants of mfq/formats/moe.py:98-134.  allow_partial: also take an expert delta
    (magic NID2, pools for some experts only), as unpack_nint_moe_delta does (cpp_runtime/mfq_decode.cpp:2484-2487)."""
    blob = bytes(blob)
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
    pools, owners = [], np.full(E, -1, dtype=np.int32)
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
        dtype = blob[off:off + dlen].decode("ascii")
        off += dlen + rlen
        tensor = unpack_tensor(dtype, blob[off:end])
        off = end
        if np.any(ids < 0) or np.any(ids >= E) or np.unique(ids).size != ids.size or np.any(owners[ids] >= 0):
            raise ValueError("invalid NINTM expert ids")
        owners[ids] = pi
        expect = (n_ids, out, K) if isinstance(tensor, NepqTensor) else (n_ids * out, K)
        if tuple(tensor.shape) != expect:
            raise ValueError(f"NINTM pool {pi} tensor shape {tensor.shape} must be {expect}")
        pools.append(MoePool(ids, dtype, tensor))
    if off != len(blob):
        raise ValueError(f"invalid NINTM tail: {len(blob) - off} extra bytes")
    if np.any(owners < 0) and not allow_partial:
        raise ValueError("NINTM pools do not cover all experts")
    return NintMoeTensor((E, out, K), pools)


def apply_expert_overlay(base: NintMoeTensor, delta: NintMoeTensor) -> NintMoeTensor:
    """load_nint_moe_cpu with an expert overlay (cpp_runtime/mfq_decode.cpp:5752-5774): the delta's pools are appended to
    the base tensor's; an expert then belongs to the last pool that lists it (the dispatch tables are filled pool by
    pool, :3355-3372), which dequantize_expertwise reproduces by assigning in pool order."""
    if tuple(delta.shape) != tuple(base.shape):
        raise ValueError("expert overlay shape mismatch")
    return NintMoeTensor(tuple(base.shape), list(base.pools) + list(delta.pools))


def dequantize_tensor(t) -> np.ndarray:
    if isinstance(t, NintTensor):
        return dequantize_nint(t)
    if isinstance(t, Nint8ZeroTensor):
        return dequantize_nint8_zero(t)
    if isinstance(t, NvqJscTensor):
        return dequantize_nvq_jsc(t)
    if isinstance(t, NvqTensor):
        return dequantize_nvq(t)
    if isinstance(t, NepqTensor):
        return dequantize_nepq(t)
    if isinstance(t, Nvq1Tensor):
        return dequantize_nvq1(t)
    if isinstance(t, Npq0Tensor):
        return dequantize_npq0(t)
    if isinstance(t, MxTensor):
        return dequantize_mx(t)
    raise TypeError(type(t))


def quantize_expertwise(weight, profiles) -> NintMoeTensor:
    """mfq/quantize/expert_nint.py:507-578, NINT cohorts only (`profiles[e]` = (bits, groupsize, sub_bits) of expert e):
    cohorts in the order their precision first appears (:528-531, a dict keyed by precision), experts ascending inside a
    cohort, the cohort's rows flattened to [n * out, K] (:559-561) and quantized weight-only like a dense tensor
    (:340-351 with importance=None)."""
    W = np.asarray(weight, dtype=np.float32)
    if W.ndim != 3:
        raise ValueError("expert-wise quantization expects [experts, out, in]")
    E, out, K = W.shape
    profiles = [tuple(int(v) for v in p) for p in profiles]
    if len(profiles) != E:
        raise ValueError(f"received {len(profiles)} precision descriptors for {E} experts")
    cohorts = {}
    for e, prof in enumerate(profiles):
        cohorts.setdefault(prof, []).append(e)
    pools = []
    for (bits, gs, sub_bits), members in cohorts.items():
        ids = np.asarray(members, dtype=np.int32)
        rows = np.ascontiguousarray(W[ids]).reshape(ids.size * out, K)
        pools.append(MoePool(ids, f"NINT{bits}", quantize_nint(rows, bits, gs, sub_bits)))
    return NintMoeTensor((E, out, K), pools)


def dequantize_expertwise(t: NintMoeTensor) -> np.ndarray:
    """mfq/quantize/expert_nint.py:605-615."""
    E, out, K = t.shape
    result = np.empty(t.shape, dtype=np.float32)
    for p in t.pools:
        result[p.expert_ids] = dequantize_tensor(p.tensor).reshape(len(p.expert_ids), out, K)
    return result


# ---------------------------------------------------------------------------
# MFQ1 container  (mfq/formats/io.py:646-685, mfq/formats/header.py:14)
# ---------------------------------------------------------------------------
def mfq_file_write(path, tensors: dict, model_arch="synthetic", version=1):
    packed = {n: (pack_tensor(t) if not isinstance(t, tuple) else t) for n, t in tensors.items()}
    with open(path, "wb") as f:
        f.write(b"MFQ1" + struct.pack("<I", version))
        a = model_arch.encode()
        f.write(struct.pack("<I", len(a)) + a)
        if version >= 2:
            f.write(struct.pack("<I", 0))
        f.write(struct.pack("<I", len(packed)))
        for n, (dt, blob) in packed.items():
            nb, db = n.encode(), dt.encode()
            f.write(struct.pack("<I", len(nb)) + nb + struct.pack("<I", len(db)) + db + struct.pack("<Q", len(blob)))
        for n, (dt, blob) in packed.items():
            f.write(blob)


def mfq_file_read(path) -> dict:
    data = Path(path).read_bytes()
    if data[:4] != b"MFQ1":
        raise ValueError("bad MFQ magic")
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
        name = data[off + 4: off + 4 + n].decode()
        off += 4 + n
        n, = struct.unpack_from("<I", data, off)
        dt = data[off + 4: off + 4 + n].decode()
        off += 4 + n
        ln, = struct.unpack_from("<Q", data, off)
        off += 8
        recs.append((name, dt, ln))
    out = {}
    for name, dt, ln in recs:
        out[name] = (dt, data[off: off + ln])
        off += ln
    return out


# ---------------------------------------------------------------------------
# the CPU matmul path  (mfq/runtime/linear.py:37-42)
# ---------------------------------------------------------------------------
def bf16_round(x) -> np.ndarray:
    """Round fp32 to the nearest bf16 (ties to even), returned as fp32."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return r.astype(np.uint32).view(np.float32)


def bf16_bits(x) -> np.ndarray:
    return (bf16_round(x).view(np.uint32) >> 16).astype(np.uint16)


def linear_forward(W: np.ndarray, x: np.ndarray) -> np.ndarray:
    """y = f32(x) @ dequant(W).T, numpy fp32 (mfq/runtime/linear.py:37-42)."""
    return np.asarray(x, dtype=np.float32) @ np.asarray(W, dtype=np.float32).T


def linear_forward_f64(W, x) -> np.ndarray:
    """The same product accumulated in fp64: the tolerance yardstick for GPU outputs."""
    return np.asarray(x, dtype=np.float64) @ np.asarray(W, dtype=np.float64).T


# ---------------------------------------------------------------------------
# MoE routing + grouped matmul  (mfq/kernels/cuda/moe.cu, tests/test_moe_kernels_cuda.py)
# ---------------------------------------------------------------------------
def moe_topk(logits, top_k, use_sigmoid=False, use_sqrt_softplus=False, normalize=False,
             delayed_softmax=False, bias=None, norm_floor=1e-20, scale=1.0):
    """mfq/kernels/cuda/moe.cu:124-263: iterative arg-max, tie -> lower expert id, NaN -> -FLT_MAX,
    bias added to the selection score only."""
    x = np.asarray(logits, dtype=np.float32)
    x = np.where(np.isnan(x), -np.finfo(np.float32).max, x).astype(np.float32)
    T, E = x.shape
    if delayed_softmax:
        w = x
    elif use_sigmoid:
        w = (1.0 / (1.0 + np.exp(-x.astype(np.float64)))).astype(np.float32)
    elif use_sqrt_softplus:
        xd = x.astype(np.float64)
        w = np.sqrt(np.where(xd > 20.0, xd, np.log1p(np.exp(np.minimum(xd, 20.0))))).astype(np.float32)
    else:
        xd = x.astype(np.float64)
        e = np.exp(xd - xd.max(-1, keepdims=True))
        w = (e / e.sum(-1, keepdims=True)).astype(np.float32)
    score = w if bias is None else (w + np.asarray(bias, dtype=np.float32)[None, :]).astype(np.float32)
    # stable sort on -score keeps the lower expert id first among equal scores
    order = np.argsort(-score, axis=-1, kind="stable")[:, :top_k]
    ids = order.astype(np.int32)
    sel = np.take_along_axis(w, order, axis=-1).astype(np.float32)
    if delayed_softmax:
        sd = sel.astype(np.float64)
        e = np.exp(sd - sd.max(-1, keepdims=True))
        sel = (e / e.sum(-1, keepdims=True)).astype(np.float32)
    elif normalize:
        sel = (sel / np.maximum(sel.sum(-1, keepdims=True), np.float32(norm_floor))).astype(np.float32)
    return ids, (sel * np.float32(scale)).astype(np.float32)


def build_expert_map(ids, n_experts, tile_m=8):
    """mfq/kernels/cuda/moe.cu:472-542: counts, exclusive bounds, tile bounds, tile->expert, and a
    grouping permutation of the (token, route) pairs (stable order inside an expert)."""
    flat = np.asarray(ids, dtype=np.int32).reshape(-1)
    valid = (flat >= 0) & (flat < n_experts)
    counts = np.bincount(flat[valid], minlength=n_experts).astype(np.int32)
    expert_bounds = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    tiles = (counts + tile_m - 1) // tile_m
    tile_bounds = np.concatenate([[0], np.cumsum(tiles)]).astype(np.int32)
    tile_experts = np.repeat(np.arange(n_experts, dtype=np.int32), tiles)
    pairs = np.flatnonzero(valid)
    ids_dst = pairs[np.argsort(flat[valid], kind="stable")].astype(np.int32)
    return ids_dst, expert_bounds, tile_bounds, tile_experts, counts


def moe_grouped_matmul(dense, x, ids):
    """tests/test_moe_kernels_cuda.py:58-68: out[t, r] = x[t(,r)] @ dense[ids[t, r]].T in fp32.
    A route with an out-of-range expert id yields zeros."""
    dense = np.asarray(dense, dtype=np.float32)
    x = np.asarray(x, dtype=np.float32)
    T, R = ids.shape
    out = np.zeros((T, R, dense.shape[1]), dtype=np.float32)
    for t in range(T):
        for r in range(R):
            e = int(ids[t, r])
            if 0 <= e < dense.shape[0]:
                src = x[t, r] if x.ndim == 3 else x[t]
                out[t, r] = src @ dense[e].T
    return out


def moe_swiglu(gate_up):
    """silu(gate) * up over [..., 2W] -> [..., W], gate = first half (mfq/kernels/cuda/moe.cu:2980-2996)."""
    g = np.asarray(gate_up, dtype=np.float32)
    W = g.shape[-1] // 2
    gate, up = g[..., :W].astype(np.float64), g[..., W:].astype(np.float64)
    return ((gate / (1.0 + np.exp(-gate))) * up).astype(np.float32)


def input_mul(x, gate, mode=0):
    """x * silu(gate) (mode 0) or x * sigmoid(gate) (mode 1) in float64: the input gate of nint_matmul_input_mul
    (cpp_runtime/mfq_decode.cpp:8395-8417; unfused form :8415-8416)."""
    x = np.asarray(x, dtype=np.float64)
    g = np.asarray(gate, dtype=np.float64)
    s = 1.0 / (1.0 + np.exp(-g))
    return x * (s if mode == 1 else g * s)


def moe_geglu(gate_up):
    """gelu_tanh(gate) * up over [..., 2W] -> [..., W], gate = first half: mfq_glu<true>
    (mfq/kernels/cuda/glu.cuh:7-12), 0.5 g (1 + tanh(sqrt(2/pi) g (1 + 0.044715 g^2)))."""
    g = np.asarray(gate_up, dtype=np.float32)
    W = g.shape[-1] // 2
    gate, up = g[..., :W].astype(np.float64), g[..., W:].astype(np.float64)
    gelu = 0.5 * gate * (1.0 + np.tanh(0.79788456080286535587989211986876 * gate * (1.0 + 0.044715 * gate * gate)))
    return (up * gelu).astype(np.float32)


def moe_weighted_reduce(pair, weights):
    """out[t] = sum_r w[t, r] * pair[t, r] in fp32, r ascending (mfq/kernels/cuda/moe.cu:2957-2978)."""
    pair = np.asarray(pair, dtype=np.float32)
    w = np.asarray(weights, dtype=np.float32)
    out = np.zeros((pair.shape[0], pair.shape[2]), dtype=np.float32)
    for r in range(pair.shape[1]):
        out += w[:, r:r + 1] * pair[:, r]
    return out


def moe_ffn(gate_up_dense, down_dense, x, router_logits, top_k, shared=None, **topk_kw):
    """cpp_runtime/mfq_decode.cpp:3394-3416 (+ ungated shared expert add, :11077-11080).
    `shared` = (gate_up_dense [2W, H], down_dense [H, W]) of the shared expert, or None."""
    ids, w = moe_topk(router_logits, top_k, **topk_kw)
    gu = moe_grouped_matmul(gate_up_dense, x, ids)
    hidden = moe_swiglu(gu)
    dn = moe_grouped_matmul(down_dense, hidden, ids)
    out = moe_weighted_reduce(dn, w)
    if shared is not None:
        sgu, sdn = shared
        h = moe_swiglu(linear_forward(sgu, x))
        out = out + linear_forward(sdn, h)
    return out, ids, w
