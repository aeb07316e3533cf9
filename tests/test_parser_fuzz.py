"""Malformed payloads: every blob and container parser of the host layers -- Python (tyloquant_amd.formats) and C++
(libmfq_runtime.so, which parses before it touches the GPU) -- answers a truncated, extended or bit-flipped input with an
error, never with a crash or an out-of-range read.  The reference's own loaders reject the same inputs with exceptions
(mfq/formats/io.py:382-446, nvq.py:586-820, nepq.py:401-474; cpp_runtime/mfq_decode.cpp:3756-4013).  Runs without a GPU:
a well-formed blob then fails at the first device call, which is an error return as well."""
import ctypes as C
import os
from pathlib import Path

import numpy as np
import pytest

import synth
from oracle import mfq_oracle as O
from tyloquant_amd import formats as F

LIBDIR = Path(__file__).resolve().parents[1] / "tyloquant_amd" / "lib"


def _blobs():
    rng = np.random.default_rng(7)
    moe = synth.moe_random(rng, 4, 16, 96, [3, 4, 4, 2])
    mixed = O.NintMoeTensor((3, 16, 96), [
        O.MoePool(np.array([0], dtype=np.int32), "NINT4", synth.nint_random(rng, 16, 96, 4, 32, 6)),
        O.MoePool(np.array([2], dtype=np.int32), "NVQ3J-512", synth.nvq_jsc_random(rng, 16, 96, "d4_512", 2)),
        O.MoePool(np.array([1], dtype=np.int32), "NEPQ0-S", synth.nepq_random(rng, "NEPQ0-S", 1, 16, 96, 2))])
    return [
        ("NINT3", O.pack_nint(synth.nint_random(rng, 5, 100, 3, 24, 5))),
        ("NINT8-0", O.pack_nint8_zero(O.quantize_nint8_zero((rng.standard_normal((8, 64)) * 0.02).astype(np.float32)))),
        ("NVQ3J-512", O.pack_tensor(synth.nvq_jsc_random(rng, 5, 100, "d4_512", 2))[1]),
        ("NVQ2J-L", O.pack_tensor(synth.nvq_jsc_random(rng, 5, 104, "e8_1024", 2))[1]),
        ("NVQ3", O.pack_tensor(synth.nvq_plain_random(rng, 5, 100))[1]),
        ("NVQ1-L", O.pack_tensor(synth.nvq1_random(rng, "NVQ1-L", 5, 100, 3, custom=True))[1]),
        ("NVQ1-S", O.pack_tensor(synth.nvq1_random(rng, "NVQ1-S", 5, 104))[1]),
        ("NPQ0-L", O.pack_tensor(synth.npq0_random(rng, "NPQ0-L", 5, 104))[1]),
        ("NPQ0-S", O.pack_tensor(synth.npq0_random(rng, "NPQ0-S", 5, 104))[1]),
        ("NEPQ1-S", O.pack_nepq(synth.nepq_random(rng, "NEPQ1-S", 1, 8, 200, 3))),
        ("NEPQ0-L", O.pack_nepq(synth.nepq_random(rng, "NEPQ0-L", 1, 8, 200, 3))),
        ("NINTM", O.pack_nint_moe(moe)),
        ("NINTM", O.pack_nint_moe(mixed)),
        ("MXFP4", O.pack_mx(synth.mx_random(rng, "MXFP4", 5, 96))),
        ("MXFP8", O.pack_mx(synth.mx_random(rng, "MXFP8", 130, 128))),
    ]


def _mutations(blob, rng, n):
    """Truncations, extensions, single-byte changes in the header region (where the counts and sizes live) and anywhere,
    and 32-bit fields overwritten with extreme values."""
    blob = bytes(blob)
    head = min(len(blob), 160)
    for _ in range(n):
        kind = rng.integers(0, 5)
        b = bytearray(blob)
        if kind == 0:
            yield bytes(b[: rng.integers(0, len(b))])
        elif kind == 1:
            yield bytes(b) + bytes(rng.integers(0, 256, rng.integers(1, 9), dtype=np.uint8))
        elif kind == 2:
            b[rng.integers(0, head)] = rng.integers(0, 256)
            yield bytes(b)
        elif kind == 3:
            b[rng.integers(0, len(b))] ^= 1 << rng.integers(0, 8)
            yield bytes(b)
        else:
            pos = int(rng.integers(0, max(1, head - 4)))
            b[pos: pos + 4] = int(rng.choice([0, 1, 0x7FFFFFFF, 0x80000000, 0xFFFFFFFF, 0xFFFFFFF0])).to_bytes(4, "little")
            yield bytes(b)


def _py_parse(dtype, blob):
    if dtype == "NINTM":
        return F.parse_nintm(blob)
    if dtype == "NINT8-0":
        return F.parse_nint8_zero(blob)
    if F.is_mx_dtype(dtype):
        return F.parse_mx(dtype, blob)
    if dtype.startswith("NINT"):
        return F.parse_nint(blob)
    if F.is_lowbit_dtype(dtype):
        return F.parse_lowbit(dtype, blob)
    if dtype.startswith("NEPQ"):
        return F.parse_nepq(blob)
    return F.parse_nvq(blob)


@pytest.mark.parametrize("case", range(15))
def test_python_parsers_raise_on_malformed_blobs(case):
    dtype, blob = _blobs()[case]
    _py_parse(dtype, blob)                                   # the well-formed blob parses
    rng = np.random.default_rng(100 + case)
    for bad in _mutations(blob, rng, 200):
        try:
            _py_parse(dtype, bad)                            # a mutation that keeps the blob consistent is fine
        except (ValueError, NotImplementedError):
            pass
        if dtype != "NINTM" and (F.is_lowbit_dtype(dtype) or dtype.startswith("NVQ")) and len(bad) != len(blob):
            with pytest.raises((ValueError, NotImplementedError)):
                F.split_rows(dtype, bad, 1)


@pytest.fixture(scope="module")
def rt():
    lib = C.CDLL(os.environ.get("MFQ_RUNTIME_LIB", str(LIBDIR / "libmfq_runtime.so")))
    lib.mfq_rt_last_error.restype = C.c_char_p
    lib.mfq_rt_load_quant_linear.argtypes = [C.c_char_p, C.c_char_p, C.c_size_t, C.POINTER(C.c_void_p)]
    lib.mfq_rt_free_quant_linear.argtypes = [C.c_void_p]
    lib.mfq_rt_load_nint_moe.argtypes = [C.c_char_p, C.c_size_t, C.POINTER(C.c_void_p)]
    lib.mfq_rt_free_nint_moe.argtypes = [C.c_void_p]
    return lib


@pytest.mark.parametrize("case", range(15))
def test_cpp_loaders_return_errors_on_malformed_blobs(rt, case):
    dtype, blob = _blobs()[case]
    rng = np.random.default_rng(200 + case)
    for bad in _mutations(blob, rng, 200):
        h = C.c_void_p()
        if dtype == "NINTM":
            rc = rt.mfq_rt_load_nint_moe(bad, len(bad), C.byref(h))
            if rc == 0:
                rt.mfq_rt_free_nint_moe(h)
        else:
            rc = rt.mfq_rt_load_quant_linear(dtype.encode(), bad, len(bad), C.byref(h))
            if rc == 0:
                rt.mfq_rt_free_quant_linear(h)
        assert rc in (0, 1)
        if len(bad) != len(blob):
            assert rc == 1 and rt.mfq_rt_last_error()        # a wrong length never gets through


def test_mfq_store_readers_reject_malformed_files(rt, tmp_path):
    """The MFQ1 container readers (Python MfqStore over a memory map, C++ MfqFile) on mutated files: header fields, the
    JSON extras of version 2, the record directory, truncations."""
    import json

    rt.mfq_rt_file_open.argtypes = [C.c_char_p, C.c_char_p, C.c_char_p, C.POINTER(C.c_void_p)]
    rt.mfq_rt_file_close.argtypes = [C.c_void_p]
    rt.mfq_rt_file_record_count.argtypes = [C.c_void_p]
    rt.mfq_rt_file_record_count.restype = C.c_int64
    rng = np.random.default_rng(31)
    tensors = {"blk.0.q": synth.nint_random(rng, 5, 100, 3, 24, 5), "blk.0.k": synth.nvq_jsc_random(rng, 5, 100, "d4_512", 2)}
    good = tmp_path / "good.mfq"
    O.mfq_file_write(good, tensors, version=2)
    data = good.read_bytes()
    with F.MfqStore(good, "", "") as st:
        assert sorted(st.records) == sorted(tensors)
    h = C.c_void_p()
    assert rt.mfq_rt_file_open(str(good).encode(), b"-", b"-", C.byref(h)) == 0, rt.mfq_rt_last_error()
    assert rt.mfq_rt_file_record_count(h) == 2
    rt.mfq_rt_file_close(h)
    bad = tmp_path / "bad.mfq"
    for i, mutated in enumerate(_mutations(data, rng, 250)):
        bad.write_bytes(mutated)
        try:
            with F.MfqStore(bad, "", "") as st:
                for name in st.records:
                    bytes(st.blob(name))                   # every listed record is readable in full
        except (ValueError, KeyError, json.JSONDecodeError, UnicodeDecodeError):
            pass
        h = C.c_void_p()
        rc = rt.mfq_rt_file_open(str(bad).encode(), b"-", b"-", C.byref(h))
        assert rc in (0, 1)
        if rc == 0:
            rt.mfq_rt_file_close(h)
        elif len(mutated) < len(data):
            assert rt.mfq_rt_last_error()
    # a refused file leaves no mapping behind: the failed opens above and 200 more of a truncated file
    bad.write_bytes(data[: len(data) // 2])

    def mappings():
        return sum(1 for line in open("/proc/self/maps") if "bad.mfq" in line)

    for _ in range(200):
        h = C.c_void_p()
        assert rt.mfq_rt_file_open(str(bad).encode(), b"-", b"-", C.byref(h)) == 1
    assert mappings() == 0
