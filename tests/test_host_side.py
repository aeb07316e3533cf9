"""Host-side product code without a GPU: payload writers/parsers against the oracle, loader errors,
and the C ABI library's exported symbols."""
import ctypes
import re
from pathlib import Path

import numpy as np
import pytest

import synth
from oracle import mfq_oracle as O
from tyloquant_amd import formats as F

ROOT = Path(__file__).resolve().parents[1]


def test_writers_are_byte_identical_to_the_oracle_packers():
    rng = np.random.default_rng(0)
    for spec in [(4, 32, 6), (3, 24, 5), (5, 28, 7), (2, 16, 5), (8, 24, 8), (6, 26, 6)]:
        t = synth.nint_random(rng, 9, 131, *spec)
        blob = F.nint_blob(t.bits, t.sub_bits, t.groupsize, t.neuron_len, t.neuron_scale, t.neuron_min, t.sub_scale,
                           t.sub_min, t.q)
        assert blob == O.pack_nint(t)
        h = F.parse_nint(blob)
        assert (h.bits, h.gs, h.sub_bits, h.out, h.ng, h.legacy) == (spec[0], spec[1], spec[2], 9, t.ng, False)
        assert h.body_bytes == O.nint_payload_nbytes(9, 131, *spec)
    j = synth.nvq_jsc_random(rng, 7, 100, "d4_512", 2)
    jb = F.nvq_jsc_blob(j.codebook, j.neuron_len, j.neuron_scale, j.scale_lut, j.bank_for_state, j.codebooks, j.state,
                        j.indices, j.signs)
    assert jb == O.pack_nvq_jsc(j)
    hj = F.parse_nvq(jb)
    assert hj.dtype == "NVQ3J-512" and hj.banks == 2 and (hj.ng, hj.nvec, hj.nsign) == (5, 25, 13)
    p = synth.nvq_plain_random(rng, 5, 96)
    assert F.nvq_plain_blob(p.codebook, p.neuron_len, p.neuron_scale, p.sub_scale, p.indices, p.signs) == O.pack_nvq_plain(p)
    for label in ("NEPQ1-S", "NEPQ1-L"):
        n = synth.nepq_random(rng, label, 2, 16, 104, 3)
        nb = F.nepq_blob(label, n.shape, n.table_payloads, n.neuron_scale, n.state, n.indices, n.aux, n.bank_ids)
        assert nb == O.pack_nepq(n)
        hn = F.parse_nepq(nb)
        assert (hn.label, hn.banks, hn.ng, hn.nvec, hn.nsuper) == (label, 3, 5, 13, 2)
    m = synth.moe_random(rng, 5, 16, 48, [4, 3, 4, 2, 3])
    mb = F.nintm_blob(5, 16, 48, [(p.expert_ids, p.dtype, O.pack_nint(p.tensor)) for p in m.pools])
    assert mb == O.pack_nint_moe(m)
    hm = F.parse_nintm(mb)
    assert [p.dtype for p in hm.pools] == ["NINT2", "NINT3", "NINT4"]
    assert bytes(mb[hm.pools[1].payload_off: hm.pools[1].payload_off + hm.pools[1].payload_bytes]) == O.pack_nint(m.pools[1].tensor)


def test_parsers_reject_what_the_reference_loaders_reject():
    rng = np.random.default_rng(1)
    t = synth.nint_random(rng, 8, 96, 4, 24, 6)
    blob = O.pack_nint(t)
    with pytest.raises(ValueError, match="invalid NINT blob tail"):
        F.parse_nint(blob[:-1])
    with pytest.raises(ValueError, match="truncated NINT header"):
        F.parse_nint(blob[:10])
    j = O.pack_nvq_jsc(synth.nvq_jsc_random(rng, 4, 48))
    with pytest.raises(ValueError, match="invalid NVQ magic"):
        F.parse_nvq(b"NOPE" + j[4:])
    bad = bytearray(j)
    bad[40 + 36] = 9                                      # state -> bank 9 of 2
    with pytest.raises(ValueError, match="state-to-bank"):
        F.parse_nvq(bytes(bad))
    bad = bytearray(j)
    bad[40 + 60] = 1                                      # reserved byte
    with pytest.raises(ValueError, match="invalid NVQ-JSC metadata"):
        F.parse_nvq(bytes(bad))
    n = O.pack_nepq(synth.nepq_random(rng, "NEPQ1-S", 1, 16, 96, 2))
    with pytest.raises(ValueError, match="truncated NEPQ header"):
        F.parse_nepq(n[:20])
    with pytest.raises(ValueError, match="invalid NEPQ tail"):
        F.parse_nepq(n[:-1])
    with pytest.raises(ValueError, match="K divisible by 8"):
        F.parse_nepq(n[:16] + (100).to_bytes(4, "little") + n[20:])
    m = O.pack_nint_moe(synth.moe_random(rng, 4, 16, 48, [4, 4, 3, 3]))
    with pytest.raises(ValueError, match="invalid NINTM magic"):
        F.parse_nintm(b"NIM1" + m[4:])
    with pytest.raises(ValueError, match="truncated NINTM"):
        F.parse_nintm(m[: len(m) // 2])


def test_mfq_container_round_trip(tmp_path):
    rng = np.random.default_rng(2)
    a = O.pack_tensor(synth.nint_random(rng, 8, 96, 3, 24, 5))
    b = O.pack_tensor(synth.nvq_jsc_random(rng, 4, 48))
    path = tmp_path / "x.mfq"
    F.write_mfq(path, {"layers.0.q": a, "layers.0.k": b}, version=2)
    data = path.read_bytes()
    d = F.read_mfq_directory(data)
    assert list(d) == ["layers.0.q", "layers.0.k"]
    assert d["layers.0.q"][0] == "NINT3" and data[d["layers.0.k"][1]: d["layers.0.k"][1] + d["layers.0.k"][2]] == b[1]
    assert O.mfq_file_read(path)["layers.0.q"] == a       # the oracle reads what the product wrote


def test_library_exports_every_symbol_the_header_declares():
    from tyloquant_amd import _lib as L
    header = (ROOT / "include" / "mfq_hip.h").read_text()
    declared = sorted(set(re.findall(r"\b(mfq_hip_\w+)\s*\(", header)))
    assert declared == L.exported_symbols()
    if not L.LIB_PATH.exists():
        pytest.skip("libmfq_hip.so is not built (run __graft_entry__.build())")
    lib = ctypes.CDLL(str(L.LIB_PATH))
    for name in declared:
        assert hasattr(lib, name), name
    assert _dynamic_symbols(L.LIB_PATH, "mfq_hip_") == declared      # and nothing is exported that the header omits
    assert L.lib().mfq_hip_version() >= 1


def _dynamic_symbols(path, prefix):
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", str(path)], check=True, capture_output=True, text=True).stdout
    return sorted({ln.split()[-1] for ln in out.splitlines() if ln.split() and ln.split()[-1].startswith(prefix)})


def test_plan_calls_need_no_gpu():
    """Layout planning is pure host arithmetic: sizes, padding and the payload accounting."""
    from tyloquant_amd import _lib as L
    if not L.LIB_PATH.exists():
        pytest.skip("libmfq_hip.so is not built")
    lib = L.lib()
    d = L.NintDesc()
    L.check(lib.mfq_hip_nint_plan(3, 5, 24, 4096, 4096, ctypes.byref(d)))
    assert (d.kind, d.dwords, d.tail_bytes, d.ng, d.ngp, d.nsteps, d.n_rowblocks) == (1, 2, 1, 171, 176, 11, 256)
    assert d.payload_bytes == 7195648 and d.step_bytes == 64 * (32 + 4 + 8)
    L.check(lib.mfq_hip_nint_plan(4, 6, 32, 12288, 4096, ctypes.byref(d)))
    assert d.payload_bytes == 27574272 and d.kind == 1 and d.dwords == 4
    L.check(lib.mfq_hip_nint_plan(5, 7, 28, 64, 112, ctypes.byref(d)))
    assert d.kind == 0 and d.dwords == 5
    with pytest.raises(L.MfqError, match="bits"):
        L.check(lib.mfq_hip_nint_plan(9, 5, 24, 8, 8, ctypes.byref(d)))
    q = L.NepqDesc()
    L.check(lib.mfq_hip_nepq_plan(2, 1, 12288, 4096, ctypes.byref(q)))
    assert q.payload_bytes - 2048 == 8944128
    with pytest.raises(L.MfqError, match="divisible by 8"):
        L.check(lib.mfq_hip_nepq_plan(2, 1, 16, 100, ctypes.byref(q)))


def test_product_quantizer_matches_the_reference_golden_vectors():
    from tyloquant_amd.quantize import nint_quantize
    g = np.load(Path(__file__).parent / "golden" / "nint_quant_vectors.npz")
    for k in sorted({n.split("_")[0] for n in g.files}):
        _, rows, K, bits, gs, sb = (int(v) for v in g[k + "_meta"])
        r = nint_quantize(g[k + "_W"], bits, gs, sb, row_chunk=5)
        assert np.array_equal(r["q"], g[k + "_q"]) and np.array_equal(r["ss"], g[k + "_ss"]), k
        assert np.array_equal(r["sm"], g[k + "_sm"]) and np.array_equal(r["ns"], g[k + "_ns"]), k
        assert np.array_equal(r["nm"], g[k + "_nm"]), k


def test_grouped_projection_blob_is_the_row_concatenation():
    rng = np.random.default_rng(5)
    a, b = synth.nint_random(rng, 16, 100, 3, 24, 5), synth.nint_random(rng, 9, 100, 3, 24, 5)
    cat = O.unpack_nint(F.nint_concat_rows([O.pack_nint(a), O.pack_nint(b)]))
    assert np.array_equal(O.dequantize_nint(cat), np.concatenate([O.dequantize_nint(a), O.dequantize_nint(b)]))
    for bits in (1, 3, 5, 7, 8, 9, 11):
        v = rng.integers(0, 1 << bits, 77)
        assert np.array_equal(F.unpack_bitstream(O.pack_bits(v, bits), 0, 77, bits), v)
    with pytest.raises(ValueError, match="must share"):
        F.nint_concat_rows([O.pack_nint(a), O.pack_nint(synth.nint_random(rng, 4, 100, 4, 24, 6))])


def test_runtime_library_exports_its_c_view():
    header = (ROOT / "include" / "mfq_runtime_c.h").read_text()
    declared = sorted(set(re.findall(r"\b(mfq_rt_\w+)\s*\(", header)))
    path = ROOT / "tyloquant_amd" / "lib" / "libmfq_runtime.so"
    if not path.exists():
        pytest.skip("libmfq_runtime.so is not built")
    lib = ctypes.CDLL(str(path))
    assert len(declared) >= 10
    for name in declared:
        assert hasattr(lib, name), name
    assert _dynamic_symbols(path, "mfq_rt_") == declared             # header and library agree both ways


def _rt():
    path = ROOT / "tyloquant_amd" / "lib" / "libmfq_runtime.so"
    if not path.exists():
        pytest.skip("libmfq_runtime.so is not built")
    lib = ctypes.CDLL(str(path))
    lib.mfq_rt_last_error.restype = ctypes.c_char_p
    return lib


def _rt_load_error(lib, fn, *args):
    handle = ctypes.c_void_p()
    rc = fn(*args, ctypes.byref(handle))
    assert rc != 0 and not handle.value
    return lib.mfq_rt_last_error().decode()


def test_cpp_parsers_reject_malformed_headers_without_touching_the_gpu():
    """Headers are validated before any division or device call: a zero groupsize, a negative
    neuron length, lengths whose sum wraps 64 bits.  Each is an error message, not a signal or an out-of-bounds read."""
    import struct
    lib = _rt()
    rng = np.random.default_rng(5)
    blob = bytearray(O.pack_tensor(synth.nvq_jsc_random(rng, 4, 48))[1])
    bad = bytearray(blob)
    struct.pack_into("<H", bad, 6, 0)                                   # groupsize 0
    msg = _rt_load_error(lib, lib.mfq_rt_load_quant_linear, b"NVQ3J-512", bytes(bad), ctypes.c_size_t(len(bad)))
    assert "must be positive" in msg
    bad = bytearray(blob)
    struct.pack_into("<i", bad, 12, -48)                                # negative neuron_len
    assert "must be positive" in _rt_load_error(lib, lib.mfq_rt_load_quant_linear, b"NVQ3J-512", bytes(bad),
                                                ctypes.c_size_t(len(bad)))
    # NINTM: payload_len + runtime_len wraps to a small number
    t = synth.moe_random(rng, 4, 16, 48, [4, 4, 3, 3])
    nim = bytearray(O.pack_nint_moe(t))
    struct.pack_into("<QQ", nim, 20 + 8, 2 ** 64 - 64, 128)
    msg = _rt_load_error(lib, lib.mfq_rt_load_nint_moe, bytes(nim), ctypes.c_size_t(len(nim)))
    assert "truncated NINTM v2 pool payload" in msg
    # an expert delta (NID2) is not a tensor; as an overlay its shape must match the tensor's
    nid = O.pack_nint_moe(O.NintMoeTensor((4, 16, 48), [O.MoePool(np.array([2], dtype=np.int32), "NINT3",
                                                                  synth.nint_random(rng, 16, 48, 3, 24, 5))]), delta=True)
    assert "delta cannot be loaded as a full tensor" in _rt_load_error(lib, lib.mfq_rt_load_nint_moe, nid, ctypes.c_size_t(len(nid)))
    with pytest.raises(ValueError, match="delta cannot be loaded as a full tensor"):
        F.parse_nintm(nid)
    d = F.parse_nintm(nid, allow_partial=True)
    assert [p.dtype for p in d.pools] == ["NINT3"] and d.pools[0].expert_ids.tolist() == [2]
    back = O.unpack_nint_moe(nid, allow_partial=True)
    over = O.apply_expert_overlay(t, back)
    dense, base = O.dequantize_expertwise(over), O.dequantize_expertwise(t)
    assert np.array_equal(dense[[0, 1, 3]], base[[0, 1, 3]]) and not np.array_equal(dense[2], base[2])
    wrong = O.pack_nint_moe(O.NintMoeTensor((4, 16, 96), [O.MoePool(np.array([2], dtype=np.int32), "NINT3",
                                                                    synth.nint_random(rng, 16, 96, 3, 24, 5))]), delta=True)
    good = O.pack_nint_moe(t)
    lib.mfq_rt_load_nint_moe_overlay.argtypes = [ctypes.c_char_p, ctypes.c_size_t, ctypes.c_char_p, ctypes.c_size_t,
                                                 ctypes.POINTER(ctypes.c_void_p)]
    assert "expert overlay shape mismatch" in _rt_load_error(lib, lib.mfq_rt_load_nint_moe_overlay, good, len(good), wrong,
                                                             len(wrong))


def test_mfq_directory_checks_of_the_reference_reader(tmp_path):
    """mfq/formats/io.py:818-828: duplicate names and a records-end != file-size are errors, in both readers."""
    import subprocess
    rng = np.random.default_rng(6)
    a = O.pack_tensor(synth.nint_random(rng, 4, 48, 3, 24, 5))
    path = tmp_path / "x.mfq"
    F.write_mfq(path, {"w": a}, version=1)
    data = path.read_bytes()
    assert list(F.read_mfq_directory(data)) == ["w"]
    with pytest.raises(ValueError, match="length mismatch"):
        F.read_mfq_directory(data + b"\0")
    with pytest.raises(ValueError, match="truncated MFQ blob"):
        F.read_mfq_directory(data[:-1])
    # two records with one name: the directory of a one-tensor file written twice
    head_end = data.index(b"NINT3") + 5 + 8
    rec = data[data.index(b"\x01\x00\x00\x00w"):head_end]               # u32 len + name, u32 len + dtype, u64 bytes
    dup = data[:data.index(b"\x01\x00\x00\x00w") - 4] + (2).to_bytes(4, "little") + rec + rec + data[head_end:] * 2
    with pytest.raises(ValueError, match="duplicate MFQ tensor record"):
        F.read_mfq_directory(dup)
    tool = ROOT / "tyloquant_amd" / "lib" / "mfq-check-linear"
    if tool.exists():
        for payload, want in ((dup, "duplicate MFQ tensor record"), (data + b"\0", "length mismatch"),
                              (data[:-1], "truncated MFQ blob")):
            bad = tmp_path / "bad.mfq"
            bad.write_bytes(payload)
            r = subprocess.run([str(tool), str(bad), "w"], capture_output=True, text=True)
            assert r.returncode == 1 and want in r.stderr, r.stderr


def test_tiled_expertwise_blob_equals_quantizing_the_full_tensor():
    """synth.nintm_quantized_blob quantizes one slab per precision and repeats the slab's streams over the cohort; the
    NINT quantizer treats every neuron on its own, so the bytes must equal the oracle's expert-wise quantization of the
    full tensor whose experts repeat the slabs -- cohort order, expert order and every stream included."""
    from tyloquant_amd import synth as psynth
    bits = [4, 3, 3, 5, 2, 4, 3, 3]
    E, out, K, slab = len(bits), 32, 100, 16
    blob, pools = psynth.nintm_quantized_blob(9, E, out, K, bits, slab_rows=slab)
    order = list(dict.fromkeys(bits))
    slabs = (np.random.default_rng(9).standard_normal((len(order), slab, K)) * 0.02).astype(np.float32)
    W = np.stack([np.tile(slabs[order.index(b)], (out // slab, 1)) for b in bits])
    t = O.quantize_expertwise(W, [psynth.MOE_PROFILES[b] for b in bits])
    assert blob == O.pack_nint_moe(t)
    assert [ids.tolist() for ids, _ in pools] == [p.expert_ids.tolist() for p in t.pools]
    assert all(payload == O.pack_nint(p.tensor) for (_, payload), p in zip(pools, t.pools))
    with pytest.raises(ValueError):
        psynth.nintm_quantized_blob(9, E, 30, K, bits, slab_rows=16)
