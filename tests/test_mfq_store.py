"""The MFQ1 store: one file or a shard set behind one record table, memory-mapped, with tensor and expert overlays
(mfq/formats/shards.py, mfq/formats/io.py:834-965, cpp_runtime/mfq_decode.cpp:1294-1527).  Pinned by files the
reference's own writer produced (tests/golden/reference_shards.npz, made by tests/golden/make_reference_shards.py):
this package's writer reproduces them byte for byte, and the Python and the C++ reader recover the records from them.
No GPU is needed."""
import ctypes
import json
import struct
from pathlib import Path

import numpy as np
import pytest

from tyloquant_amd import formats as F

ROOT = Path(__file__).resolve().parents[1]
GOLD = np.load(ROOT / "tests" / "golden" / "reference_shards.npz")
NAMES = [str(n) for n in GOLD["names"]]
DTYPES = [str(d) for d in GOLD["dtypes"]]
BLOBS = [GOLD[f"blob{i}"].tobytes() for i in range(len(NAMES))]
TENSORS = {n: (d, b) for n, d, b in zip(NAMES, DTYPES, BLOBS)}
EXTRA = {"general.name": "tiny", "block_count": 1}
LAYOUTS = {"single": {}, "by_count": {"split_max_tensors": 3}, "by_size": {"split_max_size": 2000}}


def _rt():
    path = ROOT / "tyloquant_amd" / "lib" / "libmfq_runtime.so"
    if not path.exists():
        pytest.skip("libmfq_runtime.so is not built")
    lib = ctypes.CDLL(str(path))
    lib.mfq_rt_last_error.restype = ctypes.c_char_p
    lib.mfq_rt_file_arch.restype = ctypes.c_char_p
    lib.mfq_rt_file_extra.restype = ctypes.c_char_p
    for f in ("mfq_rt_file_record_count", "mfq_rt_file_tensor_count", "mfq_rt_file_source_count"):
        getattr(lib, f).restype = ctypes.c_int64
        getattr(lib, f).argtypes = [ctypes.c_void_p]
    lib.mfq_rt_file_close.argtypes = [ctypes.c_void_p]
    lib.mfq_rt_file_arch.argtypes = [ctypes.c_void_p]
    lib.mfq_rt_file_extra.argtypes = [ctypes.c_void_p, ctypes.c_char_p]
    lib.mfq_rt_file_record.argtypes = [ctypes.c_void_p, ctypes.c_int64] + [ctypes.c_void_p] * 5
    return lib


def _cpp_open(lib, path, tensor_overlay=b"-", expert_overlay=b"-"):
    h = ctypes.c_void_p()
    rc = lib.mfq_rt_file_open(str(path).encode(), tensor_overlay, expert_overlay, ctypes.byref(h))
    if rc:
        raise RuntimeError(lib.mfq_rt_last_error().decode())
    return h


def _cpp_records(lib, h):
    out = []
    for i in range(lib.mfq_rt_file_record_count(h)):
        name, dtype, src = ctypes.c_char_p(), ctypes.c_char_p(), ctypes.c_int()
        data, n = ctypes.c_void_p(), ctypes.c_size_t()
        assert lib.mfq_rt_file_record(h, i, ctypes.byref(name), ctypes.byref(dtype), ctypes.byref(src), ctypes.byref(data),
                                      ctypes.byref(n)) == 0
        out.append((name.value.decode(), dtype.value.decode(), src.value, ctypes.string_at(data.value, n.value)))
    return out


def _golden_files(label, tmp_path):
    paths = []
    for name in GOLD[f"{label}_files"]:
        p = tmp_path / str(name)
        p.write_bytes(GOLD[f"{label}/{name}"].tobytes())
        paths.append(p)
    return paths


@pytest.mark.parametrize("label", list(LAYOUTS))
def test_writer_reproduces_the_reference_files(label, tmp_path):
    """Same records, same limits: same file names and the same bytes as write_blob_record_shards
    (mfq/formats/shards.py:254-336) -- the pre-add boundary rule, assets first in shard one, model metadata only there,
    the four split.* keys in every shard, JSON-encoded metadata values."""
    ours = F.write_mfq_shards(tmp_path / "model.mfq", TENSORS, "tiny-arch", 2, EXTRA, **LAYOUTS[label])
    assert [p.name for p in ours] == [str(n) for n in GOLD[f"{label}_files"]]
    for p in ours:
        assert p.read_bytes() == GOLD[f"{label}/{p.name}"].tobytes(), p.name


def test_shard_plan_rules():
    sizes = [("a", 10), ("b", 10), (F.ASSET_PREFIX + "x", 5), ("c", 30), ("d", 1)]
    assert F.plan_shards(sizes) == [["a", "b", F.ASSET_PREFIX + "x", "c", "d"]]
    assert F.plan_shards(sizes, split_max_tensors=2) == [[F.ASSET_PREFIX + "x", "a", "b"], ["c", "d"]]
    # size: a record larger than the limit still gets a shard of its own; the check is made before adding
    assert F.plan_shards(sizes, split_max_size=20) == [[F.ASSET_PREFIX + "x", "a", "b"], ["c"], ["d"]]
    assert F.plan_shards(sizes, split_max_size=25) == [[F.ASSET_PREFIX + "x", "a", "b"], ["c"], ["d"]]
    with pytest.raises(ValueError, match="mutually exclusive"):
        F.plan_shards(sizes, 1, 1)
    assert F.parse_shard_path("m-00002-of-00003.mfq") == (Path("m.mfq"), 2, 3)
    assert F.parse_shard_path("m.mfq") is None
    with pytest.raises(ValueError, match="invalid MFQ shard file name"):
        F.parse_shard_path("m-00004-of-00003.mfq")
    assert F.format_shard_path("dir/m.mfq", 1, 12).name == "m-00001-of-00012.mfq"


@pytest.mark.parametrize("label", list(LAYOUTS))
@pytest.mark.parametrize("entry", [0, -1])
def test_both_readers_recover_the_records_from_reference_files(label, entry, tmp_path):
    """Opened through the first or the last shard: every record with its dtype and bytes, the model metadata of the
    first shard, assets not counted as tensors; the Python store and the C++ MfqFile agree."""
    paths = _golden_files(label, tmp_path)
    with F.MfqStore(paths[entry], tensor_overlay="", expert_overlay="") as st:
        assert st.n_shards == len(paths) and [p.name for p in st.paths] == [p.name for p in paths]
        assert sorted(st.names()) == sorted(NAMES) and st.tensor_count() == len(NAMES) - 1
        assert st.model_arch == "tiny-arch" and st.version == 2
        assert st.extra["general.name"] == "tiny" and st.extra["block_count"] == 1
        for n in NAMES:
            assert st.record(n).dtype == TENSORS[n][0]
            view = st.blob(n)
            assert view.readonly and bytes(view) == TENSORS[n][1]
            view.release()
        assert json.loads(st.asset_text(F.ASSET_PREFIX + "config.json"))["hidden"] == 64
        py_order = [(r.name, r.dtype, r.source) for r in st.records.values()]
    lib = _rt()
    h = _cpp_open(lib, paths[entry])
    try:
        recs = _cpp_records(lib, h)
        assert [(n, d, s) for n, d, s, _ in recs] == py_order
        assert all(b == TENSORS[n][1] for n, _, _, b in recs)
        assert lib.mfq_rt_file_source_count(h) == len(paths) and lib.mfq_rt_file_tensor_count(h) == len(NAMES) - 1
        assert lib.mfq_rt_file_arch(h) == b"tiny-arch"
        assert lib.mfq_rt_file_extra(h, b"general.name") == b'"tiny"' and lib.mfq_rt_file_extra(h, b"nope") is None
        if len(paths) > 1:
            assert lib.mfq_rt_file_extra(h, b"split.count") == str(len(paths)).encode()
    finally:
        lib.mfq_rt_file_close(h)


def _both_fail(path, match, tmp_path, **kw):
    with pytest.raises((ValueError, FileNotFoundError), match=match):
        F.MfqStore(path, tensor_overlay=kw.get("tensor_overlay", ""), expert_overlay=kw.get("expert_overlay", ""))
    lib = _rt()
    with pytest.raises(RuntimeError, match=match):
        h = _cpp_open(lib, path, (kw.get("tensor_overlay") or "-").encode(), (kw.get("expert_overlay") or "-").encode())
        lib.mfq_rt_file_close(h)


def _rewrite_extra(path, **changes):
    """The file with metadata values replaced (None removes a key)."""
    data = path.read_bytes()
    version, arch, extra, recs, off = F.read_mfq_header(data)
    for k, v in changes.items():
        if v is None:
            extra.pop(k, None)
        else:
            extra[k] = v
    path.write_bytes(F._mfq_head(recs, changes.get("_arch", arch) if False else arch, version, extra) + data[off:])


def test_shard_set_checks(tmp_path):
    """Every inconsistency the reference names is an error in both readers: a missing shard, a file name that
    disagrees with the metadata, a shard of another set, wrong totals, a record in two shards, a lone file whose name
    claims a set."""
    import shutil
    base = tmp_path / "ok"
    base.mkdir()
    paths = _golden_files("by_count", base)

    def fresh(name):
        d = tmp_path / name
        shutil.copytree(base, d)
        return [d / p.name for p in paths]

    p = fresh("missing")
    p[1].unlink()
    _both_fail(p[0], "missing MFQ shard", tmp_path)
    p = fresh("renamed")
    p[1].rename(p[1].with_name("model-00003-of-00004.mfq"))
    _both_fail(p[1].with_name("model-00003-of-00004.mfq"), "filename/metadata mismatch", tmp_path)
    p = fresh("nosuffix")
    p[0].rename(p[0].with_name("model.mfq"))
    _both_fail(p[0].with_name("model.mfq"), "lacks -00001-of-00000 suffix", tmp_path)
    p = fresh("swapped")            # shard three under shard two's name
    shutil.copy(p[2], p[1])
    _both_fail(p[0], "shard metadata mismatch", tmp_path)
    p = fresh("totals")
    _rewrite_extra(p[2], **{"split.records.count": 9})
    _both_fail(p[0], "record count mismatch", tmp_path)
    p = fresh("total_all")
    for q in p:
        _rewrite_extra(q, **{"split.records.count": 9, "split.tensors.count": None})
    _both_fail(p[0], "record total mismatch", tmp_path)
    p = fresh("tensors_all")
    for q in p:
        _rewrite_extra(q, **{"split.tensors.count": 3})
    _both_fail(p[0], "tensor total mismatch", tmp_path)
    p = fresh("badno")
    _rewrite_extra(p[0], **{"split.no": 5})
    _both_fail(p[0], "invalid", tmp_path)
    # a record that is also in another shard: shard two rewritten with shard one's first tensor appended
    p = fresh("dup")
    d1, d2 = p[0].read_bytes(), p[1].read_bytes()
    v, arch, extra, recs2, off2 = F.read_mfq_header(d2)
    dirs1 = F.read_mfq_directory(d1)
    name = "blk.0.attn_q.weight"
    dt, o, n = dirs1[name]
    p[1].write_bytes(F._mfq_head(recs2 + [(name, dt, n)], arch, v, extra) + d2[off2:] + d1[o:o + n])
    _both_fail(p[0], "duplicate MFQ tensor", tmp_path)
    # a single (unsharded) file under a shard name
    lone = tmp_path / "lone-00001-of-00002.mfq"
    lone.write_bytes(GOLD["single/model.mfq"].tobytes())
    _both_fail(lone, "claims multiple shards", tmp_path)
    # version / architecture of a shard differ
    p = fresh("arch")
    data = p[1].read_bytes()
    v, arch, extra, recs, off = F.read_mfq_header(data)
    p[1].write_bytes(F._mfq_head(recs, "other-arch", v, extra) + data[off:])
    _both_fail(p[0], "architecture/version mismatch", tmp_path)


def test_tensor_and_expert_overlays(tmp_path, monkeypatch):
    """A tensor overlay replaces records of the same name (bytes and dtype come from the overlay file), must be
    unsharded and must not introduce names; an expert overlay holds NINTMD records over NINTM records.  Given
    explicitly or through MFQ_TENSOR_OVERLAY / MFQ_EXPERT_OVERLAY."""
    paths = _golden_files("by_size", tmp_path)
    over = tmp_path / "over.mfq"
    new_q = bytes(range(200))
    F.write_mfq(over, {"blk.0.attn_q.weight": ("NINT5", new_q)}, "tiny-arch", 2)
    exp = tmp_path / "experts.mfq"
    F.write_mfq(exp, {"blk.0.ffn_gate_up_exps.weight": ("NINTMD", b"\x01" * 77)}, "tiny-arch", 2)
    lib = _rt()
    for how in ("args", "env"):
        if how == "env":
            monkeypatch.setenv("MFQ_TENSOR_OVERLAY", str(over))
            monkeypatch.setenv("MFQ_EXPERT_OVERLAY", str(exp))
            st = F.MfqStore(paths[0])
            h = _cpp_open(lib, paths[0], None, None)
        else:
            st = F.MfqStore(paths[0], tensor_overlay=str(over), expert_overlay=str(exp))
            h = _cpp_open(lib, paths[0], str(over).encode(), str(exp).encode())
        try:
            assert st.record("blk.0.attn_q.weight").dtype == "NINT5" and bytes(st.blob("blk.0.attn_q.weight")) == new_q
            assert bytes(st.blob("blk.0.attn_k.weight")) == TENSORS["blk.0.attn_k.weight"][1]
            assert list(st.tensor_overlays) == ["blk.0.attn_q.weight"]
            assert st.expert_overlays["blk.0.ffn_gate_up_exps.weight"].nbytes == 77
            assert bytes(st.expert_overlay_blob("blk.0.ffn_gate_up_exps.weight")) == b"\x01" * 77
            assert st.expert_overlay_blob("blk.0.attn_q.weight") is None
            got = {n: (d, b) for n, d, _, b in _cpp_records(lib, h)}
            assert got["blk.0.attn_q.weight"] == ("NINT5", new_q)
            assert got["blk.0.attn_k.weight"][1] == TENSORS["blk.0.attn_k.weight"][1]
        finally:
            st.close()
            lib.mfq_rt_file_close(h)
        monkeypatch.delenv("MFQ_TENSOR_OVERLAY", raising=False)
        monkeypatch.delenv("MFQ_EXPERT_OVERLAY", raising=False)
    unknown = tmp_path / "unknown.mfq"
    F.write_mfq(unknown, {"no.such.weight": ("NINT4", b"abc")}, "tiny-arch", 2)
    _both_fail(paths[0], "tensor overlay replaces an unknown record", tmp_path, tensor_overlay=str(unknown))
    sharded = F.write_mfq_shards(tmp_path / "ov.mfq", {"blk.0.attn_q.weight": ("NINT4", b"x"), "blk.0.attn_k.weight": ("NINT4", b"y")},
                                 "tiny-arch", split_max_tensors=1)
    # a shard used as an overlay: its header says split.count 2
    with pytest.raises(ValueError, match="sharded MFQ tensor overlays are not supported"):
        F.MfqStore(paths[0], tensor_overlay=str(sharded[0]), expert_overlay="")
    with pytest.raises(RuntimeError, match="sharded MFQ tensor overlays are not supported"):
        lib.mfq_rt_file_close(_cpp_open(lib, paths[0], str(sharded[0]).encode(), b"-"))
    wrong = tmp_path / "wrong.mfq"
    F.write_mfq(wrong, {"blk.0.attn_q.weight": ("NINTMD", b"abc")}, "tiny-arch", 2)      # base record is not NINTM
    _both_fail(paths[0], "invalid expert overlay record", tmp_path, expert_overlay=str(wrong))


def test_metadata_edge_cases(tmp_path):
    """Duplicate metadata keys and non-integer split values are errors; a version 1 file has no metadata."""
    p = tmp_path / "v1.mfq"
    F.write_mfq(p, {"w": ("NINT4", b"1234")}, "a", 1)
    with F.MfqStore(p, "", "") as st:
        assert st.extra == {} and st.version == 1 and bytes(st.blob("w")) == b"1234"
    head = b"MFQ1" + struct.pack("<II", 2, 1) + b"a" + struct.pack("<I", 2)
    kv = struct.pack("<I", 1) + b"k" + struct.pack("<I", 1) + b"1"
    dup = tmp_path / "dupkey.mfq"
    dup.write_bytes(head + kv + kv + struct.pack("<I", 0))
    _both_fail(dup, "duplicate MFQ metadata key", tmp_path)
    bad = tmp_path / "bad-00001-of-00002.mfq"
    k = b"split.count"
    bad.write_bytes(b"MFQ1" + struct.pack("<II", 2, 1) + b"a" + struct.pack("<I", 1) + struct.pack("<I", len(k)) + k +
                    struct.pack("<I", 3) + b'"x"' + struct.pack("<I", 0))
    _both_fail(bad, "invalid", tmp_path)
