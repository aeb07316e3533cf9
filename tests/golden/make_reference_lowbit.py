"""Write reference-made blobs and reference-dequantized values of the 1-bit families (NVQ1-L, NVQ1-S, NPQ0-L, NPQ0-S and
the expert forms NEPQ0-S, NEPQ0-L).

As make_reference_blobs.py: the reference's own format modules are imported IN THE BUILD CONTAINER ONLY (from
/root/reference: mfq.formats.{nvq1_l,nvq1_s,npq0_l,npq0_s,nepq} and the dequantizers of mfq.quantize.{nvq1_l_quant,
nvq1_s_quant,npq0_l,npq0_s}; numpy and CPU torch, nothing else), fed seeded random fields from tests/synth.py, and the
fields, the packed bytes and the dequantized arrays are stored in tests/golden/reference_lowbit.npz.  The fixture is data;
the reference never travels.

    python tests/golden/make_reference_lowbit.py
"""
import sys
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
sys.path.insert(0, str(HERE.parent))
sys.path.insert(0, str(HERE.parents[1]))
import synth  # noqa: E402

sys.path.insert(0, "/root/reference")
from mfq.formats import npq0_l as f_pl  # noqa: E402
from mfq.formats import npq0_s as f_ps  # noqa: E402
from mfq.formats import nvq1_l as f_vl  # noqa: E402
from mfq.formats import nvq1_s as f_vs  # noqa: E402
from mfq.quantize import npq0_l as q_pl  # noqa: E402
from mfq.quantize import npq0_s as q_ps  # noqa: E402
from mfq.quantize import nvq1_l_quant as q_vl  # noqa: E402
from mfq.quantize import nvq1_s_quant as q_vs  # noqa: E402

out = {}
rng = np.random.default_rng(2025)


def put(key, **arrays):
    for name, a in arrays.items():
        out[f"{key}_{name}"] = np.asarray(a)


def blob_array(b):
    return np.frombuffer(bytes(b), dtype=np.uint8)


# NVQ1-L: built-in grid with 3-bit scales and a K that is not a multiple of 8 or 24; custom grid with 4-bit scales
for key, (rows, K, sbits, custom) in {"nvq1l_grid": (5, 100, 3, False), "nvq1l_custom": (3, 200, 4, True)}.items():
    t = synth.nvq1_random(rng, "NVQ1-L", rows, K, sbits, custom)
    rt = f_vl.Nvq1LTensor(spec=f_vl.Nvq1LSpec(groupsize=24, sub_bits=sbits), shape=t.shape, axis=0, neuron_len=K,
                          neuron_scale=t.neuron_scale, sub_scale=t.sub_scale, indices=t.indices, delta_sign=t.delta_sign,
                          codebook=t.codebook)
    put(key, meta=[rows, K, sbits, int(custom)], ns=t.neuron_scale, sub=t.sub_scale, idx=t.indices, dsg=t.delta_sign,
        cb=t.codebook if custom else np.zeros(0, np.int8), blob=blob_array(f_vl.pack_nvq1_l(rt)), deq=q_vl.dequantize(rt))

# NVQ1-S: the bank follows the delta sign; default table and a custom one
for key, (rows, K, custom) in {"nvq1s_default": (5, 104, False), "nvq1s_custom": (3, 200, True)}.items():
    t = synth.nvq1_random(rng, "NVQ1-S", rows, K, custom=custom)
    rt = f_vs.Nvq1STensor(spec=f_vs.NVQ1_S, shape=t.shape, axis=0, neuron_len=K, neuron_scale=t.neuron_scale,
                          sub_scale=t.sub_scale, indices=t.indices, delta_sign=t.delta_sign, codebook=t.codebook)
    put(key, meta=[rows, K, int(custom)], ns=t.neuron_scale, sub=t.sub_scale, idx=t.indices, dsg=t.delta_sign,
        cb=t.codebook if custom else np.zeros(0, np.int8), blob=blob_array(f_vs.pack_nvq1_s(rt)), deq=q_vs.dequantize(rt))

# NPQ0-L / NPQ0-S: product codebooks chosen by the group state
for key, label, fmod, qdeq, cls, (rows, K) in (("npq0l", "NPQ0-L", f_pl, q_pl.dequantize_npq0_l, "Npq0LTensor", (5, 104)),
                                               ("npq0s", "NPQ0-S", f_ps, q_ps.dequantize_npq0_s, "Npq0STensor", (4, 200))):
    t = synth.npq0_random(rng, label, rows, K)
    rt = getattr(fmod, cls)(shape=t.shape, axis=0, neuron_len=K, neuron_scale=t.neuron_scale, scale_lut=t.scale_lut,
                            state=t.state, indices=t.indices, first_codebooks=t.first_codebooks,
                            second_codebooks=t.second_codebooks)
    pack = fmod.pack_npq0_l if label == "NPQ0-L" else fmod.pack_npq0_s
    put(key, meta=[rows, K], ns=t.neuron_scale, lut=t.scale_lut, state=t.state, idx=t.indices, first=t.first_codebooks,
        second=t.second_codebooks, blob=blob_array(pack(rt)), deq=qdeq(rt))

# NEPQ0-S / NEPQ0-L: the NEPQ container with NPQ0 tables in its pool; two experts, three tables, K = 200 (three
# super-groups of 96 weights, the last ragged)
from mfq.formats import nepq as f_ne  # noqa: E402

for key, label in {"nepq0s": "NEPQ0-S", "nepq0l": "NEPQ0-L"}.items():
    t = synth.nepq_random(rng, label, 2, 8, 200, 3)
    rt = f_ne.NepqTensor(spec=f_ne.nepq_spec(label), shape=t.shape, neuron_scale=t.neuron_scale, state=t.state,
                         indices=t.indices, aux=t.aux, bank_ids=t.bank_ids, table_payloads=t.table_payloads)
    put(key, meta=list(t.shape) + [3], anchors=t.neuron_scale, state=t.state, indices=t.indices, aux=t.aux,
        bank_ids=t.bank_ids, tables=t.table_payloads, blob=blob_array(f_ne.pack_nepq(rt)), deq=f_ne.dequantize_nepq(rt))

np.savez_compressed(HERE / "reference_lowbit.npz", **out)
print("wrote", HERE / "reference_lowbit.npz", len(out), "arrays")
