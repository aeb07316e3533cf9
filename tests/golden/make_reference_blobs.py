"""Write reference-made packed blobs and their reference-dequantized values for tiny hand-built tensors.

Round trips of one's own packer and parser cannot catch a mistake both share (stream order inside a blob, which
96 weights a NEPQ bank id covers, how the index-parity sign bit is formed).  This script imports the reference's
own format modules IN THE BUILD CONTAINER ONLY (from /root/reference: mfq.formats.{io,nvq,nepq,moe},
mfq.quantize.{nint_quant,nvq_jsc,nvq_quant,expert_nint}; numpy and CPU torch, nothing else), builds small tensors
from seeded random fields, and stores for each: the fields, the bytes the reference packs them into, and the fp32
array the reference dequantizes them to.  The fixture (tests/golden/reference_blobs.npz) is data; the reference
itself never travels.

    python tests/golden/make_reference_blobs.py
"""
import sys
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
sys.path.insert(0, str(HERE.parent))          # tests/synth.py: the seeded field generators
sys.path.insert(0, str(HERE.parents[1]))
import synth  # noqa: E402

sys.path.insert(0, "/root/reference")
from mfq.formats import io as rio  # noqa: E402
from mfq.formats import moe as rmoe  # noqa: E402
from mfq.formats import nepq as rnepq  # noqa: E402
from mfq.formats import nvq as rnvq  # noqa: E402
from mfq.formats.nint import NintSpec  # noqa: E402
from mfq.quantize import nint_quant  # noqa: E402
from mfq.quantize import nvq_jsc  # noqa: E402
from mfq.quantize import nvq_quant  # noqa: E402
from mfq.quantize.expert_nint import dequantize_expertwise  # noqa: E402

out = {}


def put(key, **arrays):
    for name, a in arrays.items():
        out[f"{key}_{name}"] = np.asarray(a)


def blob_array(b):
    return np.frombuffer(bytes(b), dtype=np.uint8)


def ref_nint(t):
    return nint_quant.NintTensor(spec=NintSpec(bits=t.bits, groupsize=t.groupsize, sub_bits=t.sub_bits), shape=t.shape,
                                 axis=0, q=t.q, neuron_scale=t.neuron_scale, neuron_min=t.neuron_min,
                                 sub_scale=t.sub_scale, sub_min=t.sub_min, neuron_len=t.neuron_len)


rng = np.random.default_rng(2024)

# ---- NINT: odd width (3 bit), K past two groups with a ragged tail; and NINT4-32 ------------------------------
for key, (rows, K, bits, gs, sb) in {"nint3": (5, 100, 3, 24, 5), "nint4": (7, 200, 4, 32, 6), "nint5": (3, 60, 5, 28, 7)}.items():
    t = synth.nint_random(rng, rows, K, bits, gs, sb)
    rt = ref_nint(t)
    put(key, meta=[rows, K, bits, gs, sb], q=t.q, ns=t.neuron_scale, nm=t.neuron_min, ss=t.sub_scale, sm=t.sub_min,
        blob=blob_array(rio.pack_nint(rt)), deq=nint_quant.dequantize(rt))

# ---- NVQ-JSC: NVQ3J-512 (two banks) and NVQ3J (d4_256, two banks), K = 200 (ragged last group and vector) ---------
SPECS = {"d4_512": rnvq.NVQ3_D4_512, "d4_256": rnvq.NVQ3_D4}
for key, (rows, K, codebook, banks) in {"nvq3j512": (6, 200, "d4_512", 2), "nvq3j": (4, 100, "d4_256", 2)}.items():
    t = synth.nvq_jsc_random(rng, rows, K, codebook, banks)
    rt = rnvq.NvqJscTensor(shape=(rows, K), axis=0, neuron_len=K, neuron_scale=t.neuron_scale, scale_lut=t.scale_lut,
                           bank_for_state=t.bank_for_state, state=t.state, indices=t.indices, signs=t.signs,
                           codebooks=t.codebooks, base_spec=SPECS[codebook])
    put(key, meta=[rows, K, banks], codebook=np.frombuffer(codebook.encode(), dtype=np.uint8), anchors=t.neuron_scale,
        lut=t.scale_lut, bank_for_state=t.bank_for_state, state=t.state, indices=t.indices, signs=t.signs,
        codebooks=t.codebooks, blob=blob_array(rnvq.pack_nvq(rt)), deq=nvq_jsc.dequantize_nvq_jsc(rt))

# ---- plain NVQ3 (d4_256, integer relative scale) and NVQ2 with the index-parity sign rule (e8_256) ------------------
t = synth.nvq_plain_random(rng, 5, 104)
rt = rnvq.NvqTensor(spec=rnvq.NVQ3_D4, shape=(5, 104), axis=0, neuron_len=104, neuron_scale=t.neuron_scale,
                    sub_scale=t.sub_scale, indices=t.indices, signs=t.signs)
put("nvq3", meta=[5, 104], anchors=t.neuron_scale, sub_scale=t.sub_scale, indices=t.indices, signs=t.signs,
    blob=blob_array(rnvq.pack_nvq(rt)), deq=nvq_quant.dequantize(rt))
rows, K = 4, 72
spec_ip = rnvq.NvqSpec("e8_256", groupsize=24, sub_bits=4, sign_mode="index_parity")
fields = dict(anchors=rng.uniform(0.0002, 0.002, rows).astype(np.float16).astype(np.float32),
              sub_scale=rng.integers(0, 16, (rows, K // 24), dtype=np.uint8),
              indices=rng.integers(0, 256, (rows, K // 8)).astype(np.uint16),
              signs=rng.integers(0, 128, (rows, K // 8), dtype=np.uint8))
rt = rnvq.NvqTensor(spec=spec_ip, shape=(rows, K), axis=0, neuron_len=K, neuron_scale=fields["anchors"],
                    sub_scale=fields["sub_scale"], indices=fields["indices"], signs=fields["signs"])
put("nvq2ip", meta=[rows, K], blob=blob_array(rnvq.pack_nvq(rt)), deq=nvq_quant.dequantize(rt), **fields)

# ---- NEPQ1-S / NEPQ1-L: two experts, K = 200 (three super-groups of 96 weights, ragged), three banks ----------------
for key, label in {"nepq1s": "NEPQ1-S", "nepq1l": "NEPQ1-L"}.items():
    t = synth.nepq_random(rng, label, 2, 8, 200, 3)
    rt = rnepq.NepqTensor(spec=rnepq.nepq_spec(label), shape=t.shape, neuron_scale=t.neuron_scale, state=t.state,
                          indices=t.indices, aux=t.aux, bank_ids=t.bank_ids, table_payloads=t.table_payloads)
    put(key, meta=list(t.shape) + [3], anchors=t.neuron_scale, state=t.state, indices=t.indices, aux=t.aux,
        bank_ids=t.bank_ids, tables=t.table_payloads, blob=blob_array(rnepq.pack_nepq(rt)), deq=rnepq.dequantize_nepq(rt))

# ---- NINTM (NIM2): four experts in two cohorts, ids not in order ----------------------------------------------------
E, rows, K = 4, 16, 96
bits = [4, 3, 3, 4]
mt = synth.moe_random(rng, E, rows, K, bits)
pools = tuple(rmoe.NintMoePool(expert_ids=p.expert_ids, tensor=ref_nint(p.tensor)) for p in mt.pools)
rm = rmoe.NintMoeTensor(shape=(E, rows, K), pools=pools)
put("nintm", meta=[E, rows, K], bits=bits, blob=blob_array(rio.pack_nint_moe(rm)), deq=dequantize_expertwise(rm))
for pi, p in enumerate(mt.pools):
    put(f"nintm_pool{pi}", ids=p.expert_ids, q=p.tensor.q, ns=p.tensor.neuron_scale, nm=p.tensor.neuron_min,
        ss=p.tensor.sub_scale, sm=p.tensor.sub_min)

np.savez_compressed(HERE / "reference_blobs.npz", **out)
print("wrote", len(out), "arrays,", sum(a.nbytes for a in out.values()), "bytes")
