"""NINT weight-only tensor quantizer and its expert-wise form (host side, numpy), processed in row chunks.

Mirrors nint_quant.quantize with importance=None (mfq/quantize/nint_quant.py:745-823, 883-893) and
its per-group affine search make_qkx2 (mfq/formats/nint.py:119-174): per neuron row, groups of `gs`
weights get a weighted-least-squares (scale, min) pair, the row keeps two fp16 anchors and every
group a `sub_bits`-bit fraction of each.  Returns packed-domain arrays ready for formats.nint_blob.
"""
from __future__ import annotations

import numpy as np


def _group_affine(x: np.ndarray, w: np.ndarray, nmax: int):
    rmin, rdelta, nstep = (-1.0, 0.1, 20) if nmax <= 15 else (-0.5, 0.1, 15)
    mn = np.minimum(x.min(-1), 0.0)
    mx = x.max(-1)
    sum_w = w.sum(-1)
    sum_x = (w * x).sum(-1)
    degen = (mx == mn) | (sum_w <= 0)
    span = np.where(degen, 1.0, mx - mn)
    shifted = x - mn[..., None]

    def levels(iscale):
        return np.clip(np.rint(iscale[..., None] * shifted), 0, nmax).astype(np.int32)

    iscale0 = nmax / span
    best_scale = 1.0 / iscale0
    best_min = mn.copy()
    d0 = best_scale[..., None] * levels(iscale0) + mn[..., None] - x
    best_err = (w * d0 * d0).sum(-1)
    for step in range(nstep + 1):
        L = levels((rmin + rdelta * step + nmax) / span)
        Lf = L.astype(np.float32)
        sl, sl2, sxl = (w * Lf).sum(-1), (w * Lf * Lf).sum(-1), (w * Lf * x).sum(-1)
        det = sum_w * sl2 - sl * sl
        ok = det > 0
        dets = np.where(ok, det, 1.0)
        scale = (sum_w * sxl - sum_x * sl) / dets
        zero = (sl2 * sum_x - sl * sxl) / dets
        above = zero > 0                      # the minimum may not be positive: refit the scale alone
        scale = np.where(above, sxl / np.where(sl2 > 0, sl2, 1.0), scale)
        zero = np.where(above, 0.0, zero)
        resid = scale[..., None] * L + zero[..., None] - x
        err = (w * resid * resid).sum(-1)
        take = ok & (err < best_err)
        best_err = np.where(take, err, best_err)
        best_scale = np.where(take, scale, best_scale)
        best_min = np.where(take, zero, best_min)
    best_scale = np.where(degen, 0.0, best_scale)
    best_min = np.where(degen, np.minimum(mn, 0.0), best_min)
    return best_scale.astype(np.float32), best_min.astype(np.float32)


def nint_quantize(weight, bits: int = 4, gs: int = 24, sub_bits: int = 6, row_chunk: int = 512):
    """weight [out, K] fp32 -> dict(ns, nm fp32 [out] (fp16-representable), ss, sm u8 [out, ng], q u8 [out, ng, gs])."""
    bits, gs, sub_bits = int(bits), int(gs), int(sub_bits)
    W = np.asarray(weight, dtype=np.float32)
    if W.ndim != 2:
        raise ValueError(f"nint_quantize expects a rank-2 [out, in] weight, got shape {W.shape}")
    out, K = W.shape
    nmax, kmax = (1 << bits) - 1, (1 << sub_bits) - 1
    pad = (-K) % gs
    ng = (K + pad) // gs
    ns = np.empty(out, np.float32)
    nm = np.empty(out, np.float32)
    ss = np.empty((out, ng), np.uint8)
    sm = np.empty((out, ng), np.uint8)
    q = np.empty((out, ng, gs), np.uint8)
    for r0 in range(0, out, row_chunk):
        rows = W[r0: r0 + row_chunk]
        if pad:
            rows = np.concatenate([rows, np.zeros((rows.shape[0], pad), np.float32)], axis=1)
        g = rows.reshape(rows.shape[0], ng, gs)
        wts = np.sqrt((g * g).sum(-1) / gs)[..., None] + np.abs(g)
        if pad:
            wts[:, -1, gs - pad:] = 0.0        # padded tail weights do not steer the fit
        scale, zp = _group_affine(g, wts, nmax)
        the_min = -zp
        top_s, top_m = scale.max(-1), the_min.max(-1)
        d = np.where(top_s > 0, (top_s / kmax).astype(np.float16).astype(np.float32), np.float32(0.0))
        dm = np.where(top_m > 0, (top_m / kmax).astype(np.float16).astype(np.float32), np.float32(0.0))
        sub_s = np.clip(np.rint(kmax * scale / np.where(top_s > 0, top_s, 1.0)[..., None]), 0, kmax)
        sub_m = np.clip(np.rint(kmax * the_min / np.where(top_m > 0, top_m, 1.0)[..., None]), 0, kmax)
        d_eff = d[:, None] * sub_s.astype(np.float32)
        m_eff = dm[:, None] * sub_m.astype(np.float32)
        codes = np.clip(np.rint((g + m_eff[..., None]) / np.where(d_eff > 0, d_eff, 1.0)[..., None]), 0, nmax)
        sl = slice(r0, r0 + rows.shape[0])
        ns[sl], nm[sl], ss[sl], sm[sl], q[sl] = d, dm, sub_s, sub_m, codes
    return {"ns": ns, "nm": nm, "ss": ss, "sm": sm, "q": q, "bits": bits, "gs": gs, "sub_bits": sub_bits,
            "neuron_len": K}


def nint_quantize_expertwise(weight, profiles, row_chunk: int = 512):
    """weight [experts, out, K] fp32 and one (bits, groupsize, sub_bits) per expert -> (pools, blob).

    Mirrors quantize_expertwise for NINT precisions (mfq/quantize/expert_nint.py:507-578): the experts of one precision
    form a cohort -- cohorts in the order their precision first appears, experts ascending inside a cohort -- whose rows
    are flattened to [n * out, K] and quantized like a dense tensor.  `pools` is a list of (expert_ids int32,
    dtype string, dict as nint_quantize returns); `blob` the NIM2 payload holding them (mfq/formats/io.py:304-336).
    """
    from . import formats as F

    W = np.asarray(weight, dtype=np.float32)
    if W.ndim != 3:
        raise ValueError("expert-wise quantization expects [experts, out, in]")
    E, out, K = W.shape
    profiles = [tuple(int(v) for v in p) for p in profiles]
    if len(profiles) != E:
        raise ValueError(f"received {len(profiles)} precision descriptors for {E} experts")
    cohorts: dict = {}
    for e, prof in enumerate(profiles):
        cohorts.setdefault(prof, []).append(e)
    pools, packed = [], []
    for (bits, gs, sub_bits), members in cohorts.items():
        ids = np.asarray(members, dtype=np.int32)
        r = nint_quantize(W[ids].reshape(ids.size * out, K), bits, gs, sub_bits, row_chunk)
        pools.append((ids, f"NINT{bits}", r))
        packed.append((ids, f"NINT{bits}", F.nint_blob(bits, sub_bits, gs, K, r["ns"], r["nm"], r["ss"], r["sm"], r["q"])))
    return pools, F.nintm_blob(E, out, K, packed)
