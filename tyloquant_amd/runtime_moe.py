"""Expert-wise mixed-bit MoE: NINTM weights, the route plan and the FFN forward (see runtime.py)."""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import numpy as np
import torch

from . import _lib as L
from . import formats as F
from .runtime import NintWeight, _Workspace, _ptr, _stream, _x_dtype, nint_matmul

_MODE = {"softmax": L.TOPK_SOFTMAX, "sigmoid": L.TOPK_SIGMOID, "sqrt_softplus": L.TOPK_SQRT_SOFTPLUS,
         "delayed_softmax": L.TOPK_DELAYED_SOFTMAX}


def moe_topk(logits: torch.Tensor, top_k: int, use_sigmoid=False, use_sqrt_softplus=False, normalize=False,
             delayed_softmax=False, bias: torch.Tensor | None = None, norm_floor=1e-20, scale=1.0):
    """moe_topk_cuda (mfq/kernels/cuda/moe.cu:3552-3637): returns (ids int32 [T,k], weights f32 [T,k])."""
    if logits.dim() != 2 or not logits.is_cuda:
        raise ValueError("logits must be contiguous CUDA [tokens, experts]")
    if normalize and delayed_softmax:
        raise ValueError("selected-weight normalization and delayed softmax are mutually exclusive")
    if sum((use_sigmoid, use_sqrt_softplus, delayed_softmax)) > 1:
        raise ValueError("sigmoid, sqrt-softplus and delayed-softmax routing are mutually exclusive")
    logits = logits.float().contiguous()
    T, E = logits.shape
    if not 1 <= top_k <= min(16, E):
        raise ValueError("top_k must be in [1, min(16, experts)]")
    mode = L.TOPK_DELAYED_SOFTMAX if delayed_softmax else L.TOPK_SIGMOID if use_sigmoid else \
        L.TOPK_SQRT_SOFTPLUS if use_sqrt_softplus else L.TOPK_SOFTMAX
    if bias is not None:
        bias = bias.float().contiguous()
        if bias.numel() != E:
            raise ValueError("bias must be contiguous CUDA float32 [experts]")
    ids = torch.empty((T, top_k), dtype=torch.int32, device=logits.device)
    w = torch.empty((T, top_k), dtype=torch.float32, device=logits.device)
    L.check(L.lib().mfq_hip_moe_topk(_ptr(logits), _ptr(bias), T, E, top_k, mode, int(normalize), norm_floor, scale,
                                     _ptr(ids), _ptr(w), _stream()))
    return ids, w


@dataclass
class MoeRoutePlan:
    """cpp_runtime/mfq_decode.cpp:2579-2592."""
    ids: torch.Tensor
    n_experts: int
    ids_dst: torch.Tensor | None = None
    expert_bounds: torch.Tensor | None = None
    tile_bounds: torch.Tensor | None = None
    tile_experts: torch.Tensor | None = None
    counts: torch.Tensor | None = None
    map_ready: bool = False

    @property
    def tokens(self):
        return self.ids.shape[0]

    @property
    def routes(self):
        return self.ids.shape[1]


def build_expert_map(ids: torch.Tensor, n_experts: int, tile_m: int):
    """moe_build_expert_map_cuda (mfq/kernels/cuda/moe.cu:3082-3130)."""
    n_pairs = ids.numel()
    dev = ids.device
    max_tiles = -(-n_pairs // tile_m) + n_experts
    counts = torch.empty(n_experts, dtype=torch.int32, device=dev)
    eb = torch.empty(n_experts + 1, dtype=torch.int32, device=dev)
    tb = torch.empty(n_experts + 1, dtype=torch.int32, device=dev)
    te = torch.zeros(max_tiles, dtype=torch.int32, device=dev)
    dst = torch.zeros(n_pairs, dtype=torch.int32, device=dev)
    L.check(L.lib().mfq_hip_moe_route_map(_ptr(ids), n_pairs, n_experts, tile_m, _ptr(counts), _ptr(eb), _ptr(tb),
                                          _ptr(te), max_tiles, _ptr(dst), _stream()))
    return dst, eb, tb, te, counts


def build_moe_route_plan(ids: torch.Tensor, n_experts: int) -> MoeRoutePlan:
    """cpp_runtime/mfq_decode.cpp:2681-2708: the expert map is built only above 8 tokens."""
    if not ids.is_cuda or ids.dtype != torch.int32 or ids.dim() != 2:
        raise RuntimeError("MoE ids must be CUDA int32 [tokens, routes]")
    plan = MoeRoutePlan(ids.contiguous(), n_experts)
    if plan.tokens > 8:
        plan.ids_dst, plan.expert_bounds, plan.tile_bounds, plan.tile_experts, plan.counts = build_expert_map(
            plan.ids, n_experts, L.lib().mfq_hip_moe_tile_m())
    plan.map_ready = True
    return plan


class ForeignCohort:
    """A NINTM cohort of another family (NVQ, the 1-bit families, NEPQ, MXFP4): the reference runs them inside its grouped
    kernels (cpp_runtime/mfq_decode.cpp:4800-5360, mfq/kernels/cuda/nvq_matmul.cu:2588-3175); here every expert is a
    tensor of its own on that family's kernels and the host walks the experts a batch routes to -- correct, one matmul
    per expert hit, not a fast path."""

    def __init__(self, dtype, blob, expert_ids, out_per_expert, neuron_len, device):
        from .runtime import is_nepq_linear_dtype, load_quant_linear
        self.dtype, self.expert_ids = dtype, np.asarray(expert_ids, dtype=np.int32)
        self.out, self.neuron_len = out_per_expert, neuron_len
        n = len(self.expert_ids)
        self.nepq, self.mx, self.linears = None, None, []
        if F.is_mx_dtype(dtype):               # a pool is one [experts * out, K] tensor (mfq/formats/moe.py:122-124)
            from .runtime_mx import MxWeight
            h = F.parse_mx(dtype, blob)
            if (h.rows, h.cols) != (n * out_per_expert, neuron_len):
                raise ValueError(f"NINTM pool tensor shape {(h.rows, h.cols)} must be {(n * out_per_expert, neuron_len)}")
            self.mx = MxWeight.from_blob(dtype, blob, device, out=out_per_expert)
            shape = (n, out_per_expert, neuron_len)
        elif is_nepq_linear_dtype(dtype):
            from .runtime_vq import NepqWeight
            self.nepq = NepqWeight.from_blob(blob, device)
            if self.nepq.label != dtype:
                raise ValueError(f"MFQ dtype/blob mismatch: {dtype} contains {self.nepq.label}")
            shape = (self.nepq.n_experts, self.nepq.out_per_expert, self.nepq.neuron_len)
        else:
            self.linears = [load_quant_linear(dtype, b, device) for b in F.split_rows(dtype, blob, n)]
            shape = (n, self.linears[0].out, self.linears[0].neuron_len)
        if shape != (n, out_per_expert, neuron_len):
            raise ValueError(f"NINTM pool tensor shape {shape} must be {(n, out_per_expert, neuron_len)}")
        self._slot = self._wtab = None           # device tables of the one-launch decode form, built on first use
        self.live = np.ones(n, dtype=bool)       # experts an expert overlay has not given to a later cohort

    PAIRS_MAX = 64   # (token, route) pairs up to which a decode step takes one launch per cohort over all its pairs

    def matmul_pairs(self, n_experts: int, x2: torch.Tensor, routed: bool, ids: torch.Tensor, T: int, R: int,
                     flat: torch.Tensor) -> None:
        """flat[p] = W[ids[p]] . x2[p or p // R] for the pairs routed to this cohort, in one launch that reads the routing
        table on the device (mfq_hip_{nvq,nvqs,nepq,nint8z,mx}_gemv_pairs); the rows of other pairs are left alone."""
        from .runtime import Nint8ZeroWeight
        from .runtime_vq import NvqsWeight, nepq_hadamard
        lib, dev = L.lib(), x2.device
        if self._slot is None:
            slot = np.full(n_experts, -1, dtype=np.int32)
            slot[self.expert_ids[self.live]] = np.arange(len(self.expert_ids), dtype=np.int32)[self.live]
            self._slot = torch.from_numpy(slot).to(dev)
            if self.linears:
                self._wtab = torch.tensor([q.weight.data.data_ptr() for q in self.linears], dtype=torch.int64, device=dev)
        common = (_ptr(self._slot), n_experts)
        if self.nepq is not None and self.nepq.rotation_block:
            x2 = nepq_hadamard(x2, self.nepq.signs, self.nepq.rotation_block)
        tail = (_ptr(x2), _x_dtype(x2), x2.stride(0), int(routed), _ptr(ids), T, R, _ptr(flat), flat.stride(0), _stream())
        if self.mx is not None:
            w = self.mx
            L.check(lib.mfq_hip_mx_gemv_pairs(w.kind, _ptr(w.values), _ptr(w.scales), w.rows, w.neuron_len, self.out, *common, *tail))
        elif self.nepq is not None:
            w = self.nepq
            if w.streams:
                L.check(lib.mfq_hip_nvqs_gemv_pairs(C.byref(w.desc), None, _ptr(w.data), self.out, *common, *tail))
            else:
                L.check(lib.mfq_hip_nepq_gemv_pairs(C.byref(w.desc), _ptr(w.data), self.out, *common, *tail))
        else:
            w0 = self.linears[0].weight
            if isinstance(w0, Nint8ZeroWeight):
                L.check(lib.mfq_hip_nint8z_gemv_pairs(C.byref(w0.desc), _ptr(self._wtab), *common, *tail))
            elif isinstance(w0, NvqsWeight):
                L.check(lib.mfq_hip_nvqs_gemv_pairs(C.byref(w0.desc), _ptr(self._wtab), None, self.out, *common, *tail))
            else:
                L.check(lib.mfq_hip_nvq_gemv_pairs(C.byref(w0.desc), _ptr(self._wtab), *common, *tail))

    def pairs_capable(self) -> bool:
        """Whether matmul_pairs takes this cohort: every family has the launch; NEPQ1 experts must be whole row-blocks."""
        return not (self.nepq is not None and not self.nepq.streams and self.out % 16)

    @property
    def payload_bytes(self) -> int:
        if self.mx is not None:
            return self.mx.payload_bytes
        return self.nepq.payload_bytes if self.nepq is not None else sum(q.weight.payload_bytes for q in self.linears)

    def matmul(self, local: int, x: torch.Tensor) -> torch.Tensor:
        if self.mx is not None:
            from .runtime_mx import mx_matmul
            return mx_matmul(self.mx, x, local)
        if self.nepq is not None:
            from .runtime_vq import nepq_matmul
            return nepq_matmul(self.nepq, x, local)
        return self.linears[local](x)

    def dequantize(self) -> torch.Tensor:
        if self.mx is not None:
            return torch.stack([self.mx.dequantize(e) for e in range(self.mx.n_experts)])
        if self.nepq is not None:
            return self.nepq.dequantize().reshape(len(self.expert_ids), self.out, self.neuron_len)
        return torch.stack([q.dequantize() for q in self.linears])


class NintMoeWeight:
    """One logical [experts, out_per_expert, K] tensor made of cohorts (NINTM / NIM2).  NINT cohorts run on the grouped
    kernels; cohorts of other families (`foreign`) are added by the host, expert by expert."""

    def __init__(self, n_experts, out_per_expert, neuron_len, pools, expert_ids, device, foreign=(), pool_live=None):
        """pool_live[i]: which experts of NINT cohort i the cohort still owns (all of them unless an expert overlay gave
        some to a later cohort); cohorts of other families carry the same mask as `live`."""
        self.n_experts, self.out_per_expert, self.neuron_len = n_experts, out_per_expert, neuron_len
        self.pools: list[NintWeight] = pools
        self.pool_expert_ids = expert_ids
        self.pool_live = pool_live if pool_live is not None else [np.ones(len(ids), dtype=bool) for ids in expert_ids]
        self.foreign: list[ForeignCohort] = list(foreign)
        ep = np.full(n_experts, -1, dtype=np.int32)       # -1: no NINT cohort -- the kernels leave a zero row
        el = np.full(n_experts, -1, dtype=np.int32)
        for pi, (ids, live) in enumerate(zip(expert_ids, self.pool_live)):
            ep[ids[live]] = pi
            el[ids[live]] = np.arange(len(ids), dtype=np.int32)[live]
        # device dispatch tables (initialize_nint_moe_dispatch, cpp_runtime/mfq_decode.cpp:3249-3343)
        self.expert_pool = torch.from_numpy(ep).to(device)
        self.expert_local = torch.from_numpy(el).to(device)
        self._pool_array = (L.MoePool * max(len(pools), 1))()
        for i, p in enumerate(pools):
            self._pool_array[i].desc = p.desc
            self._pool_array[i].weight = p.data.data_ptr()
        self._ws = _Workspace()
        self.expert_bits = np.zeros(n_experts, dtype=np.int32)
        for pi, (ids, live) in enumerate(zip(expert_ids, self.pool_live)):
            self.expert_bits[ids[live]] = pools[pi].bits

    @property
    def payload_bytes(self) -> int:
        return sum(p.payload_bytes for p in self.pools) + sum(c.payload_bytes for c in self.foreign)

    def expert_payload_bytes(self, e: int) -> float:
        pi = int(self.expert_pool[e].item())
        if pi < 0:
            c = next(c for c in self.foreign if e in c.expert_ids[c.live])
            return c.payload_bytes / len(c.expert_ids)
        return self.pools[pi].payload_bytes / len(self.pool_expert_ids[pi])

    @staticmethod
    def from_blob(blob, device="cuda", expert_overlay=None) -> "NintMoeWeight":
        """expert_overlay: the NINTMD record of the same name from an expert overlay file (MfqFile.expert_overlays): its
        cohorts are appended and take over the experts they list (load_nint_moe_cpu, cpp_runtime/mfq_decode.cpp:5752-5774)."""
        h = F.parse_nintm(blob)
        cohorts = [(blob, p) for p in h.pools]
        if expert_overlay is not None:
            d = F.parse_nintm(expert_overlay, allow_partial=True)
            if (d.n_experts, d.out_per_expert, d.neuron_len) != (h.n_experts, h.out_per_expert, h.neuron_len):
                raise ValueError("expert overlay shape mismatch")
            cohorts += [(expert_overlay, p) for p in d.pools]
        owner = np.full(h.n_experts, -1, dtype=np.int64)        # the last cohort that lists an expert owns it
        for ci, (_, p) in enumerate(cohorts):
            owner[p.expert_ids] = ci
        device = torch.device(device)
        pools, ids, pool_live = [], [], []
        foreign = []
        for ci, (blob, p) in enumerate(cohorts):
            live = owner[p.expert_ids] == ci
            if p.runtime_bytes:
                raise ValueError("unexpected NINTM cohort runtime metadata")
            if not (p.dtype.startswith("NINT") and p.dtype[4:].isdigit()):
                from .runtime import is_nepq_linear_dtype, is_nvq_linear_dtype
                if p.dtype == "MXFP8":      # expert_tensor_family, mfq/formats/moe.py:38-47
                    raise ValueError(f"NINTM supports native MXFP4 expert pools, got {p.dtype}")
                if not (is_nvq_linear_dtype(p.dtype) or is_nepq_linear_dtype(p.dtype) or F.is_lowbit_dtype(p.dtype)
                        or p.dtype in ("MXFP4", "NINT8-0")):
                    raise NotImplementedError(f"NINTM cohort family {p.dtype} is not supported")
                foreign.append(ForeignCohort(p.dtype, bytes(blob[p.payload_off: p.payload_off + p.payload_bytes]),
                                             p.expert_ids, h.out_per_expert, h.neuron_len, device))
                foreign[-1].live = live
                continue
            w = NintWeight.from_blob(bytes(blob[p.payload_off: p.payload_off + p.payload_bytes]), device)
            if w.out != len(p.expert_ids) * h.out_per_expert or w.neuron_len != h.neuron_len:
                raise ValueError(f"NINTM pool tensor shape {(w.out, w.neuron_len)} must be "
                                 f"{(len(p.expert_ids) * h.out_per_expert, h.neuron_len)}")
            pools.append(w)
            ids.append(p.expert_ids)
            pool_live.append(live)
        return NintMoeWeight(h.n_experts, h.out_per_expert, h.neuron_len, pools, ids, device, foreign, pool_live)

    def dequantize(self) -> torch.Tensor:
        out = torch.empty((self.n_experts, self.out_per_expert, self.neuron_len), dtype=torch.float32,
                          device=self.expert_pool.device)
        for p, ids, live in zip(self.pools, self.pool_expert_ids, self.pool_live):
            mask = torch.from_numpy(live).to(out.device)
            out[torch.from_numpy(ids[live].astype(np.int64)).to(out.device)] = p.dequantize().reshape(
                len(ids), self.out_per_expert, self.neuron_len)[mask]
        for c in self.foreign:
            mask = torch.from_numpy(c.live).to(out.device)
            out[torch.from_numpy(c.expert_ids[c.live].astype(np.int64)).to(out.device)] = c.dequantize()[mask]
        return out

    def _add_foreign(self, x2: torch.Tensor, routed: bool, route: MoeRoutePlan, out: torch.Tensor) -> None:
        """The rows of the pairs routed to experts of other families: per expert, gather its activation rows, multiply
        on that family's kernels, scatter into `out` [T, R, out_per_expert]; reads the routing table on the host.  A
        decode step (up to ForeignCohort.PAIRS_MAX pairs) instead takes one launch per cohort over all pairs, with the
        routing table read on the device."""
        T, R = route.tokens, route.routes
        flat = out.view(T * R, self.out_per_expert)
        walk = list(self.foreign)
        if T * R <= ForeignCohort.PAIRS_MAX:     # a decode step: one launch per cohort, nothing read back
            for c in [c for c in walk if c.pairs_capable()]:
                c.matmul_pairs(self.n_experts, x2, routed, route.ids, T, R, flat)
                walk.remove(c)
        if not walk:
            return
        ids = route.ids.reshape(T, R).cpu().numpy()
        for c in walk:
            for local, e in enumerate(c.expert_ids):
                if not c.live[local]:
                    continue
                t_idx, r_idx = np.nonzero(ids == e)
                if t_idx.size == 0:
                    continue
                pairs = torch.from_numpy((t_idx * R + r_idx).astype(np.int64)).to(out.device)
                src = pairs if routed else torch.from_numpy(t_idx.astype(np.int64)).to(out.device)
                flat[pairs] = c.matmul(local, x2.index_select(0, src))

    def forward(self, x: torch.Tensor, route: MoeRoutePlan) -> torch.Tensor:
        """NintMoeWeight::forward (cpp_runtime/mfq_decode.cpp:2908-3071): x is [T, K] (shared by the
        routes of a token) or [T, R, K] (routed input); returns fp32 [T, R, out_per_expert]."""
        T, R = route.tokens, route.routes
        routed = x.dim() == 3
        if x.shape[-1] != self.neuron_len or x.shape[0] != T or (routed and x.shape[1] != R):
            raise ValueError("MoE activations must be [tokens, K] or [tokens, routes, K]")
        x2 = x.reshape(-1, self.neuron_len)
        if x2.stride(-1) != 1:
            x2 = x2.contiguous()
        if not self.pools:                              # no NINT cohort at all: every row comes from the host loop
            out = torch.zeros((T, R, self.out_per_expert), dtype=torch.float32, device=x.device)
            self._add_foreign(x2, routed, route, out)
            return out
        out = torch.empty((T, R, self.out_per_expert), dtype=torch.float32, device=x.device)
        mapped = route.ids_dst is not None
        lib = L.lib()
        # a workspace lets the library take the prefill kernel when a mapped call has many pairs per expert
        need = lib.mfq_hip_moe_grouped_workspace_bytes(self._pool_array, len(self.pools), self.neuron_len,
                                                       x2.shape[0]) if mapped else 0
        ws = self._ws.get(need, x.device)
        L.check(lib.mfq_hip_moe_grouped_matmul_ws(
            self._pool_array, len(self.pools), _ptr(self.expert_pool), _ptr(self.expert_local), self.n_experts,
            self.out_per_expert, self.neuron_len, _ptr(x2), _x_dtype(x2), x2.stride(0), int(routed), _ptr(route.ids),
            T, R, _ptr(route.ids_dst) if mapped else None, _ptr(route.expert_bounds) if mapped else None,
            _ptr(route.tile_bounds) if mapped else None, _ptr(route.tile_experts) if mapped else None,
            _ptr(out), self.out_per_expert, _ptr(ws), need, _stream()))
        if self.foreign:
            self._add_foreign(x2, routed, route, out)
        return out

    __call__ = forward

    def forward_glu(self, x: torch.Tensor, route: MoeRoutePlan, activation: int = L.GLU_SILU,
                    out_dtype=torch.float16) -> torch.Tensor:
        """act(gate) * up of the routed gate/up projection as 16-bit [T, R, out_per_expert / 2]
        (NintMoeWeight::forward_glu_output, cpp_runtime/mfq_decode.cpp:3073-3127): one pass of the mapped prefill
        kernels with the GLU in their epilogue; the two-call form (forward, then moe_glu) where the library
        declines -- no route map, a cohort without a prefill body, unaligned activations."""
        T, R = route.tokens, route.routes
        routed = x.dim() == 3
        if x.shape[-1] != self.neuron_len or x.shape[0] != T or (routed and x.shape[1] != R):
            raise ValueError("MoE activations must be [tokens, K] or [tokens, routes, K]")
        if self.out_per_expert % 2:
            raise RuntimeError("fused gate/up GLU needs an even number of neurons per expert")
        W = self.out_per_expert // 2
        if route.ids_dst is not None and self.out_per_expert % 32 == 0 and not self.foreign:
            x2 = x.reshape(-1, self.neuron_len)
            if x2.stride(-1) != 1:
                x2 = x2.contiguous()
            lib = L.lib()
            need = lib.mfq_hip_moe_grouped_workspace_bytes(self._pool_array, len(self.pools), self.neuron_len, x2.shape[0])
            if need:
                ws = self._ws.get(need, x.device)
                hidden = torch.empty((T, R, W), dtype=out_dtype, device=x.device)
                rc = lib.mfq_hip_moe_grouped_glu_ws(
                    self._pool_array, len(self.pools), _ptr(self.expert_pool), _ptr(self.expert_local), self.n_experts,
                    self.out_per_expert, self.neuron_len, _ptr(x2), _x_dtype(x2), x2.stride(0), int(routed),
                    _ptr(route.ids), T, R, _ptr(route.ids_dst), _ptr(route.expert_bounds), int(activation), _ptr(hidden),
                    L.X_F16 if out_dtype == torch.float16 else L.X_BF16, W, _ptr(ws), need, _stream())
                if rc == 0:
                    return hidden
                if rc != L.ERR_UNSUPPORTED:
                    L.check(rc)
        return moe_glu(self.forward(x, route), out_dtype, activation)

    def decode_capable(self, shared: NintWeight | None = None, tokens: int = 1, routes: int = 1, swiglu=False) -> bool:
        """Whether forward_decode takes these cohorts, this shared tensor and this many (token, route) pairs: the
        library's own answer (unit per cohort, shared tensor's shape, the block's LDS need, the row count)."""
        if self.foreign or (shared is not None and shared.neuron_len != self.neuron_len):
            return False
        return bool(L.lib().mfq_hip_moe_decode_capable(
            self._pool_array, len(self.pools), self.out_per_expert, self.neuron_len,
            C.byref(shared.desc) if shared is not None else None, int(tokens), int(routes), int(bool(swiglu))))

    def forward_decode(self, x: torch.Tensor, ids: torch.Tensor, shared: NintWeight | None = None, swiglu=False,
                       routed=False, out_dtype=torch.float16) -> torch.Tensor:
        """One launch for a decode step: rows t * R + r are the routed pairs, rows T * R + t the shared tensor on
        token t.  x is [T, K], or with `routed` [T * R (+ T), K] with one row per output row.  Returns fp32
        [rows, out_per_expert], or with `swiglu` 16-bit [rows, out_per_expert / 2] = silu(gate) * up (swiglu = 2 or
        "gelu": gelu_tanh(gate) * up, the `gelu` flag of forward_glu_output, cpp_runtime/mfq_decode.cpp:3074-3128)."""
        swiglu = 2 if swiglu == "gelu" else int(swiglu)
        T, R = ids.shape
        rows = T * R + (T if shared is not None else 0)
        if x.dim() != 2 or x.shape[1] != self.neuron_len or x.shape[0] != (rows if routed else T):
            raise ValueError("decode activations must be [tokens, K] or one row per output row")
        if x.stride(-1) != 1:
            x = x.contiguous()
        cols = self.out_per_expert // 2 if swiglu else self.out_per_expert
        out = torch.empty((rows, cols), dtype=out_dtype if swiglu else torch.float32, device=x.device)
        L.check(L.lib().mfq_hip_moe_decode_matmul(
            self._pool_array, len(self.pools), _ptr(self.expert_pool), _ptr(self.expert_local), self.n_experts,
            self.out_per_expert, self.neuron_len, _ptr(x), _x_dtype(x), x.stride(0), int(routed), _ptr(ids), T, R,
            C.byref(shared.desc) if shared is not None else None, _ptr(shared.data) if shared is not None else None,
            int(swiglu), _ptr(out), L.X_F16 if out.dtype == torch.float16 else L.X_BF16, cols, _stream()))
        return out


def moe_glu(gate_up: torch.Tensor, out_dtype=torch.float16, activation: int = L.GLU_SILU) -> torch.Tensor:
    """act(gate) * up, gate = first half of the last axis; act = SiLU (moe_swiglu_split_cuda) or, with
    activation = GLU_GELU, the tanh form of GELU (moe_geglu_split_cuda, cpp_runtime/mfq_decode.cpp:320)."""
    W = gate_up.shape[-1] // 2
    g2 = gate_up.reshape(-1, 2 * W)
    hidden = torch.empty((g2.shape[0], W), dtype=out_dtype, device=gate_up.device)
    if g2.shape[0] == 0:
        return hidden.reshape(*gate_up.shape[:-1], W)
    L.check(L.lib().mfq_hip_moe_glu(_ptr(g2), g2.stride(0), g2.shape[0], W, _ptr(hidden),
                                    L.X_F16 if out_dtype == torch.float16 else L.X_BF16, W, activation, _stream()))
    return hidden.reshape(*gate_up.shape[:-1], W)


def moe_swiglu(gate_up: torch.Tensor, out_dtype=torch.float16) -> torch.Tensor:
    """silu(gate) * up, gate = first half of the last axis (moe_swiglu_split_cuda)."""
    return moe_glu(gate_up, out_dtype, L.GLU_SILU)


def moe_geglu(gate_up: torch.Tensor, out_dtype=torch.float16) -> torch.Tensor:
    """gelu_tanh(gate) * up (moe_geglu_split_cuda)."""
    return moe_glu(gate_up, out_dtype, L.GLU_GELU)


def moe_weighted_reduce(pair: torch.Tensor, weights: torch.Tensor, shared: torch.Tensor | None = None,
                        gate_logits: torch.Tensor | None = None) -> torch.Tensor:
    T, R, H = pair.shape
    out = torch.empty((T, H), dtype=torch.float32, device=pair.device)
    L.check(L.lib().mfq_hip_moe_weighted_reduce(_ptr(pair.contiguous()), _ptr(weights.contiguous()), T, R, H,
                                                _ptr(shared), _ptr(gate_logits), _ptr(out), _stream()))
    return out


def nint_moe_ffn_forward(gate_up: NintMoeWeight, down: NintMoeWeight, x: torch.Tensor, router_logits: torch.Tensor,
                         top_k: int, use_sigmoid=False, use_sqrt_softplus=False, normalize=False,
                         delayed_softmax=False, router_bias=None, router_scale=1.0, shared=None):
    """cpp_runtime/mfq_decode.cpp:3394-3416.  `shared` = (gate_up NintWeight [2W, H], down NintWeight [H, W]) of the
    shared expert, added ungated (cpp_runtime/mfq_decode.cpp:11077-11080).  Returns (out, ids, weights)."""
    if gate_up.n_experts != down.n_experts or gate_up.out_per_expert != 2 * down.neuron_len or \
            down.out_per_expert != gate_up.neuron_len:
        raise RuntimeError("incompatible fused gate_up/down NINTM tensors")
    ids, w = moe_topk(router_logits, top_k, use_sigmoid, use_sqrt_softplus, normalize, delayed_softmax, router_bias,
                      1e-20, router_scale)
    route = build_moe_route_plan(ids, gate_up.n_experts)
    sgu, sdn = shared if shared is not None else (None, None)
    T_, R_ = ids.shape
    if route.ids_dst is None and gate_up.decode_capable(sgu, T_, R_, True) and down.decode_capable(sdn, T_, R_):
        # decode step: gate/up + SwiGLU of the routes and of the shared expert in one launch, the down projections in
        # a second one, then the weighted sum
        T, R = ids.shape
        hidden = gate_up.forward_decode(x, ids, sgu, swiglu=True)
        dn = down.forward_decode(hidden, ids, sdn, routed=True)
        pair = dn[: T * R].reshape(T, R, -1)
        return moe_weighted_reduce(pair, w, dn[T * R:] if shared is not None else None), ids, w
    hidden = gate_up.forward_glu(x, route)
    dn = down.forward(hidden, route)
    sh = None
    if shared is not None:
        sgu, sdn = shared
        sh = nint_matmul(sdn, moe_swiglu(nint_matmul(sgu, x)))
    return moe_weighted_reduce(dn, w, sh), ids, w


# ---------------------------------------------------------------------------------------
# Expert residency: experts in pinned host memory, a GPU arena of slots for the ones in use
# ---------------------------------------------------------------------------------------
class _HostCohort:
    """One cohort of a cached NINTM tensor: its experts' device-layout bytes in pinned host memory, and the arena
    (a NintWeight of `slots` experts) its resident experts live in."""

    def __init__(self, pool: NintWeight, expert_ids, out_per_expert):
        self.src_desc, self.expert_ids, self.out = pool.desc, np.asarray(expert_ids, dtype=np.int32), out_per_expert
        self.host = torch.empty(pool.data.numel(), dtype=torch.uint8, pin_memory=True)
        self.host.copy_(pool.data)
        rbe = out_per_expert // 16
        self.body_bytes = rbe * int(pool.desc.rowblock_bytes)
        self.slot_bytes = self.body_bytes + 2 * out_per_expert * 4
        self.arena: NintWeight | None = None
        self.slot_of: dict[int, int] = {}        # local expert index -> slot
        self.lru: list[int] = []                  # local indices, least recently used first
        self.free: list[int] = []

    def segments(self, local: int, slot: int):
        """(source offset in the host copy, destination offset in the arena, bytes) of an expert's body, scale
        anchors and minimum anchors."""
        s, a, out = self.src_desc, self.arena.desc, self.out
        return [(local * self.body_bytes, slot * self.body_bytes, self.body_bytes),
                (int(s.anchors_off) + local * out * 4, int(a.anchors_off) + slot * out * 4, out * 4),
                (int(s.anchors_off) + 16 * s.n_rowblocks * 4 + local * out * 4,
                 int(a.anchors_off) + 16 * a.n_rowblocks * 4 + slot * out * 4, out * 4)]


class MoeCachedSource:
    """A NINTM tensor whose experts live in host memory; `weight` is the NintMoeWeight view over the arenas, valid for
    the experts made resident by the last MoeExpertCache.prepare (MoeCachedSource, cpp_runtime/mfq_decode.cpp:6440-6915)."""

    def __init__(self, n_experts, out_per_expert, neuron_len, cohorts):
        self.n_experts, self.out_per_expert, self.neuron_len, self.cohorts = n_experts, out_per_expert, neuron_len, cohorts
        self.cohort_of = np.full(n_experts, -1, dtype=np.int32)
        self.local_of = np.full(n_experts, -1, dtype=np.int32)
        for ci, c in enumerate(cohorts):
            self.cohort_of[c.expert_ids] = ci
            self.local_of[c.expert_ids] = np.arange(len(c.expert_ids), dtype=np.int32)
        self.weight: NintMoeWeight | None = None


class MoeExpertCache:
    """GPU residency of routed experts under a byte budget (MoeExpertCache, cpp_runtime/mfq_decode.cpp:5941-7500).

    register_source() parses a NINTM blob, lets the GPU write each cohort's device layout once and keeps it in pinned
    host memory; finalize() splits the budget into per-cohort arenas of expert slots; prepare(source, experts) makes
    the given experts resident -- least recently used slots are reused, the bytes of all missing experts travel as one
    host-to-device copy of a staging buffer and one scatter launch (mfq_hip_cache_scatter), which also rewrites the
    dispatch-table words -- after which source.weight runs the ordinary grouped kernels."""

    def __init__(self, budget_bytes: int, device="cuda"):
        if budget_bytes <= 0:
            raise ValueError("MoE GPU cache budget must be positive")
        self.budget_bytes, self.device = int(budget_bytes), torch.device(device)
        self.sources: list[MoeCachedSource] = []
        self.finalized = False
        self.allocated_bytes = 0
        self.stats = {"hits": 0, "misses": 0, "evictions": 0, "bytes": 0, "launches": 0}
        self._stage_host = self._stage_dev = None

    def register_source(self, blob, minimum_slots: int = 1) -> MoeCachedSource:
        if self.finalized:
            raise RuntimeError("cannot register a MoE source after cache finalization")
        full = NintMoeWeight.from_blob(blob, self.device)
        if full.foreign:
            raise NotImplementedError("expert residency holds NINT cohorts only; this tensor has a "
                                      f"{full.foreign[0].dtype} cohort")
        cohorts = [_HostCohort(p, ids, full.out_per_expert) for p, ids in zip(full.pools, full.pool_expert_ids)]
        for c in cohorts:
            c.minimum_slots = min(int(minimum_slots), len(c.expert_ids))
        src = MoeCachedSource(full.n_experts, full.out_per_expert, full.neuron_len, cohorts)
        self.sources.append(src)
        del full                                   # the device copies of the pools go away; the host copies stay
        return src

    def finalize(self):
        """Slots per cohort: its minimum, plus a share of what the budget leaves in proportion to the cohort's bytes
        (never more slots than it has experts)."""
        if self.finalized:
            return
        cohorts = [c for s in self.sources for c in s.cohorts]
        need = sum(c.minimum_slots * c.slot_bytes for c in cohorts)
        if need > self.budget_bytes:
            raise RuntimeError(f"MoE GPU cache budget {self.budget_bytes} is below the minimum working set {need}")
        spare, total = self.budget_bytes - need, sum(len(c.expert_ids) * c.slot_bytes for c in cohorts)
        for c in cohorts:
            extra = int(spare * (len(c.expert_ids) * c.slot_bytes / total) // c.slot_bytes)
            slots = min(len(c.expert_ids), c.minimum_slots + extra)
            desc = L.NintDesc()
            d = c.src_desc
            L.check(L.lib().mfq_hip_nint_plan(d.bits, d.sub_bits, d.gs, slots * c.out, d.neuron_len, C.byref(desc)))
            c.arena = NintWeight(desc, torch.zeros(int(desc.total_bytes), dtype=torch.uint8, device=self.device),
                                 (slots * c.out, d.neuron_len))
            c.free = list(range(slots))
            self.allocated_bytes += int(desc.total_bytes)
        for s in self.sources:
            s.weight = NintMoeWeight(s.n_experts, s.out_per_expert, s.neuron_len, [c.arena for c in s.cohorts],
                                     [np.zeros(0, dtype=np.int32) for _ in s.cohorts], self.device)
            s.weight.expert_pool = torch.from_numpy(s.cohort_of.copy()).to(self.device)
            s.weight.expert_local = torch.full((s.n_experts,), -1, dtype=torch.int32, device=self.device)
        self.finalized = True

    def prepare(self, source: MoeCachedSource, experts) -> None:
        """Make `experts` (ids, any order, duplicates allowed) resident in `source`."""
        if not self.finalized:
            raise RuntimeError("MoE cache must be finalized before inference")
        wanted = sorted({int(e) for e in np.asarray(experts).reshape(-1) if 0 <= int(e) < source.n_experts})
        per_cohort: dict[int, list[int]] = {}
        for e in wanted:
            per_cohort.setdefault(int(source.cohort_of[e]), []).append(e)
        for ci, es in per_cohort.items():
            if len(es) > len(source.cohorts[ci].free) + len(source.cohorts[ci].slot_of):
                raise RuntimeError(f"MoE route needs {len(es)} experts of one cohort, its arena holds "
                                   f"{len(source.cohorts[ci].free) + len(source.cohorts[ci].slot_of)}")
        copies, table = [], []                     # (host tensor, src off, dst address, bytes), (expert, slot)
        for ci, es in per_cohort.items():
            c = source.cohorts[ci]
            keep = {int(source.local_of[e]) for e in es}
            for e in es:
                local = int(source.local_of[e])
                if local in c.slot_of:
                    self.stats["hits"] += 1
                    c.lru.remove(local)
                    c.lru.append(local)
                    continue
                self.stats["misses"] += 1
                if c.free:
                    slot = c.free.pop()
                else:
                    victim = next(v for v in c.lru if v not in keep)
                    c.lru.remove(victim)
                    slot = c.slot_of.pop(victim)
                    table.append((int(c.expert_ids[victim]), -1))
                    self.stats["evictions"] += 1
                c.slot_of[local] = slot
                c.lru.append(local)
                base = c.arena.data.data_ptr()
                for so, do, nb in c.segments(local, slot):
                    copies.append((c.host, so, base + do, nb))
                table.append((e, slot))
        if not copies and not table:
            return
        # staging image: the byte ranges (16-byte aligned), the table words, then the descriptors
        off, plan = 0, []
        for host, so, dst, nb in copies:
            plan.append((off, host, so, dst, nb))
            off += (nb + 15) & ~15
        words_off = off
        off += (4 * len(table) + 15) & ~15
        desc_off = off
        n = len(copies) + len(table)
        total = desc_off + 24 * n
        if self._stage_host is None or self._stage_host.numel() < total:
            self._stage_host = torch.empty(max(total, 1 << 20), dtype=torch.uint8, pin_memory=True)
            self._stage_dev = torch.empty(self._stage_host.numel(), dtype=torch.uint8, device=self.device)
        else:
            torch.cuda.current_stream().synchronize()      # the previous batch has left the pinned buffer
        img = self._stage_host.numpy()
        descs = np.zeros((n, 3), dtype=np.uint64)
        for i, (o, host, so, dst, nb) in enumerate(plan):
            img[o:o + nb] = host.numpy()[so:so + nb]
            descs[i] = (dst, o, nb)
        words = np.array([slot for _, slot in table], dtype=np.int32)
        img[words_off:words_off + 4 * len(table)] = words.view(np.uint8)
        local_ptr = source.weight.expert_local.data_ptr()
        for j, (e, _) in enumerate(table):
            descs[len(copies) + j] = (local_ptr + 4 * e, words_off + 4 * j, 4)
        img[desc_off:total] = descs.reshape(-1).view(np.uint8)
        self._stage_dev[:total].copy_(self._stage_host[:total], non_blocking=True)
        biggest = max([nb for *_, nb in copies] + [4])
        L.check(L.lib().mfq_hip_cache_scatter(_ptr(self._stage_dev), desc_off, n, biggest, _stream()))
        self.stats["bytes"] += sum(nb for *_, nb in copies)
        self.stats["launches"] += 1

    def forward(self, source: MoeCachedSource, x: torch.Tensor, route: MoeRoutePlan) -> torch.Tensor:
        """Grouped matmul of a cached tensor: reads the route's expert ids back to the host, makes them resident and
        runs NintMoeWeight.forward on the arenas (the readback of begin_route_experts / finish_route_experts,
        cpp_runtime/mfq_decode.cpp:6066-6180)."""
        self.prepare(source, route.ids.cpu().numpy())
        return source.weight.forward(x, route)
