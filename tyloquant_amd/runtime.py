"""Python twin of the host dispatch layer: weight objects, the dtype-string registry and the
matmul entry points, over the C ABI of libmfq_hip.so.

Mirrors the reference's operator surface for this path (names, argument meaning, errors):
  load_quant_linear / is_nint_linear_dtype / is_nvq_linear_dtype  cpp_runtime/mfq_decode.cpp:9409-9420, 9489-9771
  NintWeight / nint_matmul                                         cpp_runtime/mfq_decode.cpp:2101-2165, 8130-8315
  NvqWeight / nvq_matmul                                           cpp_runtime/mfq_decode.cpp:4019-4150, 7884-7931
  NepqWeight / nepq_matmul                                         mfq/kernels/cuda/nepq_matmul.py:215-280
  NintMoeWeight / MoeRoutePlan / build_moe_route_plan / nint_moe_ffn_forward
                                                                   cpp_runtime/mfq_decode.cpp:2579-2592, 2681-2708, 2908-3071, 3394-3416
torch is used only to own device memory and to name the current stream; every computation is a
HIP kernel behind the C ABI, and nothing here falls back to the CPU.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import numpy as np
import torch

from . import _lib as L
from . import formats as F


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def _x_dtype(x: torch.Tensor) -> int:
    if x.dtype == torch.bfloat16:
        return L.X_BF16
    if x.dtype == torch.float16:
        return L.X_F16
    raise TypeError(f"activations must be bfloat16 or float16, got {x.dtype}")


def _as_2d(x: torch.Tensor, K: int) -> torch.Tensor:
    if x.shape[-1] != K:
        raise ValueError(f"activation width {x.shape[-1]} != neuron length {K}")
    x2 = x.reshape(-1, K)
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    return x2


def _upload(blob, off: int, nbytes: int, device) -> torch.Tensor:
    arr = np.frombuffer(blob, dtype=np.uint8, count=nbytes, offset=off)
    return torch.from_numpy(arr.copy()).to(device, non_blocking=False)


class _Workspace:
    """Grow-only device scratch, cached per weight like the reference's per-M workspaces
    (cpp_runtime/mfq_decode.cpp:2120-2132)."""

    def __init__(self):
        self.buf = None

    def get(self, nbytes: int, device) -> torch.Tensor | None:
        if nbytes == 0:
            return None
        if self.buf is None or self.buf.numel() < nbytes or self.buf.device != device:
            self.buf = torch.empty(nbytes, dtype=torch.uint8, device=device)
        return self.buf


# ---------------------------------------------------------------------------------------
# NINT
# ---------------------------------------------------------------------------------------
class NintWeight:
    def __init__(self, desc: L.NintDesc, data: torch.Tensor, shape):
        self.desc, self.data, self.shape = desc, data, tuple(shape)
        self.out, self.neuron_len = desc.out, desc.neuron_len
        self.bits, self.gs, self.ng = desc.bits, desc.gs, desc.ng
        self._ws = _Workspace()

    @property
    def payload_bytes(self) -> int:
        return int(self.desc.payload_bytes)

    @staticmethod
    def from_blob(blob, device="cuda") -> "NintWeight":
        h = F.parse_nint(blob)
        if h.axis != 0:
            raise ValueError("NINT linear weights must be quantized along axis 0")
        desc = L.NintDesc()
        L.check(L.lib().mfq_hip_nint_plan(h.bits, h.sub_bits, h.gs, h.out, h.neuron_len, C.byref(desc)))
        device = torch.device(device)
        payload = _upload(blob, h.body_off, h.body_bytes, device)
        data = torch.empty(int(desc.total_bytes), dtype=torch.uint8, device=device)
        L.check(L.lib().mfq_hip_nint_repack(C.byref(desc), _ptr(payload), h.body_bytes, int(h.legacy), _ptr(data),
                                            _stream()))
        torch.cuda.current_stream().synchronize()  # payload may be freed after this
        return NintWeight(desc, data, h.shape)

    def dequantize(self) -> torch.Tensor:
        w = torch.empty((self.out, self.neuron_len), dtype=torch.float32, device=self.data.device)
        L.check(L.lib().mfq_hip_nint_dequant_f32(C.byref(self.desc), _ptr(self.data), _ptr(w), self.neuron_len,
                                                 _stream()))
        return w


class Nint8ZeroWeight:
    """NINT8-0 (GGML Q8_0 blocks) on the device: fp16 scales and row-major int8 codes (to_device_nint8_zero,
    cpp_runtime/mfq_decode.cpp:2309-2330)."""

    def __init__(self, desc: L.Nint8zDesc, data: torch.Tensor, shape):
        self.desc, self.data, self.shape = desc, data, tuple(shape)
        self.out, self.neuron_len, self.ng = desc.out, desc.neuron_len, desc.ng
        self.bits, self.gs = 8, 32
        self._ws = _Workspace()

    @property
    def payload_bytes(self) -> int:
        return int(self.desc.payload_bytes)

    @staticmethod
    def from_blob(blob, device="cuda") -> "Nint8ZeroWeight":
        h = F.parse_nint8_zero(blob)
        if h.axis != 0:
            raise ValueError("NINT8-0 linear weights must be quantized along axis 0")
        desc = L.Nint8zDesc()
        L.check(L.lib().mfq_hip_nint8z_plan(h.out, h.neuron_len, C.byref(desc)))
        device = torch.device(device)
        payload = _upload(blob, h.body_off, h.body_bytes, device)
        data = torch.empty(int(desc.total_bytes), dtype=torch.uint8, device=device)
        L.check(L.lib().mfq_hip_nint8z_repack(C.byref(desc), _ptr(payload), h.body_bytes, _ptr(data), _stream()))
        torch.cuda.current_stream().synchronize()  # payload may be freed after this
        return Nint8ZeroWeight(desc, data, h.shape)

    def dequantize(self) -> torch.Tensor:
        w = torch.empty((self.out, self.neuron_len), dtype=torch.float32, device=self.data.device)
        L.check(L.lib().mfq_hip_nint8z_dequant_f32(C.byref(self.desc), _ptr(self.data), _ptr(w), self.neuron_len,
                                                   _stream()))
        return w


def nint8_zero_matmul(w: Nint8ZeroWeight, x: torch.Tensor, *, force: str | None = None) -> torch.Tensor:
    """y[..., out] = x[..., K] @ W^T in fp32 for a NINT8-0 tensor (the q8_zero branch of nint_matmul,
    cpp_runtime/mfq_decode.cpp:8165-8185).  force = "gemv" pins the streaming kernel."""
    x2 = _as_2d(x, w.neuron_len)
    M = x2.shape[0]
    y = torch.empty((M, w.out), dtype=torch.float32, device=x.device)
    if M == 0:                                   # an empty batch: nothing to launch
        return y.reshape(*x.shape[:-1], w.out)
    lib = L.lib()
    if force == "gemv":
        L.check(lib.mfq_hip_nint8z_gemv(C.byref(w.desc), _ptr(w.data), _ptr(x2), _x_dtype(x2), x2.stride(0), M, _ptr(y),
                                        w.out, _stream()))
    else:
        need = lib.mfq_hip_nint8z_gemm_workspace_bytes(C.byref(w.desc), M)
        ws = w._ws.get(need, x.device)
        L.check(lib.mfq_hip_nint8z_gemm(C.byref(w.desc), _ptr(w.data), _ptr(x2), _x_dtype(x2), x2.stride(0), M, _ptr(y),
                                        w.out, _ptr(ws), need, _stream()))
    return y.reshape(*x.shape[:-1], w.out)


def nint_matmul(w: NintWeight, x: torch.Tensor, *, force: str | None = None) -> torch.Tensor:
    """y[..., out] = x[..., K] @ W^T in fp32 (cpp_runtime/mfq_decode.cpp:8130).  `force` = "gemv"
    or "gemm" pins the kernel family (the reference's MFQ_* path overrides)."""
    x2 = _as_2d(x, w.neuron_len)
    M = x2.shape[0]
    y = torch.empty((M, w.out), dtype=torch.float32, device=x.device)
    if M == 0:                                   # an empty batch: nothing to launch
        return y.reshape(*x.shape[:-1], w.out)
    lib = L.lib()
    if force == "gemv":
        L.check(lib.mfq_hip_nint_gemv(C.byref(w.desc), _ptr(w.data), _ptr(x2), _x_dtype(x2), x2.stride(0), M, _ptr(y),
                                      w.out, _stream()))
    else:
        Mq = max(M, 9) if force == "gemm" else M
        need = lib.mfq_hip_nint_gemm_workspace_bytes(C.byref(w.desc), Mq)
        ws = w._ws.get(need, x.device)
        if force == "gemm" and M < 9:
            raise ValueError("force='gemm' needs at least 9 activation rows")
        L.check(lib.mfq_hip_nint_gemm(C.byref(w.desc), _ptr(w.data), _ptr(x2), _x_dtype(x2), x2.stride(0), M, _ptr(y),
                                      w.out, _ptr(ws), need, _stream()))
    return y.reshape(*x.shape[:-1], w.out)


def _nint_matmul_glu(w: NintWeight, x: torch.Tensor, out_dtype, activation: int) -> torch.Tensor:
    x2 = _as_2d(x, w.neuron_len)
    M, W = x2.shape[0], w.out // 2
    d = w.desc
    if M == 0:
        return torch.empty((*x.shape[:-1], W), dtype=out_dtype, device=x.device)
    unit = w.out % 32 == 0 and (d.kind == 1 or (d.bits == 5 and d.gs == 28))
    o16 = L.X_F16 if out_dtype == torch.float16 else L.X_BF16
    if unit and M > 2:
        # prefill batches: the GLU runs in the epilogue of the block-tiled matmul where that kernel takes the call
        lib = L.lib()
        need = lib.mfq_hip_nint_gemm_workspace_bytes(C.byref(d), M)
        ws = w._ws.get(need, x.device)
        hidden = torch.empty((M, W), dtype=out_dtype, device=x.device)
        rc = lib.mfq_hip_nint_gemm_glu(C.byref(d), _ptr(w.data), _ptr(x2), _x_dtype(x2), x2.stride(0), M, activation,
                                       _ptr(hidden), o16, W, _ptr(ws), need, _stream())
        if rc == L.OK:
            return hidden.reshape(*x.shape[:-1], W)
        if rc != L.ERR_UNSUPPORTED:
            L.check(rc)
    if not unit or M > 2:
        from .runtime_moe import moe_glu
        return moe_glu(nint_matmul(w, x), out_dtype, activation)
    hidden = torch.empty((M, W), dtype=out_dtype, device=x.device)
    L.check(L.lib().mfq_hip_nint_gemv_glu(C.byref(w.desc), _ptr(w.data), _ptr(x2), _x_dtype(x2), x2.stride(0), M,
                                          _ptr(hidden), L.X_F16 if out_dtype == torch.float16 else L.X_BF16, W,
                                          activation, _stream()))
    return hidden.reshape(*x.shape[:-1], W)


def nint_matmul_swiglu(w: NintWeight, x: torch.Tensor, out_dtype=torch.float16) -> torch.Tensor:
    """silu(gate) * up of a [2W, K] gate/up tensor (gate rows first) in one launch for one or two rows
    (nint_gemv_packed_swiglu_ws_cuda, cpp_runtime/mfq_decode.cpp:393-396); matmul + SwiGLU kernel otherwise."""
    return _nint_matmul_glu(w, x, out_dtype, L.GLU_SILU)


def nint_matmul_geglu(w: NintWeight, x: torch.Tensor, out_dtype=torch.float16) -> torch.Tensor:
    """gelu_tanh(gate) * up of a [2W, K] gate/up tensor, as nint_matmul_swiglu (nint_matmul_geglu,
    cpp_runtime/mfq_decode.cpp:8462-8485; the reference fuses it for one row, here for one or two)."""
    return _nint_matmul_glu(w, x, out_dtype, L.GLU_GELU)


def nint_ffn_decode(gate_up: NintWeight, down: NintWeight, x: torch.Tensor, activation: int = L.GLU_SILU,
                    one_launch: bool = False, verify: bool = False) -> torch.Tensor:
    """y = down(act(gate x) * up x) in fp32 for a [2W, H] gate/up tensor and a [N, W] down tensor: the dense FFN of
    FFN::forward_impl (cpp_runtime/mfq_decode.cpp:11199-11209): the fused gate/up launch (or matmul + GLU kernel)
    followed by the down matmul.  one_launch=True runs one activation row on a pair of tensors the kernel takes as a
    single launch with a grid barrier (mfq_hip_nint_ffn_decode); it is not the default because crossing the barrier
    costs what the launch boundary costs (measured: 23.7 us against 19.3 us on 12288 x 4096 NINT4-32).  The barrier
    needs the device to itself; when it gives up the output is NaN.  verify=True waits for the launch, asks
    mfq_hip_nint_ffn_decode_status and runs the two launches instead if a barrier gave up."""
    if gate_up.out != 2 * down.neuron_len:
        raise ValueError("gate/up rows must be twice the down tensor's neuron length")
    x2 = _as_2d(x, gate_up.neuron_len)
    lib = L.lib()
    if one_launch and x2.shape[0] == 1 and x2.data_ptr() % 16 == 0:
        need = lib.mfq_hip_nint_ffn_decode_workspace_bytes(C.byref(gate_up.desc), C.byref(down.desc))
        if need:
            ws = getattr(gate_up, "_ffn_ws", None)
            if ws is None or ws.numel() < need or ws.device != x.device:
                ws = gate_up._ffn_ws = torch.zeros(need, dtype=torch.uint8, device=x.device)   # barrier words start at zero
            y = torch.empty((1, down.out), dtype=torch.float32, device=x.device)
            L.check(lib.mfq_hip_nint_ffn_decode(C.byref(gate_up.desc), _ptr(gate_up.data), C.byref(down.desc), _ptr(down.data),
                                                _ptr(x2), _x_dtype(x2), activation, _ptr(y), _ptr(ws), need, _stream()))
            if not verify or lib.mfq_hip_nint_ffn_decode_status(_ptr(ws), _stream()) == 0:
                return y.reshape(*x.shape[:-1], down.out)
    return nint_matmul(down, _nint_matmul_glu(gate_up, x, torch.float16, activation))


def nint_matmul_input_mul(w: NintWeight, x: torch.Tensor, gate: torch.Tensor, mode: int = 0, fused=True) -> torch.Tensor:
    """(x * silu(gate)) . W^T, or with mode 1 (x * sigmoid(gate)) . W^T (nint_matmul_input_mul,
    cpp_runtime/mfq_decode.cpp:8395-8417).  One or two rows: one GEMV launch whose waves gate their slice of the
    activations as they stage it.  More rows (or rows the fused launch declines): the gated activations are formed by one
    elementwise launch (fp32 product, one rounding to the dtype of x) and go through nint_matmul."""
    if gate.shape != x.shape:
        raise ValueError("gate and activations must have the same shape")
    x2 = _as_2d(x, w.neuron_len)
    g2 = _as_2d(gate.to(x2.dtype), w.neuron_len)
    if x2.shape[0] == 0:
        return nint_matmul(w, x)
    if x2.shape[0] <= 2 and fused:
        y = torch.empty((x2.shape[0], w.out), dtype=torch.float32, device=x2.device)
        rc = L.lib().mfq_hip_nint_gemv_gate(C.byref(w.desc), _ptr(w.data), _ptr(x2), _ptr(g2), _x_dtype(x2), x2.stride(0),
                                            g2.stride(0), x2.shape[0], int(mode), _ptr(y), y.stride(0), _stream())
        if rc == 0:
            return y.reshape(*x.shape[:-1], w.out)
        if rc != L.ERR_UNSUPPORTED:
            L.check(rc)
    out = torch.empty((x2.shape[0], w.neuron_len), dtype=x2.dtype, device=x2.device)
    L.check(L.lib().mfq_hip_input_gate(_ptr(x2), _ptr(g2), _x_dtype(x2), x2.stride(0), g2.stride(0), x2.shape[0],
                                       w.neuron_len, int(mode), _ptr(out), out.stride(0), _stream()))
    return nint_matmul(w, out.reshape(x.shape))


def _embedding_rows(entry, w, ids: torch.Tensor, out_dtype) -> torch.Tensor:
    codes = {torch.bfloat16: L.X_BF16, torch.float16: L.X_F16, torch.float32: L.X_F32}
    if out_dtype not in codes:
        raise TypeError(f"embedding rows are bfloat16, float16 or float32, got {out_dtype}")
    flat = ids.to(device=w.data.device, dtype=torch.int64).reshape(-1).contiguous()
    out = torch.empty((flat.numel(), w.neuron_len), dtype=out_dtype, device=w.data.device)
    L.check(entry(C.byref(w.desc), _ptr(w.data), _ptr(flat), flat.numel(), _ptr(out), codes[out_dtype], w.neuron_len,
                  _stream()))
    return out.reshape(*ids.shape, w.neuron_len)


def nint_embedding(w: NintWeight, ids: torch.Tensor, out_dtype=torch.float16) -> torch.Tensor:
    """Rows ids of the dequantized table as out_dtype, shape ids.shape + [neuron_len]; ids outside the table give
    zeros (embed_forward, cpp_runtime/mfq_decode.cpp:13929-13957)."""
    return _embedding_rows(L.lib().mfq_hip_nint_embedding, w, ids, out_dtype)


def embedding(w, ids: torch.Tensor, out_dtype=torch.float16) -> torch.Tensor:
    """Token-embedding rows of any table format embed_forward takes (cpp_runtime/mfq_decode.cpp:13929-13957): NINT,
    NINT8-0 and the NVQ families; shape ids.shape + [neuron_len], ids outside the table give zeros.  Like the
    reference, MX and NEPQ tables are refused."""
    from .runtime_vq import NvqsWeight, NvqWeight
    lib = L.lib()
    if isinstance(w, QuantLinear):
        w = w.weight
    if isinstance(w, NintWeight):
        return _embedding_rows(lib.mfq_hip_nint_embedding, w, ids, out_dtype)
    if isinstance(w, Nint8ZeroWeight):
        return _embedding_rows(lib.mfq_hip_nint8z_embedding, w, ids, out_dtype)
    if isinstance(w, NvqsWeight):
        return _embedding_rows(lib.mfq_hip_nvqs_embedding, w, ids, out_dtype)
    if isinstance(w, NvqWeight):
        return _embedding_rows(lib.mfq_hip_nvq_embedding, w, ids, out_dtype)
    raise TypeError(f"token embeddings are not supported for {type(w).__name__} tables")


def nint_matmul_argmax(w: NintWeight, x: torch.Tensor, return_logits: bool = False):
    """Greedy next token of an LM head: argmax over the neurons of x . W^T per row of x, int64, ties to the lower
    index (next_token_from_hidden, cpp_runtime/mfq_decode.cpp:14107-14130).  With return_logits also the fp32
    logits the arg-max was taken from."""
    x2 = _as_2d(x, w.neuron_len)
    M = x2.shape[0]
    lib = L.lib()
    need = lib.mfq_hip_nint_gemv_argmax_workspace_bytes(C.byref(w.desc), M)
    ws = w._ws.get(need, x.device)
    token = torch.empty((M,), dtype=torch.int64, device=x.device)
    logits = torch.empty((M, w.out), dtype=torch.float32, device=x.device) if return_logits else None
    L.check(lib.mfq_hip_nint_gemv_argmax(C.byref(w.desc), _ptr(w.data), _ptr(x2), _x_dtype(x2), x2.stride(0), M,
                                         _ptr(logits), w.out, _ptr(token), _ptr(ws), need, _stream()))
    token = token.reshape(x.shape[:-1])
    return (token, logits.reshape(*x.shape[:-1], w.out)) if return_logits else token


class NintLinearGroup:
    """Projections that share their input (gate/up, Q/K/V) kept as one concatenated NintWeight and run as
    one matmul whose output is split afterwards (cpp_runtime/mfq_decode.cpp:8618-8660)."""

    def __init__(self, weight: NintWeight, outs):
        self.w, self.outs = weight, [int(o) for o in outs]

    @staticmethod
    def from_blobs(blobs, device="cuda") -> "NintLinearGroup":
        outs = [F.parse_nint(b).out for b in blobs]
        return NintLinearGroup(NintWeight.from_blob(F.nint_concat_rows(blobs), device), outs)

    def forward(self, x: torch.Tensor):
        return list(nint_matmul(self.w, x).split(self.outs, dim=-1))

    __call__ = forward


# ---------------------------------------------------------------------------------------
# dtype registry
# ---------------------------------------------------------------------------------------
def is_nint_linear_dtype(dtype: str) -> bool:
    """NINT<bits> for any bit width (cpp_runtime/mfq_decode.cpp:9409-9412); NINT8-0 and NINTM are
    separate families."""
    return dtype.startswith("NINT") and dtype[4:].isdigit()


def is_nvq_linear_dtype(dtype: str) -> bool:
    return dtype in ("NVQ3", "NVQ3J", "NVQ3J-512", "NVQ3J-L", "NVQ2", "NVQ2J", "NVQ2J-L", "NVQ2J-XL", "NIQ3", "NIQ2", "NIQ2J")


def is_nepq_linear_dtype(dtype: str) -> bool:
    return dtype in ("NEPQ1-S", "NEPQ1-L", "NEPQ0-S", "NEPQ0-L")


@dataclass
class QuantLinear:
    kind: str
    weight: object

    @property
    def out(self):
        return self.weight.out

    @property
    def neuron_len(self):
        return self.weight.neuron_len

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return _MATMUL[self.kind](self.weight, x)

    __call__ = forward

    def reserve(self, max_rows: int) -> None:
        """Grow the weight's workspace to the largest need of any batch of 1 .. max_rows rows, so that forward() of such
        a batch does not allocate: call once before capturing forward() into a HIP graph.  (The output tensor still comes
        from torch's allocator, which is capture-aware.)"""
        lib, w = L.lib(), self.weight
        query = {"nint": lambda M: lib.mfq_hip_nint_gemm_workspace_bytes(C.byref(w.desc), M),
                 "nint8z": lambda M: lib.mfq_hip_nint8z_gemm_workspace_bytes(C.byref(w.desc), M),
                 "nvq": lambda M: (lib.mfq_hip_nvqs_gemm_workspace_bytes if type(w).__name__ == "NvqsWeight"
                                   else lib.mfq_hip_nvq_gemm_workspace_bytes)(C.byref(w.desc), M),
                 # NEPQ0-S / NEPQ0-L keep their bit streams (an NvqsDesc) and run on the stream kernels' row-range form
                 "nepq": lambda M: (lib.mfq_hip_nvqs_gemm_rows_workspace_bytes if getattr(w, "streams", False)
                                    else lib.mfq_hip_nepq_gemm_workspace_bytes)(C.byref(w.desc), w.out_per_expert, M),
                 "mx": lambda M: lib.mfq_hip_mx_gemm_rows_workspace_bytes(w.neuron_len, w.out, M)}[self.kind]
        sizes = set(range(1, min(max_rows, 512) + 1)) | set(range(576, max_rows, 64)) | {max_rows}
        need = max((int(query(M)) for M in sizes if M > 0), default=0)
        w._ws.get(need, w.data.device)

    def dequantize(self) -> torch.Tensor:
        return self.weight.dequantize()

    def embedding(self, ids: torch.Tensor, out_dtype=torch.float16) -> torch.Tensor:
        """The tensor as a token-embedding table: rows ids of its dequantized values (see embedding())."""
        return embedding(self.weight, ids, out_dtype)


def load_quant_linear(dtype: str, blob, device="cuda") -> QuantLinear:
    """Switch on the MFQ dtype string and build the device weight (cpp_runtime/mfq_decode.cpp:9489-9771)."""
    dtype = {"NIQ3": "NVQ3", "NIQ2": "NVQ2", "NIQ2J": "NVQ2J"}.get(dtype, dtype)
    if is_nint_linear_dtype(dtype):
        w = NintWeight.from_blob(blob, device)
        if f"NINT{w.bits}" != dtype:
            raise ValueError(f"MFQ dtype/blob mismatch: {dtype} contains NINT{w.bits}")
        return QuantLinear("nint", w)
    if dtype == "NINT8-0":
        return QuantLinear("nint8z", Nint8ZeroWeight.from_blob(blob, device))
    if is_nvq_linear_dtype(dtype):
        from .runtime_vq import NvqWeight
        w = NvqWeight.from_blob(blob, device)
        if w.dtype != dtype:
            raise ValueError(f"MFQ dtype/blob mismatch: {dtype} contains {w.dtype}")
        return QuantLinear("nvq", w)
    if F.is_lowbit_dtype(dtype):
        from .runtime_vq import NvqsWeight
        return QuantLinear("nvq", NvqsWeight.from_lowbit_blob(dtype, blob, device))
    if is_nepq_linear_dtype(dtype):
        from .runtime_vq import NepqWeight
        w = NepqWeight.from_blob(blob, device)
        if w.label != dtype:
            raise ValueError(f"MFQ dtype/blob mismatch: {dtype} contains {w.label}")
        if w.n_experts != 1:
            raise ValueError(f"a {dtype} linear must hold one expert, the blob holds {w.n_experts} "
                             "(multi-expert NEPQ tensors are NINTM cohorts)")
        return QuantLinear("nepq", w)
    if F.is_mx_dtype(dtype):
        from .runtime_mx import MxWeight
        return QuantLinear("mx", MxWeight.from_blob(dtype, blob, device))
    raise ValueError(f"unsupported quantized linear dtype: {dtype}")


def _mx_mm(w, x):
    from .runtime_mx import mx_matmul
    return mx_matmul(w, x)


def _nvq_mm(w, x):
    from .runtime_vq import nvq_matmul
    return nvq_matmul(w, x)


def _nepq_mm(w, x):
    from .runtime_vq import nepq_matmul
    return nepq_matmul(w, x)


_MATMUL = {"nint": nint_matmul, "nint8z": nint8_zero_matmul, "nvq": _nvq_mm, "nepq": _nepq_mm, "mx": _mx_mm}
