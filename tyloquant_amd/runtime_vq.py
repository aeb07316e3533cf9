"""NVQ (D4 and E8 families) and NEPQ1 weights and their matmul entry points (see runtime.py)."""
from __future__ import annotations

import ctypes as C
from pathlib import Path

import numpy as np
import torch

from . import _lib as L
from . import formats as F
from .runtime import _Workspace, _as_2d, _ptr, _stream, _upload, _x_dtype

_DATA = Path(__file__).resolve().parent / "data"


def builtin_grid(name: str) -> np.ndarray:
    """The magnitude grids of the non-JSC formats, decoded as 2*digit+1 from the raw tables
    (mfq/formats/nvq.py:102-129)."""
    raw = np.frombuffer((_DATA / f"{name}.bin").read_bytes(), dtype="<u2")
    dims, digit_bits = (8, 2) if name.startswith("e8_") else (4, 3)
    digits = (raw[:, None] >> (digit_bits * np.arange(dims, dtype=np.uint16))[None, :]) & ((1 << digit_bits) - 1)
    return np.ascontiguousarray(2 * digits + 1, dtype=np.int8)


class NvqWeight:
    def __init__(self, desc, data, dtype):
        self.desc, self.data, self.dtype = desc, data, dtype
        self.out, self.neuron_len = desc.out, desc.neuron_len
        self._ws = _Workspace()

    @property
    def payload_bytes(self) -> int:
        return int(self.desc.payload_bytes)

    @staticmethod
    def from_blob(blob, device="cuda") -> "NvqWeight":
        h = F.parse_nvq(blob)
        if h.vector_size != 4 or h.index_bits > 9:
            return NvqsWeight.from_header(h, blob, device)       # E8 family, d4_1024: read from the streams in place
        device = torch.device(device)
        desc = L.NvqDesc()
        lib = L.lib()
        L.check(lib.mfq_hip_nvq_plan(h.index_bits, h.banks if h.jsc else 1, h.out, h.neuron_len, C.byref(desc)))
        payload = _upload(blob, h.body_off, h.body_bytes, device)
        data = torch.empty(int(desc.total_bytes), dtype=torch.uint8, device=device)
        if h.jsc:
            L.check(lib.mfq_hip_nvq_repack(C.byref(desc), _ptr(payload), h.body_bytes, _ptr(data), _stream()))
        else:
            if h.gs != 24 or h.sub_bits != 4 or h.sign_mode != "even":
                raise NotImplementedError("plain NVQ3 runs only with gs24, 4-bit sub-scales and parity signs")
            grid = torch.from_numpy(builtin_grid(h.codebook)).to(device)
            L.check(lib.mfq_hip_nvq_repack_plain(C.byref(desc), _ptr(payload), h.body_bytes, _ptr(grid), _ptr(data),
                                                 _stream()))
        torch.cuda.current_stream().synchronize()
        return NvqWeight(desc, data, h.dtype)

    def dequantize(self) -> torch.Tensor:
        w = torch.empty((self.out, self.neuron_len), dtype=torch.float32, device=self.data.device)
        L.check(L.lib().mfq_hip_nvq_dequant_f32(C.byref(self.desc), _ptr(self.data), _ptr(w), self.neuron_len, _stream()))
        return w


class NvqsWeight:
    """NVQ tensors whose streams are read in place (mfq_hip_nvqs_*): NVQ2 (e8_256; parity or index-parity signs),
    NVQ2J / NVQ2J-L / NVQ2J-XL (e8_256 / e8_1024 / e8_4096, JSC) and NVQ3J-L (d4_1024, JSC) -- formats 2, 5, 13, 14, 15
    of the reference's unpack_nvq (cpp_runtime/mfq_decode.cpp:3756-3769)."""

    def __init__(self, desc, data, dtype):
        self.desc, self.data, self.dtype = desc, data, dtype
        self.out, self.neuron_len = desc.out, desc.neuron_len
        self._ws = _Workspace()

    @property
    def payload_bytes(self) -> int:
        return int(self.desc.payload_bytes)

    @staticmethod
    def from_header(h: F.NvqHeader, blob, device="cuda") -> "NvqsWeight":
        if h.gs != 24 or h.sub_bits != 4:
            raise NotImplementedError(f"{h.dtype}: NVQ runs only with gs24 and 4-bit states")
        if not h.jsc and h.codebook not in ("e8_256", "d4_256"):
            raise NotImplementedError(f"plain NVQ with the {h.codebook} codebook has no dtype in the runtime")
        device = torch.device(device)
        desc = L.NvqsDesc()
        lib = L.lib()
        L.check(lib.mfq_hip_nvqs_plan(h.vector_size, h.index_bits, h.banks if h.jsc else 1,
                                      int(h.sign_mode == "index_parity"), h.out, h.neuron_len, C.byref(desc)))
        payload = _upload(blob, h.body_off, h.body_bytes, device)
        data = torch.empty(int(desc.total_bytes), dtype=torch.uint8, device=device)
        grid = None if h.jsc else torch.from_numpy(builtin_grid(h.codebook)).to(device)
        L.check(lib.mfq_hip_nvqs_repack(C.byref(desc), _ptr(payload), h.body_bytes, int(h.jsc), _ptr(grid), _ptr(data),
                                        _stream()))
        torch.cuda.current_stream().synchronize()
        return NvqsWeight(desc, data, h.dtype)

    @staticmethod
    def from_lowbit_blob(dtype: str, blob, device="cuda") -> "NvqsWeight":
        """NVQ1-L / NVQ1-S / NPQ0-L / NPQ0-S (formats 1, 8, 7, 9 of the reference's unpack_nvq,
        cpp_runtime/mfq_decode.cpp:3759-3770): the same in-place streams, ternary or product codebooks."""
        h = F.parse_lowbit(dtype, blob)
        device = torch.device(device)
        desc = L.NvqsDesc()
        lib = L.lib()
        fmt = {"NVQ1-L": L.NVQS_NVQ1_L, "NVQ1-S": L.NVQS_NVQ1_S, "NPQ0-L": L.NVQS_NPQ0_L, "NPQ0-S": L.NVQS_NPQ0_S}[dtype]
        L.check(lib.mfq_hip_nvqs_plan_lowbit(fmt, h.state_bits, h.out, h.neuron_len, C.byref(desc)))
        body = _upload(blob, h.body_off, h.body_bytes, device)
        data = torch.empty(int(desc.total_bytes), dtype=torch.uint8, device=device)
        grid = None
        if dtype == "NVQ1-L" and h.table_bytes == 0:      # the built-in 2048-entry ternary grid, packed
            raw = np.frombuffer((_DATA / "iq1s_2048.bin").read_bytes(), dtype=np.uint8)
            grid = torch.from_numpy(raw.copy()).to(device)
        L.check(lib.mfq_hip_nvqs_repack_lowbit(C.byref(desc), _ptr(body), h.body_bytes, _ptr(grid), _ptr(data), _stream()))
        torch.cuda.current_stream().synchronize()
        return NvqsWeight(desc, data, dtype)

    def dequantize(self) -> torch.Tensor:
        w = torch.empty((self.out, self.neuron_len), dtype=torch.float32, device=self.data.device)
        L.check(L.lib().mfq_hip_nvqs_dequant_f32(C.byref(self.desc), _ptr(self.data), _ptr(w), self.neuron_len, _stream()))
        return w


def nvq_matmul_multi2(first: NvqWeight, second: NvqWeight, x: torch.Tensor) -> torch.Tensor:
    """cat(x @ W0^T, x @ W1^T) for two NVQ tensors that share their input, in one launch for small batches
    (nvq_matmul_multi2, cpp_runtime/mfq_decode.cpp:7981-8003)."""
    if first.neuron_len != second.neuron_len:
        raise ValueError("NVQ multi-projection requires compatible formats and input layouts")
    x2 = _as_2d(x, first.neuron_len)
    M, N = x2.shape[0], first.out + second.out
    if M > 32 or isinstance(first, NvqsWeight) or isinstance(second, NvqsWeight):
        return torch.cat([nvq_matmul(first, x), nvq_matmul(second, x)], dim=-1)
    y = torch.empty((M, N), dtype=torch.float32, device=x.device)
    if M == 0:
        return y.reshape(*x.shape[:-1], N)
    L.check(L.lib().mfq_hip_nvq_gemv_multi2(C.byref(first.desc), _ptr(first.data), C.byref(second.desc), _ptr(second.data),
                                            _ptr(x2), _x_dtype(x2), x2.stride(0), M, _ptr(y), N, _stream()))
    return y.reshape(*x.shape[:-1], N)


def nvq_matmul_swiglu(gate: NvqWeight, up: NvqWeight, x: torch.Tensor, out_dtype=torch.float16) -> torch.Tensor:
    """silu(x @ Wg^T) * (x @ Wu^T) for an NVQ gate/up pair (nvq_matmul_swiglu, cpp_runtime/mfq_decode.cpp:8004-8029): the
    joint two-projection launch followed by the elementwise SwiGLU kernel (the reference fuses the two for one row)."""
    if gate.neuron_len != up.neuron_len or gate.out != up.out:
        raise ValueError("NVQ SwiGLU requires compatible equal-width gate/up weights")
    from .runtime_moe import moe_swiglu
    return moe_swiglu(nvq_matmul_multi2(gate, up, x), out_dtype)


def nvq_ffn_swiglu_down(gate: NvqWeight, up: NvqWeight, down: NvqWeight, x: torch.Tensor) -> torch.Tensor:
    """Wd · (silu(Wg·x) * (Wu·x)) for an NVQ feed-forward block (nvq_ffn_swiglu_down, cpp_runtime/mfq_decode.cpp:8032-8071):
    the gate/up launch, the SwiGLU kernel and the down projection on its fp16 output -- three launches where the
    reference quantizes the hidden row to int8 inside one kernel for a single row."""
    if gate.neuron_len != up.neuron_len or gate.out != up.out or gate.out != down.neuron_len:
        raise ValueError("NVQ fused FFN weight layouts are incompatible")
    return nvq_matmul(down, nvq_matmul_swiglu(gate, up, x))


def nvq_matmul(w: NvqWeight, x: torch.Tensor, *, force: str | None = None) -> torch.Tensor:
    """cpp_runtime/mfq_decode.cpp:7884: GEMV up to M = 13 for the D4 family, MFMA path above."""
    x2 = _as_2d(x, w.neuron_len)
    M = x2.shape[0]
    y = torch.empty((M, w.out), dtype=torch.float32, device=x.device)
    if M == 0:                                   # an empty batch: nothing to launch
        return y.reshape(*x.shape[:-1], w.out)
    lib = L.lib()
    if isinstance(w, NvqsWeight):
        need = lib.mfq_hip_nvqs_gemm_workspace_bytes(C.byref(w.desc), M)
        ws = w._ws.get(need, x.device)
        L.check(lib.mfq_hip_nvqs_gemm(C.byref(w.desc), _ptr(w.data), _ptr(x2), _x_dtype(x2), x2.stride(0), M, _ptr(y),
                                      w.out, _ptr(ws), need, _stream()))
        return y.reshape(*x.shape[:-1], w.out)
    if force == "gemv":
        L.check(lib.mfq_hip_nvq_gemv(C.byref(w.desc), _ptr(w.data), _ptr(x2), _x_dtype(x2), x2.stride(0), M, _ptr(y),
                                     w.out, _stream()))
    else:
        need = lib.mfq_hip_nvq_gemm_workspace_bytes(C.byref(w.desc), M)
        ws = w._ws.get(need, x.device)
        L.check(lib.mfq_hip_nvq_gemm(C.byref(w.desc), _ptr(w.data), _ptr(x2), _x_dtype(x2), x2.stride(0), M, _ptr(y),
                                     w.out, _ptr(ws), need, _stream()))
    return y.reshape(*x.shape[:-1], w.out)


class NepqWeight:
    """[experts, out_per_expert, K]; a dense linear is the experts == 1 case.  NEPQ1-S / NEPQ1-L live in the lane-major
    layout of mfq_hip_nepq_*; NEPQ0-S / NEPQ0-L (`streams`) keep their bit streams and run on mfq_hip_nvqs_*_rows."""

    def __init__(self, desc, data, header: F.NepqHeader, signs):
        self.desc, self.data, self.label = desc, data, header.label
        self.streams = isinstance(desc, L.NvqsDesc)
        self.n_experts, self.out_per_expert, self.neuron_len = header.n_experts, header.out_per_expert, header.neuron_len
        self.out = header.out_per_expert
        self.rotation_block, self.rotation_seed, self.signs = header.rotation_block, header.rotation_seed, signs
        self._ws = _Workspace()

    @property
    def payload_bytes(self) -> int:
        return int(self.desc.payload_bytes)

    @staticmethod
    def from_blob(blob, device="cuda", rotation_signs=None) -> "NepqWeight":
        h = F.parse_nepq(blob)
        device = torch.device(device)
        lib = L.lib()
        payload = _upload(blob, h.body_off, h.body_bytes, device)
        if h.profile < 2:       # NEPQ0: the product tables of NPQ0, read in place
            desc = L.NvqsDesc()
            L.check(lib.mfq_hip_nvqs_plan_nepq0(h.profile, h.banks, h.n_experts * h.out_per_expert, h.neuron_len, C.byref(desc)))
            data = torch.empty(int(desc.total_bytes), dtype=torch.uint8, device=device)
            L.check(lib.mfq_hip_nvqs_repack_nepq0(C.byref(desc), _ptr(payload), h.body_bytes, _ptr(data), _stream()))
        else:
            desc = L.NepqDesc()
            L.check(lib.mfq_hip_nepq_plan(h.profile, h.banks, h.n_experts * h.out_per_expert, h.neuron_len, C.byref(desc)))
            data = torch.empty(int(desc.total_bytes), dtype=torch.uint8, device=device)
            L.check(lib.mfq_hip_nepq_repack(C.byref(desc), _ptr(payload), h.body_bytes, _ptr(data), _stream()))
        torch.cuda.current_stream().synchronize()
        signs = None
        if h.rotation_block:
            if rotation_signs is None:
                raise ValueError("rotated NEPQ cohort lacks its runtime sign vector")
            sv = np.ascontiguousarray(rotation_signs, dtype=np.int8).reshape(-1)
            if sv.size != h.neuron_len or not np.all(np.abs(sv) == 1):
                raise ValueError("NEPQ rotation sign vector is corrupt")
            signs = torch.from_numpy(sv).to(device)
        return NepqWeight(desc, data, h, signs)

    def dequantize(self) -> torch.Tensor:
        rows = self.n_experts * self.out_per_expert
        w = torch.empty((rows, self.neuron_len), dtype=torch.float32, device=self.data.device)
        if self.streams:
            L.check(L.lib().mfq_hip_nvqs_dequant_rows_f32(C.byref(self.desc), _ptr(self.data), 0, rows, _ptr(w),
                                                          self.neuron_len, _stream()))
        else:
            L.check(L.lib().mfq_hip_nepq_dequant_f32(C.byref(self.desc), _ptr(self.data), _ptr(w), self.neuron_len, _stream()))
        return w.reshape(self.n_experts, self.out_per_expert, self.neuron_len)


def nepq_hadamard(x: torch.Tensor, signs: torch.Tensor, block: int) -> torch.Tensor:
    x2 = x.reshape(-1, x.shape[-1]).contiguous()
    out = torch.empty_like(x2)
    if x2.shape[0] == 0:
        return out.reshape(x.shape)
    L.check(L.lib().mfq_hip_nepq_hadamard(_ptr(x2), _x_dtype(x2), x2.stride(0), x2.shape[0], x2.shape[1], block,
                                          _ptr(signs), _ptr(out), out.stride(0), _stream()))
    return out.reshape(x.shape)


def nepq_matmul(w: NepqWeight, x: torch.Tensor, expert: int = 0, *, force: str | None = None) -> torch.Tensor:
    """mfq/kernels/cuda/nepq_matmul.py:215-280: rotate the input when the tensor is rotated, then
    GEMV (M <= 16) or the MFMA path."""
    if not 0 <= expert < w.n_experts:
        raise ValueError(f"expert {expert} outside [0, {w.n_experts})")
    if w.rotation_block:
        x = nepq_hadamard(x, w.signs, w.rotation_block)
    x2 = _as_2d(x, w.neuron_len)
    M = x2.shape[0]
    n = w.out_per_expert
    y = torch.empty((M, n), dtype=torch.float32, device=x.device)
    if M == 0:
        return y.reshape(*x.shape[:-1], n)
    lib = L.lib()
    row0 = expert * n
    if w.streams:
        need = lib.mfq_hip_nvqs_gemm_rows_workspace_bytes(C.byref(w.desc), n, M)
        ws = w._ws.get(need, x.device)
        L.check(lib.mfq_hip_nvqs_gemm_rows(C.byref(w.desc), _ptr(w.data), row0, n, _ptr(x2), _x_dtype(x2), x2.stride(0), M,
                                           _ptr(y), n, _ptr(ws), need, _stream()))
        return y.reshape(*x.shape[:-1], n)
    if force == "gemv":
        L.check(lib.mfq_hip_nepq_gemv(C.byref(w.desc), _ptr(w.data), row0, n, _ptr(x2), _x_dtype(x2), x2.stride(0), M,
                                      _ptr(y), n, _stream()))
    else:
        need = lib.mfq_hip_nepq_gemm_workspace_bytes(C.byref(w.desc), n, M)
        ws = w._ws.get(need, x.device)
        L.check(lib.mfq_hip_nepq_gemm(C.byref(w.desc), _ptr(w.data), row0, n, _ptr(x2), _x_dtype(x2), x2.stride(0), M,
                                      _ptr(y), n, _ptr(ws), need, _stream()))
    return y.reshape(*x.shape[:-1], n)
