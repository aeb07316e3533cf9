"""MXFP4 / MXFP8 weights of full-precision MFQ files and their matmul (see runtime.py).

Mirrors the reference's Mxfp8Weight / mxfp8_matmul_f32 (cpp_runtime/mfq_decode.cpp:2060-2100, 8784-8802) and, for MXFP4
expert pools, dequant_mxfp4_cpu / select_mxfp4_cpu_rows (:1920-1975): the payload's value and scale bytes are used on the
device as they lie in the file."""
from __future__ import annotations

import torch

from . import _lib as L
from . import formats as F
from .runtime import _Workspace, _as_2d, _ptr, _stream, _upload, _x_dtype


class MxWeight:
    """[rows, cols] (a linear), or a pool of experts of `out` rows each when `out` is given."""

    def __init__(self, header: F.MxHeader, values: torch.Tensor, scales: torch.Tensor, out: int | None = None):
        self.header, self.values, self.scales = header, values, scales
        self.dtype, self.kind, self.rows, self.neuron_len = header.dtype, header.kind, header.rows, header.cols
        self.out = self.rows if out is None else int(out)
        if self.out <= 0 or self.rows % self.out:
            raise ValueError(f"{self.dtype}: {self.rows} rows are not a whole number of experts of {self.out}")
        if self.kind == 8 and self.out != self.rows and self.out % 128:
            raise ValueError("MXFP8 expert slices must preserve 128-row blocks")
        self.n_experts = self.rows // self.out
        self.data = values                      # the device tensor other weights call `data`
        self._ws = _Workspace()

    @property
    def payload_bytes(self) -> int:
        return self.header.values_bytes + self.header.scales_bytes

    @staticmethod
    def from_blob(dtype: str, blob, device="cuda", out: int | None = None) -> "MxWeight":
        h = F.parse_mx(dtype, blob)
        device = torch.device(device)
        values = _upload(blob, h.values_off, h.values_bytes, device)
        scales = _upload(blob, h.scales_off, h.scales_bytes, device)
        torch.cuda.current_stream().synchronize()
        return MxWeight(h, values, scales, out)

    def _rows(self, expert: int):
        if not 0 <= expert < self.n_experts:
            raise IndexError(f"{self.dtype}: expert {expert} of {self.n_experts}")
        return expert * self.out, self.out

    def dequantize(self, expert: int = 0, dtype=torch.float32) -> torch.Tensor:
        """fp32: element x scale; fp16: that rounded once more, as the reference's device copy is."""
        row0, nrows = self._rows(expert)
        if dtype not in (torch.float32, torch.float16):
            raise ValueError(f"MX weights dequantize to fp32 or fp16, not {dtype}")
        w = torch.empty((nrows, self.neuron_len), dtype=dtype, device=self.values.device)
        L.check(L.lib().mfq_hip_mx_dequant_rows(self.kind, _ptr(self.values), _ptr(self.scales), self.rows, self.neuron_len,
                                                row0, nrows, L.X_F32 if dtype == torch.float32 else L.X_F16, _ptr(w),
                                                self.neuron_len, _stream()))
        return w


def mx_matmul(w: MxWeight, x: torch.Tensor, expert: int = 0) -> torch.Tensor:
    """x @ W^T in fp32 (mxfp8_matmul_f32, cpp_runtime/mfq_decode.cpp:8784-8802): the matrix-core tile kernels up to 256 rows (a
    wave per neuron for activations they cannot read in 16-byte pieces), the fp16 copy + MFMA GEMM above."""
    row0, nrows = w._rows(expert)
    x2 = _as_2d(x, w.neuron_len)
    M = x2.shape[0]
    y = torch.empty((M, nrows), dtype=torch.float32, device=x.device)
    if M == 0:
        return y.reshape(*x.shape[:-1], nrows)
    lib = L.lib()
    need = lib.mfq_hip_mx_gemm_rows_workspace_bytes(w.neuron_len, nrows, M)
    ws = w._ws.get(need, x.device)
    L.check(lib.mfq_hip_mx_gemm_rows(w.kind, _ptr(w.values), _ptr(w.scales), w.rows, w.neuron_len, row0, nrows, _ptr(x2),
                                     _x_dtype(x2), x2.stride(0), M, _ptr(y), nrows, _ptr(ws), need, _stream()))
    return y.reshape(*x.shape[:-1], nrows)
