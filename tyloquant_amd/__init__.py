"""tyloquant_amd: MI355X (gfx950) implementation of the MFQ packed-weight matmul path.

`tyloquant_amd.runtime` holds the operator surface (load_quant_linear, nint_matmul, nvq_matmul,
nepq_matmul, build_moe_route_plan, nint_moe_ffn_forward); `tyloquant_amd.formats` the MFQ payload
writers/parsers; the kernels live in tyloquant_amd/csrc behind the C ABI of include/mfq_hip.h.
"""
__version__ = "0.1.0"
