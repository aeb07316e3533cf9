"""CPU oracle of the MFQ packed-weight matmul path: test infrastructure, never shipped code."""
