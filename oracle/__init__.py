"""CPU oracle for the VQ-GEMM path: test infrastructure, never part of the product."""
