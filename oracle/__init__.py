"""CPU oracle of the quantized-GEMM path: test infrastructure, not part of the product."""
