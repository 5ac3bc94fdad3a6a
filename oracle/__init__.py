"""CPU oracle for the quantized-matmul path. Test infrastructure only."""
