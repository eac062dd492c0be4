"""CPU oracle for candy's quantized-matmul path. Test infrastructure only."""
