"""candy_amd: candy's quantized-matmul path on one MI355X (gfx950).

The product is libcandy_hip.so (hand-written HIP behind a C ABI, include/candy_hip.h).
`candy_amd.hip` is the ctypes binding the tests and the benchmark drive it through;
`candy_amd.synth` draws seeded inputs in candy's block formats.
"""
