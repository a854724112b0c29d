"""CPU oracle for the W4A16 Marlin-surface hot path.

TEST INFRASTRUCTURE ONLY.  This package restates, in numpy / CPU torch, the
pure functions of the reference that define what the GPU path must compute:
the RTN quantizers and checkpoint packers, the Marlin weight / scale /
zero-point / bias layouts, "dequantize then fp32 matmul", and the MoE glue.
Only tests, the smoke check and the benchmark's CPU-baseline leg may import
it; nothing in the shipped `vllm_amd` package does.

Pin status (what independently fixes each function is listed in the module
docstrings): every function here is pinned by hand-derived known answers,
dual formulations, algebraic invariants or brute force; none is
"parity unpinned".
"""
