"""CPU oracle of the FP8 quantized-matmul path (test infrastructure only).

Only tests, the smoke test and the CPU-baseline leg of the benchmark import this package; the
shipped library (llmq_amd) never does.
"""
