"""CPU oracle for the quantized-weight LoRA matmul path.  TEST INFRASTRUCTURE ONLY: nothing under
the product package imports this; it exists so tests, the smoke check and the CPU-baseline leg of
the benchmark have an independent statement of the reference's arithmetic."""
