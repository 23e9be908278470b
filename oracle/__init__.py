"""CPU checker for the FP8 quantized-collective path: test infrastructure only."""
