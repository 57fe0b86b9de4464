"""CPU oracle for the W8A8 quantized-linear path: test infrastructure, never shipped."""
