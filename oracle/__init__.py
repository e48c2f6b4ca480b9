"""CPU oracle for the quantized linear path: test infrastructure, not product code."""
