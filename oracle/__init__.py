"""CPU oracle for the group-quantized linear path: test infrastructure, never shipped."""
