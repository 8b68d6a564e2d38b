"""CPU oracle for the INT8-X hot path (test infrastructure, never shipped)."""
