"""CPU oracle for the sub-2-bit hot path: test infrastructure, never shipped code."""
