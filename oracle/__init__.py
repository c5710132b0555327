"""CPU oracle for the ternary-linear hot path (test infrastructure only)."""
