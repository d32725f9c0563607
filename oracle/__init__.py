"""CPU checker for the optimizer step (test infrastructure only)."""
