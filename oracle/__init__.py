"""CPU oracle of the int8 transformer-layer forward path (test infrastructure only)."""
