"""CPU oracle: test infrastructure only (the checker and the timed CPU port)."""
