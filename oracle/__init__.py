"""CPU oracle of the lpmm 4-bit optimizer-state hot path: test infrastructure only."""
