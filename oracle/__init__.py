"""CPU oracle of the attention hot path: test infrastructure only."""
