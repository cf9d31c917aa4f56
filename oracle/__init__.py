"""CPU checkers for the DP hot path: test infrastructure only (see dp_oracle.c)."""
