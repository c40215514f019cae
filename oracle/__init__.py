"""CPU oracle: test infrastructure only (see xft_oracle.c header)."""
