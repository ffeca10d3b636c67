"""CPU oracle: test infrastructure only (see mni_oracle.c)."""
