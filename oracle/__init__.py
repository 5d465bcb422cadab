"""CPU oracle (test infrastructure only; see mx_oracle.py and ref_scalar.c)."""
