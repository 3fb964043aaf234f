"""CPU oracle (test infrastructure only; see xlite_oracle.py)."""
