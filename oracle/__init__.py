"""CPU oracle (test infrastructure only; see sq_oracle.py)."""
