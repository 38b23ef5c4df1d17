"""CPU oracle (test infrastructure only; see q4_oracle.py)."""
