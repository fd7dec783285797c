"""CPU oracle (test infrastructure only; see cutile_oracle.py)."""
