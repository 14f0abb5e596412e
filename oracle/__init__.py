"""CPU oracle (test infrastructure only; see hyc_oracle.py)."""
