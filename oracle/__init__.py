"""CPU oracle (test infrastructure only; see fp8_oracle.py)."""
