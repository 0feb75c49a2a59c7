"""CPU oracle: test infrastructure only (see cpu_oracle.py)."""
