"""CPU oracle package: test infrastructure only (see mx_oracle.py)."""
