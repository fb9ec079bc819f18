"""CPU oracle for the GCA hot path: test infrastructure only (see gca_oracle.py)."""
