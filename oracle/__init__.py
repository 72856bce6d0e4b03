"""CPU oracle for the AWQ W4A16 path: test infrastructure only (see awq_oracle.py)."""
