"""CPU oracle (test infrastructure only; see nq_oracle.py)."""
