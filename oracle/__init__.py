"""CPU restatement of the reference hot path: test infrastructure only (see culsh_oracle.py)."""
