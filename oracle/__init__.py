"""CPU oracle of the gated-attention path: test infrastructure only (see oracle/oracle.py)."""
