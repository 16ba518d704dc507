"""CPU oracle for the MoE path: test infrastructure only (see moe_oracle.py)."""
