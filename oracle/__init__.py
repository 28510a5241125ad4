"""CPU oracle package -- test infrastructure only (see mccl_oracle.c header)."""
