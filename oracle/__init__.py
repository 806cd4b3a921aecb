"""CPU oracle for the attention / RMSNorm / RoPE hot path — test infrastructure only (see tprime_oracle.py)."""
