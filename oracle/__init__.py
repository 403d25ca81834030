"""CPU oracle (test infrastructure only; see pskv_oracle.h)."""
