"""CPU oracle (test infrastructure only).  See rk_oracle.h."""
