"""CPU oracle (test infrastructure only; see insc_oracle.c)."""
