"""CPU oracle: test infrastructure only (see zmi_oracle.c)."""
