"""CPU oracle package (test infrastructure only; see st_oracle.h)."""
