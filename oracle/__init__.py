"""CPU oracle package (test infrastructure only; see infr_cpu_oracle.h)."""
