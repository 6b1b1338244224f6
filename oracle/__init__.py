"""CPU oracle (test infrastructure only): see custos_cpu_oracle.h."""
