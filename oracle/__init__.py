"""CPU oracle (test infrastructure only): see tuna_oracle.c and oracle.py."""
