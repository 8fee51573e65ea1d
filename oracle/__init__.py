"""CPU oracle (test infrastructure). See kvx_oracle.py."""
