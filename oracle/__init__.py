"""CPU oracle (test infrastructure only): see tile_oracle.py."""
