"""CPU oracle (test infrastructure).  See fp8_oracle.py for what it restates and how it is pinned."""
