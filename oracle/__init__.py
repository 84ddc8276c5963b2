"""CPU oracles for the periodic-attention hot path: test infrastructure, never the product path."""
