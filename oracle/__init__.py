"""CPU oracle of the 4-bit GPTQ hot path: test infrastructure, never the product path."""
