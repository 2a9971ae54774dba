"""CPU oracle of the SC convolution hot path: test infrastructure, not product code."""
