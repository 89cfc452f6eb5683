"""CPU oracle of the array-kernel path: test infrastructure, never shipped or measured as the product."""
