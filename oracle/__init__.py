"""CPU oracle of the reference arithmetic: test infrastructure, never imported by the product."""
