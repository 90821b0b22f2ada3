"""CPU checker for the hip backend (test infrastructure; never imported by the product)."""
