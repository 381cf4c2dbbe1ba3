"""CPU checker for the HIP path (test infrastructure only; never imported by the product)."""
