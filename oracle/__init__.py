"""CPU oracle for Evoformer attention (test infrastructure; never imported by the product)."""
