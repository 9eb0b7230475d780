"""CPU oracle for the fused temporal SNN operators (test infrastructure; never imported by the product package)."""
