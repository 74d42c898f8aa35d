"""CPU oracle for the MoE layer: test infrastructure, never part of the product path."""
