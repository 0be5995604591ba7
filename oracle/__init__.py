"""CPU checker for the MoE hot path: test infrastructure, never part of the product."""
