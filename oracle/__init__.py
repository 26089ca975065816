"""CPU oracle of the mixed-precision MoE GroupGEMM path — test infrastructure, never a product path."""
