"""CPU oracle of the EP=1 MoE hot path -- test infrastructure, never imported by the product."""
