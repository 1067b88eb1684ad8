"""CPU oracle of the pair-stack path: test infrastructure, never imported by the shipped package."""
