"""CPU oracle of the HashAttention decode path: test infrastructure, never imported by the shipped package."""
