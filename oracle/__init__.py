"""CPU oracle of the fused linear-logprob path: test infrastructure, never shipped code."""
