"""Model-level measurement harnesses around the blockwise int8 linear layer (synthetic data, random weights)."""
