"""Toy models using the fused layers (counterparts of atex/nv_norms/examples/*.py)."""
