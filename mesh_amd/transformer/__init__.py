"""Transformer layers built on mesh_amd; only the Mixture-of-Experts layers."""
