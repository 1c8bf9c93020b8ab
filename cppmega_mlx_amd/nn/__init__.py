"""Operator layer: the sparse-MLA dispatcher and the kernel-facing ``_tilelang`` modules."""
