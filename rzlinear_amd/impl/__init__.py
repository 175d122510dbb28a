"""Launchers of the gfx950 kernels, one module per launcher file of the reference package."""
