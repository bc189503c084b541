"""Kernel backend interface (mirror of ``boilerplate/kernels``)."""
