"""Ternary operator layer (mirror of ``boilerplate/ternary``)."""
