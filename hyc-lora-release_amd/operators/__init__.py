"""Operator API with the reference's function names (reference: operators/*.py)."""
