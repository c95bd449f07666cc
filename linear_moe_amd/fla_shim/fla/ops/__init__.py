"""Operator namespace of the shim."""
