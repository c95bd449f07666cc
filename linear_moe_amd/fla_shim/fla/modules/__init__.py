"""Module namespace of the shim."""
