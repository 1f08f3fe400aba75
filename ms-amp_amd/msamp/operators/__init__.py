"""Operators of the FP8 hot path."""
