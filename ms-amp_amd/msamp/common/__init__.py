"""Common building blocks: dtypes, scaling tensors, utilities."""
