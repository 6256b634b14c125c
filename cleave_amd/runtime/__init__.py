"""Compile, validate and time generated kernels."""
