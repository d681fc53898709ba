"""Bindings of the hand-written HIP kernels (sources under ``csrc/``)."""
