"""Compute kernels of the chunk-scheduled path: thin Python launchers over the C ABI."""
