"""TEST INFRASTRUCTURE: the CPU checker for the gfx950 matrix-multiplication kernels.

Nothing in the shipped package imports this. Only the tests, the smoke check
and the CPU-baseline leg of the benchmark do.
"""
