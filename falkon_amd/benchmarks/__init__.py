"""Timing scripts for the kernel-vector products (the reference ships its own under falkon/benchmarks)."""
