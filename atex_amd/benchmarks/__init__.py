"""Benchmarks with the shape tables and the timing protocol of the reference's own scripts
(atex/nv_norms/benchmarks/benchmark_layer_norm.py, benchmark_instance_norm.py)."""
