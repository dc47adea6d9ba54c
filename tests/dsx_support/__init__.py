"""Helpers shared by the tests, bench.py and the smoke check: seeded synthetic workloads (synth) and a driver of the C ABI for
one workload (pipeline).  Not part of the product package; the package must already be loaded (as amazon_dsstne_amd)."""
