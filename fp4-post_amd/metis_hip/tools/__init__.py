"""Small runnable helpers that ship with the package (profiling workloads)."""
