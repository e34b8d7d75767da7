"""CPU checker for the half-Gaussian rasterizer.  Test infrastructure only: importable from
tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py, never from the
shipped package."""
