"""CPU oracle of the MatGPTQ bit-sliced GEMM path.  Test infrastructure only:
imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg."""
