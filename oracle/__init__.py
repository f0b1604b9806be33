"""CPU restatements of the reference's step math.  Test infrastructure: imported only by tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg; never by flashoptim_amd."""
