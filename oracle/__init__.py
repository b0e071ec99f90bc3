"""CPU restatements of the reference algorithms.  Test infrastructure only:
importable from tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
leg, never from moonep_amd."""
