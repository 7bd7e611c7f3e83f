"""CPU checkers for the bound-propagation kernels.  Test infrastructure only:
importable from tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
leg, never from the faith_amd package."""
