"""CPU checker for the K-Quant packed-linear path.  Test infrastructure only:
imported by tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline
leg, never by the neuralfn_amd package."""
