"""TEST INFRASTRUCTURE. CPU oracles of the two reference algorithms.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this package; nothing under proteusai_amd/ does.
"""
