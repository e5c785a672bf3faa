"""CPU restatement of the reference's masked incremental path.

Test infrastructure: only tests/, __graft_entry__.smoke() and the cpu_baseline
leg of bench.py import this package, as the checker / reported baseline.
"""
