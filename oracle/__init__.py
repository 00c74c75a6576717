"""CPU oracle for the K-FAC hot path: test infrastructure, not product code.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import
this package; chainerkfac_amd never does.
"""
