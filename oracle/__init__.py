"""CPU oracle for the trittention hot path: test infrastructure only.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import
this package; the HIP library and its Python host code never do.
"""
