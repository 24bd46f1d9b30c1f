"""TEST INFRASTRUCTURE ONLY: CPU / eager restatements of the dynamic-mask attention hot path.

Nothing in the product package imports this directory.  It is used by tests/, by
__graft_entry__.smoke() and by the cpu_baseline leg of bench.py, always as the checker.
"""
