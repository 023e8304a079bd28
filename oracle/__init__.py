"""CPU oracle for the CASTLE attention hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package may import this
directory; it is used by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py, always as the checker, never as the thing that is
measured or shipped.
"""
