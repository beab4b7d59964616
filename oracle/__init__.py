"""CPU oracle for the SAPA upsampling operators.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package may import this:
only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg use it,
and only as the checker, never as the thing being measured or shipped.
"""
