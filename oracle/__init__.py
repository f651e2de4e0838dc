"""CPU oracle for the SVC -> SpMM path.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this package; the shipped package never does.
"""
