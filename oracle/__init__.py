"""CPU checker for the DGE query path.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this package; the shipped package (vtpack_amd) never does.
"""
