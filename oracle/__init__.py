"""CPU checker for the Q4_K x Q8_K path.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this package; the product (densecore_amd, the HIP library) never does.
"""
