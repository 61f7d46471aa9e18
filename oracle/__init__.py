"""CPU oracle for the MatConvNet backward hot path.  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the CPU-baseline leg of the benchmark may import this package; the
shipped library never does.
"""
