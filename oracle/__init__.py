"""CPU oracle of the FP8 quantized-linear path. TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this package; the shipped package (cache_dit_amd) never does.
"""
