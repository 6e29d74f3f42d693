"""CPU oracle of the save/load hot path. TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this package; the product
(tair_kvcache_amd) never does.
"""
