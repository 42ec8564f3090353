"""TEST INFRASTRUCTURE ONLY: CPU oracle of the fused merge-path SpMV / map + reducer + aggregator
path (a restatement of the reference's CPU path) and the recipes that build it.  Only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg may import this package."""
