"""CPU oracle of the reshard path: test infrastructure, never shipped or measured as product.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this package.
"""
