"""Parity oracle (test infrastructure): CPU restatement + optional compiled reference.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this package.
"""
