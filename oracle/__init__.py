"""CPU oracle of the dispatch/combine hot path — test infrastructure only.

Importable from tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg;
never from the product package.
"""
