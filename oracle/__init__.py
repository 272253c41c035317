"""CPU oracle for the DiffLUT hot path: test infrastructure only.

Importable from tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg;
the shipped package (difflut_amd/) never imports it.
"""
