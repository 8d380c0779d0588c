"""TEST INFRASTRUCTURE: CPU oracle for the Tucker-convolution path.

Importable only from tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg.  The product package never imports it.
"""
