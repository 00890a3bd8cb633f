"""CPU oracle for the QUIK MixedQLinear forward path.

Test infrastructure: only tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg may import this package.  The product (quik_amd, quik) never does.
"""
