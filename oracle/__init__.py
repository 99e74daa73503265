"""CPU oracle for ring-attention forward.  Test infrastructure only: never imported by
the product package (ringattention_amd); only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py use it."""
