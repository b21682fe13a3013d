"""TEST INFRASTRUCTURE: CPU oracle of the reference semantics (see tcbnn_oracle.cpp).
Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this."""
