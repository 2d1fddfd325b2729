"""CPU oracle for the HSTU jagged attention forward path.  Test infrastructure only:
imported by tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py."""
