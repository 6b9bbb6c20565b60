"""CPU oracle of XCCL's host reduction path.  Test infrastructure, not product:
only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import it."""
