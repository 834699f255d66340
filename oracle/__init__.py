"""CPU restatement of the reference's mesh conv / pool arithmetic.  TEST INFRASTRUCTURE ONLY:
imported by tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline leg, never by the
product package."""
