"""CPU oracle for the ragged batched decode step: test infrastructure only.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this package; the
product path (goinfer_amd) never does.
"""
