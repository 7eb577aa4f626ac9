"""CPU oracle for the hashmap / DOK hot path.  TEST INFRASTRUCTURE ONLY: imported by tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg, never by the doksparse_amd package."""
