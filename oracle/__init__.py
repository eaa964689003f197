"""TEST INFRASTRUCTURE — the CPU oracle for the scoring + verify path.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this package; verl_amd never does.
"""
