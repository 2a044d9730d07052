"""CPU oracle for the llama forward + reverse-mode path.

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg, never by the product package (which must fail
loudly when its HIP library is missing rather than fall back to this code).
"""
