"""CPU oracle of the tuned operators. TEST INFRASTRUCTURE ONLY: imported by
tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg, never by the
flextensor_amd package."""
