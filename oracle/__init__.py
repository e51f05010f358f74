"""Test infrastructure only: the CPU oracle (hostref) of the HIP tensor backend.  Not imported by the product."""
