"""CPU oracle for the cosine-linear-attention hot path -- test infrastructure only.

Nothing under this package is part of the shipped GPU path.  Only tests, the smoke check and the
benchmark's ``cpu_baseline`` leg import it, and only as the checker.
"""
