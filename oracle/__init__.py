"""CPU oracle for the ring-attention block step. TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package imports this; only tests/, the smoke check and the
benchmark's CPU-baseline leg do, and only as the checker.
"""
