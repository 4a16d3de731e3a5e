"""CPU checker for the W8A8-dynamic fused-MoE layer.

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
benchmark's CPU-baseline leg.  The shipped package never imports it.
"""
