"""CPU oracle for the GPT-OSS attention hot path.

Test infrastructure: imported only by tests/, by the smoke check and by the
benchmark's CPU-baseline leg.  The shipped package never imports it.
"""
