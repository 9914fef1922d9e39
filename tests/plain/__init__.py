"""Plain, slow LFM2 implementation used as the oracle by the tests.

Written from the reference's formulas (every function cites file:line of the
reference).  It shares no code with the product package: it runs on the CPU,
on whole sequences, without any cache.
"""
