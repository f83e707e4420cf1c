"""Plain, slow implementations written from the reference's formulas.

Nothing in here imports the product package: every function is whole-sequence,
cache-free, and exists only so the engine has something independent to be
compared with.
"""
