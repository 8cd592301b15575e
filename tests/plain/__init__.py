"""Plain, slow, whole-sequence implementation used only as the test oracle.

Nothing under this folder is imported by the product package, and nothing here
imports the product package: the two meet only in the tests that compare them.
"""
