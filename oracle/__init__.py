"""CPU oracle (test infrastructure only): see ref_ops.py.  Never imported by the product path."""
