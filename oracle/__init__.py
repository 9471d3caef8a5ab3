"""CPU oracle of the WTConv layer: test infrastructure only (see wtconv_ref.py)."""
