"""Oracle of the NDC hot path: test infrastructure only (see ndc_oracle.py)."""
