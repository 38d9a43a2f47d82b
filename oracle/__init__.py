"""Test-only CPU checker (see skl_oracle.h). Never imported by the product."""
