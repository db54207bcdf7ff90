"""Test-side stand-in for the reference's naive dot-product-sum module (test infrastructure only)."""
