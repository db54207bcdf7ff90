"""Test-side stand-in for the reference's naive triple-dot-product module (test infrastructure only)."""
