"""Test package (parity tests of the fused sparse operators)."""
