"""Operator benchmark rows in the reference's schema."""
