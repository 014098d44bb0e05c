"""Helpers that mirror the reference's `natten.utils` for the forward path."""
