"""Tiny argument helpers."""


def value_or(value, default):
    """`default` stands in for a missing (None) `value`."""
    if value is None:
        return default
    return value
