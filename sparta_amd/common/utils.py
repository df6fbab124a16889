"""Small helpers shared by the host-side modules."""
from typing import Any


def check_type(value: Any, expected: type):
    """Raise AssertionError unless `value` is an instance of `expected`
    (sparta/common/utils.py: check_type)."""
    assert isinstance(value, expected), f'expected {expected}, got {type(value)}'
