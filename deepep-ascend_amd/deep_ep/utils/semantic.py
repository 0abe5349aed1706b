"""Small helpers for optional arguments."""
from typing import Optional, TypeVar

T = TypeVar('T')


def value_or(value: Optional[T], default: T) -> T:
    """The argument the caller gave, or `default` where they left it at None."""
    if value is None:
        return default
    return value
