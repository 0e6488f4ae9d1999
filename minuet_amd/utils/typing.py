"""Type aliases used in signatures (mirrors minuet/utils/typing.py)."""
from typing import Iterable, Tuple, TypeVar, Union

__all__ = ["ScalarOrIterable", "ScalarOrTuple"]

T = TypeVar("T")
ScalarOrTuple = Union[T, Tuple[T, ...]]
ScalarOrIterable = Union[T, Iterable[T]]
