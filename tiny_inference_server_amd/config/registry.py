"""A name -> object table with errors that list what is known.

Every kind of part (mixer, feed-forward, norm, position encoding, block
arrangement) and the architectures themselves are looked up in one of these,
so that a new one is added by registering it, from inside or outside the
package, without editing the code that does the lookup.
"""
from __future__ import annotations

from typing import Dict, Generic, Iterator, TypeVar

T = TypeVar("T")


class Registry(Generic[T]):
    def __init__(self, what: str):
        self.what = what
        self._items: Dict[str, T] = {}

    def register(self, name: str, item: T | None = None, *, replace: bool = False):
        """`reg.register("x", obj)` or `@reg.register("x")` above a class or function."""
        def put(obj: T) -> T:
            if name in self._items and not replace:
                raise KeyError(f"{self.what} {name!r} is already registered")
            self._items[name] = obj
            return obj
        if item is not None:
            return put(item)
        return put

    def unregister(self, name: str) -> None:
        self._items.pop(name, None)

    def get(self, name: str) -> T:
        try:
            return self._items[name]
        except KeyError:
            known = ", ".join(sorted(self._items)) or "<none>"
            raise KeyError(f"unknown {self.what} {name!r}; known: {known}") from None

    def __contains__(self, name: str) -> bool:
        return name in self._items

    def __iter__(self) -> Iterator[str]:
        return iter(sorted(self._items))
