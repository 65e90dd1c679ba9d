"""Name -> factory tables.  Everything that can be chosen by a configuration
(an architecture, a mixer, a feed-forward, a norm, a position encoding, a block
arrangement) is looked up in one of these, so a new kind is added by one
`register` call and no change to the code that uses it."""
from __future__ import annotations

from typing import Callable, Dict, Generic, Iterable, TypeVar

T = TypeVar("T")


class UnknownName(KeyError):
    def __str__(self) -> str:  # KeyError would quote the message
        return self.args[0]


class Registry(Generic[T]):
    def __init__(self, what: str):
        self.what = what
        self._items: Dict[str, T] = {}

    def register(self, names: str | Iterable[str], item: T | None = None, *, replace: bool = False):
        """`register(name, item)` or `@register(name)` above a class or function."""
        if isinstance(names, str):
            names = (names,)
        names = tuple(names)

        def put(obj: T) -> T:
            for n in names:
                if n in self._items and not replace:
                    raise ValueError(f"{self.what} {n!r} is already registered")
                self._items[n] = obj
            return obj

        return put if item is None else put(item)

    def unregister(self, name: str) -> None:
        self._items.pop(name, None)

    def get(self, name: str) -> T:
        try:
            return self._items[name]
        except KeyError:
            known = ", ".join(sorted(self._items)) or "(none)"
            raise UnknownName(f"unknown {self.what} {name!r}; known: {known}") from None

    def __contains__(self, name: str) -> bool:
        return name in self._items

    def names(self):
        return sorted(self._items)
