"""Which kernel runs an operation: one table keyed by (operation, dtypes).

The reference keeps a kernel registry keyed by (op type, dtype) and asks it once per
command (src/optype.hpp:51-104, src/engine.cpp:40-57). Here a key holds an ordered list of
routes, because one (operation, dtypes) pair has several kernels that differ by the size of
the step: a route is a named way to run the operation together with the rule that says
which cases it takes. A part describes its case (rows, sizes, flags), asks
:func:`choose`, and calls the route's ``run``. The first registered route whose ``takes``
holds wins, so a route for a narrower case is registered in front of the general one
(``before=``), and another precision or another kernel is added by registering routes: no
part is edited for it.

``dtypes`` is a tuple of torch dtypes whose meaning belongs to the operation ("linear":
(weight, activations); "attention": (cache,)). ``traits`` are names a part may ask a route
for without running it ("pieces": reads piece-major rows, "gated": has the gated epilogue).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable


@dataclass(frozen=True)
class Route:
    name: str
    takes: Callable[[Any], bool]
    run: Callable[..., Any]
    traits: frozenset = field(default_factory=frozenset)


_table: dict[tuple[str, tuple], list[Route]] = {}
_version = 0      # counts the changes of the table: what a part remembers of a choice holds for one version


def version() -> int:
    return _version


def register_route(op: str, dtypes: tuple, name: str, takes: Callable[[Any], bool],
                   run: Callable[..., Any], *, traits=(), before: str | None = None) -> Route:
    """Add a route for (op, dtypes). It goes to the end of the key's list, or in front of the
    route called `before`. A name can be registered once per key."""
    routes = _table.setdefault((op, tuple(dtypes)), [])
    if any(r.name == name for r in routes):
        raise ValueError(f"route {name!r} of {op!r} {_names(dtypes)} is registered already")
    global _version
    _version += 1
    route = Route(name, takes, run, frozenset(traits))
    if before is None:
        routes.append(route)
    else:
        at = [i for i, r in enumerate(routes) if r.name == before]
        if not at:
            raise ValueError(f"route {before!r} of {op!r} {_names(dtypes)} is not registered")
        routes.insert(at[0], route)
    return route


def unregister_route(op: str, dtypes: tuple, name: str) -> None:
    routes = _table.get((op, tuple(dtypes)), [])
    left = [r for r in routes if r.name != name]
    if len(left) == len(routes):
        raise ValueError(f"route {name!r} of {op!r} {_names(dtypes)} is not registered")
    global _version
    _version += 1
    _table[(op, tuple(dtypes))] = left


def routes_of(op: str, dtypes: tuple) -> list[Route]:
    return list(_table.get((op, tuple(dtypes)), ()))


def choose(op: str, dtypes: tuple, case: Any) -> Route:
    """The first route of (op, dtypes) that takes the case. Unknown dtypes and a case that no
    route takes are errors that say what is registered."""
    routes = _table.get((op, tuple(dtypes)))
    if not routes:
        known = sorted(_names(k[1]) for k in _table if k[0] == op)
        raise TypeError(f"{op}: no kernel for {_names(dtypes)}; registered: {', '.join(known) or 'nothing'}")
    for route in routes:
        if route.takes(case):
            return route
    raise ValueError(f"{op}: none of the routes {[r.name for r in routes]} for {_names(dtypes)} takes {case}")


def table() -> dict[str, list[str]]:
    """'op (dtypes)' -> route names in the order they are tried; for documentation and tests."""
    return {f"{op} {_names(dt)}": [r.name for r in routes] for (op, dt), routes in sorted(
        _table.items(), key=lambda kv: (kv[0][0], _names(kv[0][1])))}


def _names(dtypes) -> str:
    return "(" + ", ".join(str(d).replace("torch.", "") for d in dtypes) + ")"
