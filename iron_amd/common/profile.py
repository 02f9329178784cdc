"""Tunable values by operator shape (iron/common/declare/profile.py:26-200).

A profile is a list of entries, each naming an operator class, the ``param()`` values it applies to
and the ``tunable()`` values it gives.  A graph holding one (``Graph.profile``) fills every open
tunable of the steps it records from the most specific entry that matches.  The reference's
per-device files (``profiles/<device>.json``) load as they are: their tunables are AIE tile and
column counts, which the operator classes here accept and carry and no HIP launch reads.
"""

from __future__ import annotations

import json
from collections.abc import Mapping
from enum import Enum
from pathlib import Path
from typing import Any

from .declare import _MISSING, _is_factory


class Profile:
    def __init__(self) -> None:
        self._entries: list[tuple[type, dict[str, Any], dict[str, Any]]] = []

    def __len__(self) -> int:
        return len(self._entries)

    def add(self, cls: type, **fields: Any) -> None:
        """An entry for ``cls``: its ``param()`` values to match (one left out matches any) and the
        ``tunable()`` values it gives.

        Raises:
            TypeError: a field ``cls`` does not declare, or no tunable among them.
        """
        params = cls.declaration.params
        unknown = [n for n in fields if n not in params]
        if unknown:
            raise TypeError(f"{cls.__name__} declares no field {unknown}")
        tunables = {n: v for n, v in fields.items() if params[n].tunable}
        dims = {n: v for n, v in fields.items() if not params[n].tunable}
        if not tunables:
            raise TypeError(f"an entry for {cls.__name__} must give a tunable")
        self._entries.append((cls, dims, tunables))

    @staticmethod
    def dims(cls: type, given: Mapping[str, Any]) -> dict[str, Any]:
        """Every dimension a ``cls(**given)`` call makes, as an entry is matched against them: one
        left out is its default, ``None`` where a function computes it."""
        out = {}
        for name, p in cls.declaration.params.items():
            if p.tunable:
                continue
            if given.get(name) is not None:
                out[name] = given[name]
            elif p.derive is not None or _is_factory(p.default):
                out[name] = None
            elif p.default is not _MISSING:
                out[name] = p.default
        return out

    def tunables_for(self, cls: type, given: Mapping[str, Any]) -> dict[str, Any]:
        """The tunables of the ``cls`` a call with ``given`` keywords makes, each from the most
        specific entry that names it.

        Raises:
            ValueError: two entries of equal specificity disagree.
        """
        dims = self.dims(cls, given)
        chosen: dict[str, tuple[int, Any]] = {}
        for base, matched, tunables in self._entries:
            if not issubclass(cls, base) or any(n not in dims or dims[n] != v for n, v in matched.items()):
                continue
            rank = len(matched)
            for name, value in tunables.items():
                if name not in chosen or rank > chosen[name][0]:
                    chosen[name] = (rank, value)
                elif rank == chosen[name][0] and chosen[name][1] != value:
                    raise ValueError(f"profile is ambiguous for {cls.__name__} {dims}: {name}={chosen[name][1]} and "
                                     f"{name}={value} from entries of equal specificity")
        return {name: value for name, (_, value) in chosen.items()}

    #: What a graph's recorder asks for each step it constructs.
    lookup = tunables_for

    def make(self, cls: type, **kwargs: Any):
        """``cls(**kwargs)`` with its open tunables filled from this profile."""
        given = {n: v for n, v in kwargs.items() if v is not None}
        return cls(**{**self.tunables_for(cls, given), **given})

    @classmethod
    def load(cls, path) -> "Profile":
        """The profile ``save`` (or the reference) wrote to ``path``: ``{"entries": [{"operator": name,
        field: value, ...}, ...]}``.

        Raises:
            ValueError: not that form, or an operator the catalog does not hold.
        """
        from ..operators import CATALOG

        data = json.loads(Path(path).read_text())
        if not isinstance(data, dict) or set(data) != {"entries"}:
            raise ValueError(f"{path}: a profile is {{'entries': [...]}}")
        profile = cls()
        for entry in data["entries"]:
            fields = dict(entry)
            name = fields.pop("operator")
            if name not in CATALOG:
                raise ValueError(f"{path}: no operator {name!r} in the catalog")
            op = CATALOG[name]
            for key, p in op.declaration.params.items():   # an Enum's member is its value in JSON
                if key in fields and isinstance(p.domain, type) and issubclass(p.domain, Enum):
                    fields[key] = p.domain(fields[key])
            profile.add(op, **fields)
        return profile

    def save(self, path) -> None:
        """Write the profile as JSON, an entry a line."""
        from ..operators import CATALOG

        names = {op: name for name, op in CATALOG.items()}
        lines = []
        for op, dims, tunables in self._entries:
            if op not in names:
                raise ValueError(f"{op.__name__} is not in the catalog")
            fields = {"operator": names[op], **dims, **tunables}
            lines.append("  " + json.dumps({k: (v.value if isinstance(v, Enum) else v) for k, v in fields.items()}))
        Path(path).write_text('{"entries": [\n' + ",\n".join(lines) + "\n]}\n")
