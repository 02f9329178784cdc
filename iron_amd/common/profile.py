"""Per-shape tunable values for recorded operators (interface of iron/common/declare/profile.py:26-200).

A ``Profile`` holds rules: "for operator X with these ``param()`` values, use these ``tunable()``
values".  A graph that carries one (``Graph.profile``) consults it for every step it records and
fills whatever tunables the call left open, the rule that pins the most parameters winning.

The reference ships such rules per device as ``profiles/<device>.json``; those files load here
unchanged.  Their tunables are AIE tile and column counts: this package's operators accept and keep
them (so recordings and their names stay comparable) but no HIP launch depends on them.
"""

from __future__ import annotations

import dataclasses
import json
from collections.abc import Mapping
from enum import Enum
from pathlib import Path
from typing import Any

from .declare import _MISSING, _is_factory


@dataclasses.dataclass(frozen=True)
class _Rule:
    operator: type
    when: dict          # param name -> value that must match
    give: dict          # tunable name -> value supplied

    def applies(self, cls: type, dims: Mapping[str, Any]) -> bool:
        if not issubclass(cls, self.operator):
            return False
        return all(name in dims and dims[name] == value for name, value in self.when.items())


def _jsonable(value):
    return value.value if isinstance(value, Enum) else value


class Profile:
    def __init__(self) -> None:
        self._rules: list[_Rule] = []

    def __len__(self) -> int:
        return len(self._rules)

    def add(self, cls: type, **fields: Any) -> None:
        """Add a rule for ``cls``.  Among ``fields``, ``param()`` names say when the rule applies (a
        param not mentioned matches anything) and ``tunable()`` names say what it supplies.

        Raises:
            TypeError: a name ``cls`` does not declare, or a rule that supplies no tunable.
        """
        declared = cls.declaration.params
        foreign = [name for name in fields if name not in declared]
        if foreign:
            raise TypeError(f"{cls.__name__} declares no field {foreign}")
        when = {name: value for name, value in fields.items() if not declared[name].tunable}
        give = {name: value for name, value in fields.items() if declared[name].tunable}
        if not give:
            raise TypeError(f"an entry for {cls.__name__} must give a tunable")
        self._rules.append(_Rule(cls, when, give))

    @staticmethod
    def dims(cls: type, given: Mapping[str, Any]) -> dict[str, Any]:
        """The ``param()`` values a ``cls(**given)`` call would have, as far as they are known before
        construction: what was passed, else a plain default, else None for a value only a function
        (a derived or computed default) can tell."""
        known = {}
        for name, p in cls.declaration.params.items():
            if p.tunable:
                continue
            passed = given.get(name)
            if passed is not None:
                known[name] = passed
            elif p.derive is not None or _is_factory(p.default):
                known[name] = None
            elif p.default is not _MISSING:
                known[name] = p.default
        return known

    def tunables_for(self, cls: type, given: Mapping[str, Any]) -> dict[str, Any]:
        """Tunables for the instance ``cls(**given)`` would be: per tunable, the value from the
        applicable rule that pins the most params.

        Raises:
            ValueError: two equally specific rules supply different values for one tunable.
        """
        dims = self.dims(cls, given)
        best: dict[str, tuple[int, Any]] = {}      # tunable -> (specificity, value)
        for rule in self._rules:
            if not rule.applies(cls, dims):
                continue
            specificity = len(rule.when)
            for name, value in rule.give.items():
                held = best.get(name)
                if held is None or specificity > held[0]:
                    best[name] = (specificity, value)
                elif specificity == held[0] and held[1] != value:
                    raise ValueError(f"profile is ambiguous for {cls.__name__} {dims}: {name}={held[1]} and "
                                     f"{name}={value} from entries of equal specificity")
        return {name: value for name, (_, value) in best.items()}

    lookup = tunables_for      # the name a recorder calls it by

    def make(self, cls: type, **kwargs: Any):
        """Construct ``cls`` with the profile filling in what ``kwargs`` leaves open (None counts as
        open); anything passed explicitly wins."""
        explicit = {name: value for name, value in kwargs.items() if value is not None}
        return cls(**(self.tunables_for(cls, explicit) | explicit))

    # -- files: {"entries": [{"operator": <catalog name>, <field>: <value>, ...}, ...]}
    @classmethod
    def load(cls, path) -> "Profile":
        """Read a profile file (this package's ``save`` or the reference's).

        Raises:
            ValueError: another layout, or an operator name the catalog lacks.
        """
        from ..operators import CATALOG

        document = json.loads(Path(path).read_text())
        if not (isinstance(document, dict) and set(document) == {"entries"}):
            raise ValueError(f"{path}: a profile is {{'entries': [...]}}")
        profile = cls()
        for entry in document["entries"]:
            fields = {key: value for key, value in entry.items() if key != "operator"}
            name = entry["operator"]
            operator = CATALOG.get(name)
            if operator is None:
                raise ValueError(f"{path}: no operator {name!r} in the catalog")
            for key, p in operator.declaration.params.items():
                # JSON stores an Enum-valued field as the member's value
                if key in fields and isinstance(p.domain, type) and issubclass(p.domain, Enum):
                    fields[key] = p.domain(fields[key])
            profile.add(operator, **fields)
        return profile

    def save(self, path) -> None:
        """Write the rules as JSON, one per line."""
        from ..operators import CATALOG

        catalog_name = {operator: name for name, operator in CATALOG.items()}
        rows = []
        for rule in self._rules:
            if rule.operator not in catalog_name:
                raise ValueError(f"{rule.operator.__name__} is not in the catalog")
            record = {"operator": catalog_name[rule.operator], **rule.when, **rule.give}
            rows.append("  " + json.dumps({key: _jsonable(value) for key, value in record.items()}))
        Path(path).write_text('{"entries": [\n' + ",\n".join(rows) + "\n]}\n")
