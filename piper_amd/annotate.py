"""`piper.annotate`: tag a region of model code with a schedule name (src/piper.py:51-80).

Contract kept from the reference: the tag name is a non-empty string (anything else is a
``ValueError``); every scope gets a record ``{"name", "index", "uid"}`` where ``index`` counts
the scopes opened under that name so far and ``uid`` counts all scopes of the process; scopes
nest ("PP" around "EP") and the active ones are visible together.  The reference writes the
records into FX node metadata for its graph splitter; here they are what the executor reads to
decide which region a call belongs to.
"""
from __future__ import annotations


PP_TAG = "PP"
EP_TAG = "EP"


class _Scope:
    """One `with annotate(name):` block.  Entering registers the record, leaving removes it."""

    __slots__ = ("_registry", "_name", "record")

    def __init__(self, registry: "_Registry", name: str):
        self._registry = registry
        self._name = name
        self.record: dict | None = None

    def __enter__(self) -> dict:
        self.record = self._registry.open(self._name)
        return self.record

    def __exit__(self, *exc) -> bool:
        self._registry.close(self.record)
        return False


class _Registry:
    """Process-wide bookkeeping of annotation scopes."""

    def __init__(self):
        self.reset()

    def reset(self) -> None:
        self.active: list[dict] = []
        self.opened_per_name: dict[str, int] = {}
        self.opened = 0

    def open(self, name: str) -> dict:
        # plain ints and dicts only: the model's forward is captured by Dynamo with fullgraph=True,
        # which has to trace through this bookkeeping
        nth = self.opened_per_name.get(name, 0)
        record = {"name": name, "index": nth, "uid": self.opened}
        self.opened_per_name[name] = nth + 1
        self.opened += 1
        self.active.append(record)
        return record

    def close(self, record: dict) -> None:
        # scopes are context managers, so they close innermost first
        if not self.active or self.active[-1] is not record:
            raise RuntimeError(f"annotation scope {record!r} closed out of order")
        self.active.pop()


_REGISTRY = _Registry()


def annotate(name: str) -> _Scope:
    """Context manager that tags everything run inside it with `name`."""
    if not (isinstance(name, str) and name):
        raise ValueError(f"annotate() takes a non-empty string as tag name, not {name!r}")
    return _Scope(_REGISTRY, name)


def reset_annotation_state() -> None:
    """Forget all scopes and restart the index / uid numbering (used between model builds)."""
    _REGISTRY.reset()


def current_annotations() -> tuple[dict, ...]:
    """Snapshot of the active scopes, outermost first."""
    return tuple(dict(r) for r in _REGISTRY.active)


def current_tag() -> dict[str, int]:
    """{name: index} of the active scopes, e.g. {"PP": 0, "EP": 0} inside the expert region."""
    return {r["name"]: r["index"] for r in _REGISTRY.active}
