"""`piper.annotate`: tag a region of model code with a schedule name (src/piper.py:51-80).

Same contract as the reference: a non-empty string name, an integer index assigned per name in
the order scopes are entered, a process-wide uid, and a stack so nested scopes ("PP" around
"EP") are visible together.  The reference stores the stack in FX node metadata for its graph
splitter; here the stack is what the executor reads to decide which region a call belongs to.
"""
from __future__ import annotations

from contextlib import contextmanager
from typing import Iterator

_ANNOTATION_STACK: list[dict] = []
_ANNOTATION_COUNTS: dict[str, int] = {}
_ANNOTATION_UID = 0

PP_TAG = "PP"
EP_TAG = "EP"


def reset_annotation_state() -> None:
    global _ANNOTATION_UID
    _ANNOTATION_STACK.clear()
    _ANNOTATION_COUNTS.clear()
    _ANNOTATION_UID = 0


def current_annotations() -> tuple[dict, ...]:
    """Snapshot of the active scopes, outermost first."""
    return tuple(dict(a) for a in _ANNOTATION_STACK)


def current_tag() -> dict[str, int]:
    """{name: index} of the active scopes, e.g. {"PP": 0, "EP": 0} inside the expert region."""
    return {a["name"]: a["index"] for a in _ANNOTATION_STACK}


@contextmanager
def annotate(name: str) -> Iterator[dict]:
    if not isinstance(name, str) or not name:
        raise ValueError(f"piper.annotate requires a non-empty string tag name, got {name!r}")
    global _ANNOTATION_UID
    index = _ANNOTATION_COUNTS.get(name, 0)
    _ANNOTATION_COUNTS[name] = index + 1
    uid = _ANNOTATION_UID
    _ANNOTATION_UID += 1
    annotation = {"name": name, "index": int(index), "uid": int(uid)}
    _ANNOTATION_STACK.append(annotation)
    try:
        yield annotation
    finally:
        popped = _ANNOTATION_STACK.pop()
        if popped is not annotation:
            raise RuntimeError("piper.annotate stack corrupted")
