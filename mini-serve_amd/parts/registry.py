"""Registries of parts by category and kind. A new mixer, feed-forward, norm, position encoding,
block arrangement, embedding or head is one class plus one ``register`` call; configurations
then name it by ``kind`` in a ``PartSpec``."""

from __future__ import annotations

from ..config.spec import PartSpec

CATEGORIES = ("mixer", "feed_forward", "norm", "position", "block", "embedding", "head")
PARTS: dict[str, dict[str, type]] = {c: {} for c in CATEGORIES}


def register(category: str, kind: str):
    """Class decorator: ``@register("mixer", "gqa_attention")``."""
    if category not in PARTS:
        raise ValueError(f"unknown part category {category!r}, expected one of {CATEGORIES}")

    def deco(cls):
        known = PARTS[category].get(kind)
        if known is not None and known is not cls:
            raise ValueError(f"{category} {kind!r} is already registered")
        PARTS[category][kind] = cls
        cls.kind = kind
        return cls

    return deco


def unregister(category: str, kind: str) -> None:
    PARTS[category].pop(kind, None)


def part_class(category: str, spec: PartSpec) -> type:
    try:
        return PARTS[category][spec.kind]
    except KeyError:
        raise ValueError(
            f"unknown {category} {spec.kind!r}, expected one of {sorted(PARTS[category])}"
        ) from None
