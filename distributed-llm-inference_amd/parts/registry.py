"""Registries of part classes, one per family.

Families: ``embedding``, ``norm``, ``position``, ``mixer``, ``feed_forward``, ``block``, ``head``.
A part class is constructed as ``cls(runtime, **spec.params)``; see :mod:`dli_amd.parts.base` for
what each family must provide. Registering a part touches no file of the framework::

    @register_part("mixer", "my_mixer")
    class MyMixer(Mixer): ...
"""

from __future__ import annotations

from typing import Any, Callable, TypeVar

FAMILIES = ("embedding", "norm", "position", "mixer", "feed_forward", "block", "head")
_REGISTRY: dict[str, dict[str, type]] = {f: {} for f in FAMILIES}
T = TypeVar("T", bound=type)


class UnknownPartError(KeyError):
    def __str__(self) -> str:
        return str(self.args[0])


def register_part(family: str, kind: str, *, replace: bool = False) -> Callable[[T], T]:
    if family not in _REGISTRY:
        raise ValueError(f"unknown part family {family!r}; families: {FAMILIES}")

    def deco(cls: T) -> T:
        if kind in _REGISTRY[family] and not replace:
            raise ValueError(f"{family} part {kind!r} is already registered")
        _REGISTRY[family][kind] = cls
        cls.family = family  # type: ignore[attr-defined]
        cls.kind = kind  # type: ignore[attr-defined]
        return cls

    return deco


def unregister_part(family: str, kind: str) -> None:
    _REGISTRY[family].pop(kind, None)


def part_class(family: str, kind: str) -> type:
    try:
        return _REGISTRY[family][kind]
    except KeyError:
        raise UnknownPartError(
            f"no {family} part named {kind!r}; registered: {sorted(_REGISTRY.get(family, {}))}"
        ) from None


def build_part(family: str, spec: Any, runtime: Any) -> Any:
    """Construct the part that ``spec`` (a :class:`PartSpec`) names."""
    part = part_class(family, spec.kind)(runtime, **dict(spec.params))
    part.prefix = spec.prefix
    return part


def registered_parts(family: str) -> tuple[str, ...]:
    return tuple(sorted(_REGISTRY[family]))
