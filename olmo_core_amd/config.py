"""
Minimal configuration base for the float8 boundary.

Mirrors the behaviour of the reference's ``Config`` that ``Float8Config`` inherits and that
src/test/config_test.py:7-101 pins: ``as_dict`` / ``as_config_dict`` / ``from_dict`` / ``merge`` with
dot-list overrides, the ``_CLASS_`` field for polymorphic decoding, plus ``StrEnum`` and ``DType``
(reference: src/olmo_core/config.py:39-49, 55-237, 365-392).  The reference delegates decoding to the
``dataclass_extensions`` package, which is not a dependency here; ``_build`` below is a small typed
decoder for the field types these configs use (scalars, enums, Optional, List/Tuple/Set/Dict, nested
dataclasses).
"""

from __future__ import annotations

import copy
import dataclasses
import json
import typing
from dataclasses import dataclass
from enum import Enum
from importlib import import_module
from typing import Any, Callable, ClassVar, Collection, Dict, List, Optional, Sequence, Tuple, Type, TypeVar

import torch
import yaml

from .exceptions import OLMoConfigurationError

__all__ = ["Config", "DType", "StrEnum"]


class StrEnum(str, Enum):
    """String-valued enum whose ``str()`` is its value."""

    def __str__(self) -> str:
        return self.value

    def __repr__(self) -> str:
        return f"'{self.value}'"


C = TypeVar("C", bound="Config")

_SCALARS = (float, int, bool, str)


def _parse_override(arg: str) -> Tuple[str, Any]:
    """``--a.b-c=1`` -> ("a.b_c", 1); a bare flag means true; values are YAML scalars."""
    name, sep, raw = arg.partition("=")
    if not sep:
        raw = "true"
    name = name.strip(" -").replace("-", "_")
    value: Any = "" if (not raw or raw.isspace()) else yaml.safe_load(raw)
    return name, value


def _assign(tree: Any, dotted: str, value: Any) -> None:
    head, _, rest = dotted.partition(".")
    if isinstance(tree, dict):
        key: Any = head
    elif isinstance(tree, list):
        key = int(head)
    else:
        raise ValueError(f"Can't set value '{value}' at key '{dotted}' for object {tree}")
    if rest:
        _assign(tree[key], rest, value)
    else:
        tree[key] = value


def _build(tp: Any, value: Any) -> Any:
    """Decode ``value`` (plain python data) into the annotated type ``tp``."""
    if value is None or tp is Any:
        return value
    if dataclasses.is_dataclass(tp) and isinstance(tp, type):
        if isinstance(value, tp):
            return value
        if not isinstance(value, dict):
            raise TypeError(f"expected a mapping for {tp.__name__}, got {type(value).__name__}")
        hints = typing.get_type_hints(tp)
        known = {f.name for f in dataclasses.fields(tp) if f.init}
        unknown = set(value) - known
        if unknown:
            raise TypeError(f"unexpected field(s) for {tp.__name__}: {sorted(unknown)}")
        return tp(**{k: _build(hints.get(k, Any), v) for k, v in value.items()})
    if isinstance(tp, type) and issubclass(tp, Enum):
        return value if isinstance(value, tp) else tp(value)
    origin = typing.get_origin(tp)
    args = typing.get_args(tp)
    if origin is typing.Union:
        last: Optional[Exception] = None
        for option in args:
            if option is type(None):
                continue
            try:
                return _build(option, value)
            except (TypeError, ValueError) as e:
                last = e
        if last is not None:
            raise last
        return value
    if origin in (list, set, frozenset):
        elem = args[0] if args else Any
        return origin(_build(elem, v) for v in value)
    if origin is tuple:
        if len(args) == 2 and args[1] is Ellipsis:
            return tuple(_build(args[0], v) for v in value)
        if args:
            return tuple(_build(a, v) for a, v in zip(args, value))
        return tuple(value)
    if origin is dict:
        kt, vt = args if args else (Any, Any)
        return {_build(kt, k): _build(vt, v) for k, v in value.items()}
    if tp is float and isinstance(value, int) and not isinstance(value, bool):
        return float(value)
    return value


@dataclass
class Config:
    """
    Base class for configuration dataclasses (subclasses are themselves ``@dataclass``-decorated and
    hold only simple, serialisable field types or nested configs).
    """

    CLASS_NAME_FIELD: ClassVar[str] = "_CLASS_"
    _IGNORE_FIELDS: ClassVar[Tuple[str, ...]] = ()

    # ---- dumping ---------------------------------------------------------------------------

    def as_dict(
        self,
        *,
        exclude_none: bool = False,
        exclude_private_fields: bool = False,
        exclude: Optional[Collection[str]] = None,
        include_class_name: bool = False,
        json_safe: bool = False,
        recurse: bool = True,
    ) -> Dict[str, Any]:
        skip = set(exclude or ())

        def wanted(obj):
            for f in dataclasses.fields(obj):
                if not f.init or f.name in skip:
                    continue
                v = getattr(obj, f.name)
                if (exclude_none and v is None) or (exclude_private_fields and f.name.startswith("_")):
                    continue
                yield f.name, v

        def dump(obj: Any, deep: bool) -> Any:
            if dataclasses.is_dataclass(obj) and not isinstance(obj, type):
                out = {k: (dump(v, True) if deep else v) for k, v in wanted(obj)}
                if include_class_name:
                    out[self.CLASS_NAME_FIELD] = f"{type(obj).__module__}.{type(obj).__name__}"
                return out
            if isinstance(obj, dict):
                return {k: dump(v, True) for k, v in obj.items()}
            if isinstance(obj, (list, tuple, set)):
                items = [dump(v, True) for v in obj]
                return items if json_safe else type(obj)(items)
            if obj is None or isinstance(obj, _SCALARS):
                return obj
            return str(obj) if json_safe else obj

        return dump(self, recurse)

    def as_config_dict(self) -> Dict[str, Any]:
        """JSON-safe dump for recording a config: no ``None``s, no private fields, class names in."""
        return self.as_dict(
            exclude_none=True,
            exclude_private_fields=True,
            include_class_name=True,
            json_safe=True,
            recurse=True,
        )

    # ---- traversal / validation ------------------------------------------------------------

    def apply(self, func: Callable[["Config"], None]) -> None:
        def walk(obj: Any) -> None:
            if isinstance(obj, Config):
                func(obj)
            if dataclasses.is_dataclass(obj) and not isinstance(obj, type):
                for f in dataclasses.fields(obj):
                    walk(getattr(obj, f.name))
            elif isinstance(obj, dict):
                for v in obj.values():
                    walk(v)
            elif isinstance(obj, (list, tuple, set)):
                for v in obj:
                    walk(v)

        walk(self)

    def validate(self) -> None:
        """Hook for subclasses; may normalise fields in place."""

    # ---- construction ----------------------------------------------------------------------

    def merge(self: C, dotlist: List[str], prefix: Optional[str] = None, strict: bool = True) -> C:
        """New object with ``a.b=c`` style overrides applied (optionally only those under ``prefix``)."""
        pairs = [_parse_override(s) for s in dotlist]
        if prefix is not None:
            lead = f"{prefix}."
            pairs = [(k[len(lead):], v) for k, v in pairs if k.startswith(lead)]
        if not strict:
            names = {f.name for f in dataclasses.fields(self)}
            pairs = [(k, v) for k, v in pairs if k.split(".", 1)[0] in names]
        data = self.as_dict(include_class_name=True)
        for k, v in pairs:
            _assign(data, k, v)
        return type(self).from_dict(data)

    def replace(self: C, **changes: Any) -> C:
        return dataclasses.replace(self, **changes)

    def copy(self: C, deep: bool = True) -> C:
        return copy.deepcopy(self) if deep else copy.copy(self)

    @classmethod
    def from_dict(cls: Type[C], data: Dict[str, Any], overrides: Optional[Sequence[str]] = None) -> C:
        if overrides:
            data = copy.deepcopy(data)
            for k, v in (_parse_override(s) for s in overrides):
                _assign(data, k, v)

        def lookup(path: str) -> Optional[type]:
            module_name, _, name = path.rpartition(".")
            if not module_name:
                return None
            try:
                return getattr(import_module(module_name), name, None)
            except ImportError:
                return None

        def decode(node: Any, where: str) -> Any:
            if isinstance(node, dict):
                node = {(int(k) if isinstance(k, str) and k.isdigit() else k): v for k, v in node.items()}
                body = {
                    k: decode(v, f"{where}.{k}" if where else str(k))
                    for k, v in node.items()
                    if k != cls.CLASS_NAME_FIELD
                }
                target = lookup(node[cls.CLASS_NAME_FIELD]) if cls.CLASS_NAME_FIELD in node else None
                if target is None:
                    return body
                for name in getattr(target, "_IGNORE_FIELDS", ()):
                    body.pop(name, None)
                try:
                    return _build(target, body)
                except Exception as e:
                    what = f"Failed to construct '{where}' in config: {e}" if where else f"Error building config: {e}"
                    raise OLMoConfigurationError(what) from e
            if isinstance(node, (list, tuple, set)):
                return type(node)(decode(v, f"{where}.{i}" if where else str(i)) for i, v in enumerate(node))
            return node

        decoded = decode(data, "")
        if isinstance(decoded, cls):
            return decoded
        try:
            return _build(cls, decoded)
        except (TypeError, ValueError) as e:
            raise OLMoConfigurationError(f"Error building config: {e}") from e

    @classmethod
    def from_file(cls: Type[C], path: Any, overrides: Optional[Sequence[str]] = None) -> C:
        text = str(path)
        with open(text) as f:
            if text.endswith((".yml", ".yaml")):
                data = yaml.safe_load(f)
            elif text.endswith(".json"):
                data = json.load(f)
            else:
                raise OLMoConfigurationError(f"Unsupported config file type: {path}")
        return cls.from_dict(data, overrides=overrides)


class DType(StrEnum):
    """Names of the torch dtypes a config may mention (reference: src/olmo_core/config.py:365-392)."""

    float32 = "float32"
    bfloat16 = "bfloat16"
    float16 = "float16"
    float8_e4m3fn = "float8_e4m3fn"
    float8_e5m2 = "float8_e5m2"

    @classmethod
    def from_pt(cls, dtype: torch.dtype) -> "DType":
        for member in cls:
            if getattr(torch, member.value) == dtype:
                return member
        raise NotImplementedError(dtype)

    def as_pt(self) -> torch.dtype:
        return getattr(torch, self.value)
