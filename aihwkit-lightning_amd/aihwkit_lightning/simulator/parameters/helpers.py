"""Pretty printing shared by the parameter dataclasses."""
from dataclasses import field, fields, is_dataclass
from typing import Any


def shown(default: Any):
    """A dataclass field with an immutable default that printing never leaves out (the reference
    marks such fields with the ``always_show`` metadata key)."""
    return field(default=default, metadata={"always_show": True})


class _PrintableMixin:
    """Gives a dataclass a nested, indented ``str()`` (role of reference ``helpers.py:23-108``)."""

    def __str__(self) -> str:
        parts = []
        for fld in fields(self):  # type: ignore[arg-type]
            value = getattr(self, fld.name)
            text = str(value) if is_dataclass(value) else repr(value)
            parts.append(f"{fld.name}={text}")
        name = type(self).__name__
        if len(parts) <= 3 and not any("\n" in p for p in parts):
            return f"{name}({', '.join(parts)})"
        body = ",\n".join("    " + p.replace("\n", "\n    ") for p in parts)
        return f"{name}(\n{body}\n)"
