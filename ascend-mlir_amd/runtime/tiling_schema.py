"""Tiling parameter packer for tiling_space.json files (reference:
python/runtime/tiling_schema.py:17-128; C++ twin TilingSchema::pack)."""
from __future__ import annotations

import json
import struct
from pathlib import Path


class TilingSchema:
    def __init__(self, fields):
        self._fields = [{"name": f["name"], "type": f.get("type", "int64")} for f in fields]

    @classmethod
    def from_json(cls, path) -> "TilingSchema":
        path = Path(path)
        if not path.exists():
            raise FileNotFoundError(f"tiling_space.json not found: {path}")
        try:
            data = json.loads(path.read_text())
        except json.JSONDecodeError as e:
            raise ValueError(f"JSON parse error in '{path}': {e}") from e
        params = data.get("tiling_params") if isinstance(data, dict) else None
        if params is None:
            raise ValueError(f"'{path}': missing 'tiling_params' array")
        if not isinstance(params, list):
            raise ValueError(f"'{path}': 'tiling_params' must be a list")
        fields = []
        for i, entry in enumerate(params):
            if not isinstance(entry, dict):
                raise ValueError(f"'{path}': tiling_params[{i}] must be an object")
            if not entry.get("name"):
                raise ValueError(f"'{path}': tiling_params[{i}] missing 'name'")
            fields.append(entry)
        return cls(fields)

    @classmethod
    def for_kernel(cls, kernel_name: str) -> "TilingSchema":
        """Schema of one of the fused HIP kernels, from the kernel library's registry."""
        from .. import hip_kernels
        for k in hip_kernels.kernel_table():
            if k["name"] == kernel_name:
                return cls([{"name": n, "type": "int64"} for n in k["tiling_fields"]])
        raise KeyError(kernel_name)

    def pack(self, **kwargs: int) -> bytes:
        expected = [f["name"] for f in self._fields]
        missing = sorted(set(expected) - set(kwargs))
        extra = sorted(set(kwargs) - set(expected))
        problems = []
        if missing:
            problems.append(f"missing tiling fields: {missing}")
        if extra:
            problems.append(f"unexpected tiling fields: {extra}")
        if problems:
            raise ValueError("\n".join(problems) + f"\n  expected: {expected}")
        out = bytearray()
        for f in self._fields:
            v = int(kwargs[f["name"]])
            out += struct.pack("<i", v) if f["type"] in ("int32", "int32_t") else struct.pack("<q", v)
        return bytes(out)

    @property
    def field_names(self):
        return [f["name"] for f in self._fields]

    @property
    def fields(self):
        return [dict(f) for f in self._fields]

    def __len__(self):
        return len(self._fields)

    def __repr__(self):
        return f"TilingSchema({self.field_names})"
