"""Parameter tree handed to the layers (the accessors of sharktank/sharktank/types/theta.py:72-186 that the
MoE layers call: `theta("name")`, `theta.tensor(...)`, `theta.optional_tensor(...)`, `theta.keys`, `flatten`,
`to(device=)`).  Archive I/O is not part of the hot path and is not provided."""

from __future__ import annotations

from typing import Optional, Union

from .tensors import InferenceTensor

__all__ = ["Theta", "flat_to_nested_dict"]


def flat_to_nested_dict(flat: dict) -> dict:
    nested: dict = {}
    for key, value in flat.items():
        if isinstance(value, dict):
            value = flat_to_nested_dict(value)
        parts = str(key).split(".")
        cur = nested
        for part in parts[:-1]:
            cur = cur.setdefault(part, {})
            assert isinstance(cur, dict), f"Name collision in parameter dict: {key}"
        last = parts[-1]
        if isinstance(value, dict) and isinstance(cur.get(last), dict):
            cur[last].update(value)
        else:
            assert last not in cur, f"Name collision in parameter dict: {key}"
            cur[last] = value
    return nested


def _norm_name_path(name_path) -> list:
    parts = []
    for p in name_path:
        parts.extend(str(p).split("."))
    return parts


class Theta:
    def __init__(self, tensors):
        if not isinstance(tensors, dict):
            tensors = {t.name: t for t in tensors}
        self._tree = flat_to_nested_dict(tensors)

    def flatten(self) -> dict:
        out = {}

        def walk(prefix, node):
            for k, v in node.items():
                name = f"{prefix}.{k}" if prefix else k
                if isinstance(v, dict):
                    walk(name, v)
                else:
                    out[name] = v

        walk("", self._tree)
        return out

    def to(self, *, device=None) -> "Theta":
        return Theta({k: (v.to(device=device) if v is not None else v) for k, v in self.flatten().items()})

    def tensor(self, *name_path) -> InferenceTensor:
        path = _norm_name_path(name_path)
        t = self.optional_tensor(*path)
        if t is None:
            raise KeyError(f"Could not find tensor {path[-1]} in theta {path[0:-1]}")
        return t

    def optional_tensor(self, *name_path) -> Optional[InferenceTensor]:
        path = _norm_name_path(name_path)
        cur = self._tree
        try:
            for part in path[:-1]:
                cur = cur[part]
        except KeyError:
            raise KeyError(f"Unknown parameter {path} (in Theta object containing {self.keys})")
        return cur.get(path[-1])

    @property
    def keys(self):
        return self._tree.keys()

    def __contains__(self, key) -> bool:
        return key in self._tree

    @property
    def tree(self) -> dict:
        return self._tree

    def __call__(self, *name_path) -> Union["Theta", InferenceTensor]:
        cur = self._tree
        try:
            for part in _norm_name_path(name_path):
                cur = cur[part]
        except KeyError:
            raise KeyError(f"Sub-theta {name_path} not found (of {self._tree.keys()})")
        if isinstance(cur, InferenceTensor):
            return cur
        return Theta(cur)

    def __repr__(self):
        return f"Theta({self.keys})"
