"""Per-layer schedule parameters: the container the reference's drivers build, store as JSON and
hand to a lowering schedule (lighthouse/schedule/parameters.py: a list of dictionaries, one per
layer, each with a string "layer_kind" and values that are numbers, strings, booleans or lists of
them; `to_json` / `from_json`).  On this target the entries that act are the workgroup tile
(`wg_m`, `wg_n`) and the cut along K (`split_k`) of a matmul layer; they reach the kernels through
`lighthouse_amd.ingress.torch.with_schedule_parameters` or a descriptor's `kernel:` stage."""

from __future__ import annotations

import json
import os
from collections.abc import MutableSequence

_VALUE_TYPES = (int, float, str, bool, list, tuple)


def _checked(entry) -> dict:
    if not isinstance(entry, dict):
        raise ValueError(f"Each parameter entry must be a dictionary: found '{entry}'.")
    kind = entry.get("layer_kind")
    if kind is None:
        raise ValueError("Each parameter dictionary must contain a 'layer_kind' key.")
    if not isinstance(kind, str):
        raise ValueError("'layer_kind' must be a string.")
    for key, value in entry.items():
        if not isinstance(key, str):
            raise ValueError(f"Parameter dictionary keys must be strings: found '{key}'.")
        if not isinstance(value, _VALUE_TYPES):
            raise ValueError("Parameter dictionary values must be an int, float, str, bool, list, or tuple: "
                             f"found '{value}' for key '{key}'.")
    return entry


class ScheduleParameters(MutableSequence):
    """A list of per-layer parameter dictionaries that verifies every entry it takes."""

    def __init__(self, list_of_parameters: list[dict] | None = None):
        if list_of_parameters is not None and not isinstance(list_of_parameters, list):
            raise ValueError(f"list_of_parameters must be a list of dictionaries or None, got {type(list_of_parameters)}")
        self.list_of_parameters: list[dict] = [_checked(p) for p in (list_of_parameters or [])]

    # MutableSequence supplies append, extend, reverse, pop, remove, iteration, `in`, ... on top of these five.
    def __len__(self) -> int:
        return len(self.list_of_parameters)

    def __getitem__(self, index):
        return self.list_of_parameters[index]

    def __setitem__(self, index, value) -> None:
        self.list_of_parameters[index] = _checked(value)

    def __delitem__(self, index) -> None:
        del self.list_of_parameters[index]

    def insert(self, index: int, value: dict) -> None:
        self.list_of_parameters.insert(index, _checked(value))

    def to_json(self, filename, overwrite: bool = False) -> None:
        if os.path.exists(filename) and not overwrite:
            raise FileExistsError(f"File '{filename}' already exists. Use 'overwrite=True' to overwrite it.")
        with open(filename, "w") as f:
            json.dump(self.list_of_parameters, f, indent=4)

    @classmethod
    def from_json(cls, filename: str) -> "ScheduleParameters":
        with open(filename) as f:
            return cls(json.load(f))

    def __repr__(self) -> str:
        return f"ScheduleParameters({self.list_of_parameters!r})"
