"""Which of two ways a product of a given shape goes on a given GPU: a table, not a stopwatch at serving time.

For most shapes the hand-written few-row products win, for some the library's product plus the kernels around it
does.  Which, is measured (``HipOps.measuring()``: ``Engine.calibrate`` and ``python -m llmserver_amd.kernels.calibrate``
run it), never while a request is served, and kept per kind of GPU (architecture and number of compute units, such as ``gfx950-256cu``) in JSON files: the table that ships with the package
(``choices.json`` beside this file, measured for the shapes of the sizes that ``config/named_sizes.py`` knows by name) and, if the environment variable
``LLMSERVER_AMD_CHOICES`` names one, a table of the user's own, whose entries win.  A shape that no table knows goes
the hand-written way.  The same tables give the same kernels, so two runs round alike.
"""
from __future__ import annotations

import json
import os
from typing import Dict, Optional

SHIPPED = os.path.join(os.path.dirname(os.path.abspath(__file__)), "choices.json")
USER_TABLE_VARIABLE = "LLMSERVER_AMD_CHOICES"


def choice_key(kind: str, rows: int, out_features: int, in_features: int, scaled: bool, out_float32: bool) -> str:
    return f"{kind}/{rows}/{out_features}/{in_features}/{int(bool(scaled))}/{int(bool(out_float32))}"


class ChoiceTable:
    def __init__(self, device_name: str, entries: Optional[Dict[str, bool]] = None):
        self.device_name = device_name
        self.entries: Dict[str, bool] = dict(entries or {})
        self.measured: Dict[str, bool] = {}         # what this process has measured itself

    @classmethod
    def load(cls, device_name: str, paths=None) -> "ChoiceTable":
        """The shipped table's entries for this GPU model, overlaid with the user's table if one is named."""
        if paths is None:
            paths = [SHIPPED] + ([os.environ[USER_TABLE_VARIABLE]] if os.environ.get(USER_TABLE_VARIABLE) else [])
        table = cls(device_name)
        for path in paths:
            if not os.path.isfile(path):
                continue
            with open(path) as handle:
                stored = json.load(handle)
            table.entries.update({key: bool(value) for key, value in stored.get(device_name, {}).items()})
        return table

    def get(self, key: str) -> Optional[bool]:
        return self.entries.get(key)

    def record(self, key: str, value: bool) -> None:
        self.entries[key] = self.measured[key] = bool(value)

    def save(self, path: str, everything: bool = False) -> int:
        """Merge what was measured (or, with ``everything``, all entries) into the file at ``path``; returns how many
        entries the file then holds for this GPU model."""
        stored = {}
        if os.path.isfile(path):
            with open(path) as handle:
                stored = json.load(handle)
        mine = stored.setdefault(self.device_name, {})
        mine.update(self.entries if everything else self.measured)
        stored[self.device_name] = dict(sorted(mine.items(), key=lambda item: _natural(item[0])))
        os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
        scratch = f"{path}.{os.getpid()}.tmp"
        with open(scratch, "w") as handle:
            json.dump(stored, handle, indent=1, sort_keys=True)
            handle.write("\n")
        os.replace(scratch, path)
        return len(mine)


def _natural(key: str):
    return tuple(int(part) if part.isdigit() else part for part in key.split("/"))
