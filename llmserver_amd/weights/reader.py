"""Reads a model folder's safetensors files one tensor at a time, by tensor name.

Same job as utils/weights.py:15-55: a folder holds either one
``model.safetensors`` or shards listed in ``model.safetensors.index.json["weight_map"]``; files
are memory-mapped and tensors handed out singly, so a large model never has a second full copy
in host memory.  Only local folders are read (there is no download path).
"""
from __future__ import annotations

import json
import os
from typing import Dict, Tuple

from safetensors import safe_open

INDEX_NAME = "model.safetensors.index.json"
SINGLE_NAME = "model.safetensors"


class CheckpointReader:
    def __init__(self, directory: str):
        self.directory = directory
        self._handles = {}
        index_path = os.path.join(directory, INDEX_NAME)
        single_path = os.path.join(directory, SINGLE_NAME)
        if os.path.exists(index_path):
            with open(index_path) as handle:
                self.name_to_file: Dict[str, str] = dict(json.load(handle)["weight_map"])
        elif os.path.exists(single_path):
            self.name_to_file = {name: SINGLE_NAME for name in self._open(SINGLE_NAME).keys()}
        else:
            raise FileNotFoundError(f"{directory!r} holds neither {SINGLE_NAME} nor {INDEX_NAME}")

    def _open(self, file_name: str):
        if file_name not in self._handles:
            self._handles[file_name] = safe_open(os.path.join(self.directory, file_name), "pt")
        return self._handles[file_name]

    def names(self):
        return self.name_to_file.keys()

    def has(self, name: str) -> bool:
        return name in self.name_to_file

    def shape(self, name: str) -> Tuple[int, ...]:
        return tuple(self._open(self.name_to_file[name]).get_slice(name).get_shape())

    def get(self, name: str):
        return self._open(self.name_to_file[name]).get_tensor(name)

    def close(self):
        self._handles.clear()
