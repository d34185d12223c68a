"""Writes the parameters a model holds into a model folder under the architecture's own
file names: the inverse of ``loader.load_parameters``.

A parameter that the loader joins from several file tensors by rows (q/k/v into qkv, gate/up
into gate_up: models/llama/common/src/lib.rs:132-137, :154-157) is cut back into those
tensors; one that stands in for another (an output matrix tied to the embedding table) is
not written. With this a model whose weights were drawn on the device can be handed to any
reader of the format, e.g. a plain implementation that checks the engine.
"""
from __future__ import annotations

import json
from pathlib import Path
from typing import Dict

import torch

from .loader import Param, Source
from .safetensors_io import write_safetensors


def file_tensors(tensors: Dict[str, torch.Tensor], params: Dict[str, Param],
                 sources: Dict[str, Source]) -> Dict[str, torch.Tensor]:
    """{file tensor name: view of a parameter} in the first (canonical) form of every source."""
    out: Dict[str, torch.Tensor] = {}
    for pname, param in params.items():
        src = sources[pname]
        t = tensors[pname]
        if src.stand_in is not None and tensors.get(src.stand_in) is not None and \
                t.data_ptr() == tensors[src.stand_in].data_ptr():
            continue                                   # shared with another parameter
        if not src.options:
            raise ValueError(f"parameter {pname} has no file form and is not shared")
        if tuple(t.shape) != tuple(param.shape):
            raise ValueError(f"parameter {pname} is {tuple(t.shape)}, declared {tuple(param.shape)}")
        row = 0
        pieces = src.options[0]
        for piece in pieces:
            if len(pieces) == 1:
                out[piece.name] = t
            else:
                out[piece.name] = t[row:row + piece.shape[0]]
                row += piece.shape[0]
            if tuple(out[piece.name].shape) != tuple(piece.shape):
                raise ValueError(f"{piece.name}: cut to {tuple(out[piece.name].shape)}, the file "
                                 f"form is {tuple(piece.shape)}")
    return out


def save_model_folder(folder, config_dict: dict, tensors: Dict[str, torch.Tensor],
                      params: Dict[str, Param], sources: Dict[str, Source], metadata=None) -> Path:
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    write_safetensors(folder / "model.safetensors", file_tensors(tensors, params, sources),
                      metadata={"format": "pt", **(metadata or {})})
    (folder / "config.json").write_text(json.dumps(config_dict, indent=1))
    return folder
