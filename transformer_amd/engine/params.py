"""Parameter declarations of a model, available without a GPU."""
from __future__ import annotations

from typing import Dict

import torch

from ..config.spec import ModelSpec
from ..parts.base import build_part
from ..weights.loader import Param


def declared_params(spec: ModelSpec) -> Dict[str, Param]:
    """Names, shapes and roles of every parameter of a model, without a GPU: the
    parts are built only to be asked what they want."""
    spec.validate()
    out = {"embed.weight": Param((spec.vocab, spec.hidden), "matrix")}
    for i, b in enumerate(spec.blocks):
        out.update(build_part(b, torch.float32, "cpu").all_params(f"blocks.{i}."))
    out.update(build_part(spec.final_norm, torch.float32, "cpu").all_params("final_norm."))
    for name in ("after_embed", "on_logits"):
        if getattr(spec, name, None) is not None:
            out.update(build_part(getattr(spec, name), torch.float32, "cpu").all_params(name + "."))
    out["head.weight"] = Param((spec.vocab, spec.hidden), "matrix")
    return out
