"""Random-weights mode: writes a model folder (config.json, model.safetensors)
from a configuration and a seed.

Matrices ~ N(0, std); norm weights 1 + N(0, norm_std); biases ~ N(0, std). The
tensors carry the architecture's own file names: every parameter the model's
parts declare is cut into the pieces its registry entry reads it from. Matrices
are stored in the asked storage type, vectors always in float32 (the split the
reference's conversion recipe makes: linear tensors narrow, norm tensors float32,
docs/user-guide/doc.md:133).
"""
from __future__ import annotations

import json
from pathlib import Path

import torch

from ..config.registry import get_architecture
from ..engine.params import declared_params
from .safetensors_io import write_safetensors


def draw(param, shape, gen, storage, std, norm_std):
    """One tensor of ``shape`` drawn the way its part declares (``Param.init``)."""
    wide = storage if param.role == "matrix" else torch.float32
    if param.init == "zero":
        return torch.zeros(shape, dtype=wide)
    z = torch.randn(shape, generator=gen, dtype=torch.float32)
    if param.init == "around_one":
        return (1.0 + z * norm_std).to(wide)
    if param.init == "normal":
        return (z * std).to(wide)
    raise ValueError(f"unknown way to draw a parameter: {param.init!r}")


def random_tensors(arch, config, seed: int, storage: torch.dtype = torch.bfloat16,
                   std: float = 0.02, norm_std: float = 0.1):
    """{file tensor name: tensor} for a safetensors folder."""
    spec = arch.model_spec(config)
    params = declared_params(spec)
    sources = arch.weight_sources(config, "safetensors")
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int(seed))
    out = {}
    for pname, param in params.items():
        src = sources[pname]
        if not src.options:
            continue
        if pname == "head.weight" and src.stand_in is not None and config.tie_embeddings is None:
            continue    # undecided tying: write the tied form
        for piece in src.options[0]:
            out[piece.name] = draw(param, piece.shape, gen, storage, std, norm_std)
    return out


def write_random_model(folder, config, seed: int, storage="bfloat16", std=0.02, norm_std=0.1,
                       architecture="LlamaForCausalLM") -> Path:
    """``config``: a typed configuration (or the dict of a config.json)."""
    arch = get_architecture(architecture)
    if isinstance(config, dict):
        config = arch.config_from_dict(config)
    st = {"bfloat16": torch.bfloat16, "float32": torch.float32}[str(storage).replace("torch.", "")]
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    tensors = random_tensors(arch, config, seed, st, std, norm_std)
    write_safetensors(folder / "model.safetensors", tensors,
                      metadata={"format": "pt", "seed": seed})
    d = config.to_dict()
    d["torch_dtype"] = "bfloat16" if st == torch.bfloat16 else "float32"
    (folder / "config.json").write_text(json.dumps(d, indent=1))
    return folder
