"""Entry points in the manner of the reference's drivers: a model is loaded from
a folder or file, then stepped or asked to generate.

The reference's sequence is LlamaStorage::from_gguf -> LlamaWorker::new ->
launch -> RandomSample::launch (models/llama/cuda/src/infer.rs:41,
:88, :106, :129); here ``load_model`` covers the first two.
"""
from __future__ import annotations

import sys
import time
from pathlib import Path

import torch

from . import architectures  # noqa: F401  (registers the known architectures)
from . import parts  # noqa: F401
from .config.registry import get_architecture, read_model_folder_config
from .engine.model import DecoderModel, engine_dtype
from .weights.loader import load_parameters
from .weights.safetensors_io import TensorFolder


def open_model_source(path):
    """(architecture entry, typed config, tensor file) of a folder with
    config.json + safetensors, or of a .gguf file."""
    p = Path(path)
    if p.is_file() and p.suffix == ".gguf":
        from .weights.gguf_io import GGUFFile
        f = GGUFFile(p)
        arch = get_architecture(str(f.metadata.get("general.architecture")))
        rows = f.shape("token_embd.weight")[0] if "token_embd.weight" in f else None
        return arch, arch.config_from_gguf(f.metadata, rows), f
    arch, cfg = read_model_folder_config(p)
    return arch, cfg, TensorFolder(p)


def load_model(path, dtype=None, device="cuda:0", verbose=False) -> DecoderModel:
    """dtype None: what the configuration's ``default_engine_dtype()`` says (config.json's
    torch_dtype: float32 stays float32, everything else computes in bfloat16)."""
    arch, cfg, file = open_model_source(path)
    if dtype is None:
        dtype = getattr(cfg, "default_engine_dtype", lambda: "bfloat16")()
    spec = arch.model_spec(cfg)
    model = DecoderModel(spec, engine_dtype(dtype), device)
    model.config, model.architecture = cfg, arch
    t0, last = time.time(), [time.time()]

    def progress(name):
        if verbose and time.time() - last[0] > 10:
            last[0] = time.time()
            print(f"[transformer_amd] loading weights: {name} ({time.time() - t0:.0f}s)",
                  file=sys.stderr, flush=True)

    tensors = load_parameters(model.all_params(), arch.weight_sources(cfg, file.format), file,
                              model.dtype, model.device, where=str(path), progress=progress)
    model.bind(tensors)
    file.close()
    import resource
    nbytes = model.weight_bytes()
    dt = time.time() - t0
    # ru_maxrss is in KiB on Linux; it counts mapped file pages that are resident as well
    model.load_stats = {"seconds": dt, "bytes": nbytes, "gb_per_s": nbytes / max(dt, 1e-9) / 1e9,
                        "peak_host_rss_bytes": resource.getrusage(resource.RUSAGE_SELF).ru_maxrss * 1024}
    if verbose:
        print(f"[transformer_amd] computing in {str(model.dtype)[6:]}; loaded {nbytes / 1e9:.2f} GB of weights in {dt:.1f} s "
              f"({model.load_stats['gb_per_s']:.2f} GB/s), peak host memory "
              f"{model.load_stats['peak_host_rss_bytes'] / 1e9:.2f} GB", file=sys.stderr, flush=True)
    return model


def random_model(config, seed: int = 0, dtype="bfloat16", device="cuda:0", std: float = 0.02,
                 norm_std: float = 0.1, architecture: str = "LlamaForCausalLM",
                 num_layers=None) -> DecoderModel:
    """A model whose weights are drawn on the GPU (nothing touches the disk):
    matrices ~ N(0, std), norm weights 1 + N(0, norm_std), biases ~ N(0, std).
    ``num_layers`` builds only the first layers, for a configuration that offers
    ``with_layers(n)``."""
    import zlib
    from . import kernels
    from .weights.loader import storage_dtype
    arch = get_architecture(architecture)
    if isinstance(config, dict):
        config = arch.config_from_dict(config)
    if num_layers is not None:
        shorten = getattr(config, "with_layers", None)
        if shorten is None:
            raise ValueError(f"the configuration of {arch.name} does not offer with_layers(n)")
        config = shorten(num_layers)
    spec = arch.model_spec(config)
    model = DecoderModel(spec, engine_dtype(dtype), device)
    model.config, model.architecture = config, arch
    tied = spec.tie_embeddings is True
    tensors = {}
    with torch.cuda.device(model.device):
        for name, p in model.all_params().items():
            if name == "head.weight" and tied:
                continue
            t = torch.empty(p.shape, dtype=storage_dtype(p.role, model.dtype), device=model.device)
            sid = zlib.crc32(name.encode())
            if p.init == "normal":
                kernels.fill_normal(t, seed, sid, 0.0, std)
            elif p.init == "around_one":
                kernels.fill_normal(t, seed, sid, 1.0, norm_std)
            elif p.init == "zero":
                t.zero_()
            else:
                raise ValueError(f"parameter {name}: unknown way to draw it: {p.init!r}")
            tensors[name] = t
    if tied:
        tensors["head.weight"] = tensors["embed.weight"]
    model.bind(tensors)
    return model


def save_model(model: DecoderModel, folder, metadata=None):
    """Writes ``model`` (loaded, or drawn by ``random_model``) as a model folder: config.json
    and model.safetensors under the architecture's own tensor names, in the types the
    model holds them in. ``load_model(folder, same dtype)`` gives the same model back."""
    from .weights.save import save_model_folder
    arch, cfg = model.architecture, model.config
    if cfg.tie_embeddings is None and model.w["embed"].data_ptr() == model.w["head"].data_ptr():
        import dataclasses
        cfg = dataclasses.replace(cfg, tie_embeddings=True)
    return save_model_folder(folder, cfg.to_dict(), model.tensors, model.all_params(),
                             arch.weight_sources(cfg, "safetensors"), metadata)
