"""A small Llama engine for one MI355X: typed configuration, weights by name,
blocks assembled from parts, a paged per-sequence cache, one batched step
function, a generation loop, sampling and trace replay, on hand-written HIP
kernels for gfx950."""
from . import kernels  # noqa: F401
from .api import load_model, open_model_source, random_model, save_model  # noqa: F401
from .engine.batch import Entry  # noqa: F401
from .config.llama import LlamaConfig  # noqa: F401
from .config.registry import get_architecture, known_architectures, register_architecture  # noqa: F401
from .parts.base import PartTimers, register_part  # noqa: F401
from .llama import Llama  # noqa: F401
from .sampling.args import SampleArgs  # noqa: F401

__version__ = "0.1.0"
