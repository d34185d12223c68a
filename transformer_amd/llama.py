"""A facade with the names a user of the reference looks for: the reference's
objects are LlamaStorage::from_gguf -> LlamaWorker::new -> launch ->
RandomSample::launch (models/llama/cuda/src/infer.rs:41, :88,
:106, :129); here they are ``Llama.from_pretrained`` (or ``Llama.random``),
``step``, ``generate`` and ``replay`` over one model and one cache."""
from __future__ import annotations

from typing import Optional, Sequence

from .api import load_model, random_model
from .engine.batch import Entry
from .engine.generate import generate as _generate


class Llama:
    def __init__(self, model, cache_tokens: int = 16384, max_slots: Optional[int] = None):
        self.model = model
        self.config = getattr(model, "config", None)
        self._cache_tokens, self._max_slots = cache_tokens, max_slots
        self._cache = None

    @classmethod
    def from_pretrained(cls, path, dtype="bfloat16", device="cuda:0", **kw) -> "Llama":
        """path: a folder with config.json and safetensors, or a .gguf file."""
        return cls(load_model(path, dtype, device), **kw)

    @classmethod
    def random(cls, config, seed: int = 0, dtype="bfloat16", device="cuda:0", **kw) -> "Llama":
        return cls(random_model(config, seed, dtype, device), **kw)

    @property
    def cache(self):
        if self._cache is None:
            self._cache = self.model.new_cache(self._cache_tokens, self._max_slots)
        return self._cache

    def alloc_slot(self) -> int:
        return self.cache.alloc_slot()

    def free_slot(self, slot: int) -> None:
        self.cache.free_slot(slot)

    def reset_slot(self, slot: int) -> None:
        self.cache.reset_slot(slot)

    def step(self, batch: Sequence):
        """batch: Entry objects or (slot, tokens, want) tuples -> float32 logits [wanted, vocab]."""
        entries = [e if isinstance(e, Entry) else Entry(*e) for e in batch]
        return self.model.step(self.cache, entries)

    def generate(self, prompts, max_new_tokens: int, sample_args=None, stop_ids=None, seed: int = 0,
                 max_batch: Optional[int] = None, on_token=None):
        """Generates in the facade's own cache (its slots and recorded steps are used again
        from call to call) when every batch fits it, else in a cache made for this call."""
        from .kernels import PAGE
        cache = None
        mine = self.cache
        if not mine.pool.live_slots():
            need = sorted((-(-(len(p) + max_new_tokens) // PAGE) * PAGE for p in prompts), reverse=True)
            if need and need[0] <= mine.num_pages * PAGE:
                cache = mine
        return _generate(self.model, prompts, max_new_tokens, sample_args, stop_ids, seed,
                         cache=cache, max_batch=max_batch, on_token=on_token)

    def replay(self, trace, out_dir, max_tokens: Optional[int] = None) -> None:
        """trace: an iterable of step records (dicts) or JSON lines."""
        import json
        from .replay import Replayer
        rp = Replayer(self.model, max_tokens or self._cache_tokens, out_dir)
        for rec in trace:
            rp.run_step(json.loads(rec) if isinstance(rec, str) else rec)
