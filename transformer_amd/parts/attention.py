"""The attention mixer: qkv projection, position encoding fused with the cache
write, causal grouped-query attention over the cache, output projection.

Order and shapes follow the reference's block
(models/llama/common/src/compute.rs:210-270): one merged qkv
product whose rows are all q heads, then all k heads, then all v heads
(lib.rs:132-137, split at compute.rs:227); rotation of q and k (:232-233); per
request, the step's k and v go to cache rows pos..pos+seq and the queries read
rows 0..pos+seq (:243-264); the output projection is added to the residual
(:267-270). Scale and mask are not arguments there (:511-526); here the scale
and the window are constants of the spec.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .. import kernels
from ..cache.storage import KVNeed
from ..weights.loader import Param
from .base import Part, PartError, build_part, register_part
from .linear import adds_in_place, linear, linear_delta


@dataclass(frozen=True)
class KeyUnitPlanner:
    """The work plan of the single-token attention kernels, made on the host with every step's
    tables: the sequences of the step cut into units of work of about equal length
    (``kernels.plan_key_units``). Mixers with the same number of kv heads share one plan."""
    num_kv_heads: int

    def ints(self, batch: int) -> int:
        return kernels.UNIT_INTS * kernels.key_unit_count(batch, self.num_kv_heads) + 2 * batch

    def tables(self, kv_lens, block_table):
        units, seq_units = kernels.plan_key_units(
            kv_lens, kernels.key_unit_count(len(kv_lens), self.num_kv_heads), tables=block_table)
        return {"units": units, "seq_units": seq_units}


class CachedAttention(Part):
    @property
    def graph_safe(self) -> bool:
        return bool(getattr(self.position, "graph_safe", False))

    def __init__(self, spec, dtype, device):
        if spec.num_heads % spec.num_kv_heads:
            raise PartError(f"{spec.num_heads} heads do not divide into {spec.num_kv_heads} kv heads")
        if spec.head_dim % 16 or not 16 <= spec.head_dim <= 256:
            raise PartError(f"attention kernels take head sizes that are multiples of 16 in "
                            f"[16, 256], not {spec.head_dim}")
        if spec.window is not None and spec.window < 1:
            raise PartError(f"attention window must be >= 1, got {spec.window}")
        self.spec, self.dtype = spec, dtype
        self.nq, self.nkv, self.dh = spec.num_heads, spec.num_kv_heads, spec.head_dim
        self.position = build_part(spec.position, dtype, device)

    def params(self):
        s = self.spec
        width = (self.nq + 2 * self.nkv) * self.dh
        p = {"qkv.weight": Param((width, s.hidden), "matrix"),
             "out.weight": Param((s.hidden, self.nq * self.dh), "matrix")}
        if s.qkv_bias:
            p["qkv.bias"] = Param((width,), "vector")
        if s.out_bias:
            p["out.bias"] = Param((s.hidden,), "vector")
        return p

    def cache_need(self):
        return KVNeed(self.nkv, self.dh, self.spec.window)

    def step_planner(self):
        return KeyUnitPlanner(self.nkv)

    # a block may leave the norm in front of this part to the first product (``scale``) and
    # the norm behind it to the last (``fold``) when the few-rows product takes them
    def takes_scaled(self, nt: int) -> bool:
        return kernels.skinny_takes(nt, self.w["qkv.weight"])

    def can_fold(self, nt: int) -> bool:
        return kernels.skinny_folds(nt, self.w["out.weight"])

    # with many rows the last product can add itself to the residual stream (``into``)
    def can_add(self, nt: int) -> bool:
        return adds_in_place(nt, self.w["out.weight"])

    def _out(self, o, ctx, fold, into):
        if fold is not None:
            kernels.gemm_skinny(o, self.w["out.weight"], None, bias=self.w.get("out.bias"), fold=fold)
            return None
        return (linear_delta(o, self.w["out.weight"], ctx.ws, "attention.delta", into=into),
                self.w.get("out.bias"))

    def run(self, h, ctx, cache, layer, writes_cache=True, scale=None, fold=None, into=None):
        """h: [nt, hidden] engine dtype -> (delta float32 [nt, hidden], bias row or None);
        None with ``fold``, which has then taken the result; (None, bias) with ``into``, the
        residual stream that the output projection has then added itself to."""
        nt = h.shape[0]
        width = (self.nq + 2 * self.nkv) * self.dh
        qkv = linear(h, self.w["qkv.weight"], ctx.ws.take("attention.qkv", (nt, width), self.dtype),
                     scale=scale)
        kc, vc, group = cache.layer_kv(layer)
        meta = ctx.kv[group]
        o = ctx.ws.take("attention.o", (nt, self.nq * self.dh), self.dtype)
        fused = getattr(self.position, "rotation_of", None)
        if (ctx.all_single and fused is not None and qkv.dtype == torch.bfloat16
                and kernels.keys_kernel_fits(self.nq, self.nkv, self.dh)):
            # one token per sequence: rotation, cache write and attention in one kernel
            angles, interleaved = fused(ctx)
            plan = meta.plans.get(self.step_planner(), {})    # absent: the kernel's wrapper plans
            kernels.attention_keys(qkv, o, kc, vc, meta.block_table, ctx.cu_q, ctx.pos0,
                                   ctx.max_kv_len, self.nq, self.nkv, self.dh,
                                   float(self.spec.scale), self.spec.window, angles=angles,
                                   interleaved=interleaved, bias=self.w.get("qkv.bias"),
                                   dest=meta.dest if writes_cache else None,
                                   units=plan.get("units"), seq_units=plan.get("seq_units"))
            return self._out(o, ctx, fold, into)
        if writes_cache:
            self.position.encode_and_store(qkv, ctx, self.nq, self.nkv, meta.dest, kc, vc,
                                           self.w.get("qkv.bias"))
        else:   # this run reads keys and values that an earlier run stored
            self.position.encode_and_store(qkv, ctx, self.nq, self.nkv,
                                           bias=self.w.get("qkv.bias"))
        kernels.attention(qkv, o, kc, vc, meta.block_table, ctx.cu_q, ctx.pos0, ctx.max_qlen,
                          ctx.max_kv_len, self.nq, self.nkv, self.dh, float(self.spec.scale),
                          self.spec.window)
        return self._out(o, ctx, fold, into)


register_part("attention", CachedAttention)
