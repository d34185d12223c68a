"""y = x @ W^T, the matrix product every part uses.

float32 engine: the hand-written product of csrc/gemm_simple.hip, whose every
output element is one ascending-k chain of fused multiply-adds; no library and
no reduced-precision matrix mode is involved anywhere in that path.

bfloat16 engine: the vendor library through ``torch.mm`` (the reference's
engine also hands its products to a library: the external ``mat_mul`` operator,
models/llama/common/src/compute.rs:425-455), except for
shapes that a hand-written kernel of this package serves better.
Accumulation is float32; the output type is chosen by the caller (float32 for
what is added to the residual stream and for logits).
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import kernels


class Workspace:
    """Named scratch tensors that are reused from step to step."""

    def __init__(self, device):
        self.device = torch.device(device)
        self._bufs = {}
        self.generation = 0      # grows whenever a buffer moves; recorded graphs go stale then

    def take(self, name: str, shape, dtype: torch.dtype) -> torch.Tensor:
        n = 1
        for s in shape:
            n *= int(s)
        key = (name, dtype)
        buf = self._bufs.get(key)
        if buf is None or buf.numel() < n:
            buf = torch.empty(max(n, 1), dtype=dtype, device=self.device)
            self._bufs[key] = buf
            self.generation += 1
        return buf[:n].view(*shape)

    def reserve(self, name: str, numel: int, dtype: torch.dtype) -> None:
        self.take(name, (numel,), dtype)


def linear(x: torch.Tensor, weight: torch.Tensor, out: Optional[torch.Tensor], scale=None,
           fold=None) -> torch.Tensor:
    """out[nt, n] = x[nt, k] @ weight[n, k]^T. x and weight share a dtype, or the weight is
    a float32 matrix of a bfloat16 engine (its file stores it in 32 bits and it stays so).

    scale (``kernels.RowScale``): the rows of x still lack their norm's factor, which the
    product applies. fold (``kernels.NormFold``): the product is added to the residual stream
    and prepares the next norm instead of writing ``out``. Only the few-rows product can do
    either, so a caller asks ``kernels.skinny_takes`` before it hands them over."""
    if scale is not None or fold is not None:
        return kernels.gemm_skinny(x, weight, out, scale=scale, fold=fold)
    mixed = x.dtype == torch.bfloat16 and weight.dtype == torch.float32
    if x.dtype != weight.dtype and not mixed:
        raise kernels.KernelError(f"linear: activations are {x.dtype}, weights {weight.dtype}")
    if x.shape[0] == 0:
        return out
    if x.dtype == torch.float32 or mixed:
        return kernels.gemm_simple(x, weight, out)
    if kernels.skinny_wins(x, weight):
        return kernels.gemm_skinny(x, weight, out)
    if kernels.mid_wins_plain(x.shape[0], weight) and x.stride(1) == 1 and x.stride(0) % 8 == 0 \
            and x.data_ptr() % 16 == 0:
        return kernels.gemm_mid(x, weight, out)
    if out.dtype == x.dtype:
        torch.mm(x, weight.t(), out=out)
    else:
        torch.mm(x, weight.t(), out_dtype=out.dtype, out=out)
    return out


def library_planes(rows: int, weight: torch.Tensor) -> int:
    """Planes in which the vendor library leaves a float32 product of 65 to 1,536 rows over a
    long k (the down projection): one batched call multiplies the parts of k side by side, and
    the next norm adds the planes in order. A plain call has one tile of work per 128 x 128
    outputs, which is too few for the CUs when there are few rows, and every tile then walks
    all of k: 4,096 columns over k = 14,336 take 76 us at 128 rows, 94 at 512, 129 at 1,024 in
    one plane and 30, 61, 97 in 8, 4, 4 planes. The planes cost the norm their bytes again, so
    from 1,536 rows on (2,048: 200 -> 174 us in two planes, 100 MB more for the norm) and for
    a short k (4,096: 27 -> 23 us at 512 rows) the product stays whole. It depends on the row
    count, so only bfloat16 steps, whose bits follow the row count anyway, take it."""
    if weight.dtype != torch.bfloat16 or weight.dim() != 2 or not weight.is_contiguous():
        return 1
    n, k = weight.shape
    if not kernels.MID_MAX_ROWS < rows <= 1536 or k < 8192:
        return 1
    tiles = -(-rows // 128) * -(-n // 128)
    want = 768 // tiles
    planes = 8 if want >= 8 else 4 if want >= 3 else 2 if want >= 2 else 1
    while planes > 1 and k % (planes * 64):
        planes //= 2
    return planes


def adds_in_place(rows: int, weight: torch.Tensor) -> bool:
    """Whether ``linear_delta`` can add this product to the residual stream by itself: the
    vendor library's product in one plane, which takes what it adds to as its third operand."""
    return weight.dtype == torch.bfloat16 and rows > kernels.MID_MAX_ROWS and \
        library_planes(rows, weight) == 1


def linear_delta(x: torch.Tensor, weight: torch.Tensor, ws: Workspace, name: str,
                 into: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """x @ weight^T as float32, to be added to the residual stream by the next norm: [nt, n],
    or [planes, nt, n] whose planes the norm adds in order. Products of up to 64 rows that the
    few-rows kernel does not take go to ``kernels.gemm_mid``, which cuts a weight with few
    column tiles along k and leaves the partial sums as planes (output and down projections:
    11 and 27 us at 64 rows of the 8B shape where the vendor library takes 15 and 42).

    into (the float32 residual stream, only where ``adds_in_place`` says so): the library's
    product adds itself to it, float32 sum plus float32 stream rounded once as the norm's add
    is, and nothing is returned; a prompt's norm then reads the stream alone instead of reading
    stream and delta and writing the stream back (2,048 tokens of the 8B shape: 21 to 10 us)."""
    nt, n = x.shape[0], weight.shape[0]
    if into is not None:
        if not (x.dtype == torch.bfloat16 and adds_in_place(nt, weight)) or into.shape != (nt, n) \
                or into.dtype != torch.float32:
            raise kernels.KernelError(f"linear_delta: cannot add {tuple(x.shape)} x {tuple(weight.shape)} "
                                      f"in place into {tuple(into.shape)} {into.dtype}")
        torch.addmm(into, x, weight.t(), out_dtype=torch.float32, out=into)
        return None
    if x.dtype == torch.bfloat16 and nt > 0 and kernels.mid_takes(nt, weight) \
            and x.stride(1) == 1 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0:
        planes = kernels.mid_splits(weight)
        out = ws.take(name, (planes, nt, n) if planes > 1 else (nt, n), torch.float32)
        return kernels.gemm_mid(x, weight, out)
    planes = library_planes(nt, weight) if x.dtype == torch.bfloat16 and x.is_contiguous() else 1
    if planes > 1:
        out = ws.take(name, (planes, nt, n), torch.float32)
        k = weight.shape[1] // planes
        torch.bmm(x.view(nt, planes, k).transpose(0, 1), weight.view(n, planes, k).permute(1, 2, 0),
                  out_dtype=torch.float32, out=out)
        return out
    return linear(x, weight, ws.take(name, (nt, n), torch.float32))
