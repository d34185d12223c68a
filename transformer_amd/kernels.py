"""Python face of the HIP kernel library (ctypes, plain C ABI).

Each wrapper checks devices, dtypes, contiguity and shapes on the host, then
passes raw pointers and the current HIP stream. There is no fallback: when the
library cannot be loaded or a tensor is not on the GPU, the call raises.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_longlong, c_void_p
from typing import Optional, Sequence

import torch

from .csrc.build import ensure_built

PAGE = 64          # tokens per cache page, fixed in csrc/common.h (TA_PAGE)
F32, BF16 = 0, 1


class KernelError(RuntimeError):
    pass


_lib = None


def library():
    """Loads (and on first use builds) the kernel library."""
    global _lib
    if _lib is None:
        path = ensure_built()
        lib = ctypes.CDLL(str(path))
        lib.ta_last_error.restype = c_char_p
        if lib.ta_page_size() != PAGE:
            raise KernelError(f"kernel library pages hold {lib.ta_page_size()} tokens, "
                              f"the Python side expects {PAGE}")
        lib._path = str(path)
        _lib = lib
    return _lib


def library_path() -> str:
    return library()._path


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"kernels take float32 or bfloat16, not {dtype}")


def _dev(t: torch.Tensor, name: str, dtype=None, contiguous=True):
    if not isinstance(t, torch.Tensor):
        raise KernelError(f"{name}: expected a tensor, got {type(t).__name__}")
    if not t.is_cuda:
        raise KernelError(f"{name}: tensor is on {t.device}; kernels run on the GPU only")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: expected {dtype}, got {t.dtype}")
    if contiguous and not t.is_contiguous():
        raise KernelError(f"{name}: tensor must be contiguous")
    return t


def _ptr(t: Optional[torch.Tensor]):
    return c_void_p(t.data_ptr()) if t is not None else c_void_p(0)


def _stream():
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def _check(rc: int):
    if rc != 0:
        raise KernelError(library().ta_last_error().decode())


def _rows2d(t: torch.Tensor, name: str):
    """(rows, row stride) of a 2-D tensor whose rows are contiguous."""
    if t.dim() != 2 or t.stride(1) != 1:
        raise KernelError(f"{name}: expected a 2-D tensor with contiguous rows, got shape "
                          f"{tuple(t.shape)} strides {t.stride()}")
    return t.shape[0], t.stride(0)


def _check_cache_layer(what, kcache, vcache, num_kv_heads, head_dim):
    """keys [pages, nkv, PAGE, dh]; values transposed inside a page: [pages, nkv, dh, PAGE]."""
    wk = (kcache.shape[0], num_kv_heads, PAGE, head_dim)
    wv = (kcache.shape[0], num_kv_heads, head_dim, PAGE)
    if tuple(kcache.shape) != wk or tuple(vcache.shape) != wv:
        raise KernelError(f"{what}: cache layer is {tuple(kcache.shape)} / {tuple(vcache.shape)}, "
                          f"expected {wk} / {wv}")


# ------------------------------------------------------------------ embedding
def embed(table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t] = table[tokens[t]] as float32. tokens: int32 [nt]; out: float32 [nt, d]."""
    _dev(table, "table"); _dev(tokens, "tokens", torch.int32); _dev(out, "out", torch.float32)
    vocab, d = table.shape
    nt = tokens.numel()
    if out.shape != (nt, d):
        raise KernelError(f"embed: out is {tuple(out.shape)}, expected {(nt, d)}")
    _check(library().ta_embed(_stream(), _code(table.dtype), _ptr(table), c_int(vocab), c_int(d),
                              _ptr(tokens), c_int(nt), _ptr(out)))
    return out


# ------------------------------------------------------------------ add + norm
def add_rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
                delta: Optional[torch.Tensor] = None, delta_bias: Optional[torch.Tensor] = None,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """v = x[r] + delta[r] + delta_bias; out[i] = rmsnorm(v) * weight.

    Without ``rows`` r = i and, when there is anything to add, v is stored back
    into x (the float32 residual stream). With ``rows`` (int32) only those rows
    are normalised, into out[0..len(rows)), and x is left as it is. A delta that a
    product left in parts ([planes, nt, d]) is added plane by plane, in order.
    """
    _dev(x, "x", torch.float32); _dev(weight, "weight", torch.float32); _dev(out, "out")
    nt, d = x.shape
    if weight.shape != (d,):
        raise KernelError(f"add_rmsnorm: weight is {tuple(weight.shape)}, expected {(d,)}")
    n_out = nt
    if rows is not None:
        _dev(rows, "rows", torch.int32)
        n_out = rows.numel()
    if out.shape != (n_out, d):
        raise KernelError(f"add_rmsnorm: out is {tuple(out.shape)}, expected {(n_out, d)}")
    ddt, planes, plane = F32, 1, 0
    if delta is not None:
        _dev(delta, "delta")
        if delta.dim() == 3 and delta.shape[1:] == x.shape:
            planes, plane = delta.shape[0], nt * d
        elif delta.shape != x.shape:
            raise KernelError(f"add_rmsnorm: delta is {tuple(delta.shape)}, x is {tuple(x.shape)}")
        ddt = _code(delta.dtype)
    if delta_bias is not None:
        _dev(delta_bias, "delta_bias", torch.float32)
        if delta_bias.shape != (d,):
            raise KernelError("add_rmsnorm: delta_bias must have one entry per column")
    store = int(rows is None and (delta is not None or delta_bias is not None))
    _check(library().ta_add_rmsnorm(_stream(), c_int(ddt), c_int(_code(out.dtype)), _ptr(x),
                                    _ptr(delta), _ptr(delta_bias), _ptr(weight), _ptr(rows),
                                    _ptr(out), c_int(n_out), c_int(d), c_float(eps), c_int(store),
                                    c_int(planes), c_longlong(plane)))
    return out


# ------------------------------------------------------------------ rotary + cache write
def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t, j] = (cos a, sin a) with a = float32(positions[t]) * inv_freq[j] in float32."""
    _dev(positions, "positions", torch.int32); _dev(inv_freq, "inv_freq", torch.float32)
    _dev(out, "out", torch.float32)
    nt, half = positions.numel(), inv_freq.numel()
    if tuple(out.shape) != (nt, half, 2):
        raise KernelError(f"rope_table: out is {tuple(out.shape)}, expected {(nt, half, 2)}")
    _check(library().ta_rope_table(_stream(), _ptr(positions), _ptr(inv_freq), _ptr(out), c_int(nt),
                                   c_int(half)))
    return out


def rope_kv_write(qkv: torch.Tensor, num_q_heads: int, num_kv_heads: int, head_dim: int,
                  angles: Optional[torch.Tensor], interleaved: bool,
                  dest: Optional[torch.Tensor] = None, kcache: Optional[torch.Tensor] = None,
                  vcache: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None):
    """Rotates q and k inside qkv [nt, (nq + 2 nkv) * dh] in place by the angles of
    ``rope_table`` ([nt, dh/2, 2]; None: no rotation) and stores the step's k and v
    into one cache layer (keys [pages, nkv, PAGE, dh], values [pages, nkv, dh, PAGE])
    at dest [nt] (page * PAGE + offset)."""
    _dev(qkv, "qkv")
    nt = qkv.shape[0]
    width = (num_q_heads + 2 * num_kv_heads) * head_dim
    if qkv.shape != (nt, width):
        raise KernelError(f"rope_kv_write: qkv is {tuple(qkv.shape)}, expected {(nt, width)}")
    if angles is not None:
        _dev(angles, "angles", torch.float32)
        if tuple(angles.shape) != (nt, head_dim // 2, 2):
            raise KernelError(f"rope_kv_write: angles are {tuple(angles.shape)}, expected "
                              f"{(nt, head_dim // 2, 2)}")
    if bias is not None:
        _dev(bias, "bias", torch.float32)
        if bias.numel() != width:
            raise KernelError("rope_kv_write: bias must hold one entry per qkv column")
    if kcache is not None:
        _dev(kcache, "kcache", qkv.dtype); _dev(vcache, "vcache", qkv.dtype)
        _dev(dest, "dest", torch.int32)
        _check_cache_layer("rope_kv_write", kcache, vcache, num_kv_heads, head_dim)
        if dest.numel() != nt:
            raise KernelError("rope_kv_write: dest must hold one entry per token")
    _check(library().ta_rope_kv_write(_stream(), c_int(_code(qkv.dtype)), _ptr(qkv), _ptr(bias),
                                      _ptr(dest if kcache is not None else None), _ptr(angles),
                                      c_int(1 if interleaved else 0), _ptr(kcache), _ptr(vcache),
                                      c_int(nt), c_int(num_q_heads), c_int(num_kv_heads),
                                      c_int(head_dim)))
    return qkv


# ------------------------------------------------------------------ attention
def attention_generic(q: torch.Tensor, out: torch.Tensor, kcache: torch.Tensor,
                      vcache: torch.Tensor, block_table: torch.Tensor, cu_q: torch.Tensor,
                      pos0: torch.Tensor, max_qlen: int, num_heads: int, num_kv_heads: int,
                      head_dim: int, scale: float, window: Optional[int] = None):
    """Causal attention of each sequence's new tokens over its cached keys.

    q: [nt, >= nh*dh] (a view whose rows may be wider, e.g. the qkv buffer);
    out: [nt, nh*dh]; kcache [pages, nkv, PAGE, dh], vcache [pages, nkv, dh, PAGE];
    block_table: int32 [B, max_blocks]; cu_q: int32 [B+1]; pos0: int32 [B].
    """
    _dev(q, "q", contiguous=False); _dev(out, "out", q.dtype, contiguous=False)
    nt, qs = _rows2d(q, "q")
    nto, os_ = _rows2d(out, "out")
    if nt != nto or q.shape[1] < num_heads * head_dim or out.shape[1] != num_heads * head_dim:
        raise KernelError(f"attention: q {tuple(q.shape)} / out {tuple(out.shape)} do not fit "
                          f"{num_heads} heads of {head_dim}")
    _dev(kcache, "kcache", q.dtype); _dev(vcache, "vcache", q.dtype)
    _check_cache_layer("attention", kcache, vcache, num_kv_heads, head_dim)
    _dev(block_table, "block_table", torch.int32); _dev(cu_q, "cu_q", torch.int32)
    _dev(pos0, "pos0", torch.int32)
    B = pos0.numel()
    if cu_q.numel() != B + 1 or block_table.dim() != 2 or block_table.shape[0] != B:
        raise KernelError("attention: cu_q / pos0 / block_table disagree about the batch size")
    _check(library().ta_attention_generic(
        _stream(), c_int(_code(q.dtype)), _ptr(q), c_int(qs), _ptr(out), c_int(os_), _ptr(kcache),
        _ptr(vcache), _ptr(block_table), c_int(block_table.shape[1]), _ptr(cu_q), _ptr(pos0),
        c_int(B), c_int(max_qlen), c_int(num_heads), c_int(num_kv_heads), c_int(head_dim),
        c_float(scale), c_int(window or 0)))
    return out


def attention(q, out, kcache, vcache, block_table, cu_q, pos0, max_qlen, max_kv_len, num_heads,
              num_kv_heads, head_dim, scale, window=None):
    """Picks the attention kernel for the step's shape and storage type: bfloat16
    with a head size that is a multiple of 32 runs on the matrix cores (one kernel
    for prompts, one for single tokens that slices the keys); everything else, and
    all of float32, runs the vector-ALU kernel."""
    if q.dtype == torch.bfloat16 and head_dim % 32 == 0 and 32 <= head_dim <= 256:
        if max_qlen == 1 and keys_kernel_fits(num_heads, num_kv_heads, head_dim):
            return attention_keys(q, out, kcache, vcache, block_table, cu_q, pos0, max_kv_len,
                                  num_heads, num_kv_heads, head_dim, scale, window)
        return attention_rows(q, out, kcache, vcache, block_table, cu_q, pos0, max_qlen,
                              num_heads, num_kv_heads, head_dim, scale, window)
    return attention_generic(q, out, kcache, vcache, block_table, cu_q, pos0, max_qlen, num_heads,
                             num_kv_heads, head_dim, scale, window)


def _attention_args(q, out, kcache, vcache, block_table, cu_q, pos0, num_heads, num_kv_heads,
                    head_dim):
    _dev(q, "q", torch.bfloat16, contiguous=False); _dev(out, "out", torch.bfloat16, contiguous=False)
    nt, qs = _rows2d(q, "q")
    nto, os_ = _rows2d(out, "out")
    if nt != nto or q.shape[1] < num_heads * head_dim or out.shape[1] != num_heads * head_dim:
        raise KernelError(f"attention: q {tuple(q.shape)} / out {tuple(out.shape)} do not fit "
                          f"{num_heads} heads of {head_dim}")
    _dev(kcache, "kcache", torch.bfloat16); _dev(vcache, "vcache", torch.bfloat16)
    _check_cache_layer("attention", kcache, vcache, num_kv_heads, head_dim)
    _dev(block_table, "block_table", torch.int32); _dev(cu_q, "cu_q", torch.int32)
    _dev(pos0, "pos0", torch.int32)
    B = pos0.numel()
    if cu_q.numel() != B + 1 or block_table.dim() != 2 or block_table.shape[0] != B:
        raise KernelError("attention: cu_q / pos0 / block_table disagree about the batch size")
    return B, qs, os_


_cu_count = {}


def compute_units(device) -> int:
    """CUs of the device (workgroups that run at once when each fills a CU)."""
    idx = torch.device(device).index or 0
    if idx not in _cu_count:
        _cu_count[idx] = torch.cuda.get_device_properties(idx).multi_processor_count
    return _cu_count[idx]


def rows_kernel(max_qlen: int, num_heads: int, num_kv_heads: int, head_dim: int) -> int:
    """Which of the prompt kernels takes a launch (``through_lds`` of ``attention_rows``), by
    what was measured on MI355X with 32/8, 64/8 and 32/32 heads of 128, 12/4 of 96, 16/2 and 8/8
    of 64 and 8/8 of 32, prompts of 64 to 16,384 tokens, alone and in batches of equal and of
    unequal lengths: 0 below 256 rows; 1 for heads above 128; else 2 (8B shape: 2,048 tokens
    60 us against 79 of kernel 1, 2,304: 70 against 108, 16,384: 2.30 ms against 2.59, eight
    prompts of 128 to 2,000: 118 against 128)."""
    if max_qlen * (num_heads // num_kv_heads) < 256:
        return 0
    return 1 if head_dim > 128 else 2


def attention_rows(q, out, kcache, vcache, block_table, cu_q, pos0, max_qlen, num_heads,
                   num_kv_heads, head_dim, scale, window=None, through_lds=None):
    """Matrix-core attention for prompts: every wave owns 32 (token, head) rows.
    through_lds: 0: operands straight from memory; 1: the four waves of a workgroup share every
    page through LDS (128 rows a workgroup, two workgroups a CU; head sizes up to 192); 2: the
    same with a wave's scores, softmax and output products overlapped by half pages (head sizes
    up to 128); None: ``rows_kernel`` decides."""
    if through_lds is None:
        through_lds = rows_kernel(max_qlen, num_heads, num_kv_heads, head_dim)
    B, qs, os_ = _attention_args(q, out, kcache, vcache, block_table, cu_q, pos0, num_heads,
                                 num_kv_heads, head_dim)
    _check(library().ta_attention_rows_bf16(
        _stream(), _ptr(q), c_int(qs), _ptr(out), c_int(os_), _ptr(kcache), _ptr(vcache),
        _ptr(block_table), c_int(block_table.shape[1]), _ptr(cu_q), _ptr(pos0), c_int(B),
        c_int(max_qlen), c_int(num_heads), c_int(num_kv_heads), c_int(head_dim), c_float(scale),
        c_int(window or 0), c_int(int(through_lds))))
    return out


_scratch = {}
_scratch_moves = [0]


def scratch_generation() -> int:
    """Grows whenever kernel scratch memory moves (recorded graphs go stale then)."""
    return _scratch_moves[0]


def _scratch_floats(device, n: int) -> torch.Tensor:
    buf = _scratch.get(device)
    if buf is None or buf.numel() < n:
        buf = torch.empty(max(n, 1 << 16), dtype=torch.float32, device=device)
        _scratch[device] = buf
        _scratch_moves[0] += 1
    return buf


# a unit of work of the single-token attention has at least this many pages unless it is a whole
# sequence. The kernel's time is a floor of about 8 us (launch, the chain record -> pages -> LDS
# -> partial rows) plus its bytes; since the merge asks for all of a sequence's partial rows at
# once, runs of two pages beat runs of four (one sequence of 17 pages: 11.3 against 12.7 us)
_KEYS_MIN_PER = 2


def keys_kernel(group: int, head_dim: int) -> int:
    """Which single-token attention kernel serves ``group`` query heads per kv head: 0 and 1
    name the kernels whose four waves bring a unit's pages in together through LDS (head
    sizes up to 192): 0 gives each wave a quarter of a page's keys for up to 16 query heads
    per kv head, 1 lets every wave form the scores of the whole page for up to 32. Otherwise
    4 waves take pages in turn."""
    return (0 if group <= 16 else 1) if head_dim <= 192 else 4


def key_unit_count(batch: int, num_kv_heads: int) -> int:
    """Units of work into which the sequences of a single-token step are cut (a workgroup is
    one unit of one kv head): at least twice the sequences, so that long ones can still be cut
    when the batch alone fills the CUs, rounded up to whole rounds of one workgroup per CU.
    Measured on the 256 CUs of MI355X with 8 kv heads: 256, 512 and 768 workgroups are good and
    the counts between them bad (12 sequences: 240 workgroups 19.8 us, 288 24.2, 384 22.3; 16
    sequences: 256 23.8, 320 26.8, 512 23.9), because the CUs that get one workgroup more set
    the kernel's time. It depends on the batch size alone, so a recorded graph keeps it."""
    cus = 256
    if torch.cuda.is_available():
        cus = compute_units(torch.cuda.current_device())
    per_round = max(1, cus // max(1, num_kv_heads))
    return max(batch, per_round * -(-2 * batch // per_round))


UNIT_INTS = 8      # int32 values in a unit's record, fixed in csrc/common.h (TA_UNIT_INTS)


def plan_key_units(kv_lens: Sequence[int], n_units: int, min_pages: int = 0, tables=None):
    """Cuts sequences of ``kv_lens`` tokens (this step's token included) into at most
    ``n_units`` runs of pages of about equal length, none shorter than ``min_pages`` unless
    it is a whole sequence: a CU can ask only so much of the memory in a given time, so the
    longest run sets the kernel's time. Returns int32 arrays units [n_units, 8] = (sequence,
    first page, pages, the sequence's length, page numbers of the unit's first two pages (from
    ``tables[b]``, the sequence's row of the block table; 0 without), units of the sequence,
    0), spare units holding 0 pages, and seq_units [batch, 2] = (first unit, units); a
    sequence's units follow one another and cover its pages in order. Pure host."""
    import heapq
    import numpy as np
    min_pages = min_pages or _KEYS_MIN_PER
    B = len(kv_lens)
    if n_units < B:
        raise KernelError(f"{n_units} units of work cannot hold {B} sequences")
    pages = [max(1, -(-int(n) // PAGE)) for n in kv_lens]
    count = [1] * B
    heap = [(-pages[b], b) for b in range(B)]
    heapq.heapify(heap)
    spare = n_units - B
    while spare > 0 and heap:
        _, b = heapq.heappop(heap)
        if pages[b] < min_pages * (count[b] + 1):      # another cut would make its runs too short
            continue
        count[b] += 1
        spare -= 1
        heapq.heappush(heap, (-pages[b] / count[b], b))
    cuts = []
    # sequences with the longest runs first: workgroups start in the order of their units, so
    # where there are more units than the CUs hold at once the short ones fill the end
    for b in sorted(range(B), key=lambda b: (-(pages[b] / count[b]), b)):
        base, extra = divmod(pages[b], count[b])
        first = 0
        for i in range(count[b]):
            n = base + (1 if i < extra else 0)
            cuts.append((b, first, n))
            first += n
    return _unit_records(cuts, kv_lens, n_units, tables)


def _unit_records(cuts, kv_lens, n_units, tables):
    import numpy as np
    units = np.zeros((n_units, UNIT_INTS), dtype=np.int32)
    seq = np.zeros((len(kv_lens), 2), dtype=np.int32)
    for u, (b, first, n) in enumerate(cuts):
        if seq[b, 1] == 0:
            seq[b, 0] = u
        seq[b, 1] += 1
        pa = pb = 0
        if tables is not None:
            pa = int(tables[b][first])
            pb = int(tables[b][first + 1]) if n > 1 else pa
        units[u] = (b, first, n, int(kv_lens[b]), pa, pb, 0, 0)
    for u, (b, _, _) in enumerate(cuts):
        units[u, 6] = seq[b, 1]
    return units, seq


def uniform_key_units(kv_lens: Sequence[int], pages_per_unit: int, tables=None):
    """Units of ``pages_per_unit`` pages each (the last of a sequence may be shorter): the
    plain slicing, for tests that want a given cut. Returns (units, seq_units) as above."""
    cuts = []
    for b, n in enumerate(kv_lens):
        pages = max(1, -(-int(n) // PAGE))
        for first in range(0, pages, pages_per_unit):
            cuts.append((b, first, min(pages_per_unit, pages - first)))
    return _unit_records(cuts, kv_lens, len(cuts), tables)


def attention_keys(q, out, kcache, vcache, block_table, cu_q, pos0, max_kv_len, num_heads,
                   num_kv_heads, head_dim, scale, window=None, slices=None, angles=None,
                   interleaved=False, bias=None, dest=None, units=None, seq_units=None):
    """Matrix-core attention for single tokens (sequence b brings row b of ``q``): the
    keys are cut into units of work that workgroups take in parallel, then merged.

    units, seq_units: int32 tensors on the GPU as ``plan_key_units`` lays them out (the step's
    tables carry them). Without them they are planned here from ``pos0``, which waits for the
    GPU; ``slices`` = (pages per unit, ignored, kernel) then asks for a plain cut and names
    the kernel (see ``keys_kernel``).

    Plain: ``q`` holds rotated q heads and the cache already holds the step's keys and
    values. Fused (``dest`` given): ``q`` is the raw [q | k | v] projection; the bias is
    added, q and k are rotated by ``angles`` ([B, dh/2, 2] from ``rope_table``; None: no
    rotation) and the new key and value are stored at ``dest`` before they are read."""
    B, qs, os_ = _attention_args(q, out, kcache, vcache, block_table, cu_q, pos0, num_heads,
                                 num_kv_heads, head_dim)
    if q.shape[0] != B:
        raise KernelError("attention_keys: every sequence must bring exactly one token")
    group = num_heads // num_kv_heads
    waves = keys_kernel(group, head_dim)
    if slices is not None and len(slices) > 2:
        waves = slices[2]
    if units is None:
        lens = [int(p) + 1 for p in pos0.tolist()]
        if max(lens) > block_table.shape[1] * PAGE:
            raise KernelError("attention_keys: a sequence is longer than the block table")
        host_table = block_table.cpu().numpy()
        if slices is not None:
            u, su = uniform_key_units(lens, int(slices[0]), host_table)
        else:
            u, su = plan_key_units(lens, key_unit_count(B, num_kv_heads), tables=host_table)
        units = torch.from_numpy(u).to(q.device)
        seq_units = torch.from_numpy(su).to(q.device)
    _dev(units, "units", torch.int32); _dev(seq_units, "seq_units", torch.int32)
    if units.dim() != 2 or units.shape[1] != UNIT_INTS or tuple(seq_units.shape) != (B, 2) or units.shape[0] < B:
        raise KernelError(f"attention_keys: units {tuple(units.shape)} / {tuple(seq_units.shape)} "
                          f"for {B} sequences")
    n_units = units.shape[0]
    width = (num_heads + 2 * num_kv_heads) * head_dim
    if dest is not None:
        _dev(dest, "dest", torch.int32)
        if dest.numel() != B or q.shape[1] != width:
            raise KernelError("attention_keys: the fused form needs [q | k | v] rows and one "
                              "destination per sequence")
    if angles is not None:
        _dev(angles, "angles", torch.float32)
        if tuple(angles.shape) != (B, head_dim // 2, 2):
            raise KernelError(f"attention_keys: angles are {tuple(angles.shape)}, expected "
                              f"{(B, head_dim // 2, 2)}")
    if bias is not None:
        _dev(bias, "bias", torch.float32)
        if bias.numel() != width:
            raise KernelError("attention_keys: bias must hold one entry per qkv column")
    need = library().ta_attention_keys_scratch
    need.restype = c_longlong
    floats = need(c_int(n_units), c_int(num_heads), c_int(head_dim))
    scratch = _scratch_floats(q.device, floats)
    _check(library().ta_attention_keys_bf16(
        _stream(), _ptr(q), c_int(qs), _ptr(bias), _ptr(angles), c_int(1 if interleaved else 0),
        _ptr(dest), _ptr(out), c_int(os_), _ptr(kcache), _ptr(vcache), _ptr(block_table),
        c_int(block_table.shape[1]), _ptr(pos0), c_int(B), c_int(num_heads), c_int(num_kv_heads),
        c_int(head_dim), c_float(scale), c_int(window or 0), _ptr(units), _ptr(seq_units),
        c_int(n_units), c_int(waves), _ptr(scratch)))
    return out


def keys_kernel_fits(num_heads: int, num_kv_heads: int, head_dim: int) -> bool:
    """Whether the single-token matrix-core kernels take this geometry. Those that share pages
    through LDS (head sizes up to 192) hold a fixed amount of it whatever the group; the one
    for larger heads merges its four waves through 4 * (64 + rows * head size) floats, which
    have to fit 64 KB."""
    if head_dim % 32 or not 32 <= head_dim <= 256:
        return False
    group = num_heads // max(num_kv_heads, 1)
    if keys_kernel(group, head_dim) != 4:
        return True
    return (4 * 64 + 4 * min(group, 32) * head_dim) * 4 <= 65536


# ------------------------------------------------------------------ SwiGLU
def swiglu(gate_up: torch.Tensor, out: torch.Tensor, bias: Optional[torch.Tensor] = None):
    """out = silu(gate_up[:, :di]) * gate_up[:, di:]."""
    _dev(gate_up, "gate_up"); _dev(out, "out", gate_up.dtype)
    nt, w = gate_up.shape
    if w % 2 or out.shape != (nt, w // 2):
        raise KernelError(f"swiglu: gate_up {tuple(gate_up.shape)} / out {tuple(out.shape)}")
    if bias is not None:
        _dev(bias, "bias", torch.float32)
        if bias.numel() != w:
            raise KernelError("swiglu: bias must hold one entry per gate_up column")
    _check(library().ta_swiglu(_stream(), c_int(_code(gate_up.dtype)), _ptr(gate_up), _ptr(bias),
                               _ptr(out), c_int(nt), c_int(w // 2)))
    return out


# ------------------------------------------------------------------ matrix product (plain)
def gemm_simple(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor,
                bias: Optional[torch.Tensor] = None):
    """out = a @ w.T (+ bias), float32 accumulation in ascending k for every element. a and
    w share a dtype, or a is bfloat16 and w float32 (a matrix that stays as its file stores it)."""
    _dev(a, "a", contiguous=False)
    _dev(w, "w", None if (a.dtype == torch.bfloat16 and w.dtype == torch.float32) else a.dtype,
         contiguous=False)
    _dev(out, "out", contiguous=False)
    M, lda = _rows2d(a, "a"); N, ldw = _rows2d(w, "w"); Mo, ldc = _rows2d(out, "out")
    K = a.shape[1]
    if w.shape[1] != K or Mo != M or out.shape[1] != N:
        raise KernelError(f"gemm: a {tuple(a.shape)} w {tuple(w.shape)} out {tuple(out.shape)}")
    if bias is not None:
        _dev(bias, "bias", torch.float32)
        if bias.shape != (N,):
            raise KernelError("gemm: bias must hold one entry per output column")
    _check(library().ta_gemm_simple(_stream(), c_int(_code(a.dtype)), c_int(_code(w.dtype)),
                                    c_int(_code(out.dtype)),
                                    _ptr(a), c_int(lda), _ptr(w), c_int(ldw), _ptr(bias), _ptr(out),
                                    c_int(ldc), c_int(M), c_int(N), c_int(K)))
    return out


class RowScale:
    """Rows of activations that an RMS norm has not scaled yet: ``parts`` [tiles, 16] float32
    holds sums of squares per row (16 columns each), and the product that reads the rows
    multiplies its result by rsqrt(sum / size + eps)."""

    def __init__(self, parts: torch.Tensor, eps: float, size: int):
        self.parts, self.eps, self.size = parts, float(eps), int(size)


class NormFold:
    """What the product in front of an RMS norm needs to take the norm over: the float32
    residual stream ``x`` [m, n] that its result is added to, the norm's weight [n] and eps,
    the buffer ``h`` [m, n] (bfloat16) for the next product's activations, and scratch for
    the sums of squares. ``scale()`` is what the product behind the norm is given."""

    def __init__(self, x: torch.Tensor, weight: torch.Tensor, eps: float, h: torch.Tensor,
                 parts: torch.Tensor):
        self.x, self.weight, self.eps, self.h, self.parts = x, weight, float(eps), h, parts

    @staticmethod
    def parts_shape(size: int):
        return (-(-size // 16), 16)

    def scale(self) -> RowScale:
        return RowScale(self.parts, self.eps, self.x.shape[1])


def gemm_skinny(a: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor], swiglu: bool = False,
                bias: Optional[torch.Tensor] = None, waves: int = 0,
                scale: Optional[RowScale] = None, fold: Optional[NormFold] = None):
    """out = a @ w.T for at most 16 rows of bfloat16 ``a`` (decode steps), float32
    accumulation, out bfloat16 or float32. swiglu: w is [2*n, k] (gate rows, up rows)
    and out [m, n] = silu(a @ gate.T) * (a @ up.T). waves: 4, 8 or 16 waves of a
    workgroup split k; 0 lets the library choose by the weight's shape.

    scale: the rows of ``a`` still lack their norm's factor, which is applied to the
    product. fold: instead of writing ``out``, the product (+ bias) is added to fold.x,
    and fold.h and fold.parts are prepared for the product behind the next norm."""
    _dev(a, "a", torch.bfloat16, contiguous=False); _dev(w, "w", torch.bfloat16, contiguous=False)
    M, lda = _rows2d(a, "a"); N, ldw = _rows2d(w, "w")
    K = a.shape[1]
    n_out = N // 2 if swiglu else N
    if w.shape[1] != K or (swiglu and N % 2):
        raise KernelError(f"gemm_skinny: a {tuple(a.shape)} w {tuple(w.shape)}")
    if fold is None:
        _dev(out, "out", contiguous=False)
        Mo, ldc = _rows2d(out, "out")
        if Mo != M or out.shape[1] != n_out:
            raise KernelError(f"gemm_skinny: a {tuple(a.shape)} w {tuple(w.shape)} out {tuple(out.shape)}")
        out_code = _code(out.dtype)
    else:
        ldc, out_code = n_out, F32
    if bias is not None:
        _dev(bias, "bias", torch.float32)
        if bias.numel() != N:
            raise KernelError("gemm_skinny: bias must hold one entry per row of w")
    if scale is None and fold is None:
        _check(library().ta_gemm_skinny_bf16(_stream(), c_int(out_code), c_int(int(swiglu)),
                                             _ptr(a), c_int(lda), _ptr(w), c_int(ldw), _ptr(bias),
                                             _ptr(out), c_int(ldc), c_int(M), c_int(n_out), c_int(K),
                                             c_int(waves)))
        return out
    sp, n_parts, eps, size = None, 0, 0.0, 0
    if scale is not None:
        _dev(scale.parts, "scale.parts", torch.float32)
        if scale.parts.dim() != 2 or scale.parts.shape[1] != 16 or scale.size != K or \
                scale.parts.shape[0] != -(-K // 16):
            raise KernelError(f"gemm_skinny: partial sums {tuple(scale.parts.shape)} for rows of {K}")
        sp, n_parts, eps, size = scale.parts, scale.parts.shape[0], scale.eps, scale.size
    x = nw = h = op = None
    ldx = ldh = 0
    if fold is not None:
        if swiglu:
            raise KernelError("gemm_skinny: the activation cannot be followed by the residual")
        _dev(fold.x, "fold.x", torch.float32, contiguous=False)
        _dev(fold.h, "fold.h", torch.bfloat16, contiguous=False)
        _dev(fold.weight, "fold.weight", torch.float32); _dev(fold.parts, "fold.parts", torch.float32)
        Mx, ldx = _rows2d(fold.x, "fold.x"); Mh, ldh = _rows2d(fold.h, "fold.h")
        if Mx != M or Mh != M or fold.x.shape[1] != n_out or fold.h.shape[1] != n_out or \
                fold.weight.numel() != n_out or tuple(fold.parts.shape) != NormFold.parts_shape(n_out):
            raise KernelError(f"gemm_skinny: fold of x {tuple(fold.x.shape)} h {tuple(fold.h.shape)} "
                              f"parts {tuple(fold.parts.shape)} behind a product of {M} x {n_out}")
        x, nw, h, op = fold.x, fold.weight, fold.h, fold.parts
    _check(library().ta_gemm_skinny_norm_bf16(
        _stream(), c_int(out_code), c_int(int(swiglu)), _ptr(a), c_int(lda), _ptr(w), c_int(ldw),
        _ptr(bias), _ptr(out) if fold is None else None, c_int(ldc), c_int(M), c_int(n_out), c_int(K),
        c_int(waves), _ptr(sp), c_int(n_parts), c_float(eps), c_int(size), _ptr(x), c_int(ldx),
        _ptr(nw), _ptr(h), c_int(ldh), _ptr(op)))
    return out


SKINNY_MAX_ROWS = 16
MID_MAX_ROWS = 64


def mid_splits(w: torch.Tensor) -> int:
    """Planes in which ``gemm_mid`` leaves a float32 product of this weight (its shape alone
    decides: few column tiles are cut along k among several workgroups)."""
    return int(library().ta_gemm_mid_splits(c_int(w.shape[0]), c_int(w.shape[1])))


def gemm_mid(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, swiglu: bool = False,
             bias: Optional[torch.Tensor] = None):
    """out = a @ w.T for at most 64 rows of bfloat16 ``a``, float32 accumulation. out is
    [m, n] (bfloat16 or float32) or, float32 only, [planes, m, n] whose planes add up to the
    product (``mid_splits`` planes at most; the bias is in plane 0). swiglu: w is [2*n, k]
    (gate rows, up rows) and out [m, n] = silu(a @ gate.T) * (a @ up.T)."""
    _dev(a, "a", torch.bfloat16, contiguous=False); _dev(w, "w", torch.bfloat16, contiguous=False)
    M, lda = _rows2d(a, "a"); N, ldw = _rows2d(w, "w")
    K = a.shape[1]
    n_out = N // 2 if swiglu else N
    if w.shape[1] != K or (swiglu and N % 2):
        raise KernelError(f"gemm_mid: a {tuple(a.shape)} w {tuple(w.shape)}")
    planes, plane = 1, 0
    if out.dim() == 3:
        _dev(out, "out", torch.float32)
        planes, plane = out.shape[0], out.stride(0)
        first = out[0]
    else:
        _dev(out, "out", contiguous=False)
        first = out
    Mo, ldc = _rows2d(first, "out")
    if Mo != M or first.shape[1] != n_out:
        raise KernelError(f"gemm_mid: a {tuple(a.shape)} w {tuple(w.shape)} out {tuple(out.shape)}")
    if bias is not None:
        _dev(bias, "bias", torch.float32)
        if bias.numel() != N:
            raise KernelError("gemm_mid: bias must hold one entry per row of w")
    _check(library().ta_gemm_mid_bf16(_stream(), c_int(_code(out.dtype)), c_int(int(swiglu)), _ptr(a),
                                      c_int(lda), _ptr(w), c_int(ldw), _ptr(bias), _ptr(out), c_int(ldc),
                                      c_longlong(plane), c_int(M), c_int(n_out), c_int(K), c_int(planes)))
    return out


def mid_takes(rows: int, w: torch.Tensor) -> bool:
    """Shapes for which ``gemm_mid`` is used instead of the vendor library: more rows than the
    few-rows product takes (or a k too long for it), at most 64."""
    return (w.dtype == torch.bfloat16 and w.dim() == 2 and 0 < rows <= MID_MAX_ROWS
            and w.shape[1] % 8 == 0 and w.stride(0) % 8 == 0 and w.stride(1) == 1
            and w.data_ptr() % 16 == 0 and not skinny_takes(rows, w))


def mid_wins_plain(rows: int, w: torch.Tensor) -> bool:
    """Whether ``gemm_mid`` beats the vendor library for a plain product in one plane: 17 to 48
    rows against a weight of 65 to 128 column tiles of 64, which it cuts into workgroups of 32
    columns with four quarters of k each (the qkv product of the 8B shape, 6,144 columns: 13.7,
    14.4, 16.7, 17.3 us at 24, 32, 40, 48 rows against 15.6, 15.8, 18.0, 18.0; at 56 and 64 rows
    20.0 against 18.6: every workgroup's reading of all activations then costs more than is
    won; with fewer tiles there are too few workgroups, with more (10,240 or 12,288 columns)
    the library is level or ahead at every row count)."""
    return mid_takes(rows, w) and rows <= 48 and 64 < -(-w.shape[0] // 64) <= 128


def skinny_ok(a: torch.Tensor, w: torch.Tensor) -> bool:
    """Shapes the few-rows product takes."""
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
            and 0 < a.shape[0] <= SKINNY_MAX_ROWS and a.shape[1] % 8 == 0
            and a.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0
            and w.data_ptr() % 16 == 0)


def skinny_wins(a: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether the few-rows product is at least as fast as the library's for this shape
    (measured on MI355X with weights from 34 MB to 1 GB, k of 4096 to 28672): up to 8
    rows always; up to 16 rows while k is short, because every workgroup reads its part
    of the activations again and that grows with rows times k."""
    if not skinny_ok(a, w):
        return False
    m = a.shape[0]
    return m <= 8 or a.shape[1] <= 4096


def skinny_fits(rows: int, w: torch.Tensor) -> bool:
    """Whether the few-rows product can take ``rows`` rows of bfloat16 activations in a fresh
    workspace buffer against this weight at all (asked before the activations exist)."""
    return (w.dtype == torch.bfloat16 and w.dim() == 2 and 0 < rows <= SKINNY_MAX_ROWS
            and w.shape[1] % 8 == 0 and w.stride(0) % 8 == 0 and w.stride(1) == 1
            and w.data_ptr() % 16 == 0)


def skinny_takes(rows: int, w: torch.Tensor) -> bool:
    """``skinny_wins`` in the same terms: also at least as fast as the other products."""
    return skinny_fits(rows, w) and (rows <= 8 or w.shape[1] <= 4096)


def skinny_folds(rows: int, w: torch.Tensor) -> bool:
    """Whether the product in front of a norm should be the few-rows one with the norm folded
    in: up to 16 rows whatever k, because the alternatives pay for the norm's own kernel as
    well (down projection of the 8B shape at 16 rows: 28.6 us against 25.8 + 6.0)."""
    return skinny_fits(rows, w)


# ------------------------------------------------------------------ sampling
def argmax(logits: torch.Tensor, out: torch.Tensor):
    """out[i] = index of the highest logit of row i (lowest index among equals)."""
    _dev(logits, "logits", torch.float32, contiguous=False); _dev(out, "out", torch.int32)
    n, ld = _rows2d(logits, "logits")
    if out.numel() != n:
        raise KernelError("argmax: out must hold one entry per row")
    _check(library().ta_argmax(_stream(), _ptr(logits), c_longlong(ld), c_int(n),
                               c_int(logits.shape[1]), _ptr(out)))
    return out


def sample(logits: torch.Tensor, uniform: torch.Tensor, out: torch.Tensor, temperature: float,
           top_k: int, top_p: float):
    """Draws one token per row from softmax(logits / temperature) cut by top_k / top_p."""
    _dev(logits, "logits", torch.float32, contiguous=False); _dev(out, "out", torch.int32)
    _dev(uniform, "uniform", torch.float32)
    n, ld = _rows2d(logits, "logits")
    if out.numel() != n or uniform.numel() != n:
        raise KernelError("sample: out and uniform must hold one entry per row")
    vocab = logits.shape[1]
    _check(library().ta_sample(_stream(), _ptr(logits), c_longlong(ld), c_int(n), c_int(vocab),
                               c_float(temperature), c_int(min(int(top_k), vocab)),
                               c_float(top_p), _ptr(uniform), _ptr(out)))
    return out


# ------------------------------------------------------------------ random fill
def fill_normal(out: torch.Tensor, seed: int, stream_id: int, mean: float, std: float):
    """out[i] = mean + std * z_i, z_i standard normal, a function of (seed, stream_id, i)."""
    _dev(out, "out")
    _check(library().ta_fill_normal(_stream(), c_int(_code(out.dtype)), _ptr(out),
                                    c_longlong(out.numel()), ctypes.c_ulonglong(seed & (2**64 - 1)),
                                    ctypes.c_ulonglong(stream_id & (2**64 - 1)), c_float(mean),
                                    c_float(std)))
    return out


# ------------------------------------------------------------------ conversion at load
def read_probe(buf: torch.Tensor, workgroups: int, sink: torch.Tensor) -> None:
    """Launches a kernel that only reads ``buf`` (any dtype, contiguous, a multiple of 16
    bytes) with ``workgroups`` workgroups of 256 threads; ``sink`` is 256 int32 that stay
    untouched. For measuring what the memory gives a plain read."""
    _dev(buf, "buf"); _dev(sink, "sink", torch.int32)
    nbytes = buf.numel() * buf.element_size()
    if sink.numel() < 256:
        raise KernelError("read_probe: sink needs 256 entries")
    _check(library().ta_read_probe(_stream(), _ptr(buf), c_longlong(nbytes), c_int(workgroups), _ptr(sink)))


_CONVERT_SRC = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}


def convert_takes(src: torch.dtype, dst: torch.dtype) -> bool:
    return src in _CONVERT_SRC and dst in (torch.float32, torch.bfloat16)


def convert(src: torch.Tensor, dst: torch.Tensor) -> torch.Tensor:
    """dst[i] = src[i] in dst's floating type (float32 or bfloat16) from float32, bfloat16 or
    float16: exact when widening, round-to-nearest-even when narrowing. Flat, same count."""
    _dev(src, "src"); _dev(dst, "dst")
    if not convert_takes(src.dtype, dst.dtype):
        raise KernelError(f"convert: {src.dtype} -> {dst.dtype} is not offered")
    if src.numel() != dst.numel():
        raise KernelError(f"convert: {src.numel()} values into {dst.numel()}")
    _check(library().ta_convert(_stream(), c_int(_CONVERT_SRC[src.dtype]), c_int(_code(dst.dtype)),
                                _ptr(src), _ptr(dst), c_longlong(src.numel())))
    return dst
