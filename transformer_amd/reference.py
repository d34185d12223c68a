"""Python face of the plain C++ twins of the kernels (``csrc/*_ref.cpp``): the same
operations as ``transformer_amd.kernels`` on NumPy float32 arrays, computed on the host by
plain loops with double-precision sums. Tests compare the HIP kernels with them; nothing
on the product path imports this module.

A caller that checks a bfloat16 kernel widens its inputs to float32 (exact) and rounds the
twin's result where the kernel stores bfloat16.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_longlong, c_ulonglong, c_void_p
from typing import Optional

import numpy as np

from .csrc.build import ensure_ref_built

PAGE = 64


class ReferenceError_(RuntimeError):
    pass


_lib = None


def library():
    global _lib
    if _lib is None:
        lib = ctypes.CDLL(str(ensure_ref_built()))
        lib.ta_ref_last_error.restype = ctypes.c_char_p
        if lib.ta_ref_page_size() != PAGE:
            raise ReferenceError_("the plain twins disagree about the page size")
        _lib = lib
    return _lib


def _check(rc):
    if rc != 0:
        raise ReferenceError_(library().ta_ref_last_error().decode())


def _f(a, name):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a


def _i(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _p(a: Optional[np.ndarray]):
    return c_void_p(a.ctypes.data) if a is not None else c_void_p(0)


def embed(table, tokens):
    table, tokens = _f(table, "table"), _i(tokens)
    out = np.empty((tokens.size, table.shape[1]), dtype=np.float32)
    _check(library().ta_ref_embed(_p(table), c_int(table.shape[0]), c_int(table.shape[1]), _p(tokens),
                                  c_int(tokens.size), _p(out)))
    return out


def add_rmsnorm(x, weight, eps, delta=None, delta_bias=None, rows=None):
    """Returns (out, x after the add). delta: [nt, d] or [planes, nt, d]."""
    x = _f(x, "x").copy()
    nt, d = x.shape
    weight = _f(weight, "weight")
    planes, plane = 1, 0
    if delta is not None:
        delta = _f(delta, "delta")
        if delta.ndim == 3:
            planes, plane = delta.shape[0], nt * d
    if delta_bias is not None:
        delta_bias = _f(delta_bias, "delta_bias")
    r = _i(rows) if rows is not None else None
    n_out = r.size if r is not None else nt
    out = np.empty((n_out, d), dtype=np.float32)
    store = int(rows is None and (delta is not None or delta_bias is not None))
    _check(library().ta_ref_add_rmsnorm(_p(x), _p(delta), c_int(planes), c_longlong(plane), _p(delta_bias),
                                        _p(weight), _p(r), c_int(n_out), c_int(d), c_float(eps), c_int(store),
                                        _p(out)))
    return out, x


def rope_table(positions, inv_freq):
    positions, inv_freq = _i(positions), _f(inv_freq, "inv_freq")
    out = np.empty((positions.size, inv_freq.size, 2), dtype=np.float32)
    _check(library().ta_ref_rope_table(_p(positions), _p(inv_freq), c_int(positions.size), c_int(inv_freq.size),
                                       _p(out)))
    return out


def rope_kv_write(qkv, num_q_heads, num_kv_heads, head_dim, angles, interleaved, dest=None, kcache=None,
                  vcache=None, bias=None):
    """Returns qkv after bias and rotation; kcache [pages, nkv, 64, dh] and vcache
    [pages, nkv, dh, 64] (float32, C-contiguous) are written in place."""
    qkv = _f(qkv, "qkv").copy()
    nt = qkv.shape[0]
    for c in (kcache, vcache):
        if c is not None and (c.dtype != np.float32 or not c.flags.c_contiguous):
            raise ReferenceError_("cache arrays must be C-contiguous float32 (they are written in place)")
    ang = _f(angles, "angles") if angles is not None else None
    b = _f(bias, "bias") if bias is not None else None
    d = _i(dest) if dest is not None else None
    _check(library().ta_ref_rope_kv_write(_p(qkv), _p(b), _p(d), _p(ang), c_int(1 if interleaved else 0),
                                          _p(kcache), _p(vcache), c_int(nt), c_int(num_q_heads),
                                          c_int(num_kv_heads), c_int(head_dim)))
    return qkv


def attention(q, kcache, vcache, block_table, cu_q, pos0, num_heads, num_kv_heads, head_dim, scale,
              window=None):
    """q [nt, >= nh*dh]; kcache [pages, nkv, 64, dh]; vcache [pages, nkv, dh, 64] -> [nt, nh*dh]."""
    q, kcache, vcache = _f(q, "q"), _f(kcache, "kcache"), _f(vcache, "vcache")
    block_table, cu_q, pos0 = _i(block_table), _i(cu_q), _i(pos0)
    nt = q.shape[0]
    out = np.empty((nt, num_heads * head_dim), dtype=np.float32)
    _check(library().ta_ref_attention(_p(q), c_int(q.shape[1]), _p(out), c_int(out.shape[1]), _p(kcache),
                                      _p(vcache), _p(block_table), c_int(block_table.shape[1]), _p(cu_q),
                                      _p(pos0), c_int(pos0.size), c_int(num_heads), c_int(num_kv_heads),
                                      c_int(head_dim), c_float(scale), c_int(window or 0)))
    return out


def swiglu(gate_up, bias=None):
    gate_up = _f(gate_up, "gate_up")
    nt, w = gate_up.shape
    b = _f(bias, "bias") if bias is not None else None
    out = np.empty((nt, w // 2), dtype=np.float32)
    _check(library().ta_ref_swiglu(_p(gate_up), _p(b), _p(out), c_int(nt), c_int(w // 2)))
    return out


def gemm(a, w, bias=None, swiglu=False):
    """a [M, K] @ w [N, K]^T (+ bias); swiglu: w holds gate rows then up rows, out [M, N/2]."""
    a, w = _f(a, "a"), _f(w, "w")
    M, K = a.shape
    n_out = w.shape[0] // 2 if swiglu else w.shape[0]
    b = _f(bias, "bias") if bias is not None else None
    out = np.empty((M, n_out), dtype=np.float32)
    _check(library().ta_ref_gemm(_p(a), c_int(K), _p(w), c_int(K), _p(b), _p(out), c_int(n_out), c_int(M),
                                 c_int(n_out), c_int(K), c_int(int(swiglu))))
    return out


def argmax(logits):
    logits = _f(logits, "logits")
    out = np.empty(logits.shape[0], dtype=np.int32)
    _check(library().ta_ref_argmax(_p(logits), c_longlong(logits.shape[1]), c_int(logits.shape[0]),
                                   c_int(logits.shape[1]), _p(out)))
    return out


def sample(logits, uniform, temperature, top_k=None, top_p=1.0, return_kept=False):
    logits, uniform = _f(logits, "logits"), _f(uniform, "uniform")
    n, vocab = logits.shape
    out = np.empty(n, dtype=np.int32)
    kept = np.empty((n, vocab), dtype=np.float64) if return_kept else None
    _check(library().ta_ref_sample(_p(logits), c_longlong(vocab), c_int(n), c_int(vocab), c_float(temperature),
                                   c_int(min(int(top_k), vocab) if top_k is not None else vocab), c_float(top_p),
                                   _p(uniform), _p(out), _p(kept)))
    return (out, kept) if return_kept else out


def fill_normal(n, seed, stream_id, mean, std):
    out = np.empty(int(n), dtype=np.float32)
    _check(library().ta_ref_fill_normal(_p(out), c_longlong(int(n)), c_ulonglong(seed & (2 ** 64 - 1)),
                                        c_ulonglong(stream_id & (2 ** 64 - 1)), c_float(mean), c_float(std)))
    return out


def convert(src, dst_bfloat16: bool):
    """float32 in, float32 out holding exactly what the target type stores."""
    src = np.ascontiguousarray(src, dtype=np.float32)
    out = np.empty(src.shape, dtype=np.float32)
    _check(library().ta_ref_convert(c_int(0), c_int(1 if dst_bfloat16 else 0), _p(src), _p(out),
                                    c_longlong(src.size)))
    return out


def convert_bits(bits, src_kind: str, dst_bfloat16: bool):
    """bits: uint16 patterns of "bfloat16" or "float16" values -> float32 holding what the target stores."""
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    out = np.empty(bits.shape, dtype=np.float32)
    _check(library().ta_ref_convert(c_int({"bfloat16": 1, "float16": 2}[src_kind]), c_int(1 if dst_bfloat16 else 0),
                                    _p(bits), _p(out), c_longlong(bits.size)))
    return out
