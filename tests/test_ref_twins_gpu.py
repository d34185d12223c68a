"""Each HIP kernel against its plain C++ twin (``transformer_amd/csrc/*_ref.cpp`` through
``transformer_amd.reference``), at sizes other than the engine's. The twins themselves are
held against the NumPy functions in ``test_ref_twins.py``, which needs no GPU."""
import math

import numpy as np
import pytest
import torch

import plain_llama as P
from transformer_amd import reference as R

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
rng = np.random.default_rng(23)


def dev(a, dtype=torch.float32):
    return torch.tensor(np.ascontiguousarray(a), dtype=dtype, device=DEV).contiguous()


def host(t):
    return t.detach().float().cpu().numpy()


def stored(a, dtype):
    """What the engine would hold: float32, or rounded to bfloat16 (and widened again)."""
    return P.round_bf16(a).astype(np.float32) if dtype == "bfloat16" else np.asarray(a, np.float32)


def tol(dtype, scale=1.0):
    return (2e-5 if dtype == "float32" else 1.2e-2) * scale


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embed_and_norm_kernels_against_their_twins(dtype):
    from transformer_amd import kernels
    table = stored(rng.normal(size=(77, 104)), dtype)
    toks = [76, 0, 5, 5, 77, -3]
    out = torch.empty(6, 104, device=DEV)
    kernels.embed(dev(table, DT[dtype]), dev(toks, torch.int32), out)
    assert np.array_equal(host(out), R.embed(table, toks), equal_nan=True)
    nt, d = 9, 1000
    x = rng.normal(size=(nt, d)).astype(np.float32)
    w = (1 + 0.1 * rng.normal(size=d)).astype(np.float32)
    delta = rng.normal(size=(3, nt, d)).astype(np.float32)
    bias = rng.normal(size=d).astype(np.float32)
    xd, o = dev(x), torch.empty(nt, d, dtype=DT[dtype], device=DEV)
    kernels.add_rmsnorm(xd, dev(w), 1e-4, o, delta=dev(delta), delta_bias=dev(bias))
    want, x_new = R.add_rmsnorm(x, w, 1e-4, delta=delta, delta_bias=bias)
    assert np.abs(host(xd) - x_new).max() < 2e-6
    assert np.abs(host(o) - want).max() < tol(dtype, 4)
    rows = [7, 2, 2]
    o2 = torch.empty(3, d, dtype=DT[dtype], device=DEV)
    kernels.add_rmsnorm(dev(x), dev(w), 1e-4, o2, delta=dev(delta[1]), rows=dev(rows, torch.int32))
    want, _ = R.add_rmsnorm(x, w, 1e-4, delta=delta[1], rows=rows)
    assert np.abs(host(o2) - want).max() < tol(dtype, 4)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("style", ["half", "interleaved"])
def test_rotation_kernels_against_their_twins(dtype, style):
    from transformer_amd import kernels
    nq, nkv, dh, nt = 5, 2, 48, 11
    pos = [int(p) for p in rng.integers(0, 3000, nt)]
    inv = P.rope_inv_freq(dh, 50000.0).astype(np.float32)
    ang = kernels.rope_table(dev(pos, torch.int32), dev(inv), torch.empty(nt, dh // 2, 2, device=DEV))
    twin_ang = R.rope_table(pos, inv)
    assert np.abs(host(ang) - twin_ang).max() < 2e-6               # the device's sincosf against the host's
    qkv = stored(rng.normal(size=(nt, (nq + 2 * nkv) * dh)), dtype)
    bias = (rng.normal(size=(nq + 2 * nkv) * dh) * 0.1).astype(np.float32)
    pages = 30
    dest = [int(p) * 64 + int(o) for p, o in zip(rng.permutation(pages)[:nt], rng.integers(0, 64, nt))]
    kc = torch.full((pages, nkv, 64, dh), float("nan"), dtype=DT[dtype], device=DEV)
    vc = torch.full((pages, nkv, dh, 64), float("nan"), dtype=DT[dtype], device=DEV)
    t = dev(qkv, DT[dtype])
    kernels.rope_kv_write(t, nq, nkv, dh, ang, style == "interleaved", dev(dest, torch.int32), kc, vc, dev(bias))
    tk = np.full((pages, nkv, 64, dh), np.nan, dtype=np.float32)
    tv = np.full((pages, nkv, dh, 64), np.nan, dtype=np.float32)
    want = R.rope_kv_write(qkv, nq, nkv, dh, twin_ang, style == "interleaved", dest, tk, tv, bias)
    e = tol(dtype, 4)
    assert np.abs(host(t) - want).max() < e
    kd, vd = host(kc), host(vc)
    assert np.array_equal(np.isnan(kd), np.isnan(tk)) and np.array_equal(np.isnan(vd), np.isnan(tv))
    assert np.nanmax(np.abs(kd - tk)) < e and np.nanmax(np.abs(vd - tv)) < e


def _paged(r, totals, nkv, dh, dtype):
    need = [-(-t // 64) for t in totals]
    order = r.permutation(sum(need) + 3)
    kc = np.zeros((len(order), nkv, 64, dh), dtype=np.float32)
    vc = np.zeros((len(order), nkv, dh, 64), dtype=np.float32)
    table = np.zeros((len(totals), max(need)), dtype=np.int32)
    used = 0
    for b, t in enumerate(totals):
        table[b, :need[b]] = order[used:used + need[b]]
        used += need[b]
        k, v = stored(r.normal(size=(t, nkv, dh)), dtype), stored(r.normal(size=(t, nkv, dh)), dtype)
        for p in range(t):
            kc[table[b, p // 64], :, p % 64] = k[p]
            vc[table[b, p // 64], :, :, p % 64] = v[p]
    return kc, vc, table


ATTENTION = [
    # kernel, dtype, nh, nkv, dh, new tokens, cached tokens, window
    ("generic", "float32", 6, 3, 80, [1, 9, 40], [70, 0, 13], None),
    ("generic", "bfloat16", 4, 4, 16, [3, 1], [200, 63], 50),
    ("rows", "bfloat16", 12, 4, 96, [300, 17], [0, 90], None),
    ("rows", "bfloat16", 8, 2, 64, [130], [40], 100),
    ("keys", "bfloat16", 16, 4, 128, [1, 1, 1], [500, 64, 0], None),
    ("keys", "bfloat16", 20, 1, 64, [1, 1], [129, 1000], 300),
]


@pytest.mark.parametrize("case", ATTENTION, ids=[f"{c[0]}-{c[1]}-h{c[2]}kv{c[3]}d{c[4]}" for c in ATTENTION])
def test_attention_kernels_against_their_twin(case):
    from transformer_amd import kernels
    which, dtype, nh, nkv, dh, qlens, pos0, window = case
    r = np.random.default_rng(nh * dh)
    totals = [p + n for p, n in zip(pos0, qlens)]
    kc, vc, table = _paged(r, totals, nkv, dh, dtype)
    nt = sum(qlens)
    q = np.zeros((nt, (nh + 2 * nkv) * dh), dtype=np.float32)          # q inside the wider qkv row
    q[:, :nh * dh] = stored(r.normal(size=(nt, nh * dh)), dtype)
    cu = np.concatenate([[0], np.cumsum(qlens)])
    scale = 1 / math.sqrt(dh)
    out = torch.full((nt, nh * dh), float("nan"), dtype=DT[dtype], device=DEV)
    args = (dev(q, DT[dtype]), out, dev(kc, DT[dtype]), dev(vc, DT[dtype]), dev(table, torch.int32),
            dev(cu, torch.int32), dev(pos0, torch.int32))
    if which == "generic":
        kernels.attention_generic(*args, max(qlens), nh, nkv, dh, scale, window)
    elif which == "rows":
        kernels.attention_rows(*args, max(qlens), nh, nkv, dh, scale, window)
    else:
        kernels.attention_keys(*args, max(totals), nh, nkv, dh, scale, window)
    want = R.attention(q, kc, vc, table, cu, pos0, nh, nkv, dh, scale, window)
    got = host(out)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() < tol(dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_swiglu_kernel_against_its_twin(dtype):
    from transformer_amd import kernels
    gu = stored(rng.normal(size=(7, 2 * 301)) * 3, dtype)
    bias = rng.normal(size=602).astype(np.float32)
    out = torch.empty(7, 301, dtype=DT[dtype], device=DEV)
    rel = 2.0 ** -8 if dtype == "bfloat16" else 2.0 ** -22
    for b in (None, bias):
        kernels.swiglu(dev(gu, DT[dtype]), out, dev(b) if b is not None else None)
        want = R.swiglu(gu, b)
        assert (np.abs(host(out) - want) <= rel * np.abs(want) + 1e-5).all()


PRODUCTS = [
    # kernel, M, N (output columns), K, swiglu
    ("simple", 5, 130, 97, False),
    ("skinny", 8, 304, 1000, False),
    ("skinny", 3, 152, 520, True),
    ("mid", 40, 200, 1096, False),
    ("mid", 64, 96, 520, True),
]


@pytest.mark.parametrize("case", PRODUCTS, ids=[f"{c[0]}-m{c[1]}n{c[2]}k{c[3]}{'-swiglu' if c[4] else ''}" for c in PRODUCTS])
def test_product_kernels_against_their_twin(case):
    from transformer_amd import kernels
    which, M, N, K, swiglu = case
    dtype = "float32" if which == "simple" else "bfloat16"
    a = stored(rng.normal(size=(M, K)), dtype)
    w = stored(rng.normal(size=((2 if swiglu else 1) * N, K)) * 0.1, dtype)
    bias = rng.normal(size=(2 if swiglu else 1) * N).astype(np.float32)
    out = torch.empty(M, N, dtype=torch.float32, device=DEV)
    ad, wd, bd = dev(a, DT[dtype]), dev(w, DT[dtype]), dev(bias)
    if which == "simple":
        kernels.gemm_simple(ad, wd, out, bd)
    elif which == "skinny":
        kernels.gemm_skinny(ad, wd, out, swiglu=swiglu, bias=bd)
    else:
        kernels.gemm_mid(ad, wd, out, swiglu=swiglu, bias=bd)
    want = R.gemm(a, w, bias, swiglu=swiglu)
    # float32 sums of K products of order 0.1 in another order than the twin's double sum
    assert np.abs(host(out) - want).max() < 1e-6 * K ** 0.5 * 8 * max(1.0, np.abs(want).max())


def test_sampling_kernels_against_their_twins():
    from transformer_amd import kernels
    n, vocab = 24, 5003
    logits = (rng.normal(size=(n, vocab)) * 2.5).astype(np.float32)
    logits[3, 100] = logits[3, 4000] = logits[3].max() + 1          # equals: the lower index
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    kernels.argmax(dev(logits), out)
    assert np.array_equal(out.cpu().numpy(), R.argmax(logits))
    for temperature, top_k, top_p in ((0.9, None, 1.0), (1.2, 40, 1.0), (0.7, None, 0.85), (1.0, 200, 0.6)):
        u = rng.random(n).astype(np.float32)
        kernels.sample(dev(logits), dev(u), out, temperature, top_k if top_k is not None else vocab, top_p)
        got = out.cpu().numpy()
        want, kept = R.sample(logits, u, temperature, top_k, top_p, return_kept=True)
        for r in range(n):
            if got[r] == want[r]:
                continue
            # the kernel's masses come from the hardware's exp2, the twin's from the double
            # exponential: a draw within their last bits of a boundary may go to the neighbour,
            # which has to be a kept token whose interval ends or starts at that boundary
            p = kept[r] / kept[r].sum()
            cdf = np.cumsum(p)
            assert p[got[r]] > 0 and cdf[got[r]] - p[got[r]] - 1e-5 <= u[r] <= cdf[got[r]] + 1e-5, (r, got[r], want[r])
        assert (got == want).mean() > 0.9


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_fill_normal_kernel_against_its_twin(dtype):
    from transformer_amd import kernels
    n = 100003
    out = torch.empty(n, dtype=DT[dtype], device=DEV)
    kernels.fill_normal(out, 11, 4242, 1.0, 0.25)
    want = R.fill_normal(n, 11, 4242, 1.0, 0.25)
    # the same integer hashes and uniforms; the device's float32 logarithm and cosine against
    # the host's doubles, then the storage type's rounding
    bound = 3e-6 if dtype == "float32" else 2.0 ** -8 * 2.5
    assert np.abs(host(out) - want).max() < bound


def test_conversion_kernel_against_its_twin():
    from transformer_amd import kernels
    h = torch.randn(10007, dtype=torch.float32).mul(50).to(torch.float16)
    for dst in (torch.float32, torch.bfloat16):
        out = torch.empty(10007, dtype=dst, device=DEV)
        kernels.convert(h.to(DEV), out)
        want = R.convert_bits(h.numpy().view(np.uint16), "float16", dst == torch.bfloat16)
        assert np.array_equal(host(out), want)
    f = torch.randn(10007) * 1000
    out = torch.empty(10007, dtype=torch.bfloat16, device=DEV)
    kernels.convert(f.to(DEV), out)
    assert np.array_equal(host(out), R.convert(f.numpy(), True))
