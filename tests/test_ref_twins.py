"""The plain C++ twins of the kernels (``transformer_amd/csrc/*_ref.cpp``) against the NumPy
functions of ``plain_llama``: two independent statements of the same formulas, one in C++
beside the kernels, one in Python beside the tests. They run on the host, so this file needs
no GPU; ``test_ref_twins_gpu.py`` holds the HIP kernels against the twins."""
import math

import numpy as np
import pytest

import plain_llama as P
from transformer_amd import reference as R

rng = np.random.default_rng(17)


def f32(a):
    return np.asarray(a, dtype=np.float32)


def paged_cache(r, totals, nkv, dh):
    """Keys and values of sequences in shuffled pages, in the kernels' layout."""
    need = [-(-t // 64) for t in totals]
    order = r.permutation(sum(need) + 2)
    kc = np.full((len(order), nkv, 64, dh), np.nan, dtype=np.float32)
    vc = np.full((len(order), nkv, dh, 64), np.nan, dtype=np.float32)
    table = np.zeros((len(totals), max(need)), dtype=np.int32)
    ks, vs, used = [], [], 0
    for b, t in enumerate(totals):
        table[b, :need[b]] = order[used:used + need[b]]
        used += need[b]
        k, v = f32(r.normal(size=(t, nkv, dh))), f32(r.normal(size=(t, nkv, dh)))
        for p in range(t):
            kc[table[b, p // 64], :, p % 64] = k[p]
            vc[table[b, p // 64], :, :, p % 64] = v[p]
        ks.append(k)
        vs.append(v)
    return ks, vs, kc, vc, table


def test_embed_twin():
    table = f32(rng.normal(size=(31, 20)))
    out = R.embed(table, [30, 0, 7, 31, -1])
    assert np.array_equal(out[:3], table[[30, 0, 7]]) and np.isnan(out[3:]).all()


def test_add_rmsnorm_twin():
    x, w = f32(rng.normal(size=(6, 100))), f32(1 + 0.1 * rng.normal(size=100))
    out, _ = R.add_rmsnorm(x, w, 1e-3)
    assert np.abs(out - P.rms_norm(x, w, 1e-3)).max() < 1e-6
    delta, bias = f32(rng.normal(size=(3, 6, 100))), f32(rng.normal(size=100))
    out, x_new = R.add_rmsnorm(x, w, 1e-5, delta=delta, delta_bias=bias)
    want_x = x.astype(np.float64) + delta.astype(np.float64).sum(0) + bias
    assert np.abs(x_new - want_x).max() < 1e-6                       # the stream takes the sum
    assert np.abs(out - P.rms_norm(want_x, w, 1e-5)).max() < 1e-6
    out, x_same = R.add_rmsnorm(x, w, 1e-5, delta=delta[0], rows=[4, 1])
    assert np.array_equal(x_same, x)                                 # gathered rows leave the stream alone
    assert np.abs(out - P.rms_norm((x.astype(np.float64) + delta[0])[[4, 1]], w, 1e-5)).max() < 1e-6


@pytest.mark.parametrize("style", ["half", "interleaved"])
def test_rotation_twins(style):
    nq, nkv, dh, theta = 3, 2, 16, 5000.0
    pos = [0, 5, 64, 1000]
    inv = f32(P.rope_inv_freq(dh, theta))
    ang = R.rope_table(pos, inv)
    a = np.asarray(pos, dtype=np.float32)[:, None] * inv[None, :]
    assert np.abs(ang[..., 0] - np.cos(a.astype(np.float64))).max() < 1e-7
    qkv = f32(rng.normal(size=(4, nq + 2 * nkv, dh)))
    bias = f32(rng.normal(size=(nq + 2 * nkv, dh)) * 0.1)
    kc = np.full((20, nkv, 64, dh), np.nan, dtype=np.float32)
    vc = np.full((20, nkv, dh, 64), np.nan, dtype=np.float32)
    dest = [3 * 64 + 0, 7 * 64 + 5, 1 * 64 + 63, 19 * 64 + 40]
    got = R.rope_kv_write(qkv.reshape(4, -1), nq, nkv, dh, ang, style == "interleaved", dest, kc, vc,
                          bias.reshape(-1)).reshape(4, nq + 2 * nkv, dh)
    src = qkv.astype(np.float64) + bias
    # the twin turns by the float32 angle the kernel forms, the plain function by the float64 one
    assert np.abs(got[:, :nq + nkv] - P.rope(src[:, :nq + nkv], pos, theta, style)).max() < 2e-4
    assert np.abs(got[:, nq + nkv:] - src[:, nq + nkv:]).max() < 1e-6
    for t, d in enumerate(dest):
        assert np.array_equal(kc[d // 64, :, d % 64], got[t, nq:nq + nkv])
        assert np.array_equal(vc[d // 64, :, :, d % 64], got[t, nq + nkv:])
    assert np.isnan(kc).sum() == kc.size - 4 * nkv * dh              # nothing else was written


@pytest.mark.parametrize("window", [None, 1, 37, 64])
def test_attention_twin(window):
    nh, nkv, dh = 6, 2, 16
    qlens, pos0 = [1, 30, 70], [130, 0, 20]
    totals = [p + n for p, n in zip(pos0, qlens)]
    ks, vs, kc, vc, table = paged_cache(np.random.default_rng(3), totals, nkv, dh)
    q = f32(rng.normal(size=(sum(qlens), nh, dh)))
    cu = np.concatenate([[0], np.cumsum(qlens)])
    scale = 1 / math.sqrt(dh)
    wide = np.zeros((sum(qlens), (nh + 2 * nkv) * dh), dtype=np.float32)       # q inside a wider row
    wide[:, :nh * dh] = q.reshape(len(q), -1)
    got = R.attention(wide, kc, vc, table, cu, pos0, nh, nkv, dh, scale, window).reshape(-1, nh, dh)
    want = np.concatenate([P.attention(q[cu[b]:cu[b + 1]], ks[b], vs[b], scale, first_pos=pos0[b], window=window)
                           for b in range(3)])
    assert np.abs(got - want).max() < 1e-6


def test_swiglu_and_product_twins():
    gu, bias = f32(rng.normal(size=(4, 2 * 33)) * 3), f32(rng.normal(size=66))
    def close(got, want):        # the twin hands its double result back as float32: one rounding, relative
        return (np.abs(got - want) <= 1e-7 * np.maximum(1.0, np.abs(want))).all()
    assert close(R.swiglu(gu), P.swiglu(gu[:, :33], gu[:, 33:]))
    wide = gu.astype(np.float64)
    assert close(R.swiglu(gu, bias), P.swiglu(wide[:, :33] + bias[:33], wide[:, 33:] + bias[33:]))
    a, w, b = f32(rng.normal(size=(5, 70))), f32(rng.normal(size=(24, 70))), f32(rng.normal(size=24))
    assert np.abs(R.gemm(a, w, b) - P.linear(a, w, b)).max() < 1e-5
    full = P.linear(a, w, b)
    assert np.abs(R.gemm(a, w, b, swiglu=True) - P.swiglu(full[:, :12], full[:, 12:])).max() < 1e-5


def test_argmax_and_sampling_twins():
    logits = f32(rng.normal(size=(7, 301)) * 3)
    logits[2, 40] = logits[2, 200] = 50.0                       # equals: the lower index
    logits[3, 5] = np.nan
    got = R.argmax(logits)
    assert got[2] == 40 and all(got[r] == int(np.nanargmax(logits[r])) for r in range(7))
    for temperature, top_k, top_p in ((0.8, None, 1.0), (1.3, 20, 1.0), (0.7, None, 0.9), (1.0, 50, 0.5)):
        lg = f32(rng.normal(size=(40, 301)) * 2)
        u = f32(rng.random(40))
        tokens, kept = R.sample(lg, u, temperature, top_k, top_p, return_kept=True)
        for r in range(40):
            p = P.sample_probabilities(lg[r], float(np.float32(temperature)), float(np.float32(top_p)), top_k)
            mine = kept[r] / kept[r].sum()
            assert np.abs(mine - p).max() < 1e-9                # the same kept set, the same distribution
            cdf = np.cumsum(p)
            t = tokens[r]
            assert p[t] > 0 and cdf[t] - p[t] - 1e-9 <= u[r] <= cdf[t] + 1e-9


def test_fill_normal_twin_is_a_function_of_its_keys():
    a, b = R.fill_normal(50000, 5, 77, 1.0, 0.5), R.fill_normal(50000, 5, 77, 1.0, 0.5)
    assert np.array_equal(a, b) and not np.array_equal(a, R.fill_normal(50000, 6, 77, 1.0, 0.5))
    assert abs(a.mean() - 1.0) < 0.01 and abs(a.std() - 0.5) < 0.01
    assert np.array_equal(R.fill_normal(100, 5, 77, 1.0, 0.5), a[:100])       # element i depends on i alone


def test_conversion_twin():
    a = f32(rng.normal(size=5000) * 100)
    a[:4] = [0.0, -0.0, np.inf, 1.0 + 2.0 ** -8]                 # a tie: to even
    assert np.array_equal(R.convert(a, True), P.round_bf16(a).astype(np.float32))
    assert np.array_equal(R.convert(a, False), a)
    h = f32(rng.normal(size=5000)).astype(np.float16)
    h[:3] = [6e-8, 65504.0, -2.0 ** -14]                        # subnormal, largest, smallest normal
    assert np.array_equal(R.convert_bits(h.view(np.uint16), "float16", False), h.astype(np.float32))
    assert np.array_equal(R.convert_bits(h.view(np.uint16), "float16", True),
                          P.round_bf16(h.astype(np.float32)).astype(np.float32))


def test_twins_refuse_bad_sizes():
    with pytest.raises(R.ReferenceError_, match="bad sizes"):
        R.attention(np.zeros((1, 32), np.float32), np.zeros((1, 3, 64, 16), np.float32),
                    np.zeros((1, 3, 16, 64), np.float32), [[0]], [0, 1], [0], 2, 3, 16, 0.25)
