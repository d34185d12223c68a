"""Each HIP kernel alone against its plain reference, at sizes other than the
engine's tiny models: widths that are no power of two, head sizes in steps of
16, unequal batches, shuffled pages, planted stand-out keys, a window's edge."""
import math

import numpy as np
import pytest
import torch

import plain_llama as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
rng = np.random.default_rng(99)


def dev(a, dtype=torch.float32):
    return torch.tensor(np.ascontiguousarray(a), dtype=dtype, device=DEV).contiguous()


def f64(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


def rounded(a, dtype):
    return P.round_bf16(a) if dtype == "bfloat16" else np.asarray(a, dtype=np.float32).astype(np.float64)


def tol(dtype, scale=1.0):
    return (2e-5 if dtype == "float32" else 1.2e-2) * scale


# ------------------------------------------------------------------ embedding
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("d", [100, 104, 4096])          # rows of whole 16-byte pieces take wider loads
def test_embed(dtype, d):
    from transformer_amd import kernels
    table = rounded(rng.normal(size=(301, d)), dtype)
    toks = [300, 0, 17, 17, 299]
    out = torch.empty(5, d, device=DEV)
    kernels.embed(dev(table, DT[dtype]), dev(toks, torch.int32), out)
    assert np.array_equal(f64(out), table[toks])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embed_reads_nothing_for_an_id_outside_the_table(dtype):
    """Ids chosen on the GPU reach the kernel unchecked: one outside [0, vocab) must not be
    read through; its row becomes NaN and the other rows are as always."""
    from transformer_amd import kernels
    table = rounded(rng.normal(size=(50, 24)), dtype)
    toks = [3, 50, -1, 2 ** 31 - 1, 49]
    out = torch.zeros(5, 24, device=DEV)
    kernels.embed(dev(table, DT[dtype]), dev(toks, torch.int32), out)
    got = f64(out)
    assert np.array_equal(got[[0, 4]], table[[3, 49]])
    assert np.isnan(got[1:4]).all()


# ------------------------------------------------------------------ add + RMS norm
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("d", [100, 1000, 4097])
def test_add_rmsnorm(dtype, d):
    from transformer_amd import kernels
    nt, eps = 7, 3e-4
    x = rng.normal(size=(nt, d)).astype(np.float32)
    delta = rounded(rng.normal(size=(nt, d)), dtype)
    bias = rng.normal(size=d).astype(np.float32)
    w = (1 + 0.1 * rng.normal(size=d)).astype(np.float32)
    xs = dev(x)
    out = torch.empty(nt, d, dtype=DT[dtype], device=DEV)
    kernels.add_rmsnorm(xs, dev(w), eps, out, dev(delta, DT[dtype]), dev(bias))
    v = x.astype(np.float64) + delta + bias
    assert np.abs(f64(xs) - v).max() < 1e-6                       # the residual stream got the sum
    assert np.abs(f64(out) - P.rms_norm(v, w, eps)).max() < tol(dtype, 4)
    # plain norm of the stream, nothing to add: x stays as it is
    before = xs.clone()
    kernels.add_rmsnorm(xs, dev(w), eps, out)
    assert torch.equal(xs, before)
    assert np.abs(f64(out) - P.rms_norm(f64(xs), w, eps)).max() < tol(dtype, 4)
    # gathered rows: only those rows, x untouched
    rows = [5, 0, 5]
    o3 = torch.empty(3, d, dtype=DT[dtype], device=DEV)
    kernels.add_rmsnorm(xs, dev(w), eps, o3, dev(delta, DT[dtype]), None, dev(rows, torch.int32))
    assert torch.equal(xs, before)
    want = P.rms_norm(f64(before)[rows] + delta[rows], w, eps)
    assert np.abs(f64(o3) - want).max() < tol(dtype, 4)


def test_rmsnorm_eps_matters_and_sits_inside_the_root():
    from transformer_amd import kernels
    x = dev([[3.0, 4.0]])
    out = torch.empty(1, 2, device=DEV)
    kernels.add_rmsnorm(x, dev([2.0, 0.5]), 3.5, out)
    assert np.allclose(f64(out), [[1.5, 0.5]], atol=1e-6)


# ------------------------------------------------------------------ rotary + cache write
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("dh,style", [(16, "half"), (48, "interleaved"), (128, "half"), (256, "interleaved"),
                                      (32, "interleaved"), (128, "interleaved"), (64, "half"), (24, "half")])
@pytest.mark.parametrize("many", [False, True])
def test_rope_kv_write(dtype, dh, style, many):
    """many: enough tokens for the kernel that takes four tokens per workgroup: a run that
    crosses a page, a run that starts off a multiple of four, and a last group of two."""
    from transformer_amd import kernels
    nq, nkv, pages, theta = 3, 2, 5, 12345.0
    if many:
        pos = [60, 61, 62, 63, 64, 65, 66, 67, 5, 6, 7, 8, 1000, 1001]
        dest = [3 * 64 + 60 + i for i in range(4)] + [1 * 64 + i for i in range(4)] + \
               [4 * 64 + 5 + i for i in range(4)] + [0 * 64 + 40, 0 * 64 + 41]
    else:
        pos = [0, 1, 63, 64, 1000, 4095]
        dest = [3 * 64 + 0, 3 * 64 + 1, 3 * 64 + 63, 1 * 64 + 0, 4 * 64 + 40, 0 * 64 + 63]
    nt = len(pos)
    qkv = rounded(rng.normal(size=(nt, nq + 2 * nkv, dh)), dtype)
    bias = rng.normal(size=((nq + 2 * nkv), dh)).astype(np.float32) * 0.1
    inv = P.rope_inv_freq(dh, theta)
    for b in (None, bias):
        t = dev(qkv.reshape(nt, -1), DT[dtype])
        kc = torch.full((pages, nkv, 64, dh), float("nan"), dtype=DT[dtype], device=DEV)
        vc = torch.full((pages, nkv, dh, 64), float("nan"), dtype=DT[dtype], device=DEV)
        ang = kernels.rope_table(dev(pos, torch.int32), dev(inv), torch.empty(nt, dh // 2, 2, device=DEV))
        a64 = (np.asarray(pos, np.float32)[:, None] * inv[None, :]).astype(np.float64)
        assert np.abs(f64(ang)[..., 0] - np.cos(a64)).max() < 1e-6
        assert np.abs(f64(ang)[..., 1] - np.sin(a64)).max() < 1e-6
        kernels.rope_kv_write(t, nq, nkv, dh, ang, style == "interleaved",
                              dev(dest, torch.int32), kc, vc, None if b is None else dev(b.reshape(-1)))
        src = qkv + (0 if b is None else b[None].astype(np.float64))
        want_q = P.rope(src[:, :nq], pos, theta, style)
        want_k = P.rope(src[:, nq:nq + nkv], pos, theta, style)
        want_v = src[:, nq + nkv:]
        got = f64(t).reshape(nt, nq + 2 * nkv, dh)
        e = tol(dtype, 3)
        assert np.abs(got[:, :nq] - want_q).max() < e
        assert np.abs(got[:, nq:nq + nkv] - want_k).max() < e
        kcn, vcn = f64(kc), f64(vc).transpose(0, 1, 3, 2)          # value pages are [dh][64]
        for i, dst in enumerate(dest):
            assert np.abs(kcn[dst // 64, :, dst % 64] - want_k[i]).max() < e
            assert np.abs(vcn[dst // 64, :, dst % 64] - want_v[i]).max() < e
        written = np.zeros((pages, 64), dtype=bool)
        written[[d_ // 64 for d_ in dest], [d_ % 64 for d_ in dest]] = True
        rest_k, rest_v = kcn.transpose(0, 2, 1, 3)[~written], vcn.transpose(0, 2, 1, 3)[~written]
        assert np.isnan(rest_k).all() and np.isnan(rest_v).all()                # nothing else touched


def test_rope_without_rotation_only_stores():
    from transformer_amd import kernels
    qkv = rng.normal(size=(2, 4 * 16)).astype(np.float32)
    t = dev(qkv)
    kc = torch.zeros(1, 1, 64, 16, device=DEV)
    vc = torch.zeros(1, 1, 16, 64, device=DEV)
    kernels.rope_kv_write(t, 2, 1, 16, None, False, dev([5, 6], torch.int32), kc, vc)
    assert np.array_equal(f64(t), qkv.astype(np.float64))
    assert np.array_equal(f64(kc)[0, 0, 5], qkv[0, 32:48].astype(np.float64))


# ------------------------------------------------------------------ attention
def _attention_case(dtype, nh, nkv, dh, qlens, pos0, window=None, seed=0, sharp=None,
                    which="generic", slices=None, through_lds=None):
    """Builds a paged cache with shuffled pages, runs the kernel, returns (got, want)."""
    from transformer_amd import kernels
    r = np.random.default_rng(seed)
    B = len(qlens)
    total = [p + q for p, q in zip(pos0, qlens)]
    need = [-(-t // 64) for t in total]
    n_pages = sum(need) + 3
    order = r.permutation(n_pages)
    tables, k_all, v_all = [], [], []
    kc = np.full((n_pages, nkv, 64, dh), np.nan)
    vc = np.full((n_pages, nkv, 64, dh), np.nan)
    used = 0
    for b in range(B):
        pg = order[used:used + need[b]]
        used += need[b]
        tables.append(pg)
        k = rounded(r.normal(size=(total[b], nkv, dh)), dtype)
        v = rounded(r.normal(size=(total[b], nkv, dh)), dtype)
        k_all.append(k)
        v_all.append(v)
    nt = sum(qlens)
    q = rounded(r.normal(size=(nt, nh, dh)), dtype)
    if sharp is not None:                      # one far key gets a score that stands out
        b, qi, key, head = sharp
        g = head // (nh // nkv)
        row = sum(qlens[:b]) + qi
        k_all[b][key, g] = rounded(q[row, head] / np.linalg.norm(q[row, head]) * 40, dtype)
    for b in range(B):
        for p in range(total[b]):
            kc[tables[b][p // 64], :, p % 64] = k_all[b][p]
            vc[tables[b][p // 64], :, p % 64] = v_all[b][p]
    mb = max(need)
    table = np.zeros((B, mb), dtype=np.int32)
    for b in range(B):
        table[b, :need[b]] = tables[b]
    cu = np.concatenate([[0], np.cumsum(qlens)])
    scale = 1 / math.sqrt(dh)
    # q lives in a wider row, as in the engine's qkv buffer
    width = (nh + 2 * nkv) * dh
    qbuf = torch.zeros(nt, width, dtype=DT[dtype], device=DEV)
    qbuf[:, :nh * dh] = dev(q.reshape(nt, -1), DT[dtype])
    out = torch.full((nt, nh * dh), float("nan"), dtype=DT[dtype], device=DEV)
    args = (qbuf, out, dev(kc, DT[dtype]), dev(vc.transpose(0, 1, 3, 2), DT[dtype]), dev(table, torch.int32),
            dev(cu, torch.int32), dev(pos0, torch.int32))
    if which == "generic":
        kernels.attention_generic(*args, max(qlens), nh, nkv, dh, scale, window)
    elif which == "rows":
        kernels.attention_rows(*args, max(qlens), nh, nkv, dh, scale, window, through_lds)
    elif which == "keys":
        kernels.attention_keys(*args, max(total), nh, nkv, dh, scale, window, slices=slices)
    else:
        kernels.attention(*args, max(qlens), max(total), nh, nkv, dh, scale, window)
    want = np.concatenate([P.attention(q[cu[b]:cu[b + 1]], k_all[b], v_all[b], scale,
                                       first_pos=pos0[b], window=window) for b in range(B)])
    return f64(out).reshape(nt, nh, dh), want, (v_all, q)


ATT_SHAPES = [
    # nh, nkv, dh, qlens, pos0
    (4, 2, 16, [1, 7, 13], [0, 0, 0]),
    (3, 3, 32, [5, 2, 17, 9], [0, 0, 0, 0]),
    (10, 5, 48, [1, 1, 1], [130, 5, 63]),            # decode, unequal contexts
    (8, 1, 64, [3, 40], [64, 100]),                  # prompt continued after cached tokens
    (6, 2, 80, [70], [0]),
    (32, 8, 128, [1, 1], [700, 64]),
    (4, 4, 256, [33], [31]),
]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", ATT_SHAPES, ids=[f"h{s[0]}kv{s[1]}d{s[2]}" for s in ATT_SHAPES])
def test_attention_generic(dtype, shape):
    got, want, _ = _attention_case(dtype, *shape, seed=hash(shape[:3]) % 1000)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() < tol(dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_far_key_among_hundreds(dtype):
    # sequence 1, its only query, key 3 of 800, head 5: the output must be that key's value
    got, want, (v_all, q) = _attention_case(dtype, 8, 2, 64, [1, 1], [300, 799], seed=5,
                                            sharp=(1, 0, 3, 5))
    assert np.abs(got - want).max() < tol(dtype)
    assert np.abs(got[1, 5] - v_all[1][3, 1]).max() < 0.05


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("window", [1, 5, 64, 65])
def test_attention_window_edge(dtype, window):
    # the key just outside the window stands out: it must not be seen
    qlens, pos0 = [1, 20], [200, 100]
    got, want, _ = _attention_case(dtype, 4, 2, 32, qlens, pos0, window=window, seed=window,
                                   sharp=(0, 0, 200 - window, 1))
    assert np.abs(got - want).max() < tol(dtype)
    got2, want2, _ = _attention_case(dtype, 4, 2, 32, qlens, pos0, window=window, seed=window,
                                     sharp=(0, 0, 200 - window + 1, 1) if window > 1 else (0, 0, 200, 1))
    assert np.abs(got2 - want2).max() < tol(dtype)


MFMA_SHAPES = [
    # nh, nkv, dh, qlens, pos0
    (4, 2, 32, [1, 7, 13], [0, 0, 0]),
    (3, 3, 32, [5, 2, 17, 9], [0, 0, 0, 0]),
    (8, 1, 64, [3, 40], [64, 100]),
    (6, 2, 96, [70], [0]),
    (32, 8, 128, [200, 31], [0, 300]),
    (32, 8, 128, [1, 1], [700, 64]),               # single tokens through the prompt kernel
    (5, 5, 160, [66], [63]),
    (4, 4, 256, [33], [31]),
    (40, 1, 64, [9], [120]),                       # a group wider than one tile of rows
]


# 2: scores, softmax and output products overlap by half pages
@pytest.mark.parametrize("through_lds", [False, True, 2])
@pytest.mark.parametrize("shape", MFMA_SHAPES, ids=[f"h{s[0]}kv{s[1]}d{s[2]}q{max(s[3])}" for s in MFMA_SHAPES])
def test_attention_rows_on_matrix_cores(shape, through_lds):
    if through_lds == 2 and shape[2] > 128:
        from transformer_amd import kernels
        with pytest.raises(kernels.KernelError, match="head sizes up to 128"):
            _attention_case("bfloat16", *shape, seed=1, which="rows", through_lds=through_lds)
        return
    got, want, _ = _attention_case("bfloat16", *shape, seed=sum(shape[:3]), which="rows",
                                   through_lds=through_lds)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() < tol("bfloat16")


@pytest.mark.parametrize("through_lds", [True, 2])
@pytest.mark.parametrize("window", [None, 3, 64, 100, 1000])
def test_attention_rows_through_lds_long_prompts_and_windows(window, through_lds):
    # several workgroups per sequence, a prompt continued after 100 cached tokens, windows
    # that end inside a page, inside a workgroup's rows, and beyond everything
    got, want, (v_all, _) = _attention_case("bfloat16", 8, 2, 64, [300, 77], [0, 100], window=window,
                                            seed=7, which="rows", through_lds=through_lds)
    err = np.abs(got - want)
    bound = tol("bfloat16")
    if window is not None and window < 64:
        # An average of three values keeps the two roundings to 8 bits whole (of the probabilities
        # and of the output, each relative to the values averaged): a kernel that takes the
        # exponentials relative to the first keys' maximum rounds the largest probability too,
        # which one that takes them relative to the row's maximum does not. The mean shows
        # what is no rounding (a key too many, one too few).
        bound = 2.0 ** -8 * max(np.abs(v).max() for v in v_all)
        assert err.mean() < 1.2e-3
    assert err.max() < bound


@pytest.mark.parametrize("through_lds", [True, 2])
@pytest.mark.parametrize("window", [None, 200])
def test_attention_rows_through_lds_with_paired_row_blocks(window, through_lds):
    """Enough row blocks that a workgroup takes two of them (one from the end, one from the
    start): an even and an odd number of blocks, a prompt that continues after cached tokens."""
    # kernel 2 pairs from 1,024 blocks on: twice the tokens
    qlens = [2048, 1300, 100] if through_lds == 2 else [1024, 672, 100]
    got, want, _ = _attention_case("bfloat16", 32, 8, 32, qlens, [0, 130, 5], window=window,
                                   seed=12, which="rows", through_lds=through_lds)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() < tol("bfloat16")


@pytest.mark.parametrize("through_lds", [True, 2])
def test_attention_rows_headline_geometry(through_lds):
    """32 heads on 8 kv heads of 128: a prompt of one page, of two, one that ends on a page's
    last key, one that continues a long cached prefix, and enough rows for paired blocks."""
    got, want, _ = _attention_case("bfloat16", 32, 8, 128, [64, 65, 128, 40, 600], [0, 0, 0, 1000, 24],
                                   seed=21, which="rows", through_lds=through_lds)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() < tol("bfloat16")


def test_attention_rows_one_long_prompt_by_the_default_choice():
    """A prompt long enough that workgroups take two blocks of rows each (1,060 blocks on 8 kv
    heads), with a length that is no multiple of a page or of a block, continued after cached
    tokens; and one whose blocks fill the CUs exactly twice, so that the late half of the blocks
    is counted from the end and the early half from the start."""
    got, want, _ = _attention_case("bfloat16", 32, 8, 128, [4230], [70], seed=33, which="rows")
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() < tol("bfloat16")
    got, want, _ = _attention_case("bfloat16", 32, 8, 128, [2048], [0], seed=34, which="rows")
    assert np.abs(got - want).max() < tol("bfloat16")


KEYS_SHAPES = [
    # nh, nkv, dh, pos0 (one token each), slices (pages per slice, slices) or None
    (32, 8, 128, [700, 64, 0, 2047], None),
    (32, 8, 128, [700, 64, 0, 2047], (4, 8)),
    (32, 8, 128, [700, 64, 0, 2047], (5, 7)),
    (32, 8, 128, [700, 64, 0, 2047], (4, 8, 4)),
    (32, 8, 128, [700, 64, 0, 2047], (32, 1, 8)),
    (32, 8, 128, [700, 64, 0, 2047], (16, 2, 8)),
    (32, 8, 128, [700, 64, 0, 2047], (32, 1, 0)),           # a quarter of each page's keys per wave
    (32, 8, 128, [700, 64, 0, 2047], (3, 11, 0)),
    (6, 2, 64, [129, 5], (2, 2, 0)),
    (3, 3, 32, [300], (1, 5, 0)),
    (40, 1, 96, [333, 2], (2, 3, 0)),              # three chunks of 16 heads
    (64, 4, 192, [77, 1300], (5, 5, 0)),
    (3, 3, 32, [300, 68], (6, 1, 0)),
    (32, 8, 128, [700, 64, 0, 2047], (32, 1, 1)),           # every wave the whole page, 32 heads
    (32, 8, 128, [700, 64, 0, 2047], (3, 11, 1)),
    (6, 2, 64, [129, 5], (2, 2, 1)),
    (3, 3, 32, [300], (1, 5, 1)),
    (40, 1, 96, [333, 2], (2, 3, 1)),              # two chunks of 32 heads
    (32, 8, 128, [130], (40, 1)),
    (4, 2, 32, [63, 64, 65], (4, 1)),
    (3, 3, 64, [5, 300], (4, 2)),
    (8, 1, 96, [1000], (4, 4)),
    (40, 1, 64, [333, 2], (4, 2)),                 # two chunks of heads
    (2, 2, 256, [500], (4, 2)),
]


@pytest.mark.parametrize("shape", KEYS_SHAPES, ids=[f"h{s[0]}kv{s[1]}d{s[2]}s{s[4]}" for s in KEYS_SHAPES])
def test_attention_keys_on_matrix_cores(shape):
    nh, nkv, dh, pos0, slices = shape
    got, want, _ = _attention_case("bfloat16", nh, nkv, dh, [1] * len(pos0), pos0, seed=nh + dh,
                                   which="keys", slices=slices)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() < tol("bfloat16")


def test_single_token_attention_takes_groups_of_32_heads_of_128():
    """Which geometries the fused single-token kernels take is asked of the kernel that would
    serve them: 32 heads of 128 on one kv head go to the kernel that shares pages through LDS
    (the rule of the kernel for larger heads would have sent them to the prompt kernel)."""
    from transformer_amd import kernels
    assert kernels.keys_kernel_fits(32, 1, 128) and kernels.keys_kernel_fits(64, 2, 192)
    assert kernels.keys_kernel_fits(8, 8, 256) and not kernels.keys_kernel_fits(64, 2, 256)
    assert not kernels.keys_kernel_fits(4, 4, 48)
    got, want, _ = _attention_case("bfloat16", 32, 1, 128, [1, 1], [300, 70], seed=3, which="auto")
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() < tol("bfloat16")


@pytest.mark.parametrize("which", ["rows", "keys", "auto"])
def test_matrix_core_attention_far_key_and_window(which):
    got, want, (v_all, q) = _attention_case("bfloat16", 8, 2, 64, [1, 1], [300, 799], seed=5,
                                            sharp=(1, 0, 3, 5), which=which)
    assert np.abs(got - want).max() < tol("bfloat16")
    assert np.abs(got[1, 5] - v_all[1][3, 1]).max() < 0.05
    for window in (1, 5, 64, 65, 200):
        for key in (200 - window, 200 - window + 1):
            got, want, _ = _attention_case("bfloat16", 4, 2, 32, [1, 1], [200, 100], window=window,
                                           seed=window, sharp=(0, 0, min(key, 200), 1), which=which)
            assert np.abs(got - want).max() < tol("bfloat16"), (window, key)
    if which != "keys":
        for window in (3, 64, 100):
            got, want, _ = _attention_case("bfloat16", 4, 2, 32, [150, 20], [10, 100], window=window,
                                           seed=window, which=which)
            assert np.abs(got - want).max() < tol("bfloat16"), window


@pytest.mark.parametrize("style", ["half", "interleaved"])
@pytest.mark.parametrize("geometry", [(32, 8, 128), (6, 2, 64), (3, 3, 32), (40, 1, 64)])
def test_attention_keys_with_rotation_and_cache_write_fused(style, geometry):
    """The single-token kernel takes the raw [q | k | v] projection, adds the bias, rotates q
    and k, stores the new key and value and attends over them, in one launch."""
    from transformer_amd import kernels
    nh, nkv, dh = geometry
    r = np.random.default_rng(nh * dh)
    pos0 = [0, 63, 64, 700]                       # the new token opens a page, ends one, ...
    B, theta, scale = len(pos0), 50000.0, 1 / math.sqrt(dh)
    need = [p // 64 + 1 for p in pos0]
    n_pages = sum(need) + 2
    order = r.permutation(n_pages)
    kc = np.full((n_pages, nkv, 64, dh), np.nan)
    vc = np.full((n_pages, nkv, 64, dh), np.nan)
    table = np.zeros((B, max(need)), dtype=np.int32)
    raw = rounded(r.normal(size=(B, nh + 2 * nkv, dh)), "bfloat16")
    bias = (r.normal(size=(nh + 2 * nkv, dh)) * 0.1).astype(np.float32)
    inv = P.rope_inv_freq(dh, theta)
    want, dest, used, olds = [], [], 0, []
    for b, p in enumerate(pos0):
        pg = order[used:used + need[b]]
        used += need[b]
        table[b, :need[b]] = pg
        k_old = rounded(r.normal(size=(p, nkv, dh)), "bfloat16")
        v_old = rounded(r.normal(size=(p, nkv, dh)), "bfloat16")
        for t in range(p):
            kc[pg[t // 64], :, t % 64], vc[pg[t // 64], :, t % 64] = k_old[t], v_old[t]
        src = raw[b] + bias
        q = P.round_bf16(P.rope(src[None, :nh], [p], theta, style))
        k_new = P.round_bf16(P.rope(src[None, nh:nh + nkv], [p], theta, style))
        v_new = P.round_bf16(src[None, nh + nkv:])
        want.append(P.attention(q, np.concatenate([k_old, k_new]), np.concatenate([v_old, v_new]),
                                scale, first_pos=p)[0])
        dest.append(int(pg[p // 64]) * 64 + p % 64)
        olds.append((k_new[0], v_new[0]))
    ang = kernels.rope_table(dev(pos0, torch.int32), dev(inv), torch.empty(B, dh // 2, 2, device=DEV))
    kcd = dev(kc, torch.bfloat16)
    vcd = dev(vc.transpose(0, 1, 3, 2), torch.bfloat16)
    out = torch.full((B, nh * dh), float("nan"), dtype=torch.bfloat16, device=DEV)
    cu = dev(np.arange(B + 1), torch.int32)
    eight = (8 * 64 + 8 * min(nh // nkv, 32) * dh) * 4 <= 65536      # LDS of an 8-wave workgroup
    for slices in (None, (4, 3, 4), (2, 6, 8 if eight else 4), (2, 6, 0), (12, 1, 0), (5, 3, 0), (2, 6, 1), (12, 1, 1)):
        kernels.attention_keys(dev(raw.reshape(B, -1), torch.bfloat16), out, kcd, vcd,
                               dev(table, torch.int32), cu, dev(pos0, torch.int32), max(pos0) + 1,
                               nh, nkv, dh, scale, None, slices=slices, angles=ang,
                               interleaved=style == "interleaved", bias=dev(bias.reshape(-1)),
                               dest=dev(dest, torch.int32))
        got = f64(out).reshape(B, nh, dh)
        assert np.abs(got - np.stack(want)).max() < tol("bfloat16"), slices
        kn, vn = f64(kcd), f64(vcd).transpose(0, 1, 3, 2)
        for b, d_ in enumerate(dest):
            assert np.array_equal(kn[d_ // 64, :, d_ % 64], olds[b][0])      # the same bits as the
            assert np.array_equal(vn[d_ // 64, :, d_ % 64], olds[b][1])      # separate rotation kernel


def test_attention_refuses_sizes_it_cannot_take():
    from transformer_amd import kernels
    with pytest.raises(kernels.KernelError, match="multiple of 16"):
        _attention_case("float32", 2, 1, 24, [3], [0])
    with pytest.raises(kernels.KernelError, match="kv heads"):
        _attention_case("float32", 3, 2, 16, [3], [0])


# ------------------------------------------------------------------ SwiGLU
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("di", [301, 304, 2056])       # 8 | di: bfloat16 takes eight elements per thread
def test_swiglu(dtype, di):
    from transformer_amd import kernels
    nt = 5
    gu = rounded(rng.normal(size=(nt, 2 * di)) * 3, dtype)
    gu[0, :4] = [-200.0, 90.0, -30.0, 0.0]                # the exponential overflows, underflows, ...
    bias = rng.normal(size=2 * di).astype(np.float32)
    out = torch.empty(nt, di, dtype=DT[dtype], device=DEV)
    # one rounding of the result: half a unit in the last place, relative
    rel = 2.0 ** -8 if dtype == "bfloat16" else 2.0 ** -22
    kernels.swiglu(dev(gu, DT[dtype]), out)
    want = P.swiglu(gu[:, :di], gu[:, di:])
    assert (np.abs(f64(out) - want) <= rel * np.abs(want) + 1e-6).all()
    kernels.swiglu(dev(gu, DT[dtype]), out, dev(bias))
    want = P.swiglu(gu[:, :di] + bias[:di], gu[:, di:] + bias[di:])
    assert (np.abs(f64(out) - want) <= rel * np.abs(want) + 1e-5).all()


# ------------------------------------------------------------------ matrix product
@pytest.mark.parametrize("mnk", [(1, 5, 7), (3, 130, 97), (65, 64, 16), (70, 301, 1000)])
def test_gemm_simple(mnk):
    from transformer_amd import kernels
    M, N, K = mnk
    a, w = rng.normal(size=(M, K)).astype(np.float32), rng.normal(size=(N, K)).astype(np.float32)
    bias = rng.normal(size=N).astype(np.float32)
    out = torch.empty(M, N, device=DEV)
    kernels.gemm_simple(dev(a), dev(w), out, dev(bias))
    want = a.astype(np.float64) @ w.astype(np.float64).T + bias
    assert np.abs(f64(out) - want).max() < 1e-6 * K ** 0.5 * 8
    # a row gives the same bits alone and inside the batch
    one = torch.empty(1, N, device=DEV)
    kernels.gemm_simple(dev(a[M - 1:]), dev(w), one, dev(bias))
    assert torch.equal(one[0], out[M - 1])
    # bfloat16 inputs, float32 output
    ab, wb = P.round_bf16(a), P.round_bf16(w)
    o2 = torch.empty(M, N, device=DEV)
    kernels.gemm_simple(dev(ab, torch.bfloat16), dev(wb, torch.bfloat16), o2)
    assert np.abs(f64(o2) - ab @ wb.T).max() < 1e-6 * K ** 0.5 * 8


@pytest.mark.parametrize("mnk", [(1, 16, 128), (3, 130, 104), (8, 301, 1000), (16, 48, 4104), (5, 1000, 72),
                                 (8, 16 * 1024 + 5, 2048), (3, 16 * 2050, 1096), (16, 16 * 1030, 4096)])
@pytest.mark.parametrize("waves", [0, 4, 8, 16])
def test_gemm_few_rows(mnk, waves):
    """The matrix-core product for at most 16 rows: widths and depths that are no multiple
    of its tiles, every division of k among waves, float32 and bfloat16 output."""
    from transformer_amd import kernels
    M, N, K = mnk
    a, w = P.round_bf16(rng.normal(size=(M, K))), P.round_bf16(rng.normal(size=(N, K)))
    bias = rng.normal(size=N).astype(np.float32)
    want = a @ w.T
    out = torch.full((M, N), 7.0, device=DEV)
    kernels.gemm_skinny(dev(a, torch.bfloat16), dev(w, torch.bfloat16), out, waves=waves)
    assert np.abs(f64(out) - want).max() < 1e-5 * K ** 0.5 * 8
    kernels.gemm_skinny(dev(a, torch.bfloat16), dev(w, torch.bfloat16), out, bias=dev(bias), waves=waves)
    assert np.abs(f64(out) - want - bias).max() < 1e-5 * K ** 0.5 * 8
    ob = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    kernels.gemm_skinny(dev(a, torch.bfloat16), dev(w, torch.bfloat16), ob, waves=waves)
    assert (np.abs(f64(ob) - want) <= 2.0 ** -8 * np.abs(want) + 1e-4 * K ** 0.5).all()
    # a row gives the same bits alone and inside the batch
    one = torch.empty(1, N, device=DEV)
    kernels.gemm_skinny(dev(a[M - 1:], torch.bfloat16), dev(w, torch.bfloat16), one, bias=dev(bias), waves=waves)
    assert torch.equal(one[0], out[M - 1])


@pytest.mark.parametrize("mdk", [(7, 150, 328), (5, 8200, 256), (16, 8193, 2056)])
def test_gemm_few_rows_with_strides_and_swiglu(mdk):
    from transformer_amd import kernels
    M, di, K = mdk
    a, w = P.round_bf16(rng.normal(size=(M, K))), P.round_bf16(rng.normal(size=(2 * di, K)) * 0.2)
    bias = rng.normal(size=2 * di).astype(np.float32)
    # rows of a wider buffer on both sides
    abuf = torch.zeros(M, K + 24, dtype=torch.bfloat16, device=DEV)
    abuf[:, :K] = dev(a, torch.bfloat16)
    obuf = torch.full((M, di + 9), 5.0, dtype=torch.bfloat16, device=DEV)
    kernels.gemm_skinny(abuf[:, :K], dev(w, torch.bfloat16), obuf[:, :di], swiglu=True, bias=dev(bias))
    # the unfused path rounds the product to bfloat16 before bias and activation; the fused
    # one forms the same sums in the same order, so it must agree with that to one rounding
    gu_dev = torch.empty(M, 2 * di, dtype=torch.bfloat16, device=DEV)
    kernels.gemm_skinny(abuf[:, :K], dev(w, torch.bfloat16), gu_dev)
    assert (np.abs(f64(gu_dev) - a @ w.T) <= 2.0 ** -8 * np.abs(a @ w.T) + 1e-4 * K ** 0.5).all()
    gu = f64(gu_dev) + bias
    want = P.swiglu(gu[:, :di], gu[:, di:])
    assert (np.abs(f64(obuf[:, :di]) - want) <= 2.0 ** -8 * np.abs(want) + 1e-6).all()
    assert (obuf[:, di:] == 5.0).all()
    of = torch.empty(M, di, device=DEV)
    kernels.gemm_skinny(abuf[:, :K], dev(w, torch.bfloat16), of, swiglu=True)
    g = a @ w.T
    assert np.abs(f64(of) - P.swiglu(g[:, :di], g[:, di:])).max() < 1e-4 * K ** 0.5


@pytest.mark.parametrize("shape", [(1, 200, 72, 48), (5, 4096, 1096, 6144), (8, 4096, 14336, 5120 * 2),
                                   (16, 264, 4096, 96), (3, 1000, 256, 16 * 700)])
def test_gemm_few_rows_around_a_norm(shape):
    """One product adds its result to the residual stream and prepares the RMS norm behind it
    (rows times the norm's weight, sums of squares of 16 columns each); the next product
    applies the rows' factors. Together they must give what add, norm and product give one
    after the other; widths that are no multiple of 16, both kernels of the second product."""
    from transformer_amd import kernels
    M, d, K, N2 = shape
    eps = 3e-5
    a, w1 = P.round_bf16(rng.normal(size=(M, K))), P.round_bf16(rng.normal(size=(d, K)) * 0.1)
    x = rng.normal(size=(M, d)).astype(np.float32).astype(np.float64) * 3
    x[M - 1] *= 50                                             # rows of very different size
    nw = (1 + 0.3 * rng.normal(size=d)).astype(np.float32).astype(np.float64)
    bias = rng.normal(size=d).astype(np.float32).astype(np.float64)
    w2 = P.round_bf16(rng.normal(size=(N2, d)) * 0.1)
    xd = dev(x)
    h = torch.full((M, d), 7.0, dtype=torch.bfloat16, device=DEV)
    fold = kernels.NormFold(xd, dev(nw), eps, h, torch.full(kernels.NormFold.parts_shape(d), float("nan"), device=DEV))
    kernels.gemm_skinny(dev(a, torch.bfloat16), dev(w1, torch.bfloat16), None, bias=dev(bias), fold=fold)
    x_new = x + a @ w1.T + bias
    assert np.abs(f64(xd) - x_new).max() < 1e-5 * K ** 0.5 * 8 * 50
    x_new = f64(xd)                                            # what the kernel stored, to the bit
    assert (np.abs(f64(h) - x_new * nw) <= 2.0 ** -8 * np.abs(x_new * nw) + 1e-30).all()
    sums = f64(fold.parts)[:, :M].sum(0)
    assert np.abs(sums / (x_new ** 2).sum(1) - 1).max() < 1e-5
    # the product behind the norm: factor times the product of the unscaled rows
    rs = 1 / np.sqrt((x_new ** 2).mean(1) + eps)
    want = rs[:, None] * (f64(h) @ w2.T)
    out = torch.empty(M, N2, device=DEV)
    kernels.gemm_skinny(h, dev(w2, torch.bfloat16), out, scale=fold.scale())
    assert (np.abs(f64(out) - want) <= 1e-5 * np.abs(want) + 1e-5 * d ** 0.5 * rs[:, None] * np.abs(f64(h)).max(1)[:, None]).all()
    # and the same as norm-then-product up to the one rounding of the activations
    plain = P.round_bf16(P.rms_norm(x_new, nw, eps)) @ w2.T
    assert np.abs(f64(out) - plain).max() < 2.0 ** -7 * (np.abs(P.rms_norm(x_new, nw, eps)) @ np.abs(w2.T)).max()
    # with the activation (gate rows, then up rows)
    di = N2 // 2
    act = torch.empty(M, di, device=DEV)
    kernels.gemm_skinny(h, dev(w2, torch.bfloat16), act, swiglu=True, scale=fold.scale())
    assert np.abs(f64(act) - P.swiglu(want[:, :di], want[:, di:])).max() < 1e-4 * d ** 0.5
    # a row gives the same bits alone and inside the batch
    x1 = dev(x[M - 1:])
    h1 = torch.empty(1, d, dtype=torch.bfloat16, device=DEV)
    f1 = kernels.NormFold(x1, dev(nw), eps, h1, torch.zeros(kernels.NormFold.parts_shape(d), device=DEV))
    kernels.gemm_skinny(dev(a[M - 1:], torch.bfloat16), dev(w1, torch.bfloat16), None, bias=dev(bias), fold=f1)
    o1 = torch.empty(1, N2, device=DEV)
    kernels.gemm_skinny(h1, dev(w2, torch.bfloat16), o1, scale=f1.scale())
    assert torch.equal(x1[0], xd[M - 1]) and torch.equal(h1[0], h[M - 1]) and torch.equal(o1[0], out[M - 1])


@pytest.mark.parametrize("mnk", [(17, 200, 72), (33, 1000, 1096), (64, 4096, 4096), (9, 264, 4616), (48, 130, 520),
                                 (64, 72, 6152), (25, 8200, 256)])
def test_gemm_up_to_64_rows(mnk):
    """The matrix-core product for up to 64 rows: sizes that are no multiple of its tiles,
    every number of 16-row tiles, results in planes that add up when the weight has few
    column tiles, bfloat16 output, and the same bits for a row alone or inside a batch."""
    from transformer_amd import kernels
    M, N, K = mnk
    a, w = P.round_bf16(rng.normal(size=(M, K))), P.round_bf16(rng.normal(size=(N, K)))
    bias = rng.normal(size=N).astype(np.float32)
    want = a @ w.T + bias
    ad, wd = dev(a, torch.bfloat16), dev(w, torch.bfloat16)
    planes = kernels.mid_splits(wd)
    assert 1 <= planes <= 8 and (planes > 1) == (N <= 4096 and K >= 1024)
    out = torch.full((planes, M, N) if planes > 1 else (M, N), 7.0, device=DEV)
    kernels.gemm_mid(ad, wd, out, bias=dev(bias))
    got = f64(out).sum(0) if planes > 1 else f64(out)
    assert np.abs(got - want).max() < 1e-5 * K ** 0.5 * 8
    flat = torch.full((M, N), 7.0, device=DEV)                   # one plane is always allowed
    kernels.gemm_mid(ad, wd, flat, bias=dev(bias))
    assert np.abs(f64(flat) - want).max() < 1e-5 * K ** 0.5 * 8
    ob = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    kernels.gemm_mid(ad, wd, ob)
    assert (np.abs(f64(ob) - a @ w.T) <= 2.0 ** -8 * np.abs(a @ w.T) + 1e-4 * K ** 0.5).all()
    one = torch.empty((planes, 1, N) if planes > 1 else (1, N), device=DEV)
    kernels.gemm_mid(ad[M - 1:], wd, one, bias=dev(bias))
    assert torch.equal(one[..., 0, :], out[..., M - 1, :])
    # the planes are what the next norm adds to the residual stream, in order
    if planes > 1 and N % 4 == 0:
        x = rng.normal(size=(M, N)).astype(np.float32)
        nw = (1 + 0.1 * rng.normal(size=N)).astype(np.float32)
        xd, h = dev(x), torch.empty(M, N, device=DEV)
        kernels.add_rmsnorm(xd, dev(nw), 1e-5, h, out)
        assert np.abs(f64(xd) - (x + got)).max() < 1e-4 * K ** 0.5
        assert np.abs(f64(h) - P.rms_norm(x + got, nw.astype(np.float64), 1e-5)).max() < 1e-4
        rows = dev(np.array([M - 1, 0], dtype=np.int32), torch.int32)
        h2 = torch.empty(2, N, device=DEV)
        x2 = dev(x)
        kernels.add_rmsnorm(x2, dev(nw), 1e-5, h2, out, rows=rows)
        assert torch.equal(h2[0], h[M - 1]) and torch.equal(h2[1], h[0]) and torch.equal(x2, dev(x))


@pytest.mark.parametrize("mdk", [(40, 328, 520), (17, 40, 64), (33, 1000, 4096), (48, 72, 1096), (49, 200, 256),
                                 (64, 328, 520), (64, 96, 4096)])
def test_gemm_up_to_64_rows_with_activation(mdk):
    """Gate and up rows in one product with silu(gate) * up: both arrangements of the tiles
    (32 columns per workgroup up to 48 rows, 64 above), widths that end inside a tile, k that
    ends inside a chunk, both output types, and the same bits for a row alone or in the batch."""
    from transformer_amd import kernels
    M, di, K = mdk
    a, w = P.round_bf16(rng.normal(size=(M, K))), P.round_bf16(rng.normal(size=(2 * di, K)) * 0.2)
    bias = rng.normal(size=2 * di).astype(np.float32)
    ad, wd = dev(a, torch.bfloat16), dev(w, torch.bfloat16)
    of = torch.full((M, di), 7.0, device=DEV)
    kernels.gemm_mid(ad, wd, of, swiglu=True, bias=dev(bias))
    g = a @ w.T + bias
    assert np.abs(f64(of) - P.swiglu(g[:, :di], g[:, di:])).max() < 1e-4 * K ** 0.5
    ob = torch.full((M, di), 7.0, dtype=torch.bfloat16, device=DEV)
    kernels.gemm_mid(ad, wd, ob, swiglu=True)
    g = P.round_bf16(a @ w.T)                    # the unfused path stores the product in bfloat16
    want = P.swiglu(g[:, :di], g[:, di:])
    assert (np.abs(f64(ob) - want) <= 2.0 ** -7 * np.abs(want) + 2e-2).all()
    one = torch.empty(1, di, device=DEV)
    kernels.gemm_mid(ad[M - 1:], wd, one, swiglu=True, bias=dev(bias))
    assert torch.equal(one[0], of[M - 1])
    # rows that do not start on a 16-byte boundary of the output go out one by one
    wide = torch.full((M, di + 3), 7.0, device=DEV)
    kernels.gemm_mid(ad, wd, wide[:, 1:di + 1], swiglu=True, bias=dev(bias))
    assert torch.equal(wide[:, 1:di + 1], of) and (wide[:, 0] == 7).all() and (wide[:, di + 1:] == 7).all()


def test_gemm_up_to_64_rows_refusals():
    from transformer_amd import kernels
    w2 = torch.zeros(32, 64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(kernels.KernelError, match="outside"):
        kernels.gemm_mid(torch.zeros(65, 64, dtype=torch.bfloat16, device=DEV), w2, torch.empty(65, 32, device=DEV))
    with pytest.raises(kernels.KernelError, match="splits of 1 chunks"):
        kernels.gemm_mid(torch.zeros(20, 64, dtype=torch.bfloat16, device=DEV), w2,
                         torch.empty(2, 20, 32, device=DEV))         # more planes than chunks of k
    assert kernels.mid_takes(17, w2) and kernels.mid_takes(64, w2) and not kernels.mid_takes(65, w2)
    assert not kernels.mid_takes(8, w2) and not kernels.mid_takes(20, w2.float())


def test_gemm_few_rows_refuses_what_it_cannot_take():
    from transformer_amd import kernels
    w = torch.zeros(32, 64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(kernels.KernelError, match="outside"):
        kernels.gemm_skinny(torch.zeros(17, 64, dtype=torch.bfloat16, device=DEV), w,
                            torch.empty(17, 32, device=DEV))
    with pytest.raises(kernels.KernelError, match="multiples of 8"):
        kernels.gemm_skinny(torch.zeros(2, 60, dtype=torch.bfloat16, device=DEV),
                            torch.zeros(32, 60, dtype=torch.bfloat16, device=DEV),
                            torch.empty(2, 32, device=DEV))
    a = torch.zeros(2, 64, dtype=torch.bfloat16, device=DEV)
    assert kernels.skinny_wins(a, w) and not kernels.skinny_wins(a.float(), w.float())
    assert kernels.skinny_wins(torch.zeros(16, 64, dtype=torch.bfloat16, device=DEV), w)
    assert not kernels.skinny_wins(torch.zeros(17, 64, dtype=torch.bfloat16, device=DEV), w)


def test_library_product_for_bfloat16_matches():
    from transformer_amd.parts.linear import linear
    for M, N, K in ((1, 96, 160), (9, 1000, 304), (130, 256, 96)):
        a, w = P.round_bf16(rng.normal(size=(M, K))), P.round_bf16(rng.normal(size=(N, K)))
        for odt in (torch.float32, torch.bfloat16):
            out = torch.empty(M, N, dtype=odt, device=DEV)
            linear(dev(a, torch.bfloat16), dev(w, torch.bfloat16), out)
            lim = 1e-4 * K ** 0.5 if odt == torch.float32 else 0.02 * K ** 0.5
            assert np.abs(f64(out) - a @ w.T).max() < lim


# ------------------------------------------------------------------ sampling
def test_argmax_prefers_the_lowest_index_among_equals():
    from transformer_amd import kernels
    l = rng.normal(size=(4, 5000)).astype(np.float32)
    l[1, [4000, 17, 2999]] = 9.0
    l[2, :] = 0.0
    l[3, 4999] = 50.0
    out = torch.empty(4, dtype=torch.int32, device=DEV)
    kernels.argmax(dev(l), out)
    assert out.tolist() == [int(np.argmax(l[0])), 17, 0, 4999]


@pytest.mark.parametrize("vocab", [5003, 4097, 3])
def test_argmax_rows_that_are_not_aligned(vocab):
    """Odd widths: every other row starts off a 16-byte boundary, and the last elements fall
    outside the vector loads."""
    from transformer_amd import kernels
    l = rng.normal(size=(6, vocab)).astype(np.float32)
    l[1, vocab - 1] = 40.0                   # in the tail
    l[2, [vocab - 1, vocab - 2, 0]] = 41.0   # equal at both ends: the first wins
    l[3, vocab // 2] = 42.0
    l[4, :] = -np.inf
    l[4, vocab - 2] = -1e30
    out = torch.empty(6, dtype=torch.int32, device=DEV)
    kernels.argmax(dev(l), out)
    assert out.tolist() == [int(np.argmax(l[i])) for i in range(6)]


def _pick(p, u):
    cdf = np.cumsum(p)
    return int(np.searchsorted(cdf, u * cdf[-1], side="right"))


@pytest.mark.parametrize("vocab", [384, 5000, 128256])
def test_sample_follows_the_plain_distribution(vocab):
    from transformer_amd import kernels
    n = 64
    l = (rng.normal(size=(n, vocab)) * 2).astype(np.float32)
    u = rng.random(n).astype(np.float32)
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    for T, k, p_ in ((0.8, vocab, 1.0), (1.3, 40, 1.0), (0.7, vocab, 0.9), (1.0, 50, 0.5)):
        kernels.sample(dev(l), dev(u), out, T, k, p_)
        for i, t in enumerate(out.tolist()):
            p = P.sample_probabilities(l[i], T, top_p=p_, top_k=None if k == vocab else k)
            assert p[t] > 0, (T, k, p_, i)                     # never a token outside the kept set
            cdf = np.cumsum(p)
            lo, hi = cdf[t] - p[t], cdf[t]
            assert lo - 1e-4 <= u[i] <= hi + 1e-4, (T, k, p_, i, t, _pick(p, u[i]))


@pytest.mark.parametrize("vocab", [383, 5002, 128256])
def test_sample_rows_on_16_byte_boundaries_and_others_choose_alike(vocab):
    """Aligned rows take a kernel that reads sixteen bytes per lane, others one that reads
    single values; all sums are integer sums and ties go by index, so both choose the same
    token, also where the vocabulary is no multiple of four and where many values tie."""
    from transformer_amd import kernels
    n = 48
    l = (rng.normal(size=(n, vocab)) * 2).astype(np.float32)
    l[1] = np.round(l[1] * 2) / 2                              # many equal logits
    l[2, :] = 0.25
    l[3, :min(vocab, 900)] += 9.0                              # the likely tokens all in one wave's share of the row
    l[4] *= 6                                                  # a peaked row: few tokens carry the mass
    l[5] *= 0.05                                               # a flat row: thousands of tokens are kept
    u = dev(rng.random(n).astype(np.float32))
    ld = (vocab + 11) // 4 * 4
    aligned = torch.zeros(n, ld, device=DEV)[:, 4:4 + vocab]
    shifted = torch.zeros(n, ld, device=DEV)[:, 1:1 + vocab]
    aligned.copy_(dev(l)); shifted.copy_(dev(l))
    assert aligned.data_ptr() % 16 == 0 and shifted.data_ptr() % 16 != 0
    a = torch.empty(n, dtype=torch.int32, device=DEV)
    b = torch.empty(n, dtype=torch.int32, device=DEV)
    for T, k, p_ in ((0.8, vocab, 1.0), (1.3, 40, 1.0), (0.7, vocab, 0.9), (1.0, 50, 0.5), (1.0, 3, 1.0),
                     (0.3, 2000, 0.99), (1.0, 5000, 1.0), (2.0, vocab, 0.999)):
        kernels.sample(aligned, u, a, T, k, p_)
        kernels.sample(shifted, u, b, T, k, p_)
        assert torch.equal(a, b), (T, k, p_, (a != b).nonzero().flatten().tolist())


def test_sample_frequencies():
    from transformer_amd import kernels
    l = np.log(np.array([0.5, 0.25, 0.125, 0.0625, 0.0625], dtype=np.float64)).astype(np.float32)
    n = 20000
    u = rng.random(n).astype(np.float32)
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    kernels.sample(dev(np.tile(l, (n, 1))), dev(u), out, 1.0, 5, 1.0)
    freq = np.bincount(f64(out).astype(int), minlength=5) / n
    assert np.abs(freq - np.exp(l.astype(np.float64))).max() < 0.012
    kernels.sample(dev(np.tile(l, (n, 1))), dev(u), out, 1.0, 2, 1.0)       # top-2: 2/3, 1/3
    freq = np.bincount(f64(out).astype(int), minlength=5) / n
    assert np.abs(freq - [2 / 3, 1 / 3, 0, 0, 0]).max() < 0.012
    kernels.sample(dev(np.tile(l, (n, 1))), dev(u), out, 1.0, 5, 0.75)      # reaches 0.75 at token 1
    assert set(out.tolist()) == {0, 1}


def test_sample_ties_at_the_threshold_keep_the_lower_indices():
    from transformer_amd import kernels
    l = np.zeros((1, 1000), dtype=np.float32)
    l[0, 500] = 5.0
    n = 512
    u = np.linspace(0, 0.999, n).astype(np.float32)
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    kernels.sample(dev(np.tile(l, (n, 1))), dev(u), out, 1.0, 4, 1.0)       # 500 and the first three zeros
    assert set(out.tolist()) == {0, 1, 2, 500}


def test_fill_normal():
    from transformer_amd import kernels
    t = torch.empty(1 << 20, device=DEV)
    kernels.fill_normal(t, 3, 7, 1.0, 0.1)
    a = f64(t)
    assert abs(a.mean() - 1.0) < 1e-3 and abs(a.std() - 0.1) < 1e-3
    z = (a - 1.0) / 0.1
    assert abs((z ** 3).mean()) < 0.02 and abs((z ** 4).mean() - 3.0) < 0.05
    t2 = torch.empty(1 << 20, device=DEV)
    kernels.fill_normal(t2, 3, 7, 1.0, 0.1)
    assert torch.equal(t, t2)
    kernels.fill_normal(t2, 3, 8, 1.0, 0.1)
    assert abs(np.corrcoef(a, f64(t2))[0, 1]) < 0.01


def test_kernels_refuse_cpu_tensors():
    from transformer_amd import kernels
    with pytest.raises(kernels.KernelError, match="GPU only"):
        kernels.swiglu(torch.zeros(2, 4), torch.zeros(2, 2))


# ------------------------------------------------------------------ loading: conversion, staging
@pytest.mark.parametrize("src,dst", [("float16", "bfloat16"), ("float16", "float32"),
                                     ("float32", "bfloat16"), ("bfloat16", "float32"),
                                     ("float32", "float32")])
def test_convert(src, dst):
    from transformer_amd import kernels
    types = {"float16": torch.float16, "float32": torch.float32, "bfloat16": torch.bfloat16}
    n = 100003
    a = torch.tensor(rng.normal(size=n) * np.exp(rng.normal(size=n) * 3), dtype=torch.float32)
    a[:4] = torch.tensor([0.0, -0.0, 1.00390625, -3.0e-5])      # a tie for bfloat16 among them
    a = a.to(types[src])
    out = torch.empty(n, dtype=types[dst], device=DEV)
    kernels.convert(a.to(DEV), out)
    want = a.to(types[dst])
    assert torch.equal(out.cpu().view(torch.int16 if dst == "bfloat16" else torch.int32),
                       want.view(torch.int16 if dst == "bfloat16" else torch.int32))


@pytest.mark.parametrize("engine", ["float32", "bfloat16"])
def test_the_loader_brings_the_same_bits_to_the_gpu_as_to_the_host(engine, tmp_path):
    """Small staging buffers, so that every tensor crosses in several pieces; matrices stored
    as float16 (converted on the GPU), bfloat16 or float32; vectors stored as bfloat16."""
    import gpu_util as G
    from transformer_amd.api import open_model_source
    from transformer_amd.engine.params import declared_params
    from transformer_amd.weights.loader import load_parameters
    from transformer_amd.weights.safetensors_io import write_safetensors
    w = P.read_safetensors(G.folder("C", "float32") + "/model.safetensors")
    kinds = [torch.float16, torch.bfloat16, torch.float32]
    tensors = {}
    for i, (n, a) in enumerate(w.items()):
        t = torch.tensor(a, dtype=torch.float32)
        tensors[n] = t.to(kinds[i % 3]) if a.ndim == 2 else t.to(torch.bfloat16 if i % 2 else torch.float32)
    write_safetensors(tmp_path / "model.safetensors", tensors)
    (tmp_path / "config.json").write_text(open(G.folder("C", "float32") + "/config.json").read())
    arch, cfg, f = open_model_source(tmp_path)
    params = declared_params(arch.model_spec(cfg))
    src = arch.weight_sources(cfg, f.format)
    host = load_parameters(params, src, f, DT[engine], "cpu")
    gpu = load_parameters(params, src, f, DT[engine], DEV, chunk_bytes=4096)
    assert len({t.untyped_storage().data_ptr() for t in gpu.values()}) == 1
    for n in host:
        assert gpu[n].dtype == host[n].dtype and gpu[n].data_ptr() % 256 == 0
        assert torch.equal(gpu[n].cpu().float(), host[n].float()), n


def test_read_probe_reads_and_writes_nothing():
    """The bandwidth probe of the bench: any buffer that is a multiple of 16 bytes, any number of
    workgroups; it leaves its sink alone and refuses what it cannot read."""
    from transformer_amd import kernels
    buf = torch.arange(3 * 1024 * 1024 + 4, dtype=torch.int32, device=DEV)
    sink = torch.full((256,), 7, dtype=torch.int32, device=DEV)
    for wgs in (1, 7, 256, 2048):
        kernels.read_probe(buf, wgs, sink)
    torch.cuda.synchronize()
    assert (sink == 7).all()
    with pytest.raises(kernels.KernelError, match="bytes"):
        kernels.read_probe(buf[:3], 4, sink)                      # 12 bytes
    with pytest.raises(kernels.KernelError, match="sink"):
        kernels.read_probe(buf, 4, sink[:8])
