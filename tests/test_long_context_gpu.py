"""The lengths that the measurements quote, against the plain attention: single tokens over
8 k, 16 k, 33 k and 131 k cached keys (hundreds to thousands of pages per sequence, cut by the planner into many
units of work and merged), prompts of 8,192 and 16,384 rows (workgroups that take a block of
rows from the end and one from the start), planted stand-out keys for the prompt kernel whose
softmax reference moves in steps, and an engine run that decodes past 4,096 cached tokens.
The key range is that of models/llama/common/src/compute.rs:243-264 (keys 0..pos+seq)."""
import math

import numpy as np
import pytest
import torch

import gpu_util as G
import plain_llama as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 1.2e-2            # bfloat16 attention outputs of order 1, as in the other kernel tests


def dev(a, dtype=torch.float32):
    return torch.tensor(np.ascontiguousarray(a), dtype=dtype, device=DEV).contiguous()


def f64(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


def paged(r, totals, nkv, dh, spare=3):
    """Keys and values of sequences of ``totals`` tokens in shuffled pages: (k_all, v_all, key
    cache [pages, nkv, 64, dh], value cache (not yet transposed), table)."""
    need = [-(-t // 64) for t in totals]
    n_pages = sum(need) + spare
    order = r.permutation(n_pages)
    kc = np.full((n_pages, nkv, 64, dh), np.nan, dtype=np.float32)
    vc = np.full((n_pages, nkv, 64, dh), np.nan, dtype=np.float32)
    table = np.zeros((len(totals), max(need)), dtype=np.int32)
    k_all, v_all, used = [], [], 0
    for b, t in enumerate(totals):
        pg = order[used:used + need[b]]
        used += need[b]
        table[b, :need[b]] = pg
        k = P.round_bf16(r.normal(size=(t, nkv, dh)).astype(np.float32))
        v = P.round_bf16(r.normal(size=(t, nkv, dh)).astype(np.float32))
        k_all.append(k)
        v_all.append(v)
    return k_all, v_all, kc, vc, table, need


def store(kc, vc, table, k_all, v_all):
    for b, (k, v) in enumerate(zip(k_all, v_all)):
        t = k.shape[0]
        full, rest = divmod(t, 64)
        pg = table[b]
        if full:
            kc[pg[:full]] = k[:full * 64].reshape(full, 64, *k.shape[1:]).transpose(0, 2, 1, 3)
            vc[pg[:full]] = v[:full * 64].reshape(full, 64, *v.shape[1:]).transpose(0, 2, 1, 3)
        if rest:
            kc[pg[full], :, :rest] = k[full * 64:].transpose(1, 0, 2)
            vc[pg[full], :, :rest] = v[full * 64:].transpose(1, 0, 2)


# ------------------------------------------------------------------ single tokens over long caches
KEYS_CASES = [
    # nh, nkv, dh, cached tokens of each sequence, far key (sequence, key, head) or None
    (32, 8, 128, [8191], None),
    (32, 8, 128, [16500], (0, 5, 17)),
    (32, 8, 128, [33000], (0, 32999 - 64, 30)),
    (8, 2, 128, [33011, 100, 8192, 16383, 4096, 63, 20000], (0, 1, 6)),     # a batch of unequal lengths
    (12, 4, 96, [9000, 24000], (1, 23000, 2)),
    (40, 2, 64, [12000, 700], None),                                      # 20 heads per kv head
    (8, 2, 128, [131071], (0, 77, 5)),                                    # 2,048 pages in one sequence
]


@pytest.mark.parametrize("case", KEYS_CASES, ids=[f"h{c[0]}kv{c[1]}d{c[2]}n{max(c[3])}b{len(c[3])}" for c in KEYS_CASES])
def test_single_token_attention_over_long_caches(case):
    """The units of work are the planner's own (``plan_key_units`` with the count of the batch
    size), pages are shuffled, and where a far key is planted its value has to come out."""
    from transformer_amd import kernels
    nh, nkv, dh, pos0, far = case
    r = np.random.default_rng(sum(pos0) + nh)
    B = len(pos0)
    totals = [p + 1 for p in pos0]
    k_all, v_all, kc, vc, table, need = paged(r, totals, nkv, dh)
    q = P.round_bf16(r.normal(size=(B, nh, dh)))
    if far is not None:
        b, key, head = far
        k_all[b][key, head // (nh // nkv)] = P.round_bf16(q[b, head] / np.linalg.norm(q[b, head]) * 40)
    store(kc, vc, table, k_all, v_all)
    n_units = kernels.key_unit_count(B, nkv)
    units, seq_units = kernels.plan_key_units(totals, n_units, tables=table)
    assert seq_units[:, 1].max() >= 16                       # the longest sequence is cut into many units
    scale = 1 / math.sqrt(dh)
    qbuf = torch.zeros(B, (nh + 2 * nkv) * dh, dtype=torch.bfloat16, device=DEV)
    qbuf[:, :nh * dh] = dev(q.reshape(B, -1), torch.bfloat16)
    out = torch.full((B, nh * dh), float("nan"), dtype=torch.bfloat16, device=DEV)
    kernels.attention_keys(qbuf, out, dev(kc, torch.bfloat16), dev(vc.transpose(0, 1, 3, 2), torch.bfloat16),
                           dev(table, torch.int32), dev(np.arange(B + 1), torch.int32), dev(pos0, torch.int32),
                           max(totals), nh, nkv, dh, scale, None,
                           units=dev(units, torch.int32), seq_units=dev(seq_units, torch.int32))
    got = f64(out).reshape(B, nh, dh)
    want = np.concatenate([P.attention(q[b:b + 1], k_all[b], v_all[b], scale, first_pos=pos0[b]) for b in range(B)])
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() < TOL
    if far is not None:
        b, key, head = far
        assert np.abs(got[b, head] - v_all[b][key, head // (nh // nkv)]).max() < 0.05


# ------------------------------------------------------------------ long prompts
def sampled_rows(qlen, r, extra=()):
    """Rows to check of a long prompt: its ends, the rows around every 1,024th, and random ones."""
    rows = {0, 1, 31, 32, 63, 64, 127, 128, qlen - 1, qlen - 2, qlen - 33, qlen - 129, *extra}
    for edge in range(1024, qlen, 1024):
        rows.update((edge - 1, edge))
    rows.update(int(x) for x in r.integers(0, qlen, 48))
    return sorted(x for x in rows if 0 <= x < qlen)


ROWS_CASES = [
    # nh, nkv, dh, rows of each prompt, cached tokens before them
    (16, 4, 128, [8192], [0]),           # 1,024 blocks of 128 rows: a workgroup takes two
    (8, 2, 128, [16384], [0]),
    (8, 2, 128, [9000, 300], [130, 5]),  # an odd count of blocks, continued after cached tokens
    (8, 8, 64, [8200], [0]),
    (4, 1, 128, [40000], [17]),          # 1,250 blocks on one kv head
]


@pytest.mark.parametrize("case", ROWS_CASES, ids=[f"h{c[0]}kv{c[1]}d{c[2]}q{max(c[3])}" for c in ROWS_CASES])
def test_prompt_attention_at_8k_and_16k_rows(case):
    """``attn_rows_halves`` (the default choice at these sizes) at lengths where workgroups pair
    a late block of rows with an early one. Checked on sampled rows of every prompt, every
    head, against the plain attention over all keys the row sees."""
    from transformer_amd import kernels
    nh, nkv, dh, qlens, pos0 = case
    r = np.random.default_rng(sum(qlens) + nh)
    B = len(qlens)
    totals = [p + n for p, n in zip(pos0, qlens)]
    k_all, v_all, kc, vc, table, need = paged(r, totals, nkv, dh)
    store(kc, vc, table, k_all, v_all)
    nt = sum(qlens)
    q = P.round_bf16(r.normal(size=(nt, nh, dh)).astype(np.float32))
    cu = np.concatenate([[0], np.cumsum(qlens)])
    scale = 1 / math.sqrt(dh)
    assert kernels.rows_kernel(max(qlens), nh, nkv, dh) == 2
    qbuf = torch.zeros(nt, (nh + 2 * nkv) * dh, dtype=torch.bfloat16, device=DEV)
    qbuf[:, :nh * dh] = dev(q.reshape(nt, -1), torch.bfloat16)
    out = torch.full((nt, nh * dh), float("nan"), dtype=torch.bfloat16, device=DEV)
    kernels.attention_rows(qbuf, out, dev(kc, torch.bfloat16), dev(vc.transpose(0, 1, 3, 2), torch.bfloat16),
                           dev(table, torch.int32), dev(cu, torch.int32), dev(pos0, torch.int32),
                           max(qlens), nh, nkv, dh, scale, None)
    got = f64(out).reshape(nt, nh, dh)
    assert np.isfinite(got).all()                       # every row was written
    worst = 0.0
    for b in range(B):
        for row in sampled_rows(qlens[b], r):
            p = pos0[b] + row
            want = P.attention(q[cu[b] + row:cu[b] + row + 1], k_all[b][:p + 1], v_all[b][:p + 1], scale, first_pos=p)
            worst = max(worst, np.abs(got[cu[b] + row] - want[0]).max())
    assert worst < TOL


@pytest.mark.parametrize("rise", [3.0, 12.0])
def test_prompt_attention_with_stand_out_keys_and_a_rising_maximum(rise):
    """``attn_rows_halves`` moves the reference of its exponentials only when a half page's
    maximum lies more than 8 (in powers of two) above it. A prompt of 400 tokens after a cached
    prefix: one query has a stand-out key in the first page, whose value must come out; another
    meets keys whose scores rise from half page to half page by ``rise`` (below and above 8),
    so that the reference stays behind or moves with every half page."""
    from transformer_amd import kernels
    nh, nkv, dh, qlen, p0 = 8, 2, 128, 400, 200
    r = np.random.default_rng(int(rise))
    total = p0 + qlen
    k_all, v_all, kc, vc, table, need = paged(r, [total], nkv, dh)
    q = P.round_bf16(r.normal(size=(qlen, nh, dh)))
    scale = 1 / math.sqrt(dh)
    # query row 350 (position 550), head 5: key 7 stands out
    far_row, far_head, far_key = 350, 5, 7
    k_all[0][far_key, far_head // 4] = P.round_bf16(q[far_row, far_head] / np.linalg.norm(q[far_row, far_head]) * 40)
    # query row 399, head 2: the key in the middle of every half page scores `rise` (log2) more
    # than that of the half page before
    step_row, step_head = 399, 2
    unit = q[step_row, step_head] / np.linalg.norm(q[step_row, step_head]) ** 2
    for i, key in enumerate(range(16, total, 32)):
        k_all[0][key, step_head // 4] = P.round_bf16(unit * (i * rise * math.log(2.0) / scale))
    store(kc, vc, table, k_all, v_all)
    qbuf = torch.zeros(qlen, (nh + 2 * nkv) * dh, dtype=torch.bfloat16, device=DEV)
    qbuf[:, :nh * dh] = dev(q.reshape(qlen, -1), torch.bfloat16)
    out = torch.full((qlen, nh * dh), float("nan"), dtype=torch.bfloat16, device=DEV)
    kernels.attention_rows(qbuf, out, dev(kc, torch.bfloat16), dev(vc.transpose(0, 1, 3, 2), torch.bfloat16),
                           dev(table, torch.int32), dev([0, qlen], torch.int32), dev([p0], torch.int32),
                           qlen, nh, nkv, dh, scale, None, through_lds=2)
    got = f64(out).reshape(qlen, nh, dh)
    want = P.attention(q, k_all[0], v_all[0], scale, first_pos=p0)
    # the planted keys have large norms, so many rows of their kv head are all but one value,
    # of a size up to 4: the bound is relative to the output where that exceeds 1
    assert (np.abs(got - want) < TOL * np.maximum(1.0, np.abs(want))).all()
    assert np.abs(got[far_row, far_head] - v_all[0][far_key, far_head // 4]).max() < 0.05


# ------------------------------------------------------------------ the engine past 4,096 cached tokens
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_engine_decodes_past_4096_cached_tokens(dtype, tmp_path):
    """Tiny D with its position limit raised: a prompt of 4,090 tokens, then 40 single tokens
    (the recorded step's page table grows past 4,096 tokens on the way and is recorded again),
    beside a short sequence in the same batch. Every logit of the decoded tokens and the
    prompt's last against the plain model over the whole sequence."""
    import transformer_amd as ta
    from transformer_amd import Entry
    cfg = dict(G.TINY_D, max_position_embeddings=8192)
    folder = tmp_path / "long"
    P.make_model_folder(str(folder), cfg, 3, storage=G.MODES[dtype])
    model = ta.load_model(str(folder), dtype, DEV)
    ref = P.PlainLlama(str(folder))
    r = np.random.default_rng(4)
    long_ = [int(t) for t in r.integers(0, cfg["vocab_size"], 4130)]
    short = [int(t) for t in r.integers(0, cfg["vocab_size"], 60)]
    cache = model.new_cache(4224 + 128, max_slots=2)
    G.poison(cache)
    a, b = cache.alloc_slot(), cache.alloc_slot()
    got_a = [f64(model.step(cache, [Entry(a, long_[:4090], [4089]), Entry(b, short[:20], [])]))]
    got_b = []
    for i in range(40):
        out = f64(model.step(cache, [Entry(a, [long_[4090 + i]], [0]), Entry(b, [short[20 + i]], [0])]))
        got_a.append(out[:1])
        got_b.append(out[1:])
    assert sorted({k[2] for k in cache.graphs}) == [64, 128]            # table widths, in pages
    want_a = ref.forward(long_)[4089:]
    want_b = ref.forward(short)[20:]
    assert np.abs(np.concatenate(got_a) - want_a).max() < G.TOL[dtype]
    assert np.abs(np.concatenate(got_b) - want_b).max() < G.TOL[dtype]
