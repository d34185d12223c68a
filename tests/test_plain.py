"""Pins the plain implementation by what fixes it beside the reference's text:
special cases that reduce to a library routine, explicit small vectors, and
invariants, each chosen so that a plausible mistake fails it.

The reference holds no numeric vectors for the model (its only asserting test
compares two chat-template strings, gguf/src/chat_template.rs:104-134),
so none can be replayed here: parity with the reference's external operators is
unpinned beyond these checks.
"""
import math

import numpy as np
import pytest
import torch

import plain_llama as P

rng = np.random.default_rng(1234)


# ---------------------------------------------------------------- RMS norm
def test_rms_norm_unit_mean_square():
    x = rng.normal(size=(5, 48)) * 3
    y = P.rms_norm(x, np.ones(48), 0.0)
    assert np.allclose((y * y).mean(-1), 1.0, atol=1e-12)


def test_rms_norm_formula_and_eps_inside_sqrt():
    x = np.array([[3.0, 4.0]])
    # mean square 12.5; eps inside the root (a norm with eps outside would give 5/(sqrt(12.5)+eps))
    y = P.rms_norm(x, np.array([2.0, 0.5]), 3.5)
    assert np.allclose(y, np.array([[3.0 / 4.0 * 2.0, 4.0 / 4.0 * 0.5]]))


def test_rms_norm_is_not_layer_norm():
    x = np.array([[1.0, 1.0, 1.0, 1.0]])          # a mean-subtracting norm would give 0
    assert np.allclose(P.rms_norm(x, np.ones(4), 0.0), 1.0)


def test_rms_norm_scale_invariance():
    x = rng.normal(size=(3, 32))
    w = rng.normal(size=32)
    assert np.allclose(P.rms_norm(7.5 * x, w, 0.0), P.rms_norm(x, w, 0.0))


# ---------------------------------------------------------------- linear
def test_linear_is_x_times_w_transposed():
    x = rng.normal(size=(4, 6))
    w = rng.normal(size=(5, 6))
    b = rng.normal(size=5)
    want = torch.nn.functional.linear(torch.tensor(x), torch.tensor(w), torch.tensor(b)).numpy()
    assert np.allclose(P.linear(x, w, b), want)


# ---------------------------------------------------------------- rotary
def test_rope_position_zero_is_identity():
    t = rng.normal(size=(1, 2, 16))
    for style in ("half", "interleaved"):
        assert np.allclose(P.rope(t, [0], 10000.0, style), t)


def test_rope_explicit_vector_sign_and_pairing():
    # head size 4, theta 100: f = [1, 100^(-1/2)] = [1, 0.1]; position 2
    t = np.array([[[1.0, 0.0, 0.0, 1.0]]])
    a0, a1 = 2.0 * 1.0, np.float32(2.0) * np.float32(0.1)
    # half: pairs (t0, t2) and (t1, t3)
    h = P.rope(t, [2], 100.0, "half")[0, 0]
    assert np.allclose(h, [math.cos(a0), -math.sin(a1), math.sin(a0), math.cos(a1)], atol=1e-7)
    # interleaved: pairs (t0, t1) and (t2, t3)
    i = P.rope(t, [2], 100.0, "interleaved")[0, 0]
    assert np.allclose(i, [math.cos(a0), math.sin(a0), -math.sin(a1), math.cos(a1)], atol=1e-7)


def test_rope_is_complex_multiplication():
    dh = 8
    t = rng.normal(size=(3, 2, dh))
    pos = [5, 17, 40]
    f = P.rope_inv_freq(dh, 500000.0).astype(np.float64)
    z = t[..., 0::2] + 1j * t[..., 1::2]
    ang = np.asarray(pos, dtype=np.float32)[:, None] * f.astype(np.float32)[None, :]
    zr = z * np.exp(1j * ang.astype(np.float64))[:, None, :]
    out = P.rope(t, pos, 500000.0, "interleaved")
    assert np.allclose(out[..., 0::2], zr.real) and np.allclose(out[..., 1::2], zr.imag)


def test_rope_preserves_norm_and_composes():
    t = rng.normal(size=(1, 1, 32))
    a = P.rope(t, [9], 10000.0, "half")
    assert np.allclose(np.linalg.norm(a), np.linalg.norm(t))
    # R(3) R(4) = R(7) up to the float32 rounding of the angles
    b = P.rope(P.rope(t, [3], 10000.0, "half"), [4], 10000.0, "half")
    c = P.rope(t, [7], 10000.0, "half")
    assert np.allclose(b, c, atol=1e-5)


def test_rope_scores_depend_on_distance_only():
    q = rng.normal(size=(1, 1, 16))
    k = rng.normal(size=(1, 1, 16))
    for style in ("half", "interleaved"):
        s = [float((P.rope(q, [m], 1e4, style) * P.rope(k, [n], 1e4, style)).sum())
             for m, n in ((5, 2), (105, 102), (40, 37))]
        assert np.allclose(s, s[0], atol=1e-4)
        other = float((P.rope(q, [5], 1e4, style) * P.rope(k, [3], 1e4, style)).sum())
        assert abs(other - s[0]) > 1e-3


def test_rope_styles_are_related_by_a_permutation():
    dh = 16
    t = rng.normal(size=(4, 3, dh))
    pos = [0, 3, 7, 11]
    perm = np.concatenate([np.arange(0, dh, 2), np.arange(1, dh, 2)])   # interleaved -> half order
    a = P.rope(t, pos, 1e4, "interleaved")[..., perm]
    b = P.rope(t[..., perm], pos, 1e4, "half")
    assert np.allclose(a, b)


# ---------------------------------------------------------------- attention
def _sdpa(q, k, v, scale, causal):
    tq, tk, tv = (torch.tensor(a).transpose(0, 1) for a in (q, k, v))     # [heads, T, dh]
    o = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, is_causal=causal, scale=scale)
    return o.transpose(0, 1).numpy()


def test_attention_matches_library_routine_causal_mha():
    T, nh, dh = 9, 3, 8
    q, k, v = (rng.normal(size=(T, nh, dh)) for _ in range(3))
    assert np.allclose(P.attention(q, k, v, 1 / math.sqrt(dh)), _sdpa(q, k, v, 1 / math.sqrt(dh), True))


def test_attention_one_head_one_query_is_plain_softmax_average():
    S, dh = 6, 4
    q = rng.normal(size=(1, 1, dh))
    k, v = rng.normal(size=(S, 1, dh)), rng.normal(size=(S, 1, dh))
    s = (k[:, 0] @ q[0, 0]) * 0.5
    p = np.exp(s - s.max())
    p /= p.sum()
    assert np.allclose(P.attention(q, k, v, 0.5, first_pos=S - 1)[0, 0], p @ v[:, 0])


def test_attention_first_token_returns_its_value():
    q, k, v = (rng.normal(size=(1, 2, 8)) for _ in range(3))
    assert np.allclose(P.attention(q, k, v, 0.3), v)


def test_attention_gqa_equals_mha_with_repeated_kv_heads():
    T, nh, nkv, dh = 7, 6, 2, 8
    q = rng.normal(size=(T, nh, dh))
    k, v = rng.normal(size=(T, nkv, dh)), rng.normal(size=(T, nkv, dh))
    rep = np.repeat(k, nh // nkv, axis=1), np.repeat(v, nh // nkv, axis=1)
    assert np.allclose(P.attention(q, k, v, 0.35), _sdpa(q, rep[0], rep[1], 0.35, True))
    # head h reads kv head h // group, not h % nkv
    wrong = np.tile(k, (1, nh // nkv, 1)), np.tile(v, (1, nh // nkv, 1))
    assert not np.allclose(P.attention(q, k, v, 0.35), _sdpa(q, wrong[0], wrong[1], 0.35, True))


def test_attention_offset_queries_see_all_earlier_keys():
    S, T, dh = 10, 3, 8
    q = rng.normal(size=(S, 2, dh))
    k, v = rng.normal(size=(S, 2, dh)), rng.normal(size=(S, 2, dh))
    whole = P.attention(q, k, v, 0.4)
    tail = P.attention(q[S - T:], k, v, 0.4, first_pos=S - T)
    assert np.allclose(tail, whole[S - T:])


def test_attention_window():
    S, dh, w = 12, 4, 3
    q, k, v = (rng.normal(size=(S, 1, dh)) for _ in range(3))
    out = P.attention(q, k, v, 0.5, window=w)
    for t in (0, 5, 11):
        lo = max(0, t - w + 1)
        ref = P.attention(q[t:t + 1], k[lo:t + 1], v[lo:t + 1], 0.5, first_pos=t - lo)
        assert np.allclose(out[t], ref[0])


# ---------------------------------------------------------------- SwiGLU
def test_swiglu_matches_library_silu():
    g, u = rng.normal(size=(4, 9)) * 4, rng.normal(size=(4, 9))
    want = (torch.nn.functional.silu(torch.tensor(g)) * torch.tensor(u)).numpy()
    assert np.allclose(P.swiglu(g, u), want)
    assert np.all(P.swiglu(np.zeros(3), np.ones(3)) == 0)
    assert np.allclose(P.swiglu(np.array([30.0]), np.array([2.0])), 60.0)        # silu(z) -> z
    assert np.allclose(P.swiglu(np.array([-30.0]), np.array([2.0])), 0.0, atol=1e-10)


# ---------------------------------------------------------------- whole model
@pytest.fixture(scope="module")
def tiny(tmp_path_factory):
    out = {}
    for name, cfg, seed in (("A", P.TINY_A, 0), ("B", P.TINY_B, 1)):
        d = tmp_path_factory.mktemp(f"plain_{name}")
        P.make_model_folder(d, cfg, seed)
        out[name] = P.PlainLlama(d)
    return out


def test_model_is_causal(tiny):
    for m in tiny.values():
        a = [int(t) for t in rng.integers(0, m.vocab, 12)]
        b = a[:7] + [int(t) for t in rng.integers(0, m.vocab, 5)]
        la, lb = m.forward(a), m.forward(b)
        assert np.allclose(la[:7], lb[:7], atol=1e-12)
        assert not np.allclose(la[7:], lb[7:], atol=1e-6)


def _one_layer(tmp_path, edit=None, **over):
    cfg = {**P.TINY_A, "num_hidden_layers": 1, **over}
    P.make_model_folder(tmp_path, cfg, 9, edit=edit)
    return P.PlainLlama(tmp_path)


def test_position_enters_through_the_rotation_only(tmp_path):
    """One layer: the last token's attention is a weighted sum over the set of earlier
    tokens, so without rotation (all positions equal) swapping two earlier tokens leaves its
    output unchanged; with the real positions it changes. A second source of position
    (a position added to the embedding, a mask that is not causal-by-index) would break the
    first half, a missing rotation the second."""
    m = _one_layer(tmp_path)
    E = m.w["model.embed_tokens.weight"]
    a, b = [5, 9, 200, 31, 77], [9, 5, 200, 31, 77]
    flat = np.zeros(5, dtype=np.int64)
    assert np.allclose(m.block(0, E[a], flat)[-1], m.block(0, E[b], flat)[-1], atol=1e-12)
    real = np.arange(5)
    assert np.abs(m.block(0, E[a], real)[-1] - m.block(0, E[b], real)[-1]).max() > 1e-6


def test_default_scale_is_the_library_routines_default(tmp_path):
    """The model passes no scale to its attention (compute.rs:511-526 has no such argument):
    the constant 1/sqrt(head size) of ``PlainLlama.scale`` is the library routine's own
    default (scale=None), for a head size that differs from hidden / heads."""
    m = _one_layer(tmp_path, head_dim=24, num_attention_heads=3, num_key_value_heads=3)
    T = 6
    q, k, v = (rng.normal(size=(T, m.nh, m.dh)) for _ in range(3))
    assert m.dh == 24 and m.d // m.nh != m.dh
    assert np.allclose(P.attention(q, k, v, m.scale), _sdpa(q, k, v, None, True))
    assert not np.allclose(P.attention(q, k, v, 1 / math.sqrt(m.d // m.nh)), _sdpa(q, k, v, None, True))


def _without(suffixes):
    def edit(w):
        for n in w:
            if any(n.endswith(s) for s in suffixes):
                w[n][:] = 0
    return edit


@pytest.mark.parametrize("silenced,alive", [(("down_proj.weight",), "attention"),
                                            (("o_proj.weight",), "feed-forward")])
def test_each_half_of_a_block_reads_normalised_rows_and_adds_to_the_plain_stream(tmp_path, silenced, alive):
    """Pre-norm: with eps = 0 a norm removes any scale of its input, so what a half of the
    block adds does not change when the stream is scaled, and the stream itself passes
    through unscaled: block(c x) - c x == block(x) - x. A norm on the residual path (post-norm),
    a half that reads the stream without its norm, or a missing residual fails this. (Each half
    alone: the second half reads the first one's sum, which does not scale with c.)"""
    m = _one_layer(tmp_path, edit=_without(silenced), rms_norm_eps=0.0)
    x = rng.normal(size=(7, m.d))
    pos = np.arange(7)
    base = m.block(0, x, pos) - x
    assert np.abs(base).max() > 1e-3, alive                 # the half that is alive does add something
    for c in (0.25, 3.0):
        assert np.allclose(m.block(0, c * x, pos) - c * x, base, atol=1e-10)


def test_which_norm_feeds_which_half(tmp_path):
    """input_layernorm feeds the attention and only it; post_attention_layernorm feeds the
    feed-forward and only it: a norm weight of zero silences exactly its half (the model has
    no biases), so the block equals the one whose half is silenced at its last product."""
    x = rng.normal(size=(5, P.TINY_A["hidden_size"]))
    pos = np.arange(5)
    out = {}
    for key, edit in (("no_attn_norm", _without(("input_layernorm.weight",))),
                      ("no_o", _without(("o_proj.weight",))),
                      ("no_ffn_norm", _without(("post_attention_layernorm.weight",))),
                      ("no_down", _without(("down_proj.weight",))),
                      ("full", None)):
        d = tmp_path / key
        out[key] = _one_layer(d, edit=edit).block(0, x, pos)
    assert np.allclose(out["no_attn_norm"], out["no_o"], atol=1e-12)
    assert np.allclose(out["no_ffn_norm"], out["no_down"], atol=1e-12)
    assert not np.allclose(out["no_o"], out["no_down"], atol=1e-6)
    assert not np.allclose(out["full"], out["no_o"], atol=1e-6)


def test_output_matrix_is_used_when_the_file_has_one_and_the_table_when_not(tmp_path):
    """storage.rs:84: ``output.weight`` if the file holds it, else the embedding table.
    The same weights with and without an output matrix of their own differ exactly by that
    matrix: logits = h @ W^T with W the stored output matrix, or the table."""
    cfg = {**P.TINY_A, "tie_word_embeddings": False}
    P.make_model_folder(tmp_path / "own", cfg, 4)
    own = P.PlainLlama(tmp_path / "own")

    def drop(w):
        del w["lm_head.weight"]
    P.make_model_folder(tmp_path / "tied", cfg, 4, edit=drop)
    tied = P.PlainLlama(tmp_path / "tied")
    assert "lm_head.weight" in own.w and "lm_head.weight" not in tied.w
    toks = [1, 2, 3, 250]
    x = own.w["model.embed_tokens.weight"][toks]
    pos = np.arange(4)
    for i in range(own.n_layers):
        x = own.block(i, x, pos)
    h = P.rms_norm(x, own.w["model.norm.weight"], own.eps)
    assert np.allclose(own.forward(toks), h @ own.w["lm_head.weight"].T, atol=1e-12)
    assert np.allclose(tied.forward(toks), h @ own.w["model.embed_tokens.weight"].T, atol=1e-12)
    assert not np.allclose(own.forward(toks), tied.forward(toks), atol=1e-3)


def test_block_residuals_pass_through_when_projections_are_zero(tmp_path):
    def zero(w):
        for n in w:
            if n.endswith("o_proj.weight") or n.endswith("down_proj.weight"):
                w[n][:] = 0
    P.make_model_folder(tmp_path, P.TINY_A, 3, edit=zero)
    m = P.PlainLlama(tmp_path)
    toks = [4, 8, 15]
    x = m.w["model.embed_tokens.weight"][toks]
    want = P.linear(P.rms_norm(x, m.w["model.norm.weight"], m.eps), m.w["lm_head.weight"])
    assert np.allclose(m.forward(toks), want)


def test_greedy_stops_without_emitting_the_stop_token(tiny):
    m = tiny["A"]
    free = m.greedy([3, 1, 4], 6)
    assert len(free) == 6
    stopped = m.greedy([3, 1, 4], 6, stop_ids={free[2]})
    assert stopped == free[:free.index(free[2])]


# ---------------------------------------------------------------- sampling
def test_sample_probabilities():
    l = np.array([2.0, 1.0, 3.0, 3.0, -1.0])
    assert P.sample_probabilities(l, 0.0).tolist() == [0, 0, 1, 0, 0]          # first of equals
    assert P.sample_probabilities(l, 1.0, top_k=1).tolist() == [0, 0, 1, 0, 0]
    p = P.sample_probabilities(l, 0.5)
    assert np.allclose(p, torch.softmax(torch.tensor(l) / 0.5, -1).numpy())
    p2 = P.sample_probabilities(l, 1.0, top_k=2)
    assert np.allclose(p2, [0, 0, 0.5, 0.5, 0])
    # top_p: keep the shortest prefix of the descending order that reaches it
    full = P.sample_probabilities(l, 1.0)
    p3 = P.sample_probabilities(l, 1.0, top_p=float(full[2] + 1e-9))
    assert (p3 > 0).tolist() == [False, False, True, True, False]


def test_round_bf16_ties_to_even():
    one = np.float32(1.0)
    ulp = np.float32(2.0 ** -7)                      # bf16 spacing at 1.0
    assert P.round_bf16(np.array([one + ulp / 2]))[0] == 1.0             # tie -> even (1.0)
    assert P.round_bf16(np.array([one + 3 * ulp / 2]))[0] == 1.0 + 2 * ulp
    assert P.round_bf16(np.array([one + ulp * 0.51]))[0] == 1.0 + ulp
