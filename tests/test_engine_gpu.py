"""The engine against the plain implementation, in float32 and bfloat16: requests
alone and whole; the last 32 tokens one by one; batches of unequal lengths whose
shorter requests end earlier, one batch after another in reused slots; long
decoding; the first tokens of a sequence; greedy generation through the entry
points."""
import json
import os
import pathlib
import subprocess
import sys

import numpy as np
import pytest

import gpu_util as G
import plain_llama as P

pytestmark = pytest.mark.gpu
ROOT = pathlib.Path(__file__).resolve().parent.parent
CASES = [(n, d) for n in ("A", "B", "C", "D") for d in ("float32", "bfloat16")]


def _logits(model, cache, entries):
    return model.step(cache, entries).cpu().numpy().astype(np.float64)


@pytest.mark.parametrize("name,dtype", CASES)
def test_requests_alone_and_whole(name, dtype):
    from transformer_amd import Entry
    model, ref = G.engine(name, dtype), G.plain(name, dtype)
    cache = model.new_cache(256)
    G.poison(cache)
    for n, seed in ((1, 1), (2, 2), (63, 3), (64, 4), (65, 5), (120, 6)):
        toks = G.tokens(name, n, seed)
        s = cache.alloc_slot()
        got = _logits(model, cache, [Entry(s, toks, range(n))])
        cache.free_slot(s)
        assert np.isfinite(got).all()
        assert np.abs(got - ref.forward(toks)).max() < G.TOL[dtype], (name, dtype, n)
    cache.pool.check()


@pytest.mark.parametrize("name,dtype", CASES)
def test_last_32_tokens_one_by_one(name, dtype):
    from transformer_amd import Entry
    model, ref = G.engine(name, dtype), G.plain(name, dtype)
    cache = model.new_cache(256)
    G.poison(cache)
    toks = G.tokens(name, 100, 11)
    want = ref.forward(toks)
    s = cache.alloc_slot()
    whole = _logits(model, cache, [Entry(s, toks, range(100))])
    cache.free_slot(s)
    s = cache.alloc_slot()
    parts = [_logits(model, cache, [Entry(s, toks[:68], range(68))])]
    for t in toks[68:]:
        parts.append(_logits(model, cache, [Entry(s, [t], [0])]))
    got = np.concatenate(parts)
    err = np.abs(got - want).max(axis=1)
    assert err.max() < G.TOL[dtype], f"first wrong place {int(np.argmax(err > G.TOL[dtype]))}"
    assert np.abs(got - whole).max() < G.TOL_SPLIT[dtype]
    cache.free_slot(s)


@pytest.mark.parametrize("name,dtype", CASES)
def test_unequal_batches_one_after_another_in_reused_slots(name, dtype):
    from transformer_amd import Entry
    model, ref = G.engine(name, dtype), G.plain(name, dtype)
    cache = model.new_cache(64 * 6, max_slots=3)       # room for one batch only
    G.poison(cache)
    used = []
    limit = G.CONFIGS[name][0]["max_position_embeddings"]
    for b, lens in enumerate(([5, 70, 33], [64, 2, 40], [1, min(129, limit), 17])):
        reqs = [G.tokens(name, n, 100 * b + i) for i, n in enumerate(lens)]
        prompt = [max(1, n - 10 - 3 * i) for i, n in enumerate(lens)]   # unequal decode lengths
        slots = [cache.alloc_slot() for _ in reqs]
        used.append(sorted(slots))
        got = [[] for _ in reqs]
        out = _logits(model, cache, [Entry(s, r[:p], range(p)) for s, r, p in zip(slots, reqs, prompt)])
        off = 0
        for i, p in enumerate(prompt):
            got[i].append(out[off:off + p])
            off += p
        pos = list(prompt)
        live = [i for i in range(len(reqs)) if pos[i] < len(reqs[i])]
        for i in range(len(reqs)):
            if i not in live:
                cache.free_slot(slots[i])              # nothing left to decode
        while live:
            out = _logits(model, cache, [Entry(slots[i], [reqs[i][pos[i]]], [0]) for i in live])
            nxt = []
            for row, i in enumerate(live):
                got[i].append(out[row:row + 1])
                pos[i] += 1
                if pos[i] < len(reqs[i]):
                    nxt.append(i)
                else:
                    cache.free_slot(slots[i])          # the shorter request ends earlier
            live = nxt
        for i, r in enumerate(reqs):
            g = np.concatenate(got[i])
            err = np.abs(g - ref.forward(r)).max(axis=1)
            assert err.max() < G.TOL[dtype], (name, dtype, b, i, int(np.argmax(err > G.TOL[dtype])))
        cache.pool.check()
    assert used[0] == used[1] == used[2] == [0, 1, 2]   # the same slots served every batch


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "bfloat16"), ("C", "float32"),
                                        ("D", "bfloat16")])
def test_long_decoding(name, dtype):
    from transformer_amd import Entry
    model, ref = G.engine(name, dtype), G.plain(name, dtype)
    n = {"A": 128, "B": 256, "C": 300, "D": 700}[name]
    toks = G.tokens(name, n, 21)
    want = ref.forward(toks)
    cache = model.new_cache(n + 64)
    G.poison(cache)
    s = cache.alloc_slot()
    got = [_logits(model, cache, [Entry(s, toks[:3], range(3))])]
    for t in toks[3:]:
        got.append(_logits(model, cache, [Entry(s, [t], [0])]))
    err = np.abs(np.concatenate(got) - want).max(axis=1)
    assert err.max() < G.TOL[dtype], f"first wrong place {int(np.argmax(err > G.TOL[dtype]))}"


@pytest.mark.parametrize("name,dtype", CASES)
def test_first_tokens_of_a_sequence(name, dtype):
    from transformer_amd import Entry
    model, ref = G.engine(name, dtype), G.plain(name, dtype)
    cache = model.new_cache(128)
    G.poison(cache)
    toks = G.tokens(name, 4, 31)
    want = ref.forward(toks)
    s = cache.alloc_slot()
    for i, t in enumerate(toks):                       # token by token from the very first
        got = _logits(model, cache, [Entry(s, [t], [0])])
        assert np.abs(got[0] - want[i]).max() < G.TOL[dtype], (name, dtype, i)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharp_attention_far_keys_and_page_edges(dtype):
    """With peaked attention a wrong or missing key anywhere moves the logits."""
    from transformer_amd import Entry
    model, ref = G.engine("A", dtype, "sharp"), G.plain("A", dtype, "sharp")
    toks = G.tokens("A", 128, 41)
    want = ref.forward(toks)
    cache = model.new_cache(512)
    G.poison(cache)
    hold = [cache.alloc_slot() for _ in range(3)]       # push the test's pages away from page 0
    for h in hold:
        model.step(cache, [Entry(h, G.tokens("A", 70, h), [])])
    cache.free_slot(hold[1])
    s = cache.alloc_slot()
    got = [_logits(model, cache, [Entry(s, toks[:60], range(60))])]
    for t in toks[60:]:
        got.append(_logits(model, cache, [Entry(s, [t], [0])]))
    err = np.abs(np.concatenate(got) - want).max(axis=1)
    tol = G.TOL[dtype] * (3 if dtype == "bfloat16" else 1)   # peaked softmax amplifies rounding of scores
    assert err.max() < tol, f"first wrong place {int(np.argmax(err > tol))}"


def test_a_wanted_list_may_be_empty_and_rows_come_in_entry_order():
    from transformer_amd import Entry
    model, ref = G.engine("A", "float32"), G.plain("A", "float32")
    cache = model.new_cache(256)
    a, b, c = G.tokens("A", 9, 1), G.tokens("A", 4, 2), G.tokens("A", 6, 3)
    sa, sb, sc = (cache.alloc_slot() for _ in range(3))
    out = _logits(model, cache, [Entry(sa, a, [8]), Entry(sb, b, []), Entry(sc, c, [0, 5])])
    assert out.shape == (3, 256)
    assert np.abs(out[0] - ref.forward(a)[8]).max() < 2e-5
    assert np.abs(out[1:] - ref.forward(c)[[0, 5]]).max() < 2e-5
    none = model.step(cache, [Entry(sb, [7], [])])
    assert tuple(none.shape) == (0, 256)


def test_a_full_cache_is_refused_before_anything_runs():
    from transformer_amd import Entry
    from transformer_amd.cache.pool import CacheFull
    model = G.engine("B", "float32")
    cache = model.new_cache(128)
    s = cache.alloc_slot()
    model.step(cache, [Entry(s, G.tokens("B", 100, 1), [])])
    with pytest.raises(CacheFull):
        model.step(cache, [Entry(s, G.tokens("B", 29, 2), [])])
    assert cache.length(s) == 100
    model.step(cache, [Entry(s, G.tokens("B", 28, 2), [0])])       # exactly full is fine
    assert cache.length(s) == 128


def test_a_position_past_the_models_limit_is_refused_before_anything_runs():
    from transformer_amd import Entry
    from transformer_amd.engine.batch import PositionPastLimit
    model = G.engine("A", "float32")
    limit = G.CONFIGS["A"][0]["max_position_embeddings"]
    cache = model.new_cache(4 * limit)
    s, t = cache.alloc_slot(), cache.alloc_slot()
    with pytest.raises(PositionPastLimit, match="max_position_embeddings"):
        model.step(cache, [Entry(t, [1, 2], []), Entry(s, G.tokens("A", limit + 1, 1), [])])
    assert cache.length(s) == 0 and cache.length(t) == 0
    model.step(cache, [Entry(s, G.tokens("A", limit - 1, 1), [])])
    model.step(cache, [Entry(s, [5], [0])])                 # the last position is allowed
    with pytest.raises(PositionPastLimit):
        model.step(cache, [Entry(s, [5], [0])])
    assert cache.length(s) == limit
    cache.pool.check()


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "float32"), ("C", "float32")])
def test_greedy_generation_through_the_python_entry_point(name, dtype):
    from transformer_amd.engine.generate import generate
    model, ref = G.engine(name, dtype), G.plain(name, dtype)
    prompts = [G.tokens(name, n, 50 + n) for n in (1, 7, 13, 5)]
    res = generate(model, prompts, max_new_tokens=8, max_batch=3)
    assert res.batches == [[0, 1, 2], [3]]
    for p, got in zip(prompts, res.tokens):
        assert got == ref.greedy(p, 8)
    stop = res.tokens[1][3]
    res2 = generate(model, prompts, max_new_tokens=8, stop_ids=[stop])
    for p, got, fin in zip(prompts, res2.tokens, res2.finish):
        want = ref.greedy(p, 8, stop_ids={stop})
        assert got == want and fin == ("stop" if len(want) < 8 else "length")


def test_greedy_generation_bfloat16_stays_near_the_top():
    from transformer_amd.engine.generate import generate
    model, ref = G.engine("B", "bfloat16"), G.plain("B", "bfloat16")
    prompts = [G.tokens("B", n, 60 + n) for n in (5, 2, 17, 9)]
    res = generate(model, prompts, max_new_tokens=6)
    for p, got in zip(prompts, res.tokens):
        seq = list(p)
        for t in got:
            lg = ref.forward(seq)[-1]
            assert lg.max() - lg[t] < 2 * G.TOL["bfloat16"]
            seq.append(t)


def test_temperature_sampling_is_seeded_and_independent_of_the_batch():
    from transformer_amd.engine.generate import generate
    from transformer_amd.sampling.args import SampleArgs
    from transformer_amd.sampling.sampler import uniform
    model, ref = G.engine("B", "float32"), G.plain("B", "float32")
    prompts = [G.tokens("B", n, 70 + n) for n in (5, 2, 17, 9)]
    args = SampleArgs(temperature=0.8)
    a = generate(model, prompts, 6, args, seed=11)
    b = generate(model, prompts, 6, args, seed=11)
    c = generate(model, prompts, 6, args, seed=12)
    assert a.tokens == b.tokens and a.tokens != c.tokens
    alone = generate(model, prompts[2:3], 6, args, seed=11)
    # request 2 alone is "sequence 0" of its call, so it draws other numbers: compare
    # through the plain model instead, with the numbers each call really drew
    for res, idx in ((a, [0, 1, 2, 3]), (alone, [2])):
        for k, i in enumerate(idx):
            seq = list(prompts[i])
            for g, t in enumerate(res.tokens[k]):
                p = P.sample_probabilities(ref.forward(seq)[-1], 0.8)
                cdf = np.cumsum(p)
                u = uniform(11, k, g)
                lo = cdf[t] - p[t]
                assert lo - 1e-5 <= u <= cdf[t] + 1e-5, (k, g, t)
                seq.append(t)


def test_command_line_in_the_references_manner(tmp_path):
    folder = G.folder("A", "float32")
    ref = G.plain("A", "float32")
    env = {**os.environ, "TEST_MODEL": folder, "PROMPT": "3 1 4 1 5", "MAX_STEPS": "5",
           "TEMPERATURE": "0"}
    r = subprocess.run([sys.executable, "-m", "transformer_amd", "generate", "--dtype", "float32"],
                       capture_output=True, text=True, env=env, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    want = " ".join(map(str, ref.greedy([3, 1, 4, 1, 5], 5)))
    assert want in r.stdout and "prefill" in r.stdout and "decode" in r.stdout
    # options win over the environment
    r = subprocess.run([sys.executable, "-m", "transformer_amd", "generate", "--dtype", "float32",
                        "--prompt", "9,9", "--max-steps", "3"], capture_output=True, text=True,
                       env=env, cwd=ROOT)
    assert " ".join(map(str, ref.greedy([9, 9], 3))) in r.stdout
    # --backend ref: the plain float32 kernels, whatever the dtype asked for
    r = subprocess.run([sys.executable, "-m", "transformer_amd", "generate", "--dtype", "bfloat16",
                        "--backend", "ref"], capture_output=True, text=True, env=env, cwd=ROOT)
    assert r.returncode == 0 and want in r.stdout, r.stderr[-2000:]
    # --timers: the same tokens, and the GPU time of each kind of part
    r = subprocess.run([sys.executable, "-m", "transformer_amd", "generate", "--dtype", "float32",
                        "--timers"], capture_output=True, text=True, env=env, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    assert want in r.stdout
    for kind in ("embed", "norm", "mixer", "ffn", "head"):
        assert kind in r.stdout, r.stdout
    # without --dtype the folder's torch_dtype decides: a copy of the folder that says float32
    import json
    import shutil
    says = tmp_path / "says_float32"
    shutil.copytree(folder, says)
    cfg = json.loads((says / "config.json").read_text())
    (says / "config.json").write_text(json.dumps({**cfg, "torch_dtype": "float32"}))
    r = subprocess.run([sys.executable, "-m", "transformer_amd", "generate", "--model", str(says)],
                       capture_output=True, text=True, env=env, cwd=ROOT)
    assert r.returncode == 0 and want in r.stdout, r.stderr[-2000:]
    assert "float32" in r.stderr                                   # the loader says what it computes in
    # --random CONFIG --seed N: weights drawn on the GPU, the same tokens for the same seed
    env2 = {k: v for k, v in env.items() if k != "TEST_MODEL"}
    outs = []
    for seed in ("4", "4", "5"):
        r = subprocess.run([sys.executable, "-m", "transformer_amd", "generate", "--random",
                            os.path.join(folder, "config.json"), "--seed", seed, "--dtype", "float32"],
                           capture_output=True, text=True, env=env2, cwd=ROOT)
        assert r.returncode == 0, r.stderr[-2000:]
        outs.append([l for l in r.stdout.splitlines() if l.startswith("[0]")][0])
    assert outs[0] == outs[1] != outs[2]


@pytest.mark.parametrize("name,dtype", [("B", "float32"), ("C", "bfloat16"), ("D", "bfloat16")])
def test_recorded_single_token_steps_equal_eager_ones(name, dtype):
    """Single-token steps are replayed from a recorded graph. Every replay is checked
    against the same step run eagerly, with the program's own eager work (prompts of
    other sequences, a larger scratch need, synchronisations) between the replays."""
    import torch
    from transformer_amd import Entry
    model = G.engine(name, dtype)
    toks = [G.tokens(name, 150, 300 + i) for i in range(3)]

    def run(use_graphs):
        model.use_graphs = use_graphs
        cache = model.new_cache(1024, max_slots=4)
        slots = [cache.alloc_slot() for _ in toks]
        out = [_logits(model, cache, [Entry(s, t[:20 + 9 * i], [19 + 9 * i]) for i, (s, t) in
                                      enumerate(zip(slots, toks))])]
        pos = [20 + 9 * i for i in range(3)]
        for step in range(min(110, G.CONFIGS[name][0]["max_position_embeddings"] - 40)):
            out.append(_logits(model, cache, [Entry(s, [t[p]], [0]) for s, t, p in zip(slots, toks, pos)]))
            pos = [p + 1 for p in pos]
            if step % 25 == 7:           # eager work in between: a prompt in a fourth slot
                extra = cache.alloc_slot()
                _logits(model, cache, [Entry(extra, G.tokens(name, 70 + step, step), range(70 + step))])
                cache.free_slot(extra)
                torch.cuda.synchronize()
        n_graphs = len(cache.graphs)
        return np.concatenate(out), n_graphs

    try:
        eager, n0 = run(False)
        replay, n1 = run(True)
    finally:
        model.use_graphs = True
    assert n0 == 0 and n1 >= 1
    assert np.abs(eager - replay).max() <= G.TOL_SPLIT[dtype]


def test_a_step_is_recorded_again_when_the_page_table_grows():
    """A recording holds page tables of a fixed width; a sequence that grows past it gets a new
    recording (here every page, so that 90 single-token steps record three), each tried once
    per batch size, and every step agrees with the plain model."""
    import transformer_amd as ta
    from transformer_amd import Entry
    model = ta.load_model(G.folder("D", "bfloat16"), "bfloat16", "cuda:0")
    model.GRAPH_TABLE_STEP = 1
    ref = G.plain("D", "bfloat16")
    toks = G.tokens("D", 140, 91)
    cache = model.new_cache(256)
    s = cache.alloc_slot()
    got = [_logits(model, cache, [Entry(s, toks[:50], [49])])]
    for t in toks[50:]:
        got.append(_logits(model, cache, [Entry(s, [t], [0])]))
    assert sorted(k[2] for k in cache.graphs) == [1, 2, 3] and len(cache.graphs_checked) == 1
    assert np.abs(np.concatenate(got) - ref.forward(toks)[49:]).max() < G.TOL["bfloat16"]


def test_a_recording_that_replays_wrongly_is_not_used(monkeypatch):
    """Every new recording is replayed twice against its eager step before it is trusted. A
    replay that gives other logits (forced here from the host: the replay is followed by an add
    to the logits and by a scribble over the keys that the step stored) makes steps of that
    shape run eagerly for good, with one warning and right results: the eager step runs again,
    so the cache holds what it wrote, and nothing is recorded again when the page table grows
    (here with every page) or when the kept recordings are dropped."""
    import torch
    import transformer_amd as ta
    from transformer_amd import Entry
    model = ta.load_model(G.folder("D", "bfloat16"), "bfloat16", "cuda:0")
    model.GRAPH_TABLE_STEP = 1
    ref = G.plain("D", "bfloat16")
    toks = G.tokens("D", 150, 77)
    seen = {"replays": 0}
    forward = model._forward

    def remember(ctx, cache):
        seen["logits"] = forward(ctx, cache)
        if not torch.cuda.is_current_stream_capturing():
            seen["dest"] = [t.dest.clone() for t in ctx.kv]
        return seen["logits"]

    replay = torch.cuda.CUDAGraph.replay

    def bad_replay(graph):
        replay(graph)
        seen["replays"] += 1
        seen["logits"].add_(1.0)
        for keys, dest in zip(cache.keys, seen["dest"]):         # [layers, pages, kv heads, 64, dh]
            d = int(dest[0])
            keys[:, d // 64, :, d % 64, :] = 7.0

    monkeypatch.setattr(model, "_forward", remember)
    monkeypatch.setattr(torch.cuda.CUDAGraph, "replay", bad_replay)
    cache = model.new_cache(256)
    s = cache.alloc_slot()
    got = [_logits(model, cache, [Entry(s, toks[:30], [29])])]
    with pytest.warns(UserWarning, match="run eagerly"):
        got.append(_logits(model, cache, [Entry(s, [toks[30]], [0])]))
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("error")                           # no second try, no second warning
        for i, t in enumerate(toks[31:]):
            if i == 50:
                cache.graphs.clear()                             # as when a buffer of the workspace moves
            got.append(_logits(model, cache, [Entry(s, [t], [0])]))
    assert seen["replays"] == 1 and not cache.graphs and cache.graphs_failed == {(1, 1)}
    want = ref.forward(toks)[29:]
    assert np.abs(np.concatenate(got) - want).max() < G.TOL["bfloat16"]


def test_float32_steps_filled_up_to_a_recorded_size_equal_the_eager_steps_bit_for_bit():
    """Five sequences are recorded as a step of six (one row belongs to nobody). In float32 every
    row's bits depend on its own inputs only, so the recorded, filled-up steps give exactly the
    logits of eager steps of five. (In bfloat16 the row count chooses the products' kernels, so
    there the two agree within rounding only.)"""
    from transformer_amd import Entry
    model = G.engine("C", "float32")
    toks = [G.tokens("C", 60, 40 + i) for i in range(5)]

    def run(use_graphs):
        model.use_graphs = use_graphs
        cache = model.new_cache(1024, max_slots=6)
        slots = [cache.alloc_slot() for _ in toks]
        out = [_logits(model, cache, [Entry(s, t[:20 + 3 * i], [19 + 3 * i]) for i, (s, t) in enumerate(zip(slots, toks))])]
        for step in range(20):
            out.append(_logits(model, cache, [Entry(s, [t[20 + 3 * i + step]], [0]) for i, (s, t) in enumerate(zip(slots, toks))]))
        return np.concatenate(out), [k[0] for k in cache.graphs]

    try:
        eager, _ = run(False)
        replay, batches = run(True)
    finally:
        model.use_graphs = True
    assert batches == [6]
    assert np.array_equal(eager, replay)


@pytest.mark.parametrize("merged", [True, False])
def test_a_gguf_file_gives_the_same_logits_as_the_folder_it_was_made_from(tmp_path, merged):
    """The file rotates adjacent pairs over reordered q/k rows; the folder rotates
    half-split pairs: the logits must agree (and agree with the plain model)."""
    import transformer_amd as ta
    from transformer_amd import Entry
    from transformer_amd.architectures.llama_gguf_export import export_gguf
    with pytest.raises(ValueError, match="bias"):
        export_gguf(G.folder("C", "float32"), tmp_path / "c.gguf")
    for name in ("A",):
        path = export_gguf(G.folder(name, "float32"), tmp_path / f"{name}{merged}.gguf", merged=merged)
        model = ta.load_model(path, "float32")
        assert model.config.rope_style == "interleaved"
        toks = G.tokens(name, 70, 5)
        cache = model.new_cache(128)
        s = cache.alloc_slot()
        got = _logits(model, cache, [Entry(s, toks, range(70))])
        assert np.abs(got - G.plain(name, "float32").forward(toks)).max() < G.TOL["float32"], name


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("D", "bfloat16")])
def test_a_step_may_mix_prompts_and_single_tokens(name, dtype):
    from transformer_amd import Entry
    model, ref = G.engine(name, dtype), G.plain(name, dtype)
    cache = model.new_cache(512)
    G.poison(cache)
    a, b, c = G.tokens(name, 90, 1), G.tokens(name, 40, 2), G.tokens(name, 70, 3)
    sa, sb, sc = (cache.alloc_slot() for _ in range(3))
    _logits(model, cache, [Entry(sa, a[:60], []), Entry(sb, b[:39], [])])
    # a continues with a chunk, b with one token, c starts
    got = _logits(model, cache, [Entry(sa, a[60:], range(30)), Entry(sb, b[39:], [0]),
                                 Entry(sc, c, range(70))])
    want = np.concatenate([ref.forward(a)[60:], ref.forward(b)[39:], ref.forward(c)])
    assert np.abs(got - want).max() < G.TOL[dtype]


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("D", "bfloat16")])
def test_tokens_may_stay_on_the_gpu_between_steps(name, dtype):
    """A step fed with token values that are only on the GPU gives the logits of the same step
    fed from the host: with and without recorded graphs, for single tokens and for a prompt."""
    import torch
    from transformer_amd import Entry
    model = G.engine(name, dtype)
    a, b = G.tokens(name, 50, 7), G.tokens(name, 21, 8)
    out = {}
    for mode in ("host", "device"):
        for graphs in (True, False):
            model.use_graphs = graphs
            cache = model.new_cache(256)
            G.poison(cache)
            sa, sb = cache.alloc_slot(), cache.alloc_slot()
            rows = []
            if mode == "host":
                rows.append(_logits(model, cache, [Entry(sa, a[:40], [39]), Entry(sb, b[:11], [10])]))
                for i in range(10):
                    rows.append(_logits(model, cache, [Entry(sa, [a[40 + i]], [0]), Entry(sb, [b[11 + i]], [0])]))
            else:
                dev = torch.tensor(a[:40] + b[:11], dtype=torch.int32, device=model.device)
                fake = [Entry(sa, [0] * 40, [39]), Entry(sb, [0] * 11, [10])]
                rows.append(model.step(cache, fake, device_tokens=dev).float().cpu().numpy().copy())
                for i in range(10):
                    dev = torch.tensor([a[40 + i], b[11 + i]], dtype=torch.int32, device=model.device)
                    rows.append(model.step(cache, [Entry(sa, [0], [0]), Entry(sb, [0], [0])],
                                           device_tokens=dev).float().cpu().numpy().copy())
            out[mode, graphs] = np.concatenate(rows)
    model.use_graphs = True
    for graphs in (True, False):
        assert np.array_equal(out["host", graphs], out["device", graphs])
    cache = model.new_cache(64)
    s = cache.alloc_slot()
    with pytest.raises(ValueError, match="device_tokens"):
        model.step(cache, [Entry(s, [1, 2], [1])],
                   device_tokens=torch.zeros(3, dtype=torch.int32, device=model.device))


def test_a_bfloat16_engine_keeps_matrices_that_are_stored_in_32_bits():
    """The same folder, stored in float32, run in bfloat16: the matrices stay float32 on the GPU
    and the logits follow the plain model with unrounded weights and bfloat16 activations,
    for a prompt and for single tokens."""
    import torch
    import transformer_amd as ta
    from transformer_amd import Entry
    folder = G.folder("C", "float32")
    model = ta.load_model(folder, "bfloat16", "cuda:0")
    assert model.w["head"].dtype == torch.float32 and model.dtype == torch.bfloat16
    assert model.blocks[0].mixer.w["qkv.weight"].dtype == torch.float32
    ref = P.PlainLlama(folder, round_activations=True)
    toks = G.tokens("C", 60, 21)
    cache = model.new_cache(128)
    G.poison(cache)
    s = cache.alloc_slot()
    got = [_logits(model, cache, [Entry(s, toks[:45], range(45))])]
    for t in toks[45:]:
        got.append(_logits(model, cache, [Entry(s, [t], [0])]))
    assert np.abs(np.concatenate(got) - ref.forward(toks)).max() < G.TOL["bfloat16"]


def test_the_facade_and_reset_slot():
    import transformer_amd as ta
    llama = ta.Llama.from_pretrained(G.folder("A", "float32"), "float32", cache_tokens=256)
    ref = G.plain("A", "float32")
    toks = G.tokens("A", 20, 4)
    s = llama.alloc_slot()
    first = llama.step([(s, toks, [19])]).cpu().numpy()
    llama.reset_slot(s)
    again = llama.step([ta.Entry(s, toks, [19])]).cpu().numpy()
    assert np.array_equal(first, again) and np.abs(first[0] - ref.forward(toks)[19]).max() < 2e-5
    out = llama.generate([toks], 4)
    assert out.tokens[0] == ref.greedy(toks, 4)


def test_bfloat16_stays_close_to_float32_at_the_headline_width():
    """Two layers of the Llama-3.1-8B shape with the same random weights in both dtypes:
    the bfloat16 engine (library products, matrix-core attention, graphs) must follow the
    true 32-bit path, whose kernels share nothing with it but the cache and the step."""
    import torch
    import transformer_amd as ta
    from transformer_amd import Entry
    cfg = {"architectures": ["LlamaForCausalLM"], "num_hidden_layers": 2, "hidden_size": 4096,
           "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128,
           "intermediate_size": 14336, "vocab_size": 32000, "rope_theta": 500000.0,
           "rms_norm_eps": 1e-5, "tie_word_embeddings": True, "max_position_embeddings": 4096}
    toks = [int(t) for t in np.random.default_rng(0).integers(0, 32000, 300)]
    out = {}
    for dtype in ("float32", "bfloat16"):
        model = ta.random_model(cfg, seed=5, dtype=dtype)
        cache = model.new_cache(512)
        s = cache.alloc_slot()
        parts = [model.step(cache, [Entry(s, toks[:280], range(200, 280))]).float().cpu().numpy()]
        for t in toks[280:]:
            parts.append(model.step(cache, [Entry(s, [t], [0])]).float().cpu().numpy())
        out[dtype] = np.concatenate(parts).astype(np.float64)
        del model, cache
        torch.cuda.empty_cache()
    # Both models round differently often: weights to 8 bits of mantissa once, activations at about
    # a dozen places per layer. Each rounding is a relative error of at most 2^-9, they add in
    # quadrature over the 4096-term sums, so the logits differ by about one percent of their
    # spread; the largest of the 3.2 million compared logits lies some five deviations out.
    scale = out["float32"].std()
    diff = out["bfloat16"] - out["float32"]
    rms, err = np.sqrt((diff ** 2).mean()), np.abs(diff).max()
    print(f"bf16 vs fp32 at width 4096: rms {rms:.4f} max {err:.4f} spread {scale:.3f}")
    assert np.isfinite(out["bfloat16"]).all()
    assert rms < 0.025 * scale and err < 0.12 * scale, (rms, err, scale)
    # the two paths agree on almost every greedy choice
    same = (out["bfloat16"].argmax(-1) == out["float32"].argmax(-1)).mean()
    assert same > 0.9, same


@pytest.mark.parametrize("name", ["A", "C"])
def test_single_token_steps_leave_the_norms_to_the_products(name, monkeypatch):
    """In a bfloat16 step of a few tokens the products on either side of a norm take it over:
    only the first norm and the final one run as kernels of their own. With the hand-over
    switched off the same step gives the same logits up to the one rounding that moved."""
    from transformer_amd import Entry, kernels
    from transformer_amd.parts.block import PreNormBlock
    model = G.engine(name, "bfloat16")
    layers = G.CONFIGS[name][0]["num_hidden_layers"]
    calls = []
    real = kernels.add_rmsnorm
    monkeypatch.setattr(kernels, "add_rmsnorm", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    monkeypatch.setattr(model, "use_graphs", False)
    toks = G.tokens(name, 40, 21)

    def decode():
        cache = model.new_cache(128)
        G.poison(cache)
        s = [cache.alloc_slot(), cache.alloc_slot()]
        model.step(cache, [Entry(s[0], toks[:30], []), Entry(s[1], toks[5:20], [])])
        calls.clear()
        out = _logits(model, cache, [Entry(s[0], [toks[30]], [0]), Entry(s[1], [toks[20]], [0])])
        return out, len(calls)

    folded, n_folded = decode()
    assert n_folded == 2
    monkeypatch.setattr(PreNormBlock, "_fusable", lambda self, nt: False)
    apart, n_apart = decode()
    assert n_apart == 2 * layers + 1
    assert np.abs(folded - apart).max() < G.TOL_SPLIT["bfloat16"]
    ref = G.plain(name, "bfloat16")
    want = np.stack([ref.forward(toks[:31])[-1], ref.forward(toks[5:21])[-1]])
    assert np.abs(folded - want).max() < G.TOL["bfloat16"]
