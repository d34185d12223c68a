"""Steps of 9 to 64 sequences against the plain implementation, in float32 and bfloat16:
the products that serve 9-16, 17-32 and 33-64 rows, their partial planes added by the next
norm, the attention's units of work with many sequences, recorded steps that are filled up
to the next recorded batch size, and a batch that shrinks sequence by sequence."""
import numpy as np
import pytest

import gpu_util as G

pytestmark = pytest.mark.gpu
LIVE = (9, 16, 17, 24, 33, 49, 64)


def _run_batches(model, ref, name, dtype, live_counts, seed, max_len):
    """Batches one after another in the same slots; every sequence has a prompt and a number of
    single tokens of its own, so the batch shrinks. Every wanted row is compared."""
    from transformer_amd import Entry
    rng = np.random.default_rng(seed)
    biggest = max(live_counts)
    cache = model.new_cache(biggest * (-(-max_len // 64) * 64), max_slots=biggest)
    G.poison(cache)
    tol = G.TOL[dtype]
    for b, n_live in enumerate(live_counts):
        total = [int(x) for x in rng.integers(2, max_len + 1, n_live)]
        total[0], total[-1] = max_len, 2                    # the longest and the shortest are there
        dec = [int(min(t - 1, x)) for t, x in zip(total, rng.integers(1, 24, n_live))]
        reqs = [G.tokens(name, t, 1000 * seed + 100 * b + i) for i, t in enumerate(total)]
        want = [ref.forward(r) for r in reqs]
        slots = [cache.alloc_slot() for _ in reqs]
        # freed slots serve the next batch: no slot beyond what the largest batch so far took
        assert len(set(slots)) == n_live and max(slots) < max(live_counts[:b + 1])
        pos = [t - d for t, d in zip(total, dec)]
        out = model.step(cache, [Entry(s, r[:p], range(p)) for s, r, p in zip(slots, reqs, pos)])
        out = out.cpu().numpy().astype(np.float64)
        off = 0
        for i, p in enumerate(pos):
            err = np.abs(out[off:off + p] - want[i][:p]).max(axis=1)
            assert err.max() < tol, (name, dtype, "prompt", n_live, i, int(np.argmax(err > tol)))
            off += p
        live = list(range(n_live))
        sizes = []
        while live:
            sizes.append(len(live))
            out = model.step(cache, [Entry(slots[i], [reqs[i][pos[i]]], [0]) for i in live])
            out = out.cpu().numpy().astype(np.float64)
            assert out.shape[0] == len(live)
            nxt = []
            for row, i in enumerate(live):
                err = np.abs(out[row] - want[i][pos[i]]).max()
                assert err < tol, (name, dtype, "single", n_live, len(live), i, pos[i], err)
                pos[i] += 1
                if pos[i] < total[i]:
                    nxt.append(i)
                else:
                    cache.free_slot(slots[i])
            live = nxt
        assert sizes[0] == n_live and len(set(sizes)) > 3    # the batch did shrink
        cache.pool.check()
    return cache


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_steps_of_9_to_64_sequences(name, dtype):
    model, ref = G.engine(name, dtype), G.plain(name, dtype)
    max_len = {"A": 100, "B": 90, "C": 80, "D": 140, "E": 70}[name]
    cache = _run_batches(model, ref, name, dtype, LIVE, seed=7, max_len=max_len)
    if model._graph_safe:
        # recorded at the few sizes that steps are filled up to, not once per batch size
        assert 0 < len({k[0] for k in cache.graphs}) <= len(model.GRAPH_BATCHES)
        assert all(k[0] in model.GRAPH_BATCHES for k in cache.graphs)


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("D", "bfloat16"), ("E", "bfloat16")])
def test_the_same_steps_without_recorded_graphs(name, dtype):
    model, ref = G.engine(name, dtype), G.plain(name, dtype)
    model.use_graphs = False
    try:
        cache = _run_batches(model, ref, name, dtype, (33, 20, 64), seed=8, max_len=80)
    finally:
        model.use_graphs = True
    assert not cache.graphs


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_of_more_than_64_sequences(dtype):
    """70 and 100 sequences: prompts of several hundred rows in one step, then recorded steps of
    96 and 128 rows that shrink. In bfloat16 the down projection (k = 8,192) is the library's
    batched product in planes at every row count above 64, inside the recorded steps too, whose
    recordings must pass their check (a failed one warns)."""
    import warnings
    from transformer_amd.parts.linear import library_planes
    model, ref = G.engine("F", dtype), G.plain("F", dtype)
    if dtype == "bfloat16":
        assert library_planes(70, model.blocks[0].ffn.w["down.weight"]) == 8
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        cache = _run_batches(model, ref, "F", dtype, (70, 100), seed=9, max_len=40)
    assert {k[0] for k in cache.graphs_checked} >= {96, 128} and not cache.graphs_failed


def test_planes_of_a_cut_product_reach_both_norms():
    """The configuration E is there for this: its output and down projections leave several
    planes at 17 to 64 rows."""
    from transformer_amd import kernels
    model = G.engine("E", "bfloat16")
    blk = model.blocks[0]
    assert kernels.mid_splits(blk.mixer.w["out.weight"]) > 1
    assert kernels.mid_splits(blk.ffn.w["down.weight"]) > 1
    assert kernels.mid_takes(40, blk.ffn.w["down.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_batch_that_shrinks_through_every_size(dtype):
    """40 sequences generate greedily and end one after another: prompt i leaves room for
    i + 1 tokens below the model's last position, so the batch passes through every size from
    40 down to 1, more sizes than recorded steps are kept. The tokens are the plain model's."""
    from transformer_amd.engine.generate import generate
    name = "A"
    model, ref = G.engine(name, dtype), G.plain(name, dtype)
    limit = G.CONFIGS[name][0]["max_position_embeddings"]
    n = 40
    assert n > model.MAX_GRAPHS
    prompts = [G.tokens(name, limit - i, 500 + i) for i in range(n)]
    res = generate(model, prompts, max_new_tokens=64, max_batch=n, stop_ids=[])
    assert [len(t) for t in res.tokens] == [i + 1 for i in range(n)]
    assert res.finish == ["length"] * n and res.batches == [list(range(n))]
    for i, (p, got) in enumerate(zip(prompts, res.tokens)):
        if dtype == "float32":
            assert got == ref.greedy(p, i + 1), i
        else:
            seq = list(p)
            for t in got:
                lg = ref.forward(seq)[-1]
                assert lg.max() - lg[t] < 2 * G.TOL["bfloat16"], i
                seq.append(t)
    # one sequence stops at a token of its own in the middle of such a batch
    if dtype == "float32":
        stop = res.tokens[30][12]
        again = generate(model, prompts, max_new_tokens=64, max_batch=n, stop_ids=[stop])
        for i, (p, got, fin) in enumerate(zip(prompts, again.tokens, again.finish)):
            want = ref.greedy(p, i + 1, stop_ids={stop})
            assert got == want and fin == ("stop" if len(want) < i + 1 else "length"), i
