"""Each part alone against the plain functions, and the generality of the
assembly: a toy mixer with state of its own, defined here, is registered, built
and stepped without a change to the framework's files; a schedule names a block
twice and lets a run read another run's cache."""
import dataclasses
import math
from dataclasses import dataclass

import numpy as np
import pytest
import torch

import gpu_util as G
import plain_llama as P

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
rng = np.random.default_rng(5)


def dev(a, dtype=torch.float32):
    return torch.tensor(np.asarray(a), dtype=dtype, device=DEV)


def f64(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


class Ctx:
    """The slice of a step's context that a single part needs."""

    def __init__(self, cache, entries, vocab=1 << 30):
        from transformer_amd.engine.batch import Uploader, plan_step
        from transformer_amd.parts.linear import Workspace
        self.ctx = plan_step(entries, cache, vocab, Uploader(DEV), Workspace(DEV))


def test_norm_part():
    from transformer_amd.config.spec import NormSpec
    from transformer_amd.parts import build_part
    part = build_part(NormSpec(size=72, eps=1e-3), torch.float32, DEV)
    w = 1 + 0.1 * rng.normal(size=72)
    part.bind({"weight": dev(w)})
    x = rng.normal(size=(5, 72))
    out = torch.empty(5, 72, device=DEV)
    part.run(dev(x), out)
    assert np.abs(f64(out) - P.rms_norm(x.astype(np.float32), w.astype(np.float32), 1e-3)).max() < 1e-5


def test_position_parts():
    from transformer_amd.config.spec import PositionSpec
    from transformer_amd.parts import build_part
    from transformer_amd.parts.linear import Workspace
    qkv = rng.normal(size=(3, 4, 32)).astype(np.float32)
    pos = [0, 9, 77]

    class C:                         # what a position part reads from the step's context
        nt, positions, ws, shared = 3, dev(pos, torch.int32), Workspace(DEV), {}
    rot = build_part(PositionSpec(head_dim=32, theta=777.0, style="interleaved"), torch.float32, DEV)
    t = dev(qkv.reshape(3, -1))
    rot.encode_and_store(t, C, 2, 1)
    got = f64(t).reshape(3, 4, 32)
    assert np.abs(got[:, :3] - P.rope(qkv[:, :3], pos, 777.0, "interleaved")).max() < 1e-5
    assert np.array_equal(got[:, 3], qkv[:, 3].astype(np.float64))          # v is not rotated
    none = build_part(PositionSpec(head_dim=32, kind="none"), torch.float32, DEV)
    t = dev(qkv.reshape(3, -1))
    none.encode_and_store(t, C, 2, 1)
    assert np.array_equal(f64(t).reshape(3, 4, 32), qkv.astype(np.float64))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_part_alone(dtype):
    """One attention mixer with its own cache: a prompt, then single tokens."""
    from transformer_amd import Entry
    from transformer_amd.cache.storage import SequenceCache
    from transformer_amd.config.spec import AttentionSpec, PositionSpec
    from transformer_amd.parts import build_part
    dt = torch.float32 if dtype == "float32" else torch.bfloat16
    rd = (lambda a: P.round_bf16(a)) if dtype == "bfloat16" else (lambda a: np.asarray(a, np.float32).astype(np.float64))
    d, nh, nkv, dh = 88, 6, 3, 32
    spec = AttentionSpec(hidden=d, num_heads=nh, num_kv_heads=nkv, head_dim=dh, scale=0.2,
                         position=PositionSpec(head_dim=dh, theta=5000.0, style="half"),
                         qkv_bias=True, out_bias=True)
    part = build_part(spec, dt, DEV)
    wqkv = rd(rng.normal(size=((nh + 2 * nkv) * dh, d)) * 0.1)
    wo = rd(rng.normal(size=(d, nh * dh)) * 0.1)
    bqkv, bo = rng.normal(size=(nh + 2 * nkv) * dh) * 0.1, rng.normal(size=d)
    part.bind({"qkv.weight": dev(wqkv, dt), "out.weight": dev(wo, dt), "qkv.bias": dev(bqkv),
               "out.bias": dev(bo)})
    T = 75
    h = rd(rng.normal(size=(T, d)))
    # plain: the same chain of plain functions
    qkv = P.linear(h, wqkv, bqkv.astype(np.float32)).reshape(T, nh + 2 * nkv, dh)
    q = P.rope(qkv[:, :nh], range(T), 5000.0, "half")
    k = P.rope(qkv[:, nh:nh + nkv], range(T), 5000.0, "half")
    want = P.linear(P.attention(q, k, qkv[:, nh + nkv:], 0.2).reshape(T, -1), wo)
    cache = SequenceCache([part.cache_need()], 128, 2, dt, DEV)
    G.poison(cache)
    s = cache.alloc_slot()
    got = []
    for lo, hi in ((0, 66), (66, 67), (67, 68), (68, 75)):
        c = Ctx(cache, [Entry(s, [0] * (hi - lo))]).ctx
        delta, bias = part.run(dev(h[lo:hi], dt), c, cache, 0, True)
        got.append(f64(delta) + f64(bias))
        cache.pool.advance(s, hi - lo)
    got = np.concatenate(got)
    assert np.abs(got - (want + bo.astype(np.float32))).max() < (1e-4 if dtype == "float32" else 0.06)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_feed_forward_part_alone(dtype):
    from transformer_amd.config.spec import SwiGLUSpec
    from transformer_amd.parts import build_part
    from transformer_amd.parts.linear import Workspace
    dt = torch.float32 if dtype == "float32" else torch.bfloat16
    rd = P.round_bf16 if dtype == "bfloat16" else (lambda a: np.asarray(a, np.float32).astype(np.float64))
    d, di = 72, 200
    part = build_part(SwiGLUSpec(hidden=d, intermediate=di, bias=True), dt, DEV)
    wgu, wd = rd(rng.normal(size=(2 * di, d)) * 0.2), rd(rng.normal(size=(d, di)) * 0.2)
    bgu, bd = rng.normal(size=2 * di).astype(np.float32), rng.normal(size=d).astype(np.float32)
    part.bind({"gate_up.weight": dev(wgu, dt), "down.weight": dev(wd, dt), "gate_up.bias": dev(bgu),
               "down.bias": dev(bd)})
    h = rd(rng.normal(size=(9, d)))

    class C:
        ws = Workspace(DEV)
    delta, bias = part.run(dev(h, dt), C)
    gu = P.linear(h, wgu, bgu)
    want = P.linear(P.swiglu(gu[:, :di], gu[:, di:]), wd) + bd
    assert np.abs(f64(delta) + f64(bias) - want).max() < (1e-4 if dtype == "float32" else 0.08)


@pytest.mark.parametrize("rows", [65, 300, 1024, 1536, 1537])
def test_a_long_k_product_of_a_short_prompt_is_left_in_planes(rows):
    """The product that is added to the residual stream (`linear_delta`): 65 to 1,536 rows over
    k >= 8,192 go to the library in one batched call that leaves the parts of k as float32
    planes; more rows, or a short k, stay whole and may add themselves to the stream. Planes
    or not, the sum is the product."""
    from transformer_amd.parts.linear import Workspace, adds_in_place, library_planes, linear_delta
    n, k = 200, 8192 + 512
    g = np.random.default_rng(rows)
    a = P.round_bf16(g.normal(size=(rows, k)))
    w = P.round_bf16(g.normal(size=(n, k)) * 0.05)
    wt, at = dev(w, torch.bfloat16), dev(a, torch.bfloat16)
    planes = library_planes(rows, wt)
    assert planes == (1 if rows > 1536 else 8)              # 200 columns: few tiles of outputs at any row count
    wide = torch.empty(4096, k, dtype=torch.bfloat16, device=DEV)
    assert [library_planes(r, wide) for r in (65, 128, 384, 512, 1024, 1536, 1537, 2048)] == [8, 8, 8, 4, 4, 2, 1, 1]
    assert adds_in_place(rows, wt) == (planes == 1)
    assert library_planes(rows, dev(w[:, :4096], torch.bfloat16)) == 1            # a short k stays whole
    assert library_planes(64, wt) == 1                                           # few rows: kernels of our own
    ws = Workspace(DEV)
    want = a @ w.T
    tol = 2e-3 * np.abs(want).max()                                              # float32 sums of 8,704 products
    out = linear_delta(at, wt, ws, "t")
    assert tuple(out.shape) == ((planes, rows, n) if planes > 1 else (rows, n)) and out.dtype == torch.float32
    got = f64(out).sum(0) if planes > 1 else f64(out)
    assert np.abs(got - want).max() < tol
    if planes > 1:
        # the norm behind it adds the planes to the stream in order and normalises the sum
        from transformer_amd import kernels
        x0 = g.normal(size=(rows, n)).astype(np.float32)
        x, h = dev(x0), torch.empty(rows, n, dtype=torch.bfloat16, device=DEV)
        kernels.add_rmsnorm(x, dev(np.ones(n, np.float32)), 1e-5, h, delta=out)
        assert np.abs(f64(x) - (x0 + want)).max() < tol
        assert np.abs(f64(h) - P.rms_norm(x0 + want, np.ones(n), 1e-5)).max() < 2e-2
    else:
        x0 = g.normal(size=(rows, n)).astype(np.float32)
        x = dev(x0)
        assert linear_delta(at, wt, ws, "t", into=x) is None
        assert np.abs(f64(x) - (x0 + want)).max() < tol


# ---------------------------------------------------------------- a toy mixer with state
@dataclass(frozen=True)
class RunningSumSpec:
    hidden: int
    decay: float
    kind: str = "toy_running_sum"


def _register_toy():
    from transformer_amd import register_part
    from transformer_amd.cache.storage import StateNeed
    from transformer_amd.parts.base import Part
    from transformer_amd.weights.loader import Param

    class RunningSum(Part):
        """delta[t] = gain * s[t], s[t] = decay * s[t-1] + h[t]; s lives in the cache's
        fixed-size state of the sequence's slot."""

        def __init__(self, spec, dtype, device):
            self.spec = spec

        def params(self):
            return {"gain": Param((self.spec.hidden,), "vector")}

        def cache_need(self):
            return StateNeed((self.spec.hidden,), torch.float32)

        def run(self, h, ctx, cache, layer, writes_cache=True):
            state = cache.layer_state(layer)               # [slots, hidden]
            out = torch.empty(h.shape, dtype=torch.float32, device=h.device)
            row = 0
            for slot, n in zip(ctx.slots_host, ctx.seq_lens):
                s = state[slot].clone()
                for t in range(n):
                    s = s * self.spec.decay + h[row + t].float()
                    out[row + t] = s * self.w["gain"]
                state[slot] = s
                row += n
            return out, None

    register_part("toy_running_sum", RunningSum)


def test_a_toy_mixer_with_state_is_registered_built_and_stepped():
    from transformer_amd import Entry
    from transformer_amd.config.spec import BlockSpec, ModelSpec, NormSpec, RunSpec, SwiGLUSpec
    from transformer_amd.engine.model import DecoderModel
    _register_toy()
    d, V = 48, 50
    llama = G.engine("A", "float32").spec.blocks[0]                 # an attention block beside it
    llama = dataclasses.replace(
        llama, norm1=NormSpec(d, 1e-5), norm2=NormSpec(d, 1e-5),
        mixer=dataclasses.replace(llama.mixer, hidden=d), ffn=SwiGLUSpec(d, 64))
    toy = BlockSpec(norm1=NormSpec(d, 1e-5), mixer=RunningSumSpec(d, 0.5), norm2=NormSpec(d, 1e-5),
                    ffn=SwiGLUSpec(d, 80))
    spec = ModelSpec(vocab=V, hidden=d, blocks=(toy, llama), schedule=(RunSpec(0), RunSpec(1), RunSpec(0)),
                     final_norm=NormSpec(d, 1e-5))
    model = DecoderModel(spec, "float32", DEV)
    g = torch.Generator().manual_seed(0)
    tensors = {n: (torch.randn(p.shape, generator=g) * (0.1 if p.role == "matrix" else 1.0)).to(DEV)
               for n, p in model.all_params().items()}
    model.bind(tensors)
    assert [type(n).__name__ for n in model.cache_needs] == ["StateNeed", "KVNeed", "StateNeed"]
    cache = model.new_cache(256, max_slots=3)
    toks = [int(t) for t in rng.integers(0, V, 40)]
    a, b = cache.alloc_slot(), cache.alloc_slot()
    whole = model.step(cache, [Entry(a, toks, range(40))]).clone()
    parts = [model.step(cache, [Entry(b, toks[:25], range(25))]).clone()]
    for t in toks[25:]:
        parts.append(model.step(cache, [Entry(b, [t], [0])]).clone())
    assert torch.allclose(torch.cat(parts), whole, atol=1e-5)        # the state carries over steps
    # the state of a slot that is given back starts from zero for its next user
    cache.free_slot(b)
    c = cache.alloc_slot()
    assert c == b
    again = model.step(cache, [Entry(c, toks, range(40))])
    assert torch.allclose(again, whole, atol=1e-5)
    # and the toy's state differs between the two runs of block 0 (two cache layers)
    assert not torch.equal(cache.layer_state(0)[a], cache.layer_state(2)[a])


@dataclass(frozen=True)
class CountedSumSpec:
    hidden: int
    decay: float
    kind: str = "toy_counted_sum"


def _register_counted_sum():
    from transformer_amd import register_part
    from transformer_amd.cache.storage import StateNeed
    from transformer_amd.parts.base import Part
    from transformer_amd.weights.loader import Param

    class CountedSum(Part):
        """The running sum again, as a part that may be recorded: single tokens are served by
        tensor operations over the step's slots on the device (no host loop), and the mixer
        needs two things of different types, named in a list: the sum (float32 [hidden]) and
        the number of tokens it has seen (int64 [1])."""
        graph_safe = True

        def __init__(self, spec, dtype, device):
            self.spec = spec

        def params(self):
            return {"gain": Param((self.spec.hidden,), "vector")}

        def cache_need(self):
            return [StateNeed((self.spec.hidden,), torch.float32), StateNeed((1,), torch.int64)]

        def run(self, h, ctx, cache, layer, writes_cache=True):
            sums, counts = (cache.layer_state(l) for l in layer)      # one cache layer per need
            if ctx.all_single:
                slots = ctx.slots.long()
                s = sums.index_select(0, slots) * self.spec.decay + h.float()
                sums.index_copy_(0, slots, s)
                counts.index_add_(0, slots, torch.ones_like(slots)[:, None])
                return s * self.w["gain"], None
            out = torch.empty(h.shape, dtype=torch.float32, device=h.device)
            row = 0
            for slot, n in zip(ctx.slots_host, ctx.seq_lens):
                s = sums[slot].clone()
                for t in range(n):
                    s = s * self.spec.decay + h[row + t].float()
                    out[row + t] = s * self.w["gain"]
                sums[slot] = s
                counts[slot] += n
                row += n
            return out, None

    register_part("toy_counted_sum", CountedSum)


def test_rows_that_fill_a_recorded_step_touch_nobodys_state():
    """Five sequences step as a recorded batch of six; the sixth row belongs to nobody. Its slot
    is the spare row of the state tables, so slot 0 (live, and the lowest index) keeps exactly
    the state that eager steps of five give it, and its token count is its own. The recording is
    tried twice before it is trusted; the state is put back before every try, so trying leaves no
    trace either."""
    from transformer_amd import Entry
    from transformer_amd.config.spec import BlockSpec, ModelSpec, NormSpec, RunSpec, SwiGLUSpec
    from transformer_amd.engine.model import DecoderModel
    _register_counted_sum()
    d, V = 48, 50
    llama = G.engine("A", "float32").spec.blocks[0]
    llama = dataclasses.replace(
        llama, norm1=NormSpec(d, 1e-5), norm2=NormSpec(d, 1e-5),
        mixer=dataclasses.replace(llama.mixer, hidden=d), ffn=SwiGLUSpec(d, 64))
    toy = BlockSpec(norm1=NormSpec(d, 1e-5), mixer=CountedSumSpec(d, 0.75), norm2=NormSpec(d, 1e-5),
                    ffn=SwiGLUSpec(d, 80))
    spec = ModelSpec(vocab=V, hidden=d, blocks=(toy, llama), schedule=(RunSpec(0), RunSpec(1), RunSpec(0)),
                     final_norm=NormSpec(d, 1e-5))
    model = DecoderModel(spec, "float32", DEV)
    assert model._graph_safe
    assert model.cache_layer == [(0, 1), 2, (3, 4)]
    g = torch.Generator().manual_seed(1)
    model.bind({n: (torch.randn(p.shape, generator=g) * (0.1 if p.role == "matrix" else 1.0)).to(DEV)
                for n, p in model.all_params().items()})
    toks = [[int(t) for t in rng.integers(0, V, 40)] for _ in range(5)]
    starts = [3, 9, 1, 17, 12]

    def run(use_graphs):
        model.use_graphs = use_graphs
        cache = model.new_cache(1024, max_slots=6)
        slots = [cache.alloc_slot() for _ in toks]
        assert slots[0] == 0
        out = [model.step(cache, [Entry(s, t[:n], [n - 1]) for s, t, n in zip(slots, toks, starts)]).clone()]
        for step in range(20):
            out.append(model.step(cache, [Entry(s, [t[n + step]], [0]) for s, t, n in zip(slots, toks, starts)]).clone())
        state = [cache.layer_state(l).clone() for l in range(5) if l != 2]
        return torch.cat(out), state, cache

    eager, state_e, _ = run(False)
    replay, state_r, cache = run(True)
    assert [k[0] for k in cache.graphs] == [6]                     # five sequences, recorded as six
    assert torch.equal(eager, replay)
    for a, b in zip(state_e, state_r):
        assert torch.equal(a[:5], b[:5])                           # every live slot, slot 0 among them
    counts = cache.layer_state(1)
    assert counts[:5, 0].tolist() == [n + 20 for n in starts]
    assert int(counts[5, 0]) == 0 and int(counts[cache.spare_slot, 0]) == 20   # the filling row's own
    # whole prompts give the same logits as the steps did: the state carried over
    whole = model.step(cache, [Entry(cache.alloc_slot(), toks[0][:starts[0] + 20], range(starts[0] - 1, starts[0] + 20))])
    assert torch.allclose(whole, replay.view(21, 5, V)[:, 0], atol=1e-5)


@dataclass(frozen=True)
class LatentSpec:
    hidden: int
    latent: int
    kind: str = "toy_latent"


def _register_latent():
    from transformer_amd import register_part
    from transformer_amd.cache.storage import KVNeed
    from transformer_amd.parts.base import Part
    from transformer_amd.weights.loader import Param

    class LatentAttention(Part):
        """Keeps ONE row of `latent` numbers per token (no values, a width that is no head size
        of any kernel) and derives keys and values from it when it reads: c = h.Wc; scores
        q.c over the cached rows, output (softmax.c).Wo. The cache is asked for keys only
        (`value_dim=0`) and is read and written with tensor operations through `layer_kv`."""

        def __init__(self, spec, dtype, device):
            self.spec = spec

        def params(self):
            s = self.spec
            return {"c.weight": Param((s.latent, s.hidden), "matrix"), "q.weight": Param((s.latent, s.hidden), "matrix"),
                    "o.weight": Param((s.hidden, s.latent), "matrix")}

        def cache_need(self):
            return KVNeed(1, self.spec.latent, value_dim=0)

        def run(self, h, ctx, cache, layer, writes_cache=True):
            rows, values, group = cache.layer_kv(layer)           # [pages, 1, 64, latent], [pages, 1, 0, 64]
            assert values.numel() == 0
            flat = rows.view(-1, self.spec.latent)                # page * 64 + offset, as `dest` counts
            hf = h.float()
            c = hf @ self.w["c.weight"].float().T
            q = hf @ self.w["q.weight"].float().T
            flat[ctx.kv[group].dest.long()] = c.to(rows.dtype)
            out = torch.empty(h.shape[0], self.spec.hidden, device=h.device)
            row = 0
            for b, (slot, n) in enumerate(zip(ctx.slots_host, ctx.seq_lens)):
                p0 = cache.length(slot)
                pages = torch.tensor(cache.pool.pages(slot, group), device=h.device)
                seen = rows[pages, 0].reshape(-1, self.spec.latent)[:p0 + n].float()
                for t in range(n):
                    s = (seen[:p0 + t + 1] @ q[row + t]) / self.spec.latent ** 0.5
                    out[row + t] = (torch.softmax(s, 0) @ seen[:p0 + t + 1]) @ self.w["o.weight"].float().T
                row += n
            return out, None

    register_part("toy_latent", LatentAttention)


def test_a_mixer_that_keeps_one_row_per_token_adds_a_need_not_a_cache():
    """A cache group of keys only, 24 wide: the pool, the tables, the spare page and the
    release of slots serve it as they serve attention; whole prompts equal single tokens."""
    from transformer_amd import Entry
    from transformer_amd.config.spec import BlockSpec, ModelSpec, NormSpec, RunSpec, SwiGLUSpec
    from transformer_amd.engine.model import DecoderModel
    _register_latent()
    d, V, L = 40, 30, 24
    llama = G.engine("A", "float32").spec.blocks[0]
    llama = dataclasses.replace(
        llama, norm1=NormSpec(d, 1e-5), norm2=NormSpec(d, 1e-5),
        mixer=dataclasses.replace(llama.mixer, hidden=d), ffn=SwiGLUSpec(d, 64))
    toy = BlockSpec(norm1=NormSpec(d, 1e-5), mixer=LatentSpec(d, L), norm2=NormSpec(d, 1e-5), ffn=SwiGLUSpec(d, 48))
    spec = ModelSpec(vocab=V, hidden=d, blocks=(toy, llama), schedule=(RunSpec(0), RunSpec(1)), final_norm=NormSpec(d, 1e-5))
    model = DecoderModel(spec, "float32", DEV)
    g = torch.Generator().manual_seed(2)
    model.bind({n: (torch.randn(p.shape, generator=g) * (0.2 if p.role == "matrix" else 1.0)).to(DEV)
                for n, p in model.all_params().items()})
    cache = model.new_cache(512, max_slots=3)
    assert [(n.head_dim, n.value_dim) for n in cache.kv_groups] == [(L, 0), (16, 16)]
    assert cache.keys[0].shape[-1] == L and cache.values[0].numel() == 0
    G.poison(cache)
    toks = [[int(t) for t in rng.integers(0, V, n)] for n in (150, 70)]
    a, b, c = (cache.alloc_slot() for _ in range(3))
    whole = [model.step(cache, [Entry(s, t, range(len(t)))]).clone() for s, t in zip((a, b), toks)]
    # the two together from unequal prompts, then single tokens; the shorter one ends earlier
    got = [[], []]
    cache.free_slot(a)
    cache.free_slot(b)
    a, b = cache.alloc_slot(), cache.alloc_slot()
    out = model.step(cache, [Entry(a, toks[0][:100], range(100)), Entry(b, toks[1][:30], range(30))]).clone()
    got[0].append(out[:100]); got[1].append(out[100:])
    for i in range(50):
        es = [Entry(a, [toks[0][100 + i]], [0])] + ([Entry(b, [toks[1][30 + i]], [0])] if i < 40 else [])
        out = model.step(cache, es).clone()
        got[0].append(out[:1])
        if i < 40:
            got[1].append(out[1:])
    for k in range(2):
        assert torch.allclose(torch.cat(got[k]), whole[k], atol=2e-5)
    cache.pool.check()


def test_a_schedule_may_repeat_a_block_and_borrow_a_cache():
    """Block 1 runs twice; its second run reads the keys and values that its first
    run stored. The plain side computes the same thing with plain functions."""
    from transformer_amd import Entry
    from transformer_amd.config.spec import RunSpec
    from transformer_amd.engine.model import DecoderModel
    base = G.engine("A", "float32")
    ref = G.plain("A", "float32")
    spec = dataclasses.replace(base.spec, schedule=(RunSpec(0), RunSpec(1), RunSpec(1, cache_of=1)))
    model = DecoderModel(spec, "float32", DEV)
    tensors = {"embed.weight": base.w["embed"], "head.weight": base.w["head"],
               "final_norm.weight": base.final_norm.w["weight"]}
    for i, b in enumerate(base.blocks):
        for cname, child in b.children().items():
            for n, t in child.w.items():
                tensors[f"blocks.{i}.{cname}.{n}"] = t
    model.bind(tensors)
    assert model.cache_layer == [0, 1, 1] and len(model.cache_needs) == 2
    toks = G.tokens("A", 70, 9)
    # plain: block 0, block 1, then block 1 again with k, v taken from its first run
    w = ref.w
    x = w["model.embed_tokens.weight"][toks]
    pos = np.arange(70)
    x = ref.block(0, x, pos)
    p = "model.layers.1."
    h = P.rms_norm(x, w[p + "input_layernorm.weight"], ref.eps)
    k1 = P.rope(P.linear(h, w[p + "self_attn.k_proj.weight"]).reshape(70, ref.nkvh, ref.dh), pos, ref.theta, "half")
    v1 = P.linear(h, w[p + "self_attn.v_proj.weight"]).reshape(70, ref.nkvh, ref.dh)
    x = ref.block(1, x, pos)
    h = P.rms_norm(x, w[p + "input_layernorm.weight"], ref.eps)
    q2 = P.rope(P.linear(h, w[p + "self_attn.q_proj.weight"]).reshape(70, ref.nh, ref.dh), pos, ref.theta, "half")
    x = x + P.linear(P.attention(q2, k1, v1, ref.scale).reshape(70, -1), w[p + "self_attn.o_proj.weight"])
    h = P.rms_norm(x, w[p + "post_attention_layernorm.weight"], ref.eps)
    x = x + P.linear(P.swiglu(P.linear(h, w[p + "mlp.gate_proj.weight"]), P.linear(h, w[p + "mlp.up_proj.weight"])),
                     w[p + "mlp.down_proj.weight"])
    want = P.linear(P.rms_norm(x, w["model.norm.weight"], ref.eps), w["lm_head.weight"])
    cache = model.new_cache(128)
    s = cache.alloc_slot()
    got = [model.step(cache, [Entry(s, toks[:50], range(50))]).cpu().numpy().copy()]
    for t in toks[50:]:
        got.append(model.step(cache, [Entry(s, [t], [0])]).cpu().numpy().copy())
    assert np.abs(np.concatenate(got) - want).max() < 2e-5


# ---------------------------------------------------------------- a toy position encoding and a toy routed feed-forward
@dataclass(frozen=True)
class DecaySpec:
    """q of position p is multiplied by base^p and k by base^-p: a score between positions m >= n
    is scaled by base^(m-n). Not a rotation, so it has no ``rotation_of``."""
    head_dim: int
    base: float
    kind: str = "toy_decay"


@dataclass(frozen=True)
class Top1Spec:
    hidden: int
    intermediate: int
    experts: int
    kind: str = "toy_top1"


def _register_toys_2():
    from transformer_amd import kernels, register_part
    from transformer_amd.parts.base import Part
    from transformer_amd.parts.linear import linear
    from transformer_amd.weights.loader import Param

    class Decay(Part):
        def __init__(self, spec, dtype, device):
            self.spec = spec

        def encode_and_store(self, qkv, ctx, nq, nkv, dest=None, kcache=None, vcache=None, bias=None):
            assert bias is None
            dh = self.spec.head_dim
            f = torch.pow(torch.tensor(self.spec.base, dtype=torch.float64, device=qkv.device),
                          ctx.positions.double())[:, None]
            heads = qkv.view(qkv.shape[0], nq + 2 * nkv, dh)
            heads[:, :nq] = (heads[:, :nq].double() * f[:, None]).to(qkv.dtype)
            heads[:, nq:nq + nkv] = (heads[:, nq:nq + nkv].double() / f[:, None]).to(qkv.dtype)
            return kernels.rope_kv_write(qkv, nq, nkv, dh, None, False, dest, kcache, vcache, None)

    class Top1(Part):
        """Every token goes to the expert whose router row gives the highest score."""

        def __init__(self, spec, dtype, device):
            self.spec, self.dtype = spec, dtype

        def params(self):
            s = self.spec
            p = {"router.weight": Param((s.experts, s.hidden), "matrix")}
            for e in range(s.experts):
                p[f"experts.{e}.gate_up.weight"] = Param((2 * s.intermediate, s.hidden), "matrix")
                p[f"experts.{e}.down.weight"] = Param((s.hidden, s.intermediate), "matrix")
            return p

        def run(self, h, ctx):
            s, nt = self.spec, h.shape[0]
            score = linear(h, self.w["router.weight"], torch.empty(nt, s.experts, device=h.device))
            choice = score.argmax(dim=1)
            delta = torch.zeros(nt, s.hidden, device=h.device)
            for e in range(s.experts):
                rows = (choice == e).nonzero().flatten()
                if rows.numel() == 0:
                    continue
                he = h.index_select(0, rows).contiguous()
                gu = linear(he, self.w[f"experts.{e}.gate_up.weight"],
                            torch.empty(len(rows), 2 * s.intermediate, dtype=self.dtype, device=h.device))
                act = kernels.swiglu(gu, torch.empty(len(rows), s.intermediate, dtype=self.dtype, device=h.device))
                delta[rows] = linear(act, self.w[f"experts.{e}.down.weight"],
                                     torch.empty(len(rows), s.hidden, device=h.device))
            return delta, None

    register_part("toy_decay", Decay)
    register_part("toy_top1", Top1)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_toy_position_encoding_and_a_routed_feed_forward(dtype):
    """Two blocks: attention with a position encoding that is no rotation (so single tokens take
    the separate encode-and-store path) over a routed feed-forward, then a Llama block. Whole
    prompts, single tokens and a batch of two agree with plain functions."""
    from transformer_amd import Entry
    from transformer_amd.config.spec import (AttentionSpec, BlockSpec, ModelSpec, NormSpec, PositionSpec,
                                             RunSpec, SwiGLUSpec)
    from transformer_amd.engine.model import DecoderModel
    _register_toys_2()
    d, V, nh, nkv, dh, di, E, base = 64, 40, 4, 2, 32, 48, 3, 1.01
    toy = BlockSpec(norm1=NormSpec(d, 1e-5),
                    mixer=AttentionSpec(d, nh, nkv, dh, 1 / math.sqrt(dh), DecaySpec(dh, base)),
                    norm2=NormSpec(d, 1e-6), ffn=Top1Spec(d, di, E))
    plain_block = BlockSpec(norm1=NormSpec(d, 1e-5),
                            mixer=AttentionSpec(d, nh, nkv, dh, 1 / math.sqrt(dh), PositionSpec(dh, 1e4, "half")),
                            norm2=NormSpec(d, 1e-5), ffn=SwiGLUSpec(d, di))
    spec = ModelSpec(vocab=V, hidden=d, blocks=(toy, plain_block), schedule=(RunSpec(0), RunSpec(1)),
                     final_norm=NormSpec(d, 1e-5))
    model = DecoderModel(spec, dtype, DEV)
    assert not model.blocks[0].graph_safe
    g = np.random.default_rng(3)
    host = {}
    for n, p_ in model.all_params().items():
        a = g.normal(size=p_.shape) * (0.15 if p_.role == "matrix" else 0.1) + (0 if p_.role == "matrix" else 1)
        host[n] = P.round_bf16(a) if (dtype == "bfloat16" and p_.role == "matrix") else a.astype(np.float32).astype(np.float64)
    DT = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    model.bind({n: dev(a, DT if model.all_params()[n].role == "matrix" else torch.float32) for n, a in host.items()})

    def plain(toks):
        r = (lambda a: P.round_bf16(a)) if dtype == "bfloat16" else (lambda a: a)
        T = len(toks)
        pos = np.arange(T)
        x = host["embed.weight"][toks]
        # block 0
        pre = "blocks.0."
        h = r(P.rms_norm(x, host[pre + "norm1.weight"], 1e-5))
        qkv = r(P.linear(h, host[pre + "mixer.qkv.weight"])).reshape(T, nh + 2 * nkv, dh)
        f = base ** pos.astype(np.float64)
        q = r(qkv[:, :nh] * f[:, None, None])
        k = r(qkv[:, nh:nh + nkv] / f[:, None, None])
        o = r(P.attention(q, k, qkv[:, nh + nkv:], 1 / math.sqrt(dh)))
        x = x + P.linear(o.reshape(T, -1), host[pre + "mixer.out.weight"])
        h = r(P.rms_norm(x, host[pre + "norm2.weight"], 1e-6))
        choice = np.argmax(P.linear(h, host[pre + "ffn.router.weight"]), axis=1)
        delta = np.zeros_like(x)
        for t in range(T):
            e = choice[t]
            gu = r(P.linear(h[t:t + 1], host[pre + f"ffn.experts.{e}.gate_up.weight"]))
            delta[t] = P.linear(r(P.swiglu(gu[:, :di], gu[:, di:])), host[pre + f"ffn.experts.{e}.down.weight"])[0]
        x = x + delta
        # block 1: the Llama block
        pre = "blocks.1."
        h = r(P.rms_norm(x, host[pre + "norm1.weight"], 1e-5))
        qkv = r(P.linear(h, host[pre + "mixer.qkv.weight"])).reshape(T, nh + 2 * nkv, dh)
        q = r(P.rope(qkv[:, :nh], pos, 1e4, "half"))
        k = r(P.rope(qkv[:, nh:nh + nkv], pos, 1e4, "half"))
        o = r(P.attention(q, k, qkv[:, nh + nkv:], 1 / math.sqrt(dh)))
        x = x + P.linear(o.reshape(T, -1), host[pre + "mixer.out.weight"])
        h = r(P.rms_norm(x, host[pre + "norm2.weight"], 1e-5))
        gu = r(P.linear(h, host[pre + "ffn.gate_up.weight"]))
        x = x + P.linear(r(P.swiglu(gu[:, :di], gu[:, di:])), host[pre + "ffn.down.weight"])
        return P.linear(r(P.rms_norm(x, host["final_norm.weight"], 1e-5)), host["head.weight"]), choice

    tol = 3e-5 if dtype == "float32" else 6e-2
    cache = model.new_cache(512, max_slots=3)
    ta = [int(t) for t in g.integers(0, V, 90)]
    tb = [int(t) for t in g.integers(0, V, 37)]
    want_a, choice_a = plain(ta)
    want_b, _ = plain(tb)
    assert len(set(choice_a.tolist())) == E                  # every expert is used
    a, b = cache.alloc_slot(), cache.alloc_slot()
    whole = f64(model.step(cache, [Entry(a, ta, range(90))]))
    assert np.abs(whole - want_a).max() < tol
    cache.reset_slot(a)
    # the two together, unequal, then single tokens for both (b ends earlier)
    got_a = [f64(model.step(cache, [Entry(a, ta[:60], range(60)), Entry(b, tb[:30], range(30))]))]
    got_b = [got_a[0][60:]]
    got_a[0] = got_a[0][:60]
    for i in range(30):
        ents = [Entry(a, [ta[60 + i]], [0])]
        if 30 + i < len(tb):
            ents.append(Entry(b, [tb[30 + i]], [0]))
        out = f64(model.step(cache, ents))
        got_a.append(out[:1])
        if len(ents) == 2:
            got_b.append(out[1:])
    assert np.abs(np.concatenate(got_a) - want_a).max() < tol
    assert np.abs(np.concatenate(got_b) - want_b).max() < tol


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_windowed_layer_beside_a_full_one_has_a_cache_group_of_its_own(dtype):
    """Layer 0 reads a window of 37 keys, layer 1 all of them: two cache groups, each with its
    page tables. 150 tokens, so the window's start crosses page edges; whole, then one by one."""
    from transformer_amd import Entry
    from transformer_amd.config.spec import (AttentionSpec, BlockSpec, ModelSpec, NormSpec, PositionSpec,
                                             RunSpec, SwiGLUSpec)
    from transformer_amd.engine.model import DecoderModel
    d, V, nh, nkv, dh, di, W = 64, 40, 4, 2, 32, 48, 37
    def block(window):
        return BlockSpec(norm1=NormSpec(d, 1e-5),
                         mixer=AttentionSpec(d, nh, nkv, dh, 1 / math.sqrt(dh), PositionSpec(dh, 1e4, "half"),
                                             window=window),
                         norm2=NormSpec(d, 1e-5), ffn=SwiGLUSpec(d, di))
    spec = ModelSpec(vocab=V, hidden=d, blocks=(block(W), block(None)), schedule=(RunSpec(0), RunSpec(1)),
                     final_norm=NormSpec(d, 1e-5))
    model = DecoderModel(spec, dtype, DEV)
    g = np.random.default_rng(11)
    host = {}
    for n, p_ in model.all_params().items():
        a = g.normal(size=p_.shape) * (0.15 if p_.role == "matrix" else 0.1) + (0 if p_.role == "matrix" else 1)
        host[n] = P.round_bf16(a) if (dtype == "bfloat16" and p_.role == "matrix") else a.astype(np.float32).astype(np.float64)
    DT = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    model.bind({n: dev(a, DT if model.all_params()[n].role == "matrix" else torch.float32) for n, a in host.items()})
    cache = model.new_cache(512, max_slots=2)
    assert len(cache.kv_groups) == 2 and cache.kv_groups[0].window == W and cache.kv_groups[1].window is None
    r = (lambda a: P.round_bf16(a)) if dtype == "bfloat16" else (lambda a: a)
    def plain(toks):
        T = len(toks)
        pos = np.arange(T)
        x = host["embed.weight"][toks]
        for i, window in enumerate((W, None)):
            pre = f"blocks.{i}."
            h = r(P.rms_norm(x, host[pre + "norm1.weight"], 1e-5))
            qkv = r(P.linear(h, host[pre + "mixer.qkv.weight"])).reshape(T, nh + 2 * nkv, dh)
            q = r(P.rope(qkv[:, :nh], pos, 1e4, "half"))
            k = r(P.rope(qkv[:, nh:nh + nkv], pos, 1e4, "half"))
            o = r(P.attention(q, k, qkv[:, nh + nkv:], 1 / math.sqrt(dh), window=window))
            x = x + P.linear(o.reshape(T, -1), host[pre + "mixer.out.weight"])
            h = r(P.rms_norm(x, host[pre + "norm2.weight"], 1e-5))
            gu = r(P.linear(h, host[pre + "ffn.gate_up.weight"]))
            x = x + P.linear(r(P.swiglu(gu[:, :di], gu[:, di:])), host[pre + "ffn.down.weight"])
        return P.linear(r(P.rms_norm(x, host["final_norm.weight"], 1e-5)), host["head.weight"])

    T = 150
    toks = [int(t) for t in g.integers(0, V, T)]
    want = plain(toks)
    tol = 3e-5 if dtype == "float32" else 6e-2
    a, b = cache.alloc_slot(), cache.alloc_slot()
    for t_ in cache.keys + cache.values:               # whatever a page held before must not matter
        t_.fill_(float("nan"))
    whole = f64(model.step(cache, [Entry(a, toks, range(T))]))
    assert np.abs(whole - want).max() < tol
    parts = [f64(model.step(cache, [Entry(b, toks[:70], range(70))]))]
    for t in toks[70:]:
        parts.append(f64(model.step(cache, [Entry(b, [t], [0])])))
    assert np.abs(np.concatenate(parts) - want).max() < tol

    # pages that have left the window go back after every step, so with a bound on a step's
    # tokens the windowed group gets by with far less storage than the full one
    from transformer_amd.cache.pool import CacheFull
    small = model.new_cache(1024, max_slots=2, max_step_tokens=160)
    assert small.group_pages == [2 * (W // 64 + 3) + 2, 16]
    assert [k.shape[1] for k in small.keys] == [p + 1 for p in small.group_pages]   # and a spare page each
    for t_ in small.keys + small.values:
        t_.fill_(float("nan"))
    T2 = 330
    two = [[int(t) for t in g.integers(0, V, T2)] for _ in range(2)]
    wants = [plain(t) for t in two]
    sl = [small.alloc_slot(), small.alloc_slot()]
    got = [[], []]
    out = f64(model.step(small, [Entry(sl[0], two[0][:70], range(70)), Entry(sl[1], two[1][:61], range(61))]))
    got[0].append(out[:70]); got[1].append(out[70:])
    for t in range(61, T2):
        es = [Entry(sl[1], [two[1][t]], [0])] if t < 70 else \
            [Entry(sl[0], [two[0][t]], [0]), Entry(sl[1], [two[1][t]], [0])]
        out = f64(model.step(small, es))
        for j, e in enumerate(es):
            got[sl.index(e.slot)].append(out[j:j + 1])
        assert small.pool.held_pages(0) <= 2 * (W // 64 + 2)
    small.pool.check()
    for k_ in range(2):
        assert np.abs(np.concatenate(got[k_]) - wants[k_]).max() < tol
    pages = small.pool.pages(sl[0], 0)
    assert pages[0] < 0 and pages[-1] >= 0 and len(pages) == -(-T2 // 64)
    small.free_slot(sl[1])
    c = small.alloc_slot()
    with pytest.raises(CacheFull, match="cache group 0"):     # 600 tokens in one step break the promise
        model.step(small, [Entry(c, [1] * 600, [599])])
    small.pool.check()


@dataclass(frozen=True)
class ScaleSpec:
    kind = "toy_scale"
    factor: float


@dataclass(frozen=True)
class SoftCapSpec:
    kind = "toy_softcap"
    cap: float


def _register_model_level_toys():
    from transformer_amd import register_part
    from transformer_amd.parts.base import Part

    class Scale(Part):
        graph_safe = True

        def __init__(self, spec, dtype, device):
            self.factor = spec.factor

        def run(self, x, ctx):
            x.mul_(self.factor)

    class SoftCap(Part):
        graph_safe = True

        def __init__(self, spec, dtype, device):
            self.cap = spec.cap

        def run(self, logits, ctx):
            logits.div_(self.cap).tanh_().mul_(self.cap)

    register_part("toy_scale", lambda spec, dtype, device: Scale(spec, dtype, device))
    register_part("toy_softcap", lambda spec, dtype, device: SoftCap(spec, dtype, device))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_parts_after_the_embedding_and_on_the_logits_and_the_dump_hook(dtype):
    """An architecture with a scaled embedding or capped logits names a part for it in its
    ModelSpec; the model's forward pass is not edited. The same weights with the scale folded
    into the embedding table, and the cap applied by hand, give the same logits. `dump`
    receives every intermediate of a step in order."""
    from transformer_amd import Entry
    from transformer_amd.engine.model import DecoderModel
    _register_model_level_toys()
    base = G.engine("A", dtype)                     # untied output matrix
    spec = dataclasses.replace(base.spec, after_embed=ScaleSpec(4.0), on_logits=SoftCapSpec(3.0))
    hooked = DecoderModel(spec, dtype, DEV)
    hooked.bind(dict(base.tensors))
    plain = DecoderModel(base.spec, dtype, DEV)
    scaled = dict(base.tensors)
    assert scaled["embed.weight"].data_ptr() != scaled["head.weight"].data_ptr()
    scaled["embed.weight"] = base.tensors["embed.weight"] * 4.0      # exact in both dtypes
    plain.bind(scaled)
    toks = [int(t) for t in rng.integers(0, base.spec.vocab, 70)]
    got, want = [], []
    for model, into in ((hooked, got), (plain, want)):
        cache = model.new_cache(256, max_slots=2)
        slot = cache.alloc_slot()
        into.append(model.step(cache, [Entry(slot, toks[:66], [0, 65])]).clone())
        for t in toks[66:]:                                       # recorded steps run the parts too
            into.append(model.step(cache, [Entry(slot, [t], [0])]).clone())
    got, want = torch.cat(got), torch.cat(want)
    assert torch.allclose(got, 3.0 * torch.tanh(want / 3.0), atol=2e-6 if dtype == "float32" else 1e-5)
    assert got.abs().max() <= 3.0
    seen = []
    hooked.dump = lambda name, t: seen.append((name, tuple(t.shape), t.float().clone()))
    cache = hooked.new_cache(256, max_slots=1)
    last = hooked.step(cache, [Entry(cache.alloc_slot(), toks[:5], [4])]).clone()
    hooked.dump = None
    names = [n for n, _, _ in seen]
    runs = len(base.spec.schedule)
    assert names == ["embed"] + [f"run.{i}" for i in range(runs)] + ["final_norm", "logits"]
    assert seen[0][1] == (5, base.spec.hidden) and seen[-1][1] == (1, base.spec.vocab)
    assert torch.equal(seen[-1][2], last)
    emb = base.tensors["embed.weight"].float()[toks[:5]] * 4.0
    assert torch.equal(seen[0][2], emb)                            # the embedding after its part


def test_timers_per_kind_of_part():
    """With `model.timers` set a step records GPU events around the embedding, every norm, mixer
    and feed-forward and the output matrix, and gives the same logits as without."""
    import transformer_amd as ta
    model = G.engine("B", "bfloat16")
    toks = G.tokens("B", 40, 3)
    cache = model.new_cache(256, max_slots=2)
    a, b = cache.alloc_slot(), cache.alloc_slot()
    plain = [model.step(cache, [ta.Entry(a, toks[:39], [38])]).clone(), model.step(cache, [ta.Entry(a, toks[39:], [0])]).clone()]
    model.timers = ta.PartTimers()
    timed = [model.step(cache, [ta.Entry(b, toks[:39], [38])]).clone(), model.step(cache, [ta.Entry(b, toks[39:], [0])]).clone()]
    table = model.timers.table()
    model.timers = None
    runs = len(model.spec.schedule)
    assert set(table) == {"embed", "norm", "mixer", "ffn", "head"}
    assert table["embed"][0] == 2 and table["head"][0] == 2
    assert table["mixer"][0] == 2 * runs and table["ffn"][0] == 2 * runs
    # the prompt runs every norm as a kernel of its own; the single token leaves most to the products
    assert 2 * runs + 1 + 2 <= table["norm"][0] <= 2 * (2 * runs + 1)
    assert all(ms > 0 for _, ms in table.values())
    assert torch.equal(timed[0], plain[0])
    assert torch.allclose(timed[1], plain[1], atol=2e-2)         # recorded or eager: the same kernels


def test_unknown_part_kind_is_named():
    from transformer_amd.parts import PartError, build_part

    @dataclass(frozen=True)
    class Odd:
        kind: str = "no_such_part"
    with pytest.raises(PartError, match="no_such_part"):
        build_part(Odd(), torch.float32, DEV)
