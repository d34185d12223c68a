"""Plain, slow Llama decoder used as the oracle of the test-suite.

Whole sequences, no cache, NumPy float64 arithmetic, one function per part.
It shares no code with ``transformer_amd``: it has its own safetensors reader,
its own reading of config.json and its own formulas, written from the call
order of the reference's step function.

The reference keeps every formula inside an external operator crate, so the
formulas here are pinned by the tests in ``test_plain_*.py`` (library special
cases and invariants), not by the reference's text alone.
"""
from __future__ import annotations

import json
import struct
from pathlib import Path

import numpy as np


# --------------------------------------------------------------------------
# files
# --------------------------------------------------------------------------
def read_safetensors(path) -> dict:
    """name -> float64 ndarray (F32, F16 and BF16 payloads) or int64 for ints."""
    raw = Path(path).read_bytes()
    (hlen,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8:8 + hlen])
    body = memoryview(raw)[8 + hlen:]
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        lo, hi = info["data_offsets"]
        buf = body[lo:hi]
        dt = info["dtype"]
        if dt == "F32":
            a = np.frombuffer(buf, dtype="<f4").astype(np.float64)
        elif dt == "F16":
            a = np.frombuffer(buf, dtype="<f2").astype(np.float64)
        elif dt == "BF16":
            u = np.frombuffer(buf, dtype="<u2").astype(np.uint32) << 16
            a = u.view(np.float32).astype(np.float64)
        elif dt == "F64":
            a = np.frombuffer(buf, dtype="<f8").copy()
        elif dt in ("I32", "I64"):
            a = np.frombuffer(buf, dtype="<i4" if dt == "I32" else "<i8").astype(np.int64)
        else:
            raise ValueError(f"plain reader: dtype {dt} of {name}")
        out[name] = a.reshape(info["shape"])
    return out


def round_bf16(a: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even to bfloat16, returned as float64."""
    f = np.asarray(a, dtype=np.float32)
    u = f.view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32).astype(np.float64).reshape(f.shape)


# --------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------
def rms_norm(x, w, eps):
    """y = x * rsqrt(mean(x^2) + eps) * w over the last axis.

    Call sites: models/llama/common/src/compute.rs:206-207 (before attention),
    :274-275 (before the feed-forward), :358-363 (output norm); the argument
    struct with ``epsilon`` is filled at compute.rs:396-423.
    """
    x = np.asarray(x, dtype=np.float64)
    ms = np.mean(x * x, axis=-1, keepdims=True)
    return x / np.sqrt(ms + eps) * np.asarray(w, dtype=np.float64)


def linear(x, w, bias=None):
    """y = x @ w.T (+ bias); weights are stored [out, in] and used transposed.

    models/llama/common/src/lib.rs:168-180 (the computation view is the
    transpose of the stored [row, col] matrix); mat_mul call sites
    compute.rs:222, :270, :283, :292, :365. The bias enters as beta=1 over a
    broadcast copy of it (compute.rs:213-222).
    """
    y = np.asarray(x, dtype=np.float64) @ np.asarray(w, dtype=np.float64).T
    if bias is not None:
        y = y + np.asarray(bias, dtype=np.float64)
    return y


def rope_inv_freq(head_dim, theta):
    """f_j = theta^(-2j/head_dim), j in [0, head_dim/2), rounded to float32.

    theta is an f32 field of the model description
    (models/llama/common/src/lib.rs:39) and reaches the operator next to the
    sin/cos tables of shape [2, nctx, dh] (compute.rs:41-53, :474-484).
    """
    j = np.arange(head_dim // 2, dtype=np.float64)
    return (float(theta) ** (-2.0 * j / head_dim)).astype(np.float32)


def rope(t, positions, theta, style):
    """Rotate pairs of ``t`` [T, heads, dh] by angle pos * f_j.

    Applied to q and to k, in place, before the cache write
    (compute.rs:232-233); positions of a request are pos .. pos+seq_len
    (compute.rs:188-198). The angle is formed in float32 (position times the
    float32 frequency), its sine and cosine are then taken exactly.

    style "half":        pair (t[j], t[j + dh/2])   (safetensors convention)
    style "interleaved": pair (t[2j], t[2j + 1])    (llama-GGUF convention,
                         docs/user-guide/doc.md:133 vs :139: only qwen2 needs
                         the extra permute-qk conversion)
    """
    t = np.asarray(t, dtype=np.float64)
    dh = t.shape[-1]
    f = rope_inv_freq(dh, theta)
    ang = (np.asarray(positions, dtype=np.float32)[:, None] * f[None, :]).astype(np.float32)
    c = np.cos(ang.astype(np.float64))[:, None, :]
    s = np.sin(ang.astype(np.float64))[:, None, :]
    out = np.empty_like(t)
    if style == "half":
        u, v = t[..., : dh // 2], t[..., dh // 2:]
        out[..., : dh // 2] = u * c - v * s
        out[..., dh // 2:] = u * s + v * c
    elif style == "interleaved":
        u, v = t[..., 0::2], t[..., 1::2]
        out[..., 0::2] = u * c - v * s
        out[..., 1::2] = u * s + v * c
    else:
        raise ValueError(style)
    return out


def attention(q, k, v, scale, first_pos=0, window=None):
    """Causal grouped-query attention of one sequence, scores materialised.

    q [T, nh, dh]; k, v [S, nkvh, dh] hold the keys of positions 0..S-1 and
    the queries sit at positions first_pos .. first_pos+T-1 (S = first_pos+T).
    Query head h reads KV head h // (nh // nkvh). Query at position p sees
    keys <= p (and > p - window when a window is given).

    models/llama/common/src/compute.rs:243-264: per request, keys 0..pos+seq
    of the cache are attended (max_att_len = pos + seq_len,
    models/llama/cuda/src/infer.rs:120); no scale and no mask are passed
    (compute.rs:511-526), so 1/sqrt(dh) and the causal mask are fixed here.
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    T, nh, dh = q.shape
    S, nkvh, _ = k.shape
    assert S == first_pos + T and nh % nkvh == 0
    group = nh // nkvh
    qpos = first_pos + np.arange(T)[:, None]
    kpos = np.arange(S)[None, :]
    visible = kpos <= qpos
    if window is not None:
        visible &= kpos > qpos - window
    out = np.empty((T, nh, v.shape[-1]))
    for h in range(nh):
        g = h // group
        s = (q[:, h, :] @ k[:, g, :].T) * scale
        s = np.where(visible, s, -np.inf)
        s = s - s.max(axis=-1, keepdims=True)
        p = np.exp(s)
        p = p / p.sum(axis=-1, keepdims=True)
        out[:, h, :] = p @ v[:, g, :]
    return out


def swiglu(gate, up):
    """silu(gate) * up with silu(z) = z / (1 + exp(-z)).

    compute.rs:286-288: gate and up are the two column halves of the merged
    gate_up product, gate first; the result replaces gate.
    """
    gate = np.asarray(gate, dtype=np.float64)
    return gate / (1.0 + np.exp(-gate)) * np.asarray(up, dtype=np.float64)


# --------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------
class PlainLlama:
    """Reads a model folder (config.json + model.safetensors) by itself."""

    def __init__(self, folder, round_activations=False):
        folder = Path(folder)
        c = json.loads((folder / "config.json").read_text())
        self.raw = c
        self.n_layers = c["num_hidden_layers"]
        self.d = c["hidden_size"]
        self.nh = c["num_attention_heads"]
        # defaults as the reference applies them to its own keys:
        # models/llama/common/src/storage.rs:54 (kv heads = heads), :55
        # (head size = d / heads), :58 (eps 1e-5), :59 (theta 1e4)
        self.nkvh = c.get("num_key_value_heads", self.nh)
        self.dh = c.get("head_dim") or self.d // self.nh
        self.di = c["intermediate_size"]
        self.vocab = c["vocab_size"]
        self.eps = c.get("rms_norm_eps", 1e-5)
        self.theta = c.get("rope_theta", 1e4)
        self.rope_style = c.get("rope_style", "half")
        self.scale = 1.0 / np.sqrt(self.dh)
        self.w = read_safetensors(folder / "model.safetensors")
        self.round_activations = round_activations

    def _r(self, a):
        return round_bf16(a) if self.round_activations else a

    def block(self, i, x, positions):
        """One pre-norm block: compute.rs:204-292 in order."""
        w, p = self.w, f"model.layers.{i}."
        T = x.shape[0]
        h = self._r(rms_norm(x, w[p + "input_layernorm.weight"], self.eps))
        q = linear(h, w[p + "self_attn.q_proj.weight"], w.get(p + "self_attn.q_proj.bias"))
        k = linear(h, w[p + "self_attn.k_proj.weight"], w.get(p + "self_attn.k_proj.bias"))
        v = linear(h, w[p + "self_attn.v_proj.weight"], w.get(p + "self_attn.v_proj.bias"))
        q = self._r(q).reshape(T, self.nh, self.dh)
        k = self._r(k).reshape(T, self.nkvh, self.dh)
        v = self._r(v).reshape(T, self.nkvh, self.dh)
        q = self._r(rope(q, positions, self.theta, self.rope_style))
        k = self._r(rope(k, positions, self.theta, self.rope_style))
        o = self._r(attention(q, k, v, self.scale)).reshape(T, self.nh * self.dh)
        # x = 1*x + o @ Wo.T : compute.rs:267-270
        x = x + linear(o, w[p + "self_attn.o_proj.weight"], w.get(p + "self_attn.o_proj.bias"))
        h = self._r(rms_norm(x, w[p + "post_attention_layernorm.weight"], self.eps))
        g = self._r(linear(h, w[p + "mlp.gate_proj.weight"], w.get(p + "mlp.gate_proj.bias")))
        u = self._r(linear(h, w[p + "mlp.up_proj.weight"], w.get(p + "mlp.up_proj.bias")))
        a = self._r(swiglu(g, u))
        # x = 1*x + act @ Wdown.T : compute.rs:290-292
        return x + linear(a, w[p + "mlp.down_proj.weight"], w.get(p + "mlp.down_proj.bias"))

    def forward(self, tokens):
        """tokens [T] -> logits [T, vocab] of one whole sequence from position 0."""
        w = self.w
        tokens = np.asarray(tokens, dtype=np.int64)
        # embedding rows, no scaling: test-utils/src/llama.rs:18-23
        x = w["model.embed_tokens.weight"][tokens]
        positions = np.arange(len(tokens))
        for i in range(self.n_layers):
            x = self.block(i, x, positions)
        # output norm then output matrix: compute.rs:358-365; the output
        # matrix falls back to the embedding table: storage.rs:84
        h = self._r(rms_norm(x, w["model.norm.weight"], self.eps))
        head = w.get("lm_head.weight", w["model.embed_tokens.weight"])
        return linear(h, head)

    def greedy(self, prompt, n_new, stop_ids=()):
        """test-utils/src/lib.rs:153-173: feed, take the next token, stop on
        the stop token without emitting it."""
        seq = list(prompt)
        out = []
        for _ in range(n_new):
            nxt = int(np.argmax(self.forward(seq)[-1]))
            if nxt in stop_ids:
                break
            out.append(nxt)
            seq.append(nxt)
        return out


# --------------------------------------------------------------------------
# sampling
# --------------------------------------------------------------------------
def sample_probabilities(logits, temperature, top_p=1.0, top_k=None):
    """Distribution the sampler draws from.

    Defaults and ranges: test-utils/src/lib.rs:78-80 (temperature 0 = argmax,
    top_p 1, top_k unlimited). Tokens are ordered by descending logit (ties:
    lower index first); the first top_k are kept, then the shortest prefix
    whose probability reaches top_p; the rest gets probability 0.
    """
    logits = np.asarray(logits, dtype=np.float64)
    n = logits.shape[-1]
    if temperature == 0 or top_k == 1:
        p = np.zeros(n)
        p[int(np.argmax(logits))] = 1.0
        return p
    z = logits / temperature
    z = z - z.max()
    p = np.exp(z)
    p /= p.sum()
    order = np.argsort(-logits, kind="stable")
    keep = np.zeros(n, dtype=bool)
    k = n if top_k is None else min(int(top_k), n)
    cum = 0.0
    for r, idx in enumerate(order[:k]):
        keep[idx] = True
        cum += p[idx]
        if cum >= top_p:
            break
    p = np.where(keep, p, 0.0)
    return p / p.sum()


# --------------------------------------------------------------------------
# writing a model folder (tests make their own weights with this)
# --------------------------------------------------------------------------
def write_safetensors(path, tensors: dict, dtype="F32"):
    """tensors: name -> float ndarray; stored as F32 or BF16 (per-name dict ok)."""
    header, blobs, off = {}, [], 0
    for name, a in tensors.items():
        dt = dtype[name] if isinstance(dtype, dict) else dtype
        a = np.ascontiguousarray(a)
        if dt == "F32":
            b = a.astype("<f4").tobytes()
        elif dt == "BF16":
            u = round_bf16(a).astype(np.float32).view(np.uint32) >> 16
            b = u.astype("<u2").tobytes()
        else:
            raise ValueError(dt)
        header[name] = {"dtype": dt, "shape": list(a.shape), "data_offsets": [off, off + len(b)]}
        blobs.append(b)
        off += len(b)
    h = json.dumps(header, separators=(",", ":")).encode()
    h += b" " * ((8 - len(h) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(h)))
        f.write(h)
        for b in blobs:
            f.write(b)


def make_model_folder(folder, config: dict, seed, storage="F32", std=0.02, norm_std=0.1,
                      edit=None):
    """Random Llama weights under the safetensors names, written to ``folder``.

    Matrices ~ N(0, std), norm weights 1 + N(0, norm_std). ``edit(weights)``
    may change tensors before they are written (tests plant stand-out keys).
    With storage "BF16" matrices are stored in bfloat16 and norm weights in
    float32, the split the reference's conversion recipe makes between linear
    and norm tensors (docs/user-guide/doc.md:133).
    """
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    c = config
    rng = np.random.default_rng(seed)
    d, nh = c["hidden_size"], c["num_attention_heads"]
    nkvh = c.get("num_key_value_heads", nh)
    dh = c.get("head_dim") or d // nh
    di, V = c["intermediate_size"], c["vocab_size"]
    w = {}

    def mat(name, r, cdim):
        w[name] = rng.normal(0.0, std, size=(r, cdim))

    def vec(name, n):
        w[name] = 1.0 + rng.normal(0.0, norm_std, size=(n,))

    mat("model.embed_tokens.weight", V, d)
    for i in range(c["num_hidden_layers"]):
        p = f"model.layers.{i}."
        vec(p + "input_layernorm.weight", d)
        mat(p + "self_attn.q_proj.weight", nh * dh, d)
        mat(p + "self_attn.k_proj.weight", nkvh * dh, d)
        mat(p + "self_attn.v_proj.weight", nkvh * dh, d)
        mat(p + "self_attn.o_proj.weight", d, nh * dh)
        if c.get("attention_bias"):
            for n_, r in (("q", nh * dh), ("k", nkvh * dh), ("v", nkvh * dh), ("o", d)):
                w[p + f"self_attn.{n_}_proj.bias"] = rng.normal(0.0, std, size=(r,))
        vec(p + "post_attention_layernorm.weight", d)
        mat(p + "mlp.gate_proj.weight", di, d)
        mat(p + "mlp.up_proj.weight", di, d)
        mat(p + "mlp.down_proj.weight", d, di)
        if c.get("mlp_bias"):
            for n_, r in (("gate", di), ("up", di), ("down", d)):
                w[p + f"mlp.{n_}_proj.bias"] = rng.normal(0.0, std, size=(r,))
    vec("model.norm.weight", d)
    if not c.get("tie_word_embeddings", False):
        mat("lm_head.weight", V, d)
    if edit is not None:
        edit(w)
    if storage == "BF16":
        dts = {n: ("BF16" if a.ndim == 2 else "F32") for n, a in w.items()}
    else:
        dts = "F32"
    write_safetensors(folder / "model.safetensors", w, dts)
    (folder / "config.json").write_text(json.dumps(c, indent=1))
    return folder


TINY_A = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4,
    "num_key_value_heads": 2, "head_dim": 16, "intermediate_size": 176,
    "vocab_size": 256, "rope_theta": 10000.0, "rms_norm_eps": 1e-5,
    "tie_word_embeddings": False, "max_position_embeddings": 128,
}

TINY_B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 3,
    "num_key_value_heads": 3, "intermediate_size": 256,
    "vocab_size": 384, "rope_theta": 500000.0, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": True, "max_position_embeddings": 256,
    "rope_style": "interleaved", "attention_bias": True,
}
