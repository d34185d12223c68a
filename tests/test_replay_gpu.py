"""bin/trace_run driven the way a user drives it: the same requests whole, with the
last 32 tokens one by one, and in batches of unequal lengths, in both dtypes."""
import json
import pathlib
import subprocess
import sys

import numpy as np
import pytest

import gpu_util as G

pytestmark = pytest.mark.gpu
ROOT = pathlib.Path(__file__).resolve().parent.parent


def run_trace(folder, dtype, steps, out, max_tokens):
    text = "\n".join(json.dumps(s) for s in steps) + "\n"
    r = subprocess.run([str(ROOT / "bin" / "trace_run"), "--model", folder, "--dtype", dtype,
                        "--out", str(out), "--max-tokens", str(max_tokens)],
                       input=text, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-3000:]
    assert r.stdout.split("\n")[:-1] == [f"done {s['step']}" for s in steps]
    return r


def read(out, step, vocab):
    return np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(-1, vocab).astype(np.float64)


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("A", "bfloat16"), ("B", "bfloat16"),
                                        ("C", "float32"), ("C", "bfloat16"), ("D", "float32"),
                                        ("D", "bfloat16")])
def test_trace_replay_three_ways(name, dtype, tmp_path):
    folder, ref = G.folder(name, dtype), G.plain(name, dtype)
    vocab = G.CONFIGS[name][0]["vocab_size"]
    reqs = {f"r{i}": G.tokens(name, n, 200 + i) for i, n in enumerate((40, 97, 64, 33, 70))}
    want = {k: ref.forward(v) for k, v in reqs.items()}
    tol = G.TOL[dtype]
    # 1. each request alone and whole
    steps = [{"step": i, "entries": [{"id": k, "tokens": v, "want": list(range(len(v)))}], "end": [k]}
             for i, (k, v) in enumerate(reqs.items())]
    run_trace(folder, dtype, steps, tmp_path / "whole", 128)
    for i, k in enumerate(reqs):
        assert np.abs(read(tmp_path / "whole", i, vocab) - want[k]).max() < tol
    # 2. the last 32 tokens one by one
    k, v = "r1", reqs["r1"]
    steps = [{"step": 0, "entries": [{"id": k, "tokens": v[:-32], "want": list(range(len(v) - 32))}], "end": []}]
    for j, t in enumerate(v[-32:]):
        steps.append({"step": j + 1, "entries": [{"id": k, "tokens": [t], "want": [0]}],
                      "end": [k] if j == 31 else []})
    run_trace(folder, dtype, steps, tmp_path / "tail", 128)
    got = np.concatenate([read(tmp_path / "tail", s["step"], vocab) for s in steps])
    assert np.abs(got - want[k]).max() < tol
    # 3. batches of unequal lengths; shorter requests end earlier; the second batch
    #    starts after the first and fits only because its slots and pages came back
    steps, n = [], 0
    rows = {k: [] for k in reqs}
    for batch in (["r0", "r1", "r2"], ["r3", "r4"]):
        pre = {k: max(1, len(reqs[k]) - 20 - 7 * i) for i, k in enumerate(batch)}
        steps.append({"step": n, "entries": [{"id": k, "tokens": reqs[k][:pre[k]], "want": list(range(pre[k]))}
                                             for k in batch], "end": []})
        for k in batch:
            rows[k].append((n, batch.index(k), pre[k]))
        n += 1
        pos, live = dict(pre), list(batch)
        while live:
            ends = [k for k in live if pos[k] + 1 == len(reqs[k])]
            steps.append({"step": n, "entries": [{"id": k, "tokens": [reqs[k][pos[k]]],
                                                  "want": [0] if pos[k] % 2 else []} for k in live],
                          "end": ends})
            for k in live:
                if pos[k] % 2:
                    rows[k].append((n, pos[k]))
                pos[k] += 1
            live = [k for k in live if k not in ends]
            n += 1
    run_trace(folder, dtype, steps, tmp_path / "batch", 64 * 5)
    out = tmp_path / "batch"
    for batch in (["r0", "r1", "r2"], ["r3", "r4"]):
        first = rows[batch[0]][0][0]
        got = read(out, first, vocab)
        off = 0
        for k in batch:
            p = rows[k][0][2]
            assert np.abs(got[off:off + p] - want[k][:p]).max() < tol, (k, "prompt")
            off += p
    for s in steps:                      # a step that wants nothing writes no file
        if not any(e["want"] for e in s["entries"]):
            assert not (out / f"{s['step']}.f32").exists()
    # the index names every row of every file by (request, position in its sequence)
    index = {r["step"]: r["rows"] for r in map(json.loads, (out / "index.jsonl").read_text().splitlines())}
    assert sorted(index) == [s["step"] for s in steps if any(e["want"] for e in s["entries"])]
    for step, named in index.items():
        got = read(out, step, vocab)
        assert len(named) == len(got)
        for row, (k, p) in zip(got, named):
            assert np.abs(row - want[k][p]).max() < tol, (step, k, p)
    for k in reqs:
        for item in rows[k][1:]:
            step, p = item
            s = steps[step]
            wanted = [e["id"] for e in s["entries"] if e["want"]]
            got = read(out, step, vocab)[wanted.index(k)]
            assert np.abs(got - want[k][p]).max() < tol, (k, p)
