"""Trace replay: feeds given token ids through a model step by step and writes
logits. It samples nothing and owns no forward pass, cache or loader: it drives
``load_model``, ``DecoderModel.step`` and the ``SequenceCache`` that generation
uses.

The nearest thing in the reference is the stream of Task{nt, pos, embd, next}
messages a driver sends its workers, one per step
(test-utils/src/llama.rs:25-35, consumed at
models/llama/common-cpu/src/infer.rs:96-142).

Input, one JSON object a line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
For a step that wants logits, ``<out>/<step>.f32`` holds them as little-endian
float32 [wanted, vocab], in the order of the entries and of ``want``. ``<out>/index.jsonl``
gets one line per such step, {"step": s, "rows": [[request id, position in the sequence],
...]}, which names the rows of the step's file. After every step a line ``done <step>`` is
printed and flushed.
"""
from __future__ import annotations

import json
import sys
from pathlib import Path
from typing import Dict

from .engine.batch import Entry


class TraceError(ValueError):
    pass


class Replayer:
    def __init__(self, model, max_tokens: int, out_dir):
        self.model = model
        self.cache = model.new_cache(max_tokens)
        self.out = Path(out_dir)
        self.out.mkdir(parents=True, exist_ok=True)
        (self.out / "index.jsonl").write_text("")
        self.slots: Dict[str, int] = {}

    def run_step(self, rec: dict) -> None:
        if "step" not in rec or "entries" not in rec:
            raise TraceError("a trace line needs 'step' and 'entries'")
        step = rec["step"]
        entries, rows = [], []
        for e in rec["entries"]:
            rid = str(e["id"])
            if rid not in self.slots:
                self.slots[rid] = self.cache.alloc_slot()
            entries.append(Entry(self.slots[rid], list(e["tokens"]), list(e.get("want", ()))))
            at = self.cache.length(self.slots[rid])
            rows += [[e["id"], at + int(w)] for w in entries[-1].want]
        if entries:
            logits = self.model.step(self.cache, entries)
            if logits.shape[0]:
                arr = logits.detach().cpu().numpy().astype("<f4", copy=False)
                tmp = self.out / f"{step}.f32.tmp"
                arr.tofile(tmp)
                tmp.replace(self.out / f"{step}.f32")
                with open(self.out / "index.jsonl", "a") as f:
                    f.write(json.dumps({"step": step, "rows": rows}) + "\n")
        for rid in rec.get("end", ()):
            rid = str(rid)
            if rid not in self.slots:
                raise TraceError(f"step {step}: request {rid!r} ends but was never seen")
            self.cache.free_slot(self.slots.pop(rid))

    def run(self, lines, report=sys.stdout) -> None:
        for line in lines:
            line = line.strip()
            if not line:
                continue
            rec = json.loads(line)
            self.run_step(rec)
            print(f"done {rec['step']}", file=report, flush=True)


def main(argv=None) -> int:
    import argparse
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args(argv)
    from .api import load_model
    model = load_model(args.model, args.dtype, args.device, verbose=True)
    Replayer(model, args.max_tokens, args.out).run(sys.stdin)
    return 0
