"""Command line and Python entry point in the manner of the reference's driver.

The reference is configured by environment variables
(test-utils/src/lib.rs:31-42, :67-82; documented in
docs/user-guide/doc.md:150-159):

    TEST_MODEL   model path                          -> --model
    DEVICES      card number (cuda driver: one int)  -> --devices
    PROMPT       prompt, default "Once upon a time," -> --prompt
    AS_USER      apply the chat template             -> --as-user (needs a tokenizer; refused)
    TEMPERATURE  default 0, [0, inf)                 -> --temperature
    TOP_P        default 1, [0, 1]                   -> --top-p
    TOP_K        default unlimited, [1, inf]         -> --top-k
    MAX_STEPS    default unlimited: calls of the model, the prompt's included -> --max-steps

Every option defaults to its environment variable, then to the reference's
default. The engine's contract starts at token ids: ``--prompt`` is a list of
ids ("5,17,3"); text is taken only when the model folder holds a tokenizer.json.
``--prompt`` may be repeated to run several requests as one batch. At the end
the reference's table (total / prefill / decode: tokens, time, time per token)
is printed (test-utils/src/lib.rs:175-190).
"""
from __future__ import annotations

import argparse
import os
import sys
from dataclasses import dataclass, field
from pathlib import Path
from typing import List, Optional, Sequence

DEFAULT_PROMPT = "Once upon a time,"


def _env(name, default, typ=str):
    v = os.environ.get(name)
    if v is None:
        return default
    try:
        return typ(v)
    except ValueError:
        return default          # the reference falls back to the default on a parse failure


def _bool(s: str) -> bool:
    t = s.lower()
    if t in ("true", "t", "yes", "y", "1"):
        return True
    if t in ("false", "f", "no", "n", "0"):
        return False
    raise ValueError(f"`AS_USER` is not a boolean value: {s!r}")


@dataclass
class Inference:
    """The reference's ``Inference`` record (test-utils/src/lib.rs:20-29)."""
    model: str
    devices: Optional[str] = None
    prompt: List[str] = field(default_factory=lambda: [DEFAULT_PROMPT])
    as_user: bool = False
    temperature: float = 0.0
    top_p: float = 1.0
    top_k: Optional[int] = None
    max_steps: Optional[int] = None
    dtype: Optional[str] = None     # None: the configuration's torch_dtype decides
    seed: int = 0
    timers: bool = False        # GPU time per kind of part (steps then run eagerly)
    random: Optional[str] = None   # instead of ``model``: a config.json or a shape name; weights from ``seed``
    layers: Optional[int] = None

    @classmethod
    def load(cls) -> Optional["Inference"]:
        """From the environment alone; None when TEST_MODEL is not set (lib.rs:50-58)."""
        path = os.environ.get("TEST_MODEL")
        if path is None:
            print("TEST_MODEL not set")
            return None
        if not Path(path).exists():
            print(f"{path!r} not found")
            return None
        return cls(model=path, devices=os.environ.get("DEVICES"),
                   prompt=[os.environ.get("PROMPT", DEFAULT_PROMPT)],
                   as_user=_bool(os.environ["AS_USER"]) if "AS_USER" in os.environ else False,
                   temperature=_env("TEMPERATURE", 0.0, float), top_p=_env("TOP_P", 1.0, float),
                   top_k=_env("TOP_K", None, int), max_steps=_env("MAX_STEPS", None, int))


def prompt_to_tokens(prompt: str, model_path) -> List[int]:
    s = prompt.strip()
    try:
        return [int(t) for t in s.replace(",", " ").split()]
    except ValueError:
        pass
    tok = Path(model_path) / "tokenizer.json"
    if tok.exists():
        from tokenizers import Tokenizer
        return Tokenizer.from_file(str(tok)).encode(prompt).ids
    raise SystemExit(f"prompt {prompt!r} is not a list of token ids and {model_path} has no "
                     f"tokenizer.json; give ids such as --prompt 5,17,3")


def infer(inf: Inference, stream=sys.stdout):
    """Loads the model, generates for every prompt, prints tokens and the timing
    table, and returns the GenerationResult."""
    import torch
    from .api import load_model
    from .engine.generate import generate
    from .sampling.args import SampleArgs
    if inf.as_user:
        raise SystemExit("AS_USER needs a chat template and a tokenizer; this engine starts at "
                         "token ids")
    device = f"cuda:{int(inf.devices) if inf.devices else 0}"
    args = SampleArgs(inf.temperature, inf.top_p, inf.top_k)
    print(args, file=stream)
    print(f"using gpu{device[5:]}", file=stream)
    if inf.random:
        import json
        from .api import random_model
        from .config.registry import architecture_of_config_json
        from .config.shapes import SHAPES
        d = dict(SHAPES[inf.random][1]) if inf.random in SHAPES else json.loads(Path(inf.random).read_text())
        arch = architecture_of_config_json(d)
        model = random_model(arch.config_from_dict(d), inf.seed, inf.dtype or "bfloat16", device,
                             architecture=arch.name, num_layers=inf.layers)
        where = Path(inf.random).parent if inf.random not in SHAPES else Path(".")
    else:
        model = load_model(inf.model, inf.dtype, device, verbose=True)
        where = inf.model
    prompts = [prompt_to_tokens(p, where) for p in inf.prompt]
    # MAX_STEPS counts calls of the model; every call yields one token
    max_new = inf.max_steps if inf.max_steps is not None else \
        max(1, model.spec.max_position - max(len(p) for p in prompts)) if model.spec.max_position \
        else 256
    if inf.timers:
        from .parts.base import PartTimers
        model.timers = PartTimers()
    res = generate(model, prompts, max_new, args, seed=inf.seed)
    torch.cuda.synchronize()
    for i, (p, out) in enumerate(zip(prompts, res.tokens)):
        print(f"[{i}] prompt {len(p)} tokens -> {' '.join(map(str, out))}  ({res.finish[i]})",
              file=stream)
    print(f"\n{'':10}{'num tokens':>12}{'elapse':>14}{'time per token':>18}", file=stream)
    for row in res.timing.table():
        print(f"{row['']:10}{row['num tokens']:>12}{row['elapse'] * 1e3:>12.3f}ms"
              f"{row['time per token'] * 1e3:>16.3f}ms", file=stream)
    if inf.timers:
        print(f"\n{'part':10}{'calls':>10}{'GPU time':>14}", file=stream)
        for name, (calls, ms) in sorted(model.timers.table().items(), key=lambda kv: -kv[1][1]):
            print(f"{name:10}{calls:>10}{ms:>12.3f}ms", file=stream)
        model.timers = None
    return res


def main(argv: Optional[Sequence[str]] = None) -> int:
    ap = argparse.ArgumentParser(prog="transformer_amd", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd")
    g = sub.add_parser("generate", help="generate from token-id prompts (the reference's test_infer)")
    g.add_argument("--model", default=os.environ.get("TEST_MODEL"))
    g.add_argument("--random", default=None, metavar="CONFIG",
                   help="instead of --model: a model with random weights, drawn on the GPU from --seed, "
                        "of a config.json or of one of the shapes 8b, 7b, 70b")
    g.add_argument("--layers", type=int, default=None, help="with --random: only the first layers")
    g.add_argument("--devices", default=os.environ.get("DEVICES"))
    g.add_argument("--prompt", action="append", default=None)
    g.add_argument("--as-user", action="store_true",
                   default=_bool(os.environ["AS_USER"]) if "AS_USER" in os.environ else False)
    g.add_argument("--temperature", type=float, default=_env("TEMPERATURE", 0.0, float))
    g.add_argument("--top-p", type=float, default=_env("TOP_P", 1.0, float))
    g.add_argument("--top-k", type=int, default=_env("TOP_K", None, int))
    g.add_argument("--max-steps", type=int, default=_env("MAX_STEPS", None, int))
    g.add_argument("--dtype", choices=["bfloat16", "float32"], default=None,
                   help="the engine's type; default: what config.json's torch_dtype says (float32 stays "
                        "float32, everything else computes in bfloat16)")
    g.add_argument("--backend", choices=["hip", "ref"], default="hip",
                   help="ref: the plain float32 kernels of the device (one sum per output element in "
                        "ascending order, attention without matrix cores), whatever --dtype says; the "
                        "role of the reference's CPU back-end (models/llama/common-cpu/src/lib.rs:48-67)")
    g.add_argument("--seed", type=int, default=0)
    g.add_argument("--timers", action="store_true",
                   help="print GPU time per kind of part (embed, norm, mixer, ffn, head); steps run eagerly")
    r = sub.add_parser("random", help="write a model folder with random weights")
    r.add_argument("--config", required=True,
                   help="a config.json to take the sizes from, or one of the shapes 8b, 7b, 70b")
    r.add_argument("--out", required=True)
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--storage", choices=["bfloat16", "float32"], default="bfloat16")
    r.add_argument("--layers", type=int, default=None, help="write only the first layers")
    r.add_argument("--on-gpu", action="store_true",
                   help="draw the weights on the GPU and stream them to the file (large models); "
                        "another stream of numbers than the host draws")
    r.add_argument("--probe", default=None,
                   help="with --on-gpu: token ids; prints the greedy continuation of the model that "
                        "was written, to compare with `generate` on the folder")
    p = sub.add_parser("replay", help="same as bin/trace_run")
    p.add_argument("rest", nargs=argparse.REMAINDER)
    b = sub.add_parser("bench", help="run bench.py of the source tree with the given options")
    b.add_argument("rest", nargs=argparse.REMAINDER)
    a = ap.parse_args(argv)
    if a.cmd == "generate":
        if a.random and a.model and "TEST_MODEL" not in os.environ:
            print("give --model or --random, not both")
            return 2
        if a.random:
            a.model = None
            inf = Inference(model="", devices=a.devices,
                            prompt=a.prompt or [os.environ.get("PROMPT", DEFAULT_PROMPT)],
                            as_user=a.as_user, temperature=a.temperature, top_p=a.top_p,
                            top_k=a.top_k, max_steps=a.max_steps,
                            dtype="float32" if a.backend == "ref" else a.dtype, seed=a.seed,
                            timers=a.timers, random=a.random, layers=a.layers)
            infer(inf)
            return 0
        if not a.model:
            print("TEST_MODEL not set")
            return 0            # the reference's driver returns quietly (lib.rs:50-53)
        inf = Inference(model=a.model, devices=a.devices,
                        prompt=a.prompt or [os.environ.get("PROMPT", DEFAULT_PROMPT)],
                        as_user=a.as_user, temperature=a.temperature, top_p=a.top_p,
                        top_k=a.top_k, max_steps=a.max_steps,
                        dtype="float32" if a.backend == "ref" else a.dtype, seed=a.seed,
                        timers=a.timers)
        infer(inf)
        return 0
    if a.cmd == "random":
        import json
        from . import architectures  # noqa: F401
        from .config.registry import architecture_of_config_json
        from .weights.random_init import write_random_model
        from .config.shapes import SHAPES
        d = dict(SHAPES[a.config][1]) if a.config in SHAPES else json.loads(Path(a.config).read_text())
        if a.layers is not None:
            d["num_hidden_layers"] = a.layers
        arch = architecture_of_config_json(d)
        if a.on_gpu:
            import time
            from .api import random_model, save_model
            from .engine.generate import generate
            model = random_model(arch.config_from_dict(d), a.seed, a.storage, architecture=arch.name)
            t0 = time.time()
            save_model(model, a.out, metadata={"seed": a.seed})
            print(f"[transformer_amd] wrote {model.weight_bytes() / 1e9:.2f} GB in {time.time() - t0:.1f} s",
                  file=sys.stderr, flush=True)
            if a.probe:
                toks = prompt_to_tokens(a.probe, a.out)
                print("probe:", " ".join(map(str, generate(model, [toks], 8, stop_ids=[]).tokens[0])))
        else:
            write_random_model(a.out, arch.config_from_dict(d), a.seed, a.storage, architecture=arch.name)
        print(a.out)
        return 0
    if a.cmd == "replay":
        from .replay import main as replay_main
        return replay_main(a.rest)
    if a.cmd == "bench":
        import runpy
        script = Path(__file__).resolve().parent.parent / "bench.py"
        if not script.exists():
            print(f"{script} not found: the bench lives in the source tree")
            return 2
        sys.argv = [str(script), *a.rest]
        runpy.run_path(str(script), run_name="__main__")
        return 0
    ap.print_help()
    return 2


if __name__ == "__main__":
    sys.exit(main())
