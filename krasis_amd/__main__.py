"""Command line: `python -m krasis_amd <command>`.

  generate  --model DIR --prompt 1,2,3 [--prompt ...] --max-new-tokens N [--dtype bfloat16|float32] [--temperature T --top-k K --top-p P --seed S]
            token ids in, token ids out (one JSON line per prompt); the model class is chosen by config.json (model_registry.load_model)
  trace     --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N
            replays a step trace from standard input through the engine's step function and writes the logits asked for (see `trace_replay`)
  models    the registered layer-described designs
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def trace_replay(engine, out_dir: str, lines, reply) -> None:
    """One JSON object per line: {"step": n, "entries": [{"id", "tokens", "want"}], "end": [ids]}.  All entries of a step are ONE batch of the engine;
    for a step with wanted places the logits go to <out_dir>/<n>.f32 (little-endian f32 [wanted, vocab], in the order of the entries and of `want`);
    after every step `done <n>` is printed.  Requests named in `end` give their slot and pages back after the step."""
    import numpy as np
    for line in lines:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        entries = [(e["id"], e["tokens"], e.get("want", [])) for e in st.get("entries", [])]
        n_want = sum(len(e[2]) for e in entries)
        if entries:
            logits, _ = engine.step(entries, logits=n_want > 0)
            if n_want:
                tmp = os.path.join(out_dir, f".{st['step']}.part")
                np.ascontiguousarray(logits, "<f4").tofile(tmp)
                os.replace(tmp, os.path.join(out_dir, f"{st['step']}.f32"))
        for rid in st.get("end", []):
            if rid in engine.live():
                engine.finish(rid)
        reply(f"done {st['step']}")


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="python -m krasis_amd")
    sub = ap.add_subparsers(dest="cmd", required=True)
    g = sub.add_parser("generate")
    g.add_argument("--model", required=True)
    g.add_argument("--prompt", action="append", required=True, help="comma-separated token ids; repeat for a batch")
    g.add_argument("--max-new-tokens", type=int, default=16)
    g.add_argument("--dtype", default="bfloat16")
    g.add_argument("--max-tokens", type=int, default=0, help="cache pool in tokens (0: sized for the prompts)")
    g.add_argument("--temperature", type=float, default=0.0)
    g.add_argument("--top-k", type=int, default=0)
    g.add_argument("--top-p", type=float, default=1.0)
    g.add_argument("--seed", type=int, default=0)
    t = sub.add_parser("trace")
    t.add_argument("--model", required=True)
    t.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    t.add_argument("--out", required=True)
    t.add_argument("--max-tokens", type=int, required=True)
    sub.add_parser("models")
    a = ap.parse_args(argv)

    from . import model_registry as R
    if a.cmd == "models":
        print("\n".join(R.architectures()))
        return 0
    if a.cmd == "generate":
        prompts = [[int(x) for x in p.split(",") if x.strip()] for p in a.prompt]
        fam = R.model_family(R.read_config(a.model))
        if fam.startswith("serve:"):
            pool = a.max_tokens or sum((len(p) + a.max_new_tokens + 63) // 64 * 64 for p in prompts[:4]) + 64
            eng = R.load_model(a.model, dtype=a.dtype, max_tokens=pool, build=True)
            outs = eng.generate(prompts, a.max_new_tokens, a.temperature, a.top_k, a.top_p, seed=a.seed)
        else:
            dec = R.load_model(a.model, max_tokens=a.max_tokens or 8192)
            outs = [dec.generate(p, a.max_new_tokens, a.temperature, a.top_k, a.top_p, rng_seed=a.seed) for p in prompts]
        for p, o in zip(prompts, outs):
            print(json.dumps({"prompt": p, "tokens": o}))
        return 0
    # trace
    cfg = R.read_config(a.model)
    if not R.model_family(cfg).startswith("serve:"):
        print("trace replay needs a design served by the batched store", file=sys.stderr)
        return 2
    os.makedirs(a.out, exist_ok=True)
    eng = R.load_model(a.model, dtype=a.dtype, max_tokens=a.max_tokens, max_slots=4, build=True)

    def reply(s: str) -> None:
        sys.stdout.write(s + "\n")
        sys.stdout.flush()
    trace_replay(eng, a.out, sys.stdin, reply)
    return 0


if __name__ == "__main__":
    sys.exit(main())
