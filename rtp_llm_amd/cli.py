"""Command line of the package.

    python -m rtp_llm_amd.cli generate --model DIR --prompt-ids 5,17,3 [--prompt-ids ...] --max-new-tokens N [--dtype bfloat16|float32]
                                       [--top-k K --top-p P --temperature T --seed S] [--no-graphs]
    python -m rtp_llm_amd.cli trace --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N      (steps on standard input)
    python -m rtp_llm_amd.cli families

`generate` prints one JSON line per prompt with the generated token ids.  `trace` replays a schedule of steps through the engine's step
function and writes the logits of the asked rows: one JSON object a line on standard input,
{"step": n, "entries": [{"id": .., "tokens": [..], "want": [..]}], "end": [ids]}; for a step with wanted rows it writes <out>/<n>.f32
(little-endian float32 [wanted, vocab], in the order of the entries and wants), then prints "done <n>"; sequences named in "end" give
their pages and state slot back after the step."""
import argparse
import json
import os
import sys

DTYPES = {"bfloat16": "bfloat16", "bf16": "bfloat16", "float32": "float32", "fp32": "float32", "float16": "float16", "fp16": "float16"}


def _dtype(name):
    import torch
    return getattr(torch, DTYPES[name])


def cmd_generate(a):
    import torch
    from . import registry
    eng = registry.load_engine(a.model, _dtype(a.dtype), a.device, max_tokens=a.max_tokens, max_seqs=a.max_seqs)
    if not a.no_graphs and hasattr(eng, "use_graphs"):
        eng.use_graphs = True                     # decode-only steps replay a captured HIP graph
    prompts = [[int(t) for t in p.split(",") if t.strip()] for p in a.prompt_ids]
    sampling = {} if a.top_k == 1 else dict(top_k=a.top_k, top_p=a.top_p, temperature=a.temperature, seed=a.seed)
    outs = eng.generate(prompts, a.max_new_tokens, **sampling)
    torch.cuda.synchronize()
    for p, o in zip(prompts, outs):
        print(json.dumps({"prompt": p, "generated": o}))
    return 0


def cmd_trace(a):
    import numpy as np
    import torch
    from . import registry
    dtype = _dtype(a.dtype)
    eng = registry.load_engine(a.model, dtype, a.device, max_tokens=a.max_tokens, max_seqs=a.max_seqs)
    if not hasattr(eng, "run_step"):
        print("this family has no ragged step function to replay a trace through", file=sys.stderr)
        return 3
    os.makedirs(a.out, exist_ok=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        logits = eng.run_step([(e["id"], e["tokens"], e.get("want", [])) for e in st["entries"]])
        if logits is not None:
            arr = logits.detach().to("cpu", torch.float32).contiguous().numpy().astype("<f4", copy=False)
            tmp = os.path.join(a.out, f".{st['step']}.f32.part")
            arr.tofile(tmp)
            os.replace(tmp, os.path.join(a.out, f"{st['step']}.f32"))
        else:
            torch.cuda.synchronize()
        for sid in st.get("end", []):
            eng.release(sid)
        sys.stdout.write(f"done {st['step']}\n")
        sys.stdout.flush()
    return 0


def main(argv=None):
    ap = argparse.ArgumentParser(prog="rtp_llm_amd")
    sub = ap.add_subparsers(dest="cmd", required=True)
    g = sub.add_parser("generate", help="generate token ids for prompts given as token ids")
    g.add_argument("--model", required=True)
    g.add_argument("--prompt-ids", action="append", required=True, help="comma-separated token ids; repeat for a batch")
    g.add_argument("--max-new-tokens", type=int, default=16)
    g.add_argument("--dtype", default="bfloat16", choices=sorted(DTYPES))
    g.add_argument("--device", default="cuda:0")
    g.add_argument("--max-tokens", type=int, default=8192, help="tokens the cache pool holds")
    g.add_argument("--max-seqs", type=int, default=4, help="live sequences (state slots)")
    g.add_argument("--top-k", type=int, default=1)
    g.add_argument("--top-p", type=float, default=1.0)
    g.add_argument("--temperature", type=float, default=1.0)
    g.add_argument("--seed", type=int, default=0)
    g.add_argument("--no-graphs", action="store_true", help="run decode-only steps eagerly instead of replaying captured HIP graphs (families with a ragged step function)")
    g.set_defaults(fn=cmd_generate)
    t = sub.add_parser("trace", help="replay a schedule of steps from standard input and write the logits of the asked rows")
    t.add_argument("--model", required=True)
    t.add_argument("--dtype", default="bfloat16", choices=sorted(DTYPES))
    t.add_argument("--out", required=True)
    t.add_argument("--max-tokens", type=int, required=True)
    t.add_argument("--max-seqs", type=int, default=4)
    t.add_argument("--device", default="cuda:0")
    t.set_defaults(fn=cmd_trace)
    f = sub.add_parser("families", help="list the registered model families")
    f.set_defaults(fn=lambda a: print("\n".join(__import__("rtp_llm_amd.registry", fromlist=["x"]).families())) or 0)
    a = ap.parse_args(argv)
    return a.fn(a)


if __name__ == "__main__":
    sys.exit(main())
