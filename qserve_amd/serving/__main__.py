"""Command line of the serving engine.

    python -m qserve_amd.serving generate --model DIR --prompt 1,2,3 [--prompt ...] [--max-new N] [--dtype ...] [--graphs]
    python -m qserve_amd.serving trace    --model DIR --dtype ... --out DIR --max-tokens N     (steps on standard input)
    python -m qserve_amd.serving models
"""
import argparse
import json
import sys


def main():
    if len(sys.argv) < 2 or sys.argv[1] in ("-h", "--help"):
        print(__doc__)
        return 0
    cmd, argv = sys.argv[1], sys.argv[2:]
    if cmd == "trace":
        from .trace import main as trace_main
        return trace_main(argv)
    if cmd == "models":
        from .registry import architectures
        for name, engine in architectures().items():
            print(f"{name}\t{engine}")
        return 0
    if cmd != "generate":
        print(__doc__)
        return 2
    ap = argparse.ArgumentParser(prog="qserve_amd.serving generate")
    ap.add_argument("--model", required=True)
    ap.add_argument("--prompt", action="append", required=True, help="token ids, comma separated (repeat for a batch)")
    ap.add_argument("--max-new", type=int, default=16)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--top-k", type=int, default=0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--seed", type=int, default=None)
    ap.add_argument("--max-tokens", type=int, default=8192)
    ap.add_argument("--max-seqs", type=int, default=4)
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--graphs", action="store_true", help="replay single-token steps from hipGraphs")
    a = ap.parse_args(argv)
    from . import Engine, SamplingParams
    eng = Engine.from_pretrained(a.model, dtype=a.dtype, device=a.device, max_tokens=a.max_tokens, max_seqs=a.max_seqs,
                                 decode_graphs=a.graphs)
    prompts = [[int(t) for t in p.split(",") if t.strip()] for p in a.prompt]
    outs = eng.generate(prompts, SamplingParams(max_new=a.max_new, temperature=a.temperature, top_k=a.top_k, top_p=a.top_p,
                                                seed=a.seed))
    for p, o in zip(prompts, outs):
        print(json.dumps({"prompt": p, "output": o}))
    return 0


if __name__ == "__main__":
    sys.exit(main())
