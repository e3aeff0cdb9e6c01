"""Replay a recorded trace of token steps through the engine and write the logits asked for.

    python -m qserve_amd.serving trace --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Standard input: one JSON object a line,
    {"step": n, "entries": [{"id": ..., "tokens": [...], "want": [...]}], "end": [ids]}
All entries of a step run as one batch from the cache earlier steps left; a request is admitted at its first entry and
gives its pages and slot back when a step lists it under "end".  For a step with wanted positions the float32 logits
[wanted, vocab] go to DIR/<step>.f32 (little-endian, entries' order); after every step `done <step>` is printed.
Nothing is sampled.
"""
import argparse
import json
import os
import sys


def main(argv=None):
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n")[0])
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--max-seqs", type=int, default=4)
    ap.add_argument("--device", default="cuda:0")
    a = ap.parse_args(argv)
    import torch

    from .engine import Engine
    if not torch.cuda.is_available():
        print("trace_run: no GPU visible (served models have no CPU path)", file=sys.stderr)
        return 4
    eng = Engine.from_pretrained(a.model, dtype=a.dtype, device=a.device, max_tokens=a.max_tokens, max_seqs=a.max_seqs)
    os.makedirs(a.out, exist_ok=True)
    slots = {}
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        items, want, at = [], [], 0
        for e in step.get("entries", []):
            if e["id"] not in slots:
                slots[e["id"]] = eng.open_sequence()
            items.append((slots[e["id"]], e["tokens"]))
            want += [at + int(k) for k in e.get("want", [])]
            at += len(e["tokens"])
        logits = eng.execute(items, want)
        if want:
            data = logits.to(torch.float32).cpu().contiguous().numpy().astype("<f4", copy=False)
            tmp = os.path.join(a.out, f".{step['step']}.part")
            with open(tmp, "wb") as f:
                f.write(data.tobytes())
            os.replace(tmp, os.path.join(a.out, f"{step['step']}.f32"))
        for rid in step.get("end", []):
            if rid in slots:
                eng.close_sequence(slots.pop(rid))
        sys.stdout.write(f"done {step['step']}\n")
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
