"""Trace replay: feed given token ids through a model step by step and write the logits that are asked for.  Nothing is sampled.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N [--state-slots 4]

Standard input carries one JSON object per line, `{"step": n, "entries": [{"id": "a", "tokens": [..], "want": [..]}], "end": ["a"]}`: every entry brings a request's next
tokens (a request is admitted at its first entry) and the places among them whose logits are wanted; all entries of a step run as ONE ragged batch through the model's
step function, from the K / V pages and state slots that earlier steps left.  `<out>/<step>.f32` receives the wanted logits ([wanted, vocab], little-endian f32, in entry
and `want` order); after every step a line `done <step>` is printed.  Requests named in `end` return their pages and slot.  The page pool is sized for `--max-tokens`
live tokens (per request rounded up to whole pages) and `--state-slots` live requests, so long traces reuse both.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--state-slots", type=int, default=4)
    ap.add_argument("--block-size", type=int, default=32)
    a = ap.parse_args(argv)

    import numpy as np
    import torch
    from . import registry
    from .hybrid import HybridCache, HybridDecoder, RaggedBatch

    if not torch.cuda.is_available():
        print("trace_run: no GPU (there is no CPU path)", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    bs = a.block_size
    # every live request may round up to a whole page; one more page for the pool's null block
    blocks = -(-a.max_tokens // bs) + a.state_slots + 1
    model = registry.load_model(a.model, dev, a.dtype, num_blocks=blocks, block_size=bs, state_slots=a.state_slots)
    if not isinstance(model, HybridDecoder):
        print("trace_run: this architecture has no ragged step function", file=sys.stderr)
        return 2
    cache = HybridCache(model)
    os.makedirs(a.out, exist_ok=True)
    ids: dict = {}
    length: dict = {}
    admitted = 0
    with torch.inference_mode():
        for line in sys.stdin:
            line = line.strip()
            if not line:
                continue
            step = json.loads(line)
            entries = []
            for e in step.get("entries", []):
                if not e["tokens"]:
                    continue
                if e["id"] not in ids:
                    admitted += 1
                    ids[e["id"]] = admitted
                rid = ids[e["id"]]
                p0 = length.get(rid, 0)
                if not cache.reserve(rid, p0 + len(e["tokens"])):
                    print(f"trace_run: no pages or state slot left for request {e['id']!r}", file=sys.stderr)
                    return 1
                entries.append(cache.entry(rid, e["tokens"], p0, e.get("want", ())))
                length[rid] = p0 + len(e["tokens"])
            if entries:
                batch = RaggedBatch.build(entries, bs, dev)
                logits = model.forward_batch(batch)
                if logits.shape[0]:
                    out = logits.float().cpu().numpy().astype("<f4")
                    tmp = os.path.join(a.out, f".{step['step']}.part")
                    out.tofile(tmp)
                    os.replace(tmp, os.path.join(a.out, f"{step['step']}.f32"))
                else:
                    torch.cuda.current_stream().synchronize()
            for name in step.get("end", []):
                rid = ids.pop(name, None)
                if rid is not None:
                    cache.release(rid)
                    length.pop(rid, None)
            print(f"done {step['step']}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
