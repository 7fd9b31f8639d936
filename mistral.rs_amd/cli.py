"""Command line of the package (bin/mistralrs):

    bin/mistralrs generate --model PATH --prompt-ids 1,2,3 [--prompt-ids 4,5 ...] [--max-new-tokens 16] [--top-k 1] [--temperature 1.0] [--top-p 1.0] [--min-p 0.0]
                           [--seed 0] [--dtype bfloat16|float32] [--max-tokens 4096] [--max-seqs 4]
    bin/mistralrs trace    --model DIR --dtype ... --out DIR --max-tokens N          (the same program as bin/trace_run)
    bin/mistralrs build    [--only libmrs_hybrid.so]

`generate` picks the loader from the checkpoint (registry.load_model), puts every prompt into the paged-attention scheduler and runs the engine until all are done;
prompts and results are token ids (the package has no tokenizer).  One JSON line per request goes to standard output.
"""
from __future__ import annotations

import argparse
import json
import sys


def make_engine(model, max_tokens: int, max_seqs: int, sampler=None, max_batched_tokens: int = 2048, use_graphs: bool = True):
    """Scheduler + engine around a loaded model with a ragged step function (hybrid.HybridDecoder): pages for `max_tokens` live tokens, `max_seqs` state slots."""
    from .hybrid import HybridCache
    from .scheduler import PagedAttentionScheduler, PagedEngine, SchedulerConfig
    cache = HybridCache(model)
    sched = PagedAttentionScheduler(SchedulerConfig(max_num_seqs=max_seqs, max_num_batched_tokens=max_batched_tokens, uniform_prompt_batches=False), cache.kv,
                                    prefix_caching=False, state_pool=cache.slots if model.has_recurrent_state else None)
    eng = PagedEngine(model, sched, sampler=sampler, use_graphs=use_graphs)
    eng.cache = cache
    return eng


def _generate(a) -> int:
    import torch
    from . import registry
    from .sampler import SequenceSampler
    from .scheduler import Sequence
    if not torch.cuda.is_available():
        print("generate: no GPU (there is no CPU path)", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    prompts = [[int(t) for t in p.split(",") if t.strip()] for p in a.prompt_ids]
    arch = registry.architecture_of(a.model)
    with torch.inference_mode():
        if arch in ("llama", "mistral"):
            from . import sampler as S
            model = registry.load_model(a.model, dev, max_context_len=a.max_tokens)
            for i, p in enumerate(prompts):
                toks, probs = S.generate(model, p, a.max_new_tokens, a.top_k, a.temperature, a.top_p, a.min_p, a.seed)
                print(json.dumps({"request": i, "tokens": toks, "probs": probs}), flush=True)
            return 0
        bs = 32
        model = registry.load_model(a.model, dev, a.dtype, num_blocks=-(-a.max_tokens // bs) + a.max_seqs + 1, block_size=bs, state_slots=a.max_seqs)
        smp = SequenceSampler(model.spec.vocab, dev, a.top_k, a.temperature, a.top_p, a.min_p, a.seed)
        eng = make_engine(model, a.max_tokens, a.max_seqs, sampler=smp)
        seqs = [Sequence(id=i + 1, tokens=list(p), max_new_tokens=a.max_new_tokens) for i, p in enumerate(prompts)]
        for s in seqs:
            eng.s.add_seq(s)
        eng.run()
        for i, s in enumerate(seqs):
            print(json.dumps({"request": i, "tokens": s.generated, "error": s.error}), flush=True)
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="mistralrs", description="MI355X-native inference: generate from token ids, replay a trace, build the HIP libraries")
    sub = ap.add_subparsers(dest="cmd", required=True)
    g = sub.add_parser("generate")
    g.add_argument("--model", required=True)
    g.add_argument("--prompt-ids", action="append", required=True, help="comma-separated token ids; repeat for more requests")
    g.add_argument("--max-new-tokens", type=int, default=16)
    g.add_argument("--top-k", type=int, default=1)
    g.add_argument("--temperature", type=float, default=1.0)
    g.add_argument("--top-p", type=float, default=1.0)
    g.add_argument("--min-p", type=float, default=0.0)
    g.add_argument("--seed", type=int, default=0)
    g.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    g.add_argument("--max-tokens", type=int, default=4096)
    g.add_argument("--max-seqs", type=int, default=4)
    t = sub.add_parser("trace", add_help=False)
    b = sub.add_parser("build")
    b.add_argument("--only", default=None)
    a, rest = ap.parse_known_args(argv)
    if a.cmd == "trace":
        from .trace import main as trace_main
        return trace_main(rest)
    if rest:
        ap.error("unrecognized arguments: " + " ".join(rest))
    if a.cmd == "build":
        import importlib.util
        import os
        spec = importlib.util.spec_from_file_location("mrs_build", os.path.join(os.path.dirname(os.path.abspath(__file__)), "build.py"))
        m = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(m)
        for k, v in m.build(only=a.only.split(",") if a.only else None).items():
            print(k, "->", v)
        return 0
    return _generate(a)


if __name__ == "__main__":
    sys.exit(main())
