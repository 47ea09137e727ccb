"""Command line of the package.

    python -m zhilight_amd models                                  the registered model names
    python -m zhilight_amd generate --model DIR --prompt 1,2,3 [--prompt ...] [--max-new-tokens N] [--temperature T] [--top-k K]
                                    [--top-p P] [--seed S] [--dtype bfloat16|float32] [--max-tokens N]
    python -m zhilight_amd trace --model DIR --dtype D --out DIR --max-tokens N      (steps on standard input; see trace.py)
    python -m zhilight_amd build [--force]                         compile every library in-tree
"""
import argparse
import json
import sys


def main(argv=None):
    ap = argparse.ArgumentParser(prog="python -m zhilight_amd")
    sub = ap.add_subparsers(dest="cmd", required=True)
    sub.add_parser("models")
    b = sub.add_parser("build")
    b.add_argument("--force", action="store_true")
    for name in ("generate", "trace"):
        p = sub.add_parser(name)
        p.add_argument("--model", required=True)
        p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
        p.add_argument("--max-tokens", type=int, default=4096, help="tokens that live requests may hold in the cache at any time")
        p.add_argument("--max-seqs", type=int, default=4)
        p.add_argument("--device", default="cuda:0")
        if name == "trace":
            p.add_argument("--out", required=True)
        else:
            p.add_argument("--prompt", action="append", required=True, help="token ids with commas between them; may be given several times")
            p.add_argument("--max-new-tokens", type=int, default=16)
            p.add_argument("--temperature", type=float, default=0.0)
            p.add_argument("--top-k", type=int, default=0)
            p.add_argument("--top-p", type=float, default=1.0)
            p.add_argument("--seed", type=int, default=0)
            p.add_argument("--max-step-tokens", type=int, default=512)
    a = ap.parse_args(argv)
    if a.cmd == "models":
        from . import registry
        print("\n".join(registry.registered()))
        return 0
    if a.cmd == "build":
        from . import build
        print(build.build(force=a.force, verbose=True))
        return 0
    if a.cmd == "trace":
        from . import trace
        return trace.replay(a.model, a.dtype, a.out, a.max_tokens, a.max_seqs, device=a.device)
    from . import registry
    from .engine import Engine, SamplingParams
    model = registry.load_model(a.model, dtype=a.dtype, device=a.device)
    if not getattr(model, "ragged", False):
        print("generate: this model class is driven through its own context (llama.LLaMA.new_context / prefill / step_greedy)", file=sys.stderr)
        return 2
    engine = Engine(model, max_tokens=a.max_tokens, max_seqs=a.max_seqs, max_step_tokens=a.max_step_tokens)
    prompts = [[int(t) for t in p.split(",") if t.strip()] for p in a.prompt]
    outs = engine.generate(prompts, SamplingParams(a.max_new_tokens, a.temperature, a.top_k, a.top_p, a.seed))
    for p, o in zip(prompts, outs):
        print(json.dumps({"prompt": p, "tokens": o}))
    return 0


if __name__ == "__main__":
    sys.exit(main())
