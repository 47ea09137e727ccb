"""Replay a trace of steps through the engine's step function and write the logits that the trace asks for.

    python -m zhilight_amd trace --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N < steps.jsonl

One JSON object per input line: {"step": n, "entries": [{"id", "tokens", "want"}], "end": [ids]}.  All entries of a line are ONE step of the
engine (portions of prompts beside single tokens); a request is admitted at its first entry and gives its pages and its state slot back when
a line names it under "end".  For a line that wants logits, OUT/<step>.f32 holds them as little-endian fp32, (wanted, vocab), in the order
of the entries; after every line "done <step>" is printed.  Nothing is sampled.
"""
import json
import os
import sys

import numpy as np


def replay(model_dir, dtype, out_dir, max_tokens, max_seqs=4, stream=None, device="cuda:0"):
    import torch
    from . import registry
    from .engine import Engine, Entry
    stream = stream or sys.stdin
    model = registry.load_model(model_dir, dtype=dtype, device=device)
    engine = Engine(model, max_tokens=max_tokens, max_seqs=max_seqs)
    os.makedirs(out_dir, exist_ok=True)
    for line in stream:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        entries = [Entry(str(e["id"]), [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])]) for e in step.get("entries", [])]
        logits = engine.run_step(entries)
        if logits is not None:
            arr = logits.to(torch.float32).cpu().numpy().astype("<f4")
            tmp = os.path.join(out_dir, ".%s.part" % step["step"])
            with open(tmp, "wb") as fh:
                fh.write(np.ascontiguousarray(arr).tobytes())
            os.replace(tmp, os.path.join(out_dir, "%s.f32" % step["step"]))
        else:
            torch.cuda.synchronize()
        for rid in step.get("end", []):
            engine.release(str(rid))
        sys.stdout.write("done %s\n" % step["step"])
        sys.stdout.flush()
    return 0
