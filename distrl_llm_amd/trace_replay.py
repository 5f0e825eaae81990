"""Trace replay: feed given token ids through an engine step by step and
write the logits it produces. Nothing is sampled.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

The model class and engine are chosen from ``DIR/config.json`` exactly as
the server chooses them; the replay only drives the engine's own
``open_sequence`` / ``step`` / ``close_sequence``. Steps arrive on standard
input, one JSON object per line::

    {"step": 7, "entries": [{"id": "req1", "tokens": [11, 4], "want": [1]},
                            {"id": "req2", "tokens": [9], "want": []}], "end": ["req2"]}

(each object on one line)

All entries of a step run as one batch (prompt portions beside single
tokens). A request is admitted at its first entry and may skip steps;
requests named in ``end`` return their pages and state slot after the
step. When a step wants logits they are written to ``<out>/<step>.f32``
(little-endian fp32, ``[wanted, vocab]``, entry order then ``want``
order); every step is acknowledged with a ``done <step>`` line.

``--max-tokens`` sizes the cache pool (tokens held by live requests, each
request rounded up to whole pages); ``--slots`` the state slots.
"""

from __future__ import annotations

import argparse
import json
import os
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", choices=("bfloat16", "float32"), default="bfloat16")
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--slots", type=int, default=4,
                    help="state slots = most live requests")
    ap.add_argument("--block-size", type=int, default=16)
    args = ap.parse_args(argv)

    import torch

    from .config import EngineConfig
    from .models.registry import load_model_and_engine

    device = torch.device("cuda:0" if torch.cuda.is_available() else "cpu")
    dtype = torch.bfloat16 if args.dtype == "bfloat16" else torch.float32
    if dtype == torch.float32:
        # true fp32 products: no reduced-precision matrix mode
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
    bs = args.block_size
    cfg = EngineConfig(max_seq_length=max(args.max_tokens, bs), kv_block_size=bs,
                       num_kv_blocks=max(1, (args.max_tokens + bs - 1) // bs),
                       num_state_slots=args.slots, max_num_seqs=args.slots)
    _model, engine = load_model_and_engine(args.model, cfg, dtype=dtype,
                                           device=device)
    if not hasattr(engine, "step"):
        sys.stderr.write("this model's engine has no mixed-batch step\n")
        return 4
    os.makedirs(args.out, exist_ok=True)

    live = {}
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        msg = json.loads(line)
        work, want = [], []
        for e in msg.get("entries", []):
            q = live.get(e["id"])
            if q is None:
                q = live[e["id"]] = engine.open_sequence()
            work.append((q, e["tokens"]))
            want.append(list(e.get("want", [])))
        if work:
            logits = engine.step(work, want)
            if logits.shape[0]:
                data = logits.to(torch.float32).cpu().contiguous().numpy()
                tmp = os.path.join(args.out, ".%s.part" % msg["step"])
                with open(tmp, "wb") as f:
                    f.write(data.astype("<f4").tobytes())
                os.replace(tmp, os.path.join(args.out, "%s.f32" % msg["step"]))
            elif device.type == "cuda":
                torch.cuda.synchronize()
        for rid in msg.get("end", []):
            q = live.pop(rid, None)
            if q is not None:
                engine.close_sequence(q)
        sys.stdout.write("done %s\n" % msg["step"])
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
