"""Trace replay: feed given token ids through a served model step by step
and write the logits at chosen places. Nothing is sampled.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps arrive on standard input, one JSON object a line:

    {"step": 7, "entries": [{"id": "req-1", "tokens": [41, 8], "want": [1]},
                            {"id": "req-2", "tokens": [300], "want": []}],
     "end": ["req-2"]}

`entries` bring each request's next tokens and the indices (`want`) among
them whose logits to report; `end` names requests that release their pages
and state slot after the step. The entries of a step form one packed batch
through the engine's chunk forward (InferenceEngine.feed) — prompt portions
next to single decode tokens — continuing from whatever earlier steps left
in the cache. Logits go to OUT/<step>.f32 (rows in entry order, then `want`
order; little-endian fp32, [rows, vocab]) when a step wants any, and every
step is acknowledged with a flushed `done <step>` line on standard output.

The engine is built with a page pool for --max-tokens tokens (each live
request rounded up to whole pages) and state slots for four requests, so
pages and slots are reused as requests end.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

MAX_LIVE = 4


def build_engine(model_dir: str, dtype_name: str, max_tokens: int):
    import torch

    from ..models.spec import resolve_spec
    from . import kv as kv_mod
    from .engine import InferenceEngine

    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype_name]
    if dtype is torch.float32:
        # true fp32 products: no reduced-precision matrix mode
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")
    name = os.path.basename(os.path.normpath(model_dir))
    spec = resolve_spec(name, model_dir)
    device = "cuda" if torch.cuda.is_available() else "cpu"
    if device == "cuda" and not spec.is_hybrid and dtype is torch.float32:
        # the dense-transformer kernels are bf16-only on the GPU
        print("float32 is not available for this model family on the GPU",
              file=sys.stderr)
        sys.exit(3)
    bs = kv_mod.BLOCK_SIZE
    spec.max_seq_len = max(spec.max_seq_len, max_tokens)
    return InferenceEngine(
        spec, device=device, dtype=dtype, model_path=model_dir,
        max_batch=MAX_LIVE, max_seq_len=max_tokens, use_graphs=False,
        # every live request may leave its last page partly empty
        kv_blocks=-(-max_tokens // bs) + MAX_LIVE, kv_margin_blocks=1,
    )


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__,
                                 formatter_class=argparse.RawTextHelpFormatter)
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", choices=("bfloat16", "float32"),
                    default="bfloat16")
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    a = ap.parse_args(argv)
    os.makedirs(a.out, exist_ok=True)
    engine = build_engine(a.model, a.dtype, a.max_tokens)
    import numpy as np

    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        entries = [(e["id"], e["tokens"], e.get("want") or [])
                   for e in step.get("entries", [])]
        logits = engine.feed(entries, step.get("end") or ())
        if logits is not None:
            arr = logits.detach().to("cpu").numpy().astype("<f4")
            path = os.path.join(a.out, "%d.f32" % step["step"])
            with open(path + ".part", "wb") as f:
                f.write(np.ascontiguousarray(arr).tobytes())
            os.replace(path + ".part", path)
        print("done %d" % step["step"], flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
