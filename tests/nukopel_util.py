"""Helpers shared by the Nukopel tests: write a small random checkpoint,
serve it with the engine, replay token schedules through feed() and compare
with the plain whole-sequence oracle."""
from __future__ import annotations

import random
from typing import Dict, List, Sequence, Tuple

import torch

from tests import nukopel_oracle as O


def make_engine(tmp_path, cfg, W, device="cpu", dtype=torch.float32,
                max_batch=4, block_size=16, kv_blocks=64, max_seq_len=1024,
                **kw):
    from bee2bee_amd.engine.engine import InferenceEngine

    path = str(tmp_path / "ckpt")
    O.save_checkpoint(path, cfg, W)
    return InferenceEngine(
        "nk-test", device=device, dtype=dtype, model_path=path,
        max_batch=max_batch, max_seq_len=max_seq_len, use_graphs=kw.pop(
            "use_graphs", False),
        kv_block_size=block_size, kv_blocks=kv_blocks, kv_margin_blocks=1, **kw)


def oracle_logits(cfg, W, tokens: Sequence[int]) -> torch.Tensor:
    return O.forward(list(tokens), W, cfg, dtype=torch.float64)[0]


def row_errs(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Per row: RMS difference relative to the RMS of the expected logits."""
    got, want = got.double().cpu(), want.double().cpu()
    d = (got - want).pow(2).mean(-1).sqrt()
    return d / want.pow(2).mean(-1).sqrt().clamp_min(1e-12)


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    return float(row_errs(got, want).max())


def assert_logits(got: torch.Tensor, want: torch.Tensor, dtype,
                  what: str = "") -> None:
    """fp32 runs must match the oracle row by row. bf16 runs carry rounding
    noise, and a row whose router sees a near-tie may pick another expert:
    they must be close on average with few outliers."""
    e = row_errs(got, want)
    if dtype is torch.float32:
        assert float(e.max()) < 2e-4, (what, float(e.max()))
    else:
        assert float(e.mean()) < 0.05, (what, float(e.mean()))
        assert float((e > 0.12).float().mean()) <= 0.1, (what, e)


def replay(engine, requests: Dict[str, List[int]],
           schedule: List[List[Tuple[str, int]]]) -> Dict[str, torch.Tensor]:
    """schedule: steps of (request id, token count). Every position's logits
    are collected; a request is ended when its tokens run out."""
    at = {r: 0 for r in requests}
    rows: Dict[str, List[torch.Tensor]] = {r: [] for r in requests}
    for step in schedule:
        entries, end = [], []
        for rid, n in step:
            lo, hi = at[rid], at[rid] + n
            entries.append((rid, requests[rid][lo:hi], list(range(n))))
            at[rid] = hi
            if hi == len(requests[rid]):
                end.append(rid)
        logits = engine.feed(entries, end)
        o = 0
        for rid, n in step:
            rows[rid].append(logits[o:o + n].cpu())
            o += n
    return {r: torch.cat(v) for r, v in rows.items() if v}


def random_tokens(n: int, vocab: int, seed: int) -> List[int]:
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


def chunk_schedule(rid: str, total: int, sizes: Sequence[int]):
    """Portions of the given sizes (cycled) until `total` tokens are fed."""
    out, at, i = [], 0, 0
    while at < total:
        n = min(sizes[i % len(sizes)], total - at)
        out.append([(rid, n)])
        at += n
        i += 1
    return out
