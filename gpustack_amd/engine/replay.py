"""Trace replay: feed recorded token ids through the engine step by step
and write the logits of chosen positions — nothing is sampled.

The driver reads one JSON object per line on its input,

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}],
     "end": []}

runs all entries of a step as ONE engine batch (LLMEngine.replay_step: the
scheduler's forced-token path, the model runner, the paged pool and the
kernels that serve generation), writes OUT/<step>.f32 (little-endian fp32
[wanted, vocab]) when something was wanted, and prints `done <step>`.
Requests named in "end" give their blocks back to the pool after the step.
The pool is sized for `max_tokens` live tokens, so blocks are re-used while
a trace runs.
"""
from __future__ import annotations

import json
import sys
from pathlib import Path


def build_engine(model_dir: str, dtype: str, max_tokens: int,
                 max_requests: int = 4, device: str | None = None):
    import torch

    from .config import EngineConfig
    from .engine import LLMEngine

    if device is None:
        device = "cuda" if torch.cuda.is_available() else "cpu"
    if dtype == "float32":
        # true fp32 products: no reduced-precision matrix modes
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")
    bs = EngineConfig.block_size
    # every live request may leave its last block partly empty; one more
    # block is the pool's reserved padding block
    blocks = (max_tokens + bs - 1) // bs + max_requests + 1
    cfg = EngineConfig(
        model=model_dir, dtype=dtype, device=device,
        enforce_random_weights=False, kv_cache_blocks=blocks,
        max_num_seqs=max_requests, max_model_len=max(max_tokens, 1),
        max_prefill_tokens=max(max_tokens, 1))
    return LLMEngine(cfg)


def run_trace(model_dir: str, dtype: str, out_dir: str, max_tokens: int,
              lines=None, out=None, device: str | None = None) -> int:
    lines = sys.stdin if lines is None else lines
    out = sys.stdout if out is None else out
    eng = build_engine(model_dir, dtype, max_tokens, device=device)
    outp = Path(out_dir)
    outp.mkdir(parents=True, exist_ok=True)
    for line in lines:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        entries = [(e["id"], e["tokens"], e.get("want") or [])
                   for e in step.get("entries", []) if e.get("tokens")]
        logits = eng.replay_step(entries, step.get("end") or [])
        if logits is not None and logits.shape[0] > 0:
            arr = logits.detach().float().cpu().contiguous().numpy()
            arr.astype("<f4").tofile(outp / f"{step['step']}.f32")
        print(f"done {step['step']}", file=out, flush=True)
    return 0
