"""Trace replay: feed given token ids through the serving engine step by step and write the
logits of chosen positions - no sampling.  Each step is one batch of the engine's model
runner (portions of prompts next to single tokens), run from the paged cache and the state
slots that earlier steps left; requests are admitted at their first portion and release
their pages and slot when the trace ends them.

Input (stdin), one JSON object per line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
Output: ``<out>/<step>.f32`` (little-endian fp32 [wanted rows, vocab], entries' order) for
steps that want rows, and a flushed line ``done <step>`` on stdout after every step.

    python -m agentic_traffic_testing_amd.engine.trace_replay --model DIR \\
        --dtype bfloat16|float32 --out DIR --max-tokens N
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys

import numpy as np


class TraceReplayer:
    def __init__(self, model: str, dtype: str = "bfloat16", max_tokens: int = 4096,
                 max_seqs: int = 4, device: str | None = None, block_size: int = 16):
        import torch

        from ..config import EngineConfig
        from .llm_engine import LLMEngine

        if device is None:
            device = "cuda" if torch.cuda.is_available() else "cpu"
        pool = max(block_size, int(math.ceil(max_tokens / block_size)) * block_size)
        cfg = EngineConfig(model=model, dtype=dtype, device=device, block_size=block_size,
                           max_model_len=pool, max_num_seqs=max_seqs,
                           max_num_batched_tokens=max(pool, 2048),
                           num_kv_blocks=pool // block_size, enable_prefix_caching=False,
                           use_graphs=False, async_decode=False, startup_warmup=False,
                           gemm_tuning="")
        self.engine = LLMEngine(cfg)
        self.vocab = self.engine.model_cfg.vocab_size

    def step(self, entries: list, end: list) -> np.ndarray | None:
        """Run one step; returns the wanted logits [rows, vocab] (None when nothing is wanted)."""
        portions = [(e["id"], [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])])
                    for e in entries]
        out = self.engine.replay_step(portions)
        for rid in end:
            self.engine.finish_request(rid)
        return out


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, default=4096)
    ap.add_argument("--max-seqs", type=int, default=4)
    ap.add_argument("--device", default=None)
    a = ap.parse_args(argv)
    os.makedirs(a.out, exist_ok=True)
    rp = TraceReplayer(a.model, a.dtype, a.max_tokens, a.max_seqs, a.device)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        msg = json.loads(line)
        logits = rp.step(msg.get("entries", []), msg.get("end", []))
        if logits is not None:
            path = os.path.join(a.out, f"{msg['step']}.f32")
            with open(path + ".part", "wb") as f:
                f.write(np.ascontiguousarray(logits, dtype="<f4").tobytes())
            os.replace(path + ".part", path)
        sys.stdout.write(f"done {msg['step']}\n")
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
