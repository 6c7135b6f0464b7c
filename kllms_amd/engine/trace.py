"""Replay of a recorded step schedule through the engine.

A schedule is a stream of JSON lines, one per engine step:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

Every entry continues request ``id`` by its next tokens (a prompt portion or
one decoded token); all entries of a line run as ONE batch through
LLMEngine.step_segments — the engine's own step function, cache / state
manager and kernels. ``want`` lists the places among the entry's tokens whose
logits are written (fp32 little-endian, [wanted, vocab], entry order) to
``<out>/<step>.f32``; ``end`` names requests whose cache blocks and state slot
are returned after the step. Nothing is sampled. After each step the line
``done <step>`` is printed and flushed.

The engine is sized by ``max_tokens`` (live tokens, each request rounded up
to whole cache blocks) and ``max_live`` state slots, so blocks and slots are
reused across requests.
"""

from __future__ import annotations

import json
import os
import sys
from typing import Dict, IO, Optional

import torch

from .config import EngineConfig
from .engine import LLMEngine
from .kvcache import SequenceKV


def build_engine(model_dir: str, dtype: str, max_tokens: int, max_live: int = 4,
                 device: Optional[str] = None) -> LLMEngine:
    cfg = EngineConfig(model=model_dir, dtype=dtype, device=device, use_hip_graphs=False,
                       enable_prefix_caching=False, max_state_slots=max_live,
                       max_batch_size=max_live, max_seq_len=max(max_tokens, 1))
    bs = cfg.kv_block_size
    # every live request may waste up to one block of rounding
    cfg.max_kv_blocks = (max_tokens + bs - 1) // bs + max_live
    if dtype == "float32":
        # true fp32 matrix products: no reduced-precision matmul mode
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")
    return LLMEngine(cfg)


class TraceSession:
    def __init__(self, engine: LLMEngine, out_dir: str):
        self.engine = engine
        self.out_dir = out_dir
        self.live: Dict[str, SequenceKV] = {}

    def step(self, line: dict) -> None:
        eng = self.engine
        entries = []
        for e in line.get("entries", []):
            seq = self.live.get(e["id"])
            if seq is None:
                seq = self.live[e["id"]] = eng.open_sequence()
            entries.append((seq, [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])]))
        logits = eng.step_segments(entries)
        if logits is not None:
            data = logits.to(torch.float32).contiguous().cpu().numpy().astype("<f4")
            tmp = os.path.join(self.out_dir, f".{line['step']}.part")
            with open(tmp, "wb") as f:
                f.write(data.tobytes())
            os.replace(tmp, os.path.join(self.out_dir, f"{line['step']}.f32"))
        elif eng.device.type == "cuda":
            torch.cuda.synchronize()
        for rid in line.get("end", []):
            seq = self.live.pop(rid, None)
            if seq is not None:
                eng.kv.free_sequence(seq)

    def run(self, inp: IO[str], out: IO[str]) -> None:
        for raw in inp:
            raw = raw.strip()
            if not raw:
                continue
            line = json.loads(raw)
            self.step(line)
            out.write(f"done {line['step']}\n")
            out.flush()


def main(argv=None) -> int:
    import argparse

    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--out", required=True, help="folder for the <step>.f32 logit files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (sizes the cache pool)")
    ap.add_argument("--max-live", type=int, default=4, help="state slots = most requests live at once")
    ap.add_argument("--device", default=None, help="default: cuda if present, else cpu")
    a = ap.parse_args(argv)
    os.makedirs(a.out, exist_ok=True)
    engine = build_engine(a.model, a.dtype, a.max_tokens, a.max_live, a.device)
    TraceSession(engine, a.out).run(sys.stdin, sys.stdout)
    return 0


if __name__ == "__main__":
    sys.exit(main())
