"""Replay of a recorded token schedule through the engine.

A trace is a sequence of steps; each step lists, per request, the next
tokens to feed (a prompt portion, or one decoded token) and the places among
them whose logits are wanted, plus the requests that end after the step.
Nothing is sampled: the tokens are given. Every step is one engine batch run
by ``LLMEngine.forced_step`` on the engine's own scheduler structures, block
and state-slot managers, model runner and kernels.

Step format (one JSON object per line)::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}],
     "end": ["a"]}

For a step with wanted places the logits are written as little-endian fp32
``[wanted, vocab]`` to ``<out>/<step>.f32``; after every step the line
``done <step>`` is printed.
"""

from __future__ import annotations

import json
import os
import sys
from typing import Dict, List, Optional

import torch

from kserve_amd.engine.config import CacheConfig, EngineConfig, SchedulerConfig
from kserve_amd.engine.request import Request
from kserve_amd.engine.sampling_params import SamplingParams

# live requests a replayed trace may hold at once (state slots of the engine)
MAX_LIVE_REQUESTS = 4


def engine_config_for_trace(
    model_dir: str, dtype: str, max_tokens: int, device: str,
    block_size: Optional[int] = None, enforce_eager: bool = False,
) -> EngineConfig:
    from kserve_amd.models.registry import load_model_config

    model_cfg = load_model_config(model_dir)
    model_cfg.dtype = dtype
    cache = CacheConfig() if block_size is None else CacheConfig(block_size=block_size)
    bs = cache.block_size
    # the pool holds max_tokens (each request rounded up to whole pages by
    # the caller's accounting) plus the reserved scratch block 0
    cache.num_gpu_blocks = -(-max_tokens // bs) + 1
    sched = SchedulerConfig(
        max_num_seqs=MAX_LIVE_REQUESTS,
        max_num_batched_tokens=max(max_tokens, 1),
        max_model_len=max(max_tokens, 1),
        enable_chunked_prefill=True,
        multi_step=1,
    )
    return EngineConfig(
        model=model_cfg, cache=cache, scheduler=sched, device=device,
        model_path=model_dir, enforce_eager=enforce_eager, eos_token_id=-1,
    )


class TraceReplayer:
    def __init__(self, engine):
        self.engine = engine
        self.live: Dict[str, Request] = {}

    def step(self, entries: List[dict], end: List[str]) -> Optional[torch.Tensor]:
        items = []
        rows: List[int] = []
        decode_only = True
        off = 0
        for e in entries:
            toks = [int(t) for t in e["tokens"]]
            req = self.live.get(e["id"])
            if req is None:
                req = Request(
                    e["id"], [], SamplingParams(max_tokens=None, ignore_eos=True),
                    eos_token_id=None,
                )
                self.live[e["id"]] = req
            req.prompt_token_ids.extend(toks)
            if not (len(toks) == 1 and req.num_computed_tokens > 0):
                decode_only = False
            items.append((req, len(toks)))
            rows.extend(off + int(w) for w in e.get("want", []))
            off += len(toks)
        logits = None
        if items:
            if decode_only:
                # decode batches yield one row per request
                rows = []
                for i, e in enumerate(entries):
                    rows.extend(i for _ in e.get("want", []))
            logits = self.engine.forced_step(items, rows)
        done = [self.live.pop(i) for i in end if i in self.live]
        if done:
            self.engine.release(done)
        return logits


def run(args) -> int:
    import torch

    if args.dtype not in ("bfloat16", "float32"):
        print(f"unsupported dtype {args.dtype}", file=sys.stderr)
        return 2
    if args.dtype == "float32":
        # true fp32 matrix products: no reduced-precision matmul modes
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")
    device = args.device or ("cuda" if torch.cuda.is_available() else "cpu")
    from kserve_amd.engine.engine import LLMEngine

    cfg = engine_config_for_trace(
        args.model, args.dtype, args.max_tokens, device,
        block_size=args.block_size, enforce_eager=args.enforce_eager,
    )
    engine = LLMEngine(cfg)
    replayer = TraceReplayer(engine)
    os.makedirs(args.out, exist_ok=True)
    proto = getattr(args, "proto", None) or sys.stdout
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        logits = replayer.step(step.get("entries", []), step.get("end", []))
        if logits is not None:
            data = logits.detach().to(torch.float32).cpu().contiguous().numpy()
            tmp = os.path.join(args.out, f".{step['step']}.part")
            with open(tmp, "wb") as f:
                f.write(data.astype("<f4").tobytes())
            os.replace(tmp, os.path.join(args.out, f"{step['step']}.f32"))
        proto.write(f"done {step['step']}\n")
        proto.flush()
    return 0
