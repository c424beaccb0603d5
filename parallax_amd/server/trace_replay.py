"""Replay a token trace through the engine and write logits.

Reads one JSON object per line from a stream,

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}],
     "end": []}

feeds every entry's tokens through Engine.replay_step (the scheduler's batch
formation, the cache manager's pages and state slots, the model's prefill and
decode forwards — nothing is sampled), writes the fp32 logits at the wanted
places to <out>/<step>.f32 ([wanted, vocab], little-endian) and prints
'done <step>' after each step. Useful to compare engines, dtypes or batching
schedules position by position.
"""

from __future__ import annotations

import json
import os
import sys
from typing import IO, Optional

import torch

from ..models.config import ModelConfig
from ..utils.logging_config import get_logger
from .engine import Engine, EngineArgs

logger = get_logger("server.trace_replay")


def needed_extensions(cfg: ModelConfig, dtype: torch.dtype):
    """The HIP extensions a model's forward loads on a GPU."""
    names = []
    if cfg.layer_specs is not None:
        names.append("_mix")
        if dtype == torch.bfloat16:
            names.append("_C")      # tuned GEMMs, grouped-GEMM experts
    else:
        names.append("_C")
    return names


def build_engine(model_path: str, dtype: torch.dtype, max_tokens: int,
                 max_requests: int = 4, device: Optional[torch.device] = None,
                 block_size: int = 32, enable_graphs: bool = True) -> Engine:
    cfg = ModelConfig.from_pretrained(model_path)
    pages = (max_tokens + block_size - 1) // block_size
    args = EngineArgs(
        block_size=block_size,
        num_kv_blocks=pages,
        max_batch_size=max_requests,
        extra_linear_slots=0,
        dtype=dtype,
        enable_prefix_cache=False,
        enable_graphs=enable_graphs and dtype != torch.float32,
        max_model_len=max(block_size, pages * block_size),
        max_num_tokens_per_batch=max(16384, max_tokens),
    )
    if device is not None:
        from ..parallel.comm import CommContext

        comm = CommContext(world_size=1, rank=0, pp_size=1, tp_size=1,
                           pp_rank=0, tp_rank=0, device=device)
        return Engine(cfg, args, comm=comm, model_path=model_path)
    return Engine(cfg, args, model_path=model_path)


def replay(engine: Engine, stream: IO[str], out_dir: str,
           done: IO[str] = sys.stdout) -> int:
    steps = 0
    for line in stream:
        line = line.strip()
        if not line:
            continue
        msg = json.loads(line)
        entries = [(e["id"], e["tokens"], e.get("want", []))
                   for e in msg.get("entries", [])]
        logits = None
        if entries:
            logits = engine.replay_step(entries, msg.get("end", []))
        else:
            for rid in msg.get("end", []):
                engine.scheduler.finish_forced(rid)
        if logits is not None and logits.numel():
            data = logits.to(torch.float32).cpu().contiguous().numpy()
            if sys.byteorder != "little":
                data = data.byteswap()
            tmp = os.path.join(out_dir, ".%s.part" % msg["step"])
            with open(tmp, "wb") as f:
                f.write(data.tobytes())
            os.replace(tmp, os.path.join(out_dir, "%s.f32" % msg["step"]))
        done.write("done %s\n" % msg["step"])
        done.flush()
        steps += 1
    return steps


def main(argv=None) -> int:
    import argparse

    ap = argparse.ArgumentParser(
        prog="trace_run",
        description="replay a token trace (JSON lines on stdin) through the "
                    "engine and write logits")
    ap.add_argument("--model", required=True, help="folder with config.json "
                    "and model.safetensors")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="tokens the cache pool is sized for")
    ap.add_argument("--max-requests", type=int, default=4,
                    help="requests live at once (batch rows, state slots)")
    ap.add_argument("--device", default=None,
                    help="torch device (default: cuda:0; a CPU run must be "
                         "asked for explicitly)")
    ap.add_argument("--no-graphs", action="store_true",
                    help="run decode steps eagerly instead of from hipGraphs")
    a = ap.parse_args(argv)

    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[a.dtype]
    # keep our own chatter off stdout: the caller reads 'done <step>' there
    real_stdout = sys.stdout
    sys.stdout = sys.stderr
    device = torch.device(a.device) if a.device else None
    on_gpu = device is None or device.type == "cuda"
    if on_gpu:
        from ..ops.build import ensure_extensions

        cfg = ModelConfig.from_pretrained(a.model)
        ensure_extensions(needed_extensions(cfg, dtype))
        if not torch.cuda.is_available():
            print("trace_run: no GPU visible (pass --device cpu to run the "
                  "eager CPU engine)", file=sys.stderr)
            return 2
        # true fp32 products: no reduced-precision matrix modes
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
        torch.set_float32_matmul_precision("highest")
    os.makedirs(a.out, exist_ok=True)
    engine = build_engine(a.model, dtype, a.max_tokens, a.max_requests,
                          device=device, enable_graphs=not a.no_graphs)
    replay(engine, sys.stdin, a.out, done=real_stdout)
    return 0


if __name__ == "__main__":
    sys.exit(main())
