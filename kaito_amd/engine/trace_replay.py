"""Replay a step trace through the serving engine and write the logits.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Each line of standard input is one step,

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

naming, per request, its next tokens and the offsets among them whose
logits are wanted; `end` lists requests that are finished after the step.
All entries of a step run as ONE engine batch (prompt portions beside
single tokens). For a step with wanted rows the logits are written to
<out>/<step>.f32 (little-endian f32, [rows, vocab], in entry/offset
order); after every step `done <step>` is printed.

The replay owns only the composition of steps. Admission, page and
state-slot bookkeeping, batch preparation and the forward pass are the
engine's (LLMEngine.extend_request / step_explicit / release).
"""
from __future__ import annotations

import argparse
import json
import os
import sys

EXIT_UNSUPPORTED_DTYPE = 3


def build_engine(model_dir: str, dtype: str, max_tokens: int,
                 device: str = "cuda", max_live: int = 4):
    import torch

    from ..models.registry import config_from_checkpoint
    from ..parallel.state import init_parallel
    from .config import EngineConfig
    from .engine import LLMEngine

    tdtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
    with open(os.path.join(model_dir, "config.json")) as f:
        mcfg = config_from_checkpoint(json.load(f), name="trace-model",
                                      dtype=tdtype)
    if mcfg.runtime != "native":
        raise SystemExit(f"no native model class for {model_dir}")
    if tdtype == torch.float32 and mcfg.arch == "llama":
        # the rotary-model kernels are bf16-only
        raise SystemExit(EXIT_UNSUPPORTED_DTYPE)
    if tdtype == torch.float32:
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
    init_parallel(1)
    cfg = EngineConfig(
        model=mcfg, device=device, max_num_seqs=max_live,
        max_model_len=mcfg.max_position,
        num_gpu_blocks=-(-max_tokens // EngineConfig.block_size),
        enforce_eager=True, enable_prefix_caching=False)
    return LLMEngine(cfg, weights_path=model_dir)


def replay(engine, lines, out_dir: str, say=print) -> None:
    import numpy as np

    ids = {}                     # request name → engine sequence id
    next_id = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        portions, want = [], []
        for i, e in enumerate(step["entries"]):
            if e["id"] not in ids:
                ids[e["id"]] = next_id
                next_id += 1
            sid = ids[e["id"]]
            engine.extend_request(sid, e["tokens"])
            portions.append((sid, len(e["tokens"])))
            want.extend((i, int(o)) for o in e.get("want", ()))
        logits = engine.step_explicit(portions, want) if portions else None
        if logits is not None:
            arr = logits.detach().to("cpu").numpy().astype("<f4")
            tmp = os.path.join(out_dir, f".{step['step']}.f32.part")
            arr.tofile(tmp)
            os.replace(tmp, os.path.join(out_dir, f"{step['step']}.f32"))
        elif engine.runner.is_gpu:
            import torch
            torch.cuda.synchronize()
        for name in step.get("end", ()):
            if name in ids:
                engine.release(ids.pop(name))
        say(f"done {step['step']}")


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__,
                                 formatter_class=argparse.RawTextHelpFormatter)
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", choices=("bfloat16", "float32"),
                    default="bfloat16")
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--device", default="cuda",
                    help="cuda (serving path) or cpu (reference ops, "
                         "development only)")
    a = ap.parse_args(argv)
    os.makedirs(a.out, exist_ok=True)
    engine = build_engine(a.model, a.dtype, a.max_tokens, a.device)

    def say(text):
        sys.stdout.write(text + "\n")
        sys.stdout.flush()

    replay(engine, sys.stdin, a.out, say)
    return 0


if __name__ == "__main__":
    sys.exit(main())
