"""`trace_run` -- replay a token trace through the engine and write logits.

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps arrive on standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

Every step is one `LLMEngine.forced_step`: all entries form one batch
(several tokens: a prompt chunk; one token of a live request: a decode row),
through the scheduler's page management, the model runner and the model's
kernels -- the path generation takes, with the tokens given instead of
sampled.  For a step that wants logits, `<out>/<step>.f32` holds them as
little-endian float32 [wanted, vocab], in the order of the entries and of
`want`; after every step `done <step>` is printed.  The KV pool holds
--max-tokens tokens (requests rounded up to whole blocks) and four live
requests, so pages are reused as requests end.

Exit code 3: the model's class has no kernels for --dtype.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

LIVE_REQUESTS = 4
BLOCK_SIZE = 64


def main(argv: list[str] | None = None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run")
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--device", default=None, help="default: cuda when a GPU is visible, else cpu")
    a = ap.parse_args(argv)

    from ..models.config import get_config
    from ..models.registry import supports_dtype

    mcfg = get_config(a.model)
    if not supports_dtype(mcfg.architecture, a.dtype):
        print(f"trace_run: {mcfg.architecture} has no {a.dtype} kernels", file=sys.stderr)
        return 3

    import numpy as np
    import torch

    from ..engine.engine import EngineConfig, LLMEngine

    if a.dtype == "float32":  # true fp32 products, no reduced-precision matrix mode
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
    device = a.device or ("cuda" if torch.cuda.is_available() else "cpu")
    blocks = max(1, -(-a.max_tokens // BLOCK_SIZE))
    eng = LLMEngine(EngineConfig(
        model=a.model, random_init=False, dtype=a.dtype, device=device, block_size=BLOCK_SIZE,
        num_gpu_blocks=blocks, max_model_len=blocks * BLOCK_SIZE, max_num_seqs=LIVE_REQUESTS,
        enable_prefix_caching=False, use_cuda_graph=False, async_schedule=False), model_cfg=mcfg)
    os.makedirs(a.out, exist_ok=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        entries = [(e["id"], e["tokens"], e.get("want") or []) for e in st["entries"]]
        got = eng.forced_step(entries, st.get("end") or [])
        parts = [got[rid] for rid, _, want in entries if want]
        if parts:
            out = torch.cat(parts, 0).to("cpu", torch.float32).numpy().astype("<f4")
            tmp = os.path.join(a.out, f".{st['step']}.tmp")
            out.tofile(tmp)
            os.replace(tmp, os.path.join(a.out, f"{st['step']}.f32"))
        elif device == "cuda":
            torch.cuda.synchronize()
        print(f"done {st['step']}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
