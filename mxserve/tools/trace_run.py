"""Trace runner: `bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N`.

Reads steps from standard input, one JSON object a line (mxserve/engine/replay.py), runs each
through the engine and, for a step in which logits are wanted, writes OUT/<step>.f32: the wanted
rows' logits as little-endian fp32 [wanted, vocab].  After every step it prints `done <step>`.
The KV pool holds --max-tokens tokens (rounded up to whole blocks) and the engine admits four live
requests, so blocks and state slots are used again as requests end.  Missing native extensions are
built in-tree on the first call."""
from __future__ import annotations

import argparse
import json
import os
import sys


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--max-live", type=int, default=4, help="requests live at any time (state slots)")
    ap.add_argument("--device", default="auto")
    ap.add_argument("--enforce-eager", action="store_true", help="no hipGraph replay of single-token steps")
    a = ap.parse_args(argv)

    import numpy as np
    import torch
    from mxserve.config import EngineArgs
    from mxserve.engine.engine import LLMEngine
    from mxserve.engine.replay import TraceReplayer

    if a.dtype == "float32":  # true fp32 products in the library GEMMs
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
    bs = 16
    blocks = -(-a.max_tokens // bs)
    args = EngineArgs(model=os.path.abspath(a.model), device=a.device, dtype=a.dtype, block_size=bs,
                      num_gpu_blocks=blocks, cpu_num_blocks=blocks, max_model_len=max(a.max_tokens, bs),
                      max_num_seqs=a.max_live, max_num_batched_tokens=max(a.max_tokens, bs),
                      enable_prefix_caching=False, async_scheduling=False, load_format="safetensors",
                      enforce_eager=a.enforce_eager, cuda_graph_max_bs=a.max_live)
    eng = LLMEngine(args)
    rp = TraceReplayer(eng)
    os.makedirs(a.out, exist_ok=True)
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        st = json.loads(line)
        logits = rp.step(st.get("entries") or [], st.get("end") or [])
        if logits is not None:
            arr = np.ascontiguousarray(logits.numpy(), dtype="<f4")
            tmp = os.path.join(a.out, f".{st['step']}.part")
            with open(tmp, "wb") as f:
                f.write(arr.tobytes())
            os.replace(tmp, os.path.join(a.out, f"{st['step']}.f32"))
        sys.stdout.write(f"done {st['step']}\n")
        sys.stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
