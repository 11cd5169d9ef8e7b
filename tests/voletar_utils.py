"""Helpers of the Voletar tests: small configurations, checkpoints on disk, an engine over them and
replay of arbitrary step schedules."""
from __future__ import annotations

import json
import os

import numpy as np
import torch

from mxserve.config import EngineArgs
from mxserve.engine.engine import LLMEngine
from mxserve.engine.replay import TraceReplayer
from mxserve.models.voletar import random_state


def lightning(heads=3, dim=32, vdim=48, ff=None, decay=None):
    decay = decay or [0.5 + 0.499 * (i + 1) / heads for i in range(heads)]
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def parallel(heads=4, kv_heads=2, dim=40, vdim=56, size=24, keep=5, scale=0.2, rheads=2, rdim=24, rvdim=40, cap=10.0,
             ff=320):
    return {"type": "parallel",
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                               "mask": {"size": size, "keep_first": keep}},
                      "right": {"heads": rheads, "dim": rdim, "vdim": rvdim, "gate_cap": cap}},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def config(layers, width=192, vocab=384, loop=None, softcap=20.0, eps=1e-5):
    c = {"architecture": "Voletar", "width": width, "vocab": vocab, "layers": layers, "norm": {"eps": eps}}
    if loop:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    if softcap:
        c["logit_softcap"] = softcap
    return c


BASE = config([lightning(), parallel(), lightning(heads=2, dim=48, vdim=32, ff=256),
               parallel(heads=3, kv_heads=3, dim=32, vdim=32, size=17, keep=0, rheads=3, rdim=40, rvdim=24, ff=None)],
              loop=(1, 3, 3))


def write_checkpoint(path, cfg: dict, seed: int = 0, tweak=None) -> dict:
    """config.json + model.safetensors (bf16) under `path`; returns the stored weights as float64 arrays."""
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    sd = {k: v.to(torch.bfloat16).contiguous() for k, v in random_state(cfg, seed).items()}
    if tweak:
        tweak(sd)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file(sd, os.path.join(path, "model.safetensors"))
    return {k: v.double().numpy() for k, v in sd.items()}


def engine(path, device="cpu", dtype="float32", max_tokens=512, max_live=4, eager=True, **kw) -> LLMEngine:
    bs = 16
    blocks = -(-max_tokens // bs)
    args = EngineArgs(model=str(path), device=device, dtype=dtype, block_size=bs, num_gpu_blocks=blocks,
                      cpu_num_blocks=blocks, max_model_len=max(max_tokens, 64), max_num_seqs=max_live,
                      max_num_batched_tokens=max(max_tokens, 64), enable_prefix_caching=False, async_scheduling=False,
                      load_format="safetensors", enforce_eager=eager, cuda_graph_max_bs=max_live, **kw)
    return LLMEngine(args)


def replay(eng: LLMEngine, steps: list) -> dict:
    """steps: [[(request id, tokens, end?)]] -> {request id: logits [n, vocab]} of every token fed."""
    rp = TraceReplayer(eng)
    got: dict = {}
    for n, step in enumerate(steps):
        entries = [{"id": rid, "tokens": list(toks), "want": list(range(len(toks)))} for rid, toks, _ in step]
        lg = rp.step(entries, [rid for rid, _, end in step if end])
        at = 0
        for rid, toks, _ in step:
            got.setdefault(rid, []).append(lg[at:at + len(toks)].double().numpy())
            at += len(toks)
    return {rid: np.concatenate(v) for rid, v in got.items()}


def cut(tokens, sizes):
    """tokens in portions of the given sizes, the last size repeated to the end."""
    out, at, i = [], 0, 0
    while at < len(tokens):
        n = sizes[min(i, len(sizes) - 1)]
        out.append(tokens[at:at + n])
        at += n
        i += 1
    return out


def rel_err(got: np.ndarray, want: np.ndarray) -> float:
    """Largest row error: rms of the difference (mean removed) over the rms of the expected logits."""
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    return float((np.sqrt((d ** 2).mean(-1)) / np.sqrt((want ** 2).mean())).max())
