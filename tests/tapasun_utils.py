"""Helpers of the Tapasun tests: small configurations and checkpoints on disk.  The engine, replay
and error helpers are those of the Voletar tests (they know nothing of a design)."""
from __future__ import annotations

import json
import os

import torch

from mxserve.models.tapasun import random_state
from tests.voletar_utils import cut, engine, rel_err, replay  # noqa: F401

BANDS = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 48}


def ff(n):
    return {"kind": "dense", "ff": n} if n else None


def mamba2(heads=4, vdim=24, state=40, groups=2, conv=4, norm_groups=2, mlp=96):
    return {"type": "mamba2", "mlp": ff(mlp),
            "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}}


def rot(dims, base=10000.0, scaling=None):
    r = {"dims": dims, "base": base}
    if scaling:
        r["scaling"] = scaling
    return r


def attention(heads=6, kv_heads=3, dim=24, vdim=40, scale=0.25, dims=16, base=10000.0, scaling=BANDS, kv_from=None, mlp=96):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": rot(dims, base, scaling)}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mlp": ff(mlp), "mixer": m}


def parallel(heads=4, kv_heads=2, dim=24, vdim=16, scale=0.3, dims=8, base=500.0, factor=2.0, rheads=4, rkv=2, rdim=24,
             rvdim=40, conv=3, ls=0.7, rs=1.2, mlp=96):
    return {"type": "parallel", "mlp": ff(mlp), "mixer": {
        "left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                 "rot": rot(dims, base, {"factor": factor})},
        "right": {"heads": rheads, "kv_heads": rkv, "dim": rdim, "vdim": rvdim, "conv": conv},
        "left_scale": ls, "right_scale": rs}}


def config(layers, width=112, vocab=320, eps=1e-5, embed_scale=3.0):
    return {"architecture": "Tapasun", "width": width, "vocab": vocab, "layers": layers, "norm": {"eps": eps},
            "embedding": {"scale": embed_scale}}


BASE = config([mamba2(), attention(), parallel(), attention(kv_from=1, mlp=None), mamba2(heads=3, vdim=16, state=24, groups=3,
                                                                                         conv=2, norm_groups=1, mlp=None),
               parallel(heads=2, kv_heads=1, dim=16, vdim=24, dims=16, rheads=2, rkv=2, rdim=40, rvdim=16, conv=4, ls=1.1, rs=0.4)])


def write_checkpoint(path, cfg: dict, seed: int = 0, ranks=(12, 20), tweak=None) -> dict:
    """config.json + model.safetensors (bf16) under `path`; returns the stored weights as float64
    arrays.  ranks: the inner sizes of the delta rule's low-rank pairs, which only the tensors tell."""
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    g = torch.Generator().manual_seed(seed + 1000)
    sd = random_state(cfg, seed)
    for name in [n for n in sd if n.endswith(".a1") or n.endswith(".g1")]:
        r = ranks[0] if name.endswith(".a1") else ranks[1]
        two = name[:-1] + "2"
        sd[name] = torch.randn(r, sd[name].shape[1], generator=g) * sd[name].shape[1] ** -0.5
        sd[two] = torch.randn(sd[two].shape[0], r, generator=g) * r ** -0.5
    sd = {k: v.to(torch.bfloat16).contiguous() for k, v in sd.items()}
    if tweak:
        tweak(sd)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file(sd, os.path.join(path, "model.safetensors"))
    return {k: v.double().numpy() for k, v in sd.items()}
