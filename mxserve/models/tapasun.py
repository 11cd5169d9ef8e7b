"""Tapasun: a decoder whose config.json lists its layers.  A layer is
    x <- x + norm1b(mixer(norm1(x))),   x <- x + norm2b(ff(norm2(x)))        (the second when it has a feed-forward)
with RMS norms that have one weight for all coordinates, and one of three mixers:

  mamba2      selective state space (mixers.Mamba2)
  attention   rotary softmax attention with per-head q/k norm, band-scaled frequencies and one more
              exp(0) in the denominator; `kv_from: j` reads layer j's pages (mixers.RotaryAttention)
  parallel    left_scale * attention (linearly scaled rotary, learned sink per head, values turned by
              their position) + right_scale * gated delta rule (mixers.ScaledPair, GatedDeltaRule)

The embedding is multiplied by `embedding.scale`; the feed-forward is W_down(SiLU(W_gate h) * W_up h);
the logits are head(norm(x)).  The residual stream is fp32 from the embedding to the final norm: a
sublayer's output is RMS-normed, weighed, added, and the next norm taken in one kernel
(seqmix.resid_update).  A layer's input projections are one GEMM, so are a feed-forward's gate and up,
and a parallel layer's two output projections.  One forward = one engine step over a flattened token
batch: paged K/V through the block tables, fp32 recurrent and convolution state in the runner's slots.
"""
from __future__ import annotations

import sys
from typing import Optional

import torch

from .. import ops
from ..ops import seqmix
from .config import ModelConfig
from .hybrid import HybridLM, LayerPlan, plan_runs
from .mixers import GatedDeltaRule, Mamba2, Mixer, RotaryAttention, ScaledPair, StepContext


def build_mixer(kind: str, prefix: str, width: int, mc: dict) -> Mixer:
    """A layer's mixer from its config entry (`type` and `mixer`)."""
    if kind == "mamba2":
        return Mamba2(prefix, width, int(mc["heads"]), int(mc["vdim"]), int(mc["state"]), int(mc["groups"]),
                      int(mc["conv"]), int(mc["norm_groups"]))
    if kind == "attention":
        return RotaryAttention(prefix, width, int(mc["heads"]), int(mc["kv_heads"]), int(mc["dim"]), int(mc["vdim"]),
                               float(mc["scale"]), mc["rot"], qk_norm=True, sink="zero", kv_from=mc.get("kv_from"))
    if kind == "parallel":
        l, r = mc["left"], mc["right"]
        left = RotaryAttention(prefix + "left.", width, int(l["heads"]), int(l["kv_heads"]), int(l["dim"]),
                               int(l["vdim"]), float(l["scale"]), l["rot"], qk_norm=False, sink="learned",
                               rotate_values=True, kv_from=l.get("kv_from"))
        right = GatedDeltaRule(prefix + "right.", width, int(r["heads"]), int(r["kv_heads"]), int(r["dim"]),
                               int(r["vdim"]), int(r["conv"]))
        return ScaledPair(prefix, width, left, right, float(mc["left_scale"]), float(mc["right_scale"]))
    raise ValueError(f"unknown mixer type {kind!r}")


def mixers_of(ac: dict) -> list:
    return [build_mixer(l["type"], f"l{i}.mix.", int(ac["width"]), l["mixer"]) for i, l in enumerate(ac["layers"])]


def layer_plan(ac: dict, block_size: int = 16, mixers: Optional[list] = None) -> LayerPlan:
    """Every layer runs once, in order; a layer with `kv_from` shares the pages of the layer it names."""
    mixers = mixers or mixers_of(ac)
    return plan_runs([(i, None, False) for i in range(len(mixers))], mixers, block_size)


def weight_shapes(ac: dict, mixers: Optional[list] = None) -> dict:
    """Checkpoint tensor names and shapes (a norm's weight is a single number)."""
    W, V = int(ac["width"]), int(ac["vocab"])
    mixers = mixers or mixers_of(ac)
    sh = {"embed": (V, W), "final.norm": (), "head": (V, W)}
    for i, (l, m) in enumerate(zip(ac["layers"], mixers)):
        p = f"l{i}."
        sh[p + "norm1"] = sh[p + "norm1b"] = ()
        for name, rows in m.proj_rows():
            sh[name] = (rows, W)
        sh.update(m.extra_shapes())
        mlp = l.get("mlp")
        if mlp:
            if mlp.get("kind", "dense") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            sh[p + "norm2"] = sh[p + "norm2b"] = ()
            sh[p + "mlp.gate"] = sh[p + "mlp.up"] = (int(mlp["ff"]), W)
            sh[p + "mlp.down"] = (W, int(mlp["ff"]))
    return sh


def random_state(ac: dict, seed: int = 0, device="cpu") -> dict:
    """Random weights in checkpoint naming (fp32): projections ~ N(0, 1/fan_in); norm weights, sinks,
    decays and step biases spread so that every mechanism matters."""
    g = torch.Generator(device=device).manual_seed(seed)
    rnd = lambda shape: torch.randn(shape, generator=g, device=device)  # noqa: E731
    out = {}
    for name, shape in weight_shapes(ac).items():
        leaf = name.rsplit(".", 1)[-1]
        if len(shape) == 0:
            t = 1.0 + 0.2 * rnd(())
        elif leaf == "A_log":
            t = -0.5 + 0.8 * rnd(shape)
        elif leaf == "dt_bias":
            t = -1.0 + rnd(shape)
        elif leaf in ("D", "sink"):
            t = rnd(shape)
        elif leaf == "b" and len(shape) == 1:  # convolution bias
            t = 0.1 * rnd(shape)
        elif leaf == "norm":
            t = 1.0 + 0.1 * rnd(shape)
        elif leaf == "conv":
            t = rnd(shape) * shape[1] ** -0.5
        elif name == "embed":
            t = rnd(shape) * shape[1] ** -0.5
        else:
            t = rnd(shape) * shape[1] ** -0.5
        out[name] = t
    return out


class TapasunLM(HybridLM):
    design = sys.modules[__name__]

    def __init__(self, cfg: ModelConfig, device, dtype: torch.dtype = torch.bfloat16, block_size: int = 16):
        super().__init__(cfg, device, dtype, block_size)
        self.embed_scale = float((self.ac.get("embedding") or {}).get("scale", 1.0))

    def finish_weights(self, w: dict) -> None:
        """One-number norm weights as rows of the width (what the fused residual kernel reads); a
        feed-forward's gate and up as one projection."""
        W = self.width
        for name in [n for n, t in w.items() if t.dim() == 0]:
            w[name] = w[name].reshape(1).expand(W).contiguous()
        for i in range(len(self.mixers)):
            p = f"l{i}.mlp."
            if p + "gate" in w:
                w[p + "_gu"] = torch.cat([w.pop(p + "gate"), w.pop(p + "up")]).contiguous()

    def forward(self, input_ids: torch.Tensor, md, kv_cache: torch.Tensor) -> torch.Tensor:
        """Final-normed hidden states of the rows md.logits_indices."""
        w, eps, dt = self.w, self.eps, self.dtype
        ctx = StepContext(md=md, cache=kv_cache, state=md.state, block_size=self.block_size, eps=eps)
        x = seqmix.embed_scaled(input_ids, w["embed"], self.embed_scale)
        tap = self.layer_tap
        runs = self.plan.runs
        h = seqmix.resid_update(x, None, eps, norm_w=w["l0.norm1"], out_dtype=dt) if runs else None
        for n, run in enumerate(runs):
            i = run.layer
            p = f"l{i}."
            nxt = w[f"l{runs[n + 1].layer}.norm1"] if n + 1 < len(runs) else None
            m = self.mixers[i]
            y = m.forward(self._split(ops.linear(h, w[p + "mix._in"]), m), h, w, ctx, run.koff, run.voff, run.soff)
            if p + "mlp._gu" in w:
                h = seqmix.resid_update(x, y, eps, wa=w[p + "norm1b"], norm_w=w[p + "norm2"], out_dtype=dt)
                y = ops.linear(seqmix.silu_mul(ops.linear(h, w[p + "mlp._gu"])), w[p + "mlp.down"])
                h = seqmix.resid_update(x, y, eps, wa=w[p + "norm2b"], norm_w=nxt, out_dtype=dt)
            else:
                h = seqmix.resid_update(x, y, eps, wa=w[p + "norm1b"], norm_w=nxt, out_dtype=dt)
            if tap is not None:
                tap.append(x.clone())
        xs = x.index_select(0, md.logits_indices)
        return seqmix.resid_update(xs, None, eps, norm_w=w["final.norm"], out_dtype=dt)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """fp32 logits."""
        return seqmix.softcap(ops.linear(hidden, self.w["head"]), 0.0)
