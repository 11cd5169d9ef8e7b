"""Voletar: a decoder whose layers differ from one another.  config.json lists them: `lightning`
layers (decayed linear attention) and `parallel` layers (window attention beside an mLSTM memory),
each with an optional dense feed-forward (squared ReLU).  A span of layers can be looped: it runs
`times` times over the same weights, every pass with its own K/V pages and recurrent state, and
each pass starts from W_in [x; x0] + step[t] (x0: the embedding output).

The residual stream is fp32; every sublayer's output is added, and the next sublayer's RMSNorm
taken, in one kernel (seqmix.resid_update).  A layer's input projections are one GEMM over the
concatenated weight rows of its mixer(s).  One forward = one engine step over a flattened token batch,
as for the other models: paged K/V for the attention mixers through the block tables, fp32 state
for the recurrent mixers in the runner's per-request slots.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F

from .. import ops
from ..ops import seqmix
from .config import ModelConfig
from .hybrid import HybridLM, LayerPlan, LayerRun, plan_runs  # noqa: F401  (LayerRun: part of this module's surface)
from .mixers import Mixer, StepContext, build_mixer


def mixers_of(ac: dict) -> list:
    return [build_mixer(l["type"], f"l{i}.mix.", int(ac["width"]), l["mixer"]) for i, l in enumerate(ac["layers"])]


_mixers = mixers_of


def layer_plan(ac: dict, block_size: int = 16, mixers: Optional[list] = None) -> LayerPlan:
    """Execution order with every run's place in a cache block and in a state slot."""
    mixers = mixers or _mixers(ac)
    n = len(mixers)
    loop = ac.get("loop") or None
    order = [(i, None, False) for i in range(n)]
    if loop:
        a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
        if not 0 <= a < b <= n or times < 1:
            raise ValueError(f"bad loop {loop}")
        order = [(i, None, False) for i in range(a)]
        for t in range(times):
            order += [(i, t, i == a) for i in range(a, b)]
        order += [(i, None, False) for i in range(b, n)]
    return plan_runs(order, mixers, block_size)


def weight_shapes(ac: dict, mixers: Optional[list] = None) -> dict:
    """Checkpoint tensor names and shapes."""
    W, V = int(ac["width"]), int(ac["vocab"])
    mixers = mixers or _mixers(ac)
    sh = {"embed": (V, W), "final.norm": (W,), "head": (V, W)}
    loop = ac.get("loop") or None
    if loop:
        sh["loop.in"] = (W, 2 * W)
        sh["loop.step"] = (int(loop["times"]), W)
    for i, (l, m) in enumerate(zip(ac["layers"], mixers)):
        p = f"l{i}."
        sh[p + "norm1"] = (W,)
        for name, rows in m.proj_rows():
            sh[name] = (rows, W)
        sh.update(m.extra_shapes())
        mlp = l.get("mlp")
        if mlp:
            if mlp.get("kind", "dense") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            sh[p + "norm2"] = (W,)
            sh[p + "mlp.up"] = (int(mlp["ff"]), W)
            sh[p + "mlp.down"] = (W, int(mlp["ff"]))
    return sh


def random_state(ac: dict, seed: int = 0, device="cpu") -> dict:
    """Random weights in checkpoint naming (fp32): projections ~ N(0, 1/fan_in), norm weights near 1,
    gate biases spread so that input and forget gates both matter."""
    g = torch.Generator(device=device).manual_seed(seed)
    out = {}
    for name, shape in weight_shapes(ac).items():
        if len(shape) == 1 and name.endswith(".b"):
            t = torch.randn(shape, generator=g, device=device) + (2.0 if name.endswith("f.b") else 0.0)
        elif len(shape) == 1:
            t = 1.0 + 0.1 * torch.randn(shape, generator=g, device=device)
        elif name == "loop.step":
            t = 0.1 * torch.randn(shape, generator=g, device=device)
        elif name == "embed":
            t = torch.randn(shape, generator=g, device=device)
        else:
            t = torch.randn(shape, generator=g, device=device) * shape[1] ** -0.5
        out[name] = t
    return out


class VoletarLM(HybridLM):
    """Voletar on the shared surface of the layer-list designs (mxserve/models/hybrid.py)."""

    def __init__(self, cfg: ModelConfig, device, dtype: torch.dtype = torch.bfloat16, block_size: int = 16):
        import sys
        self.design = sys.modules[__name__]
        super().__init__(cfg, device, dtype, block_size)
        self.softcap = float(self.ac.get("logit_softcap") or 0.0)

    # ------------------------------------------------------------------ forward
    def _add(self, x: torch.Tensor, pending, norm_w: Optional[torch.Tensor]):
        """Add a sublayer's output (a tensor, or the two branch outputs of a parallel mixer with their
        width norms) to the stream and return the next RMSNorm's output, if one is asked for."""
        if pending is None:
            if norm_w is None:
                return None
            return seqmix.resid_update(x, None, self.eps, norm_w=norm_w, out_dtype=self.dtype)
        if isinstance(pending, tuple):
            a, wa, b, wb = pending
            return seqmix.resid_update(x, a, self.eps, wa=wa, b=b, wb=wb, norm_w=norm_w, out_dtype=self.dtype)
        return seqmix.resid_update(x, pending, self.eps, norm_w=norm_w, out_dtype=self.dtype)

    def forward(self, input_ids: torch.Tensor, md, kv_cache: torch.Tensor) -> torch.Tensor:
        """Final-normed hidden states of the rows md.logits_indices."""
        w, W = self.w, self.width
        ctx = StepContext(md=md, cache=kv_cache, state=md.state, block_size=self.block_size, eps=self.eps)
        x0 = F.embedding(input_ids, w["embed"])
        x = x0.to(torch.float32, copy=True)  # fp32 models: never an alias of x0
        T = x.shape[0]
        pending = None
        cat = None
        tap = self.layer_tap
        for run in self.plan.runs:
            i = run.layer
            p = f"l{i}."
            if run.first_of_pass:
                self._add(x, pending, None)
                if cat is None:
                    cat = torch.empty(T, 2 * W, dtype=self.dtype, device=x.device)
                    cat[:, W:].copy_(x0)
                seqmix.cast_into(cat, x)
                y = ops.linear(cat, w["loop.in"])
                h = seqmix.resid_update(x, y, self.eps, bias=w["loop.step"][run.loop_pass], assign=True,
                                        norm_w=w[p + "norm1"], out_dtype=self.dtype)
            else:
                h = self._add(x, pending, w[p + "norm1"])
            m = self.mixers[i]
            parts = self._split(ops.linear(h, w[p + "mix._in"]), m)
            out = m.forward(parts, h, w, ctx, run.koff, run.voff, run.soff)
            if isinstance(out, tuple):
                pending = (out[0], w[p + "mix.left.out"], out[1], w[p + "mix.right.out"])
            else:
                pending = out
            if p + "mlp.up" in w:
                h = self._add(x, pending, w[p + "norm2"])
                pending = ops.linear(seqmix.relu_sq(ops.linear(h, w[p + "mlp.up"])), w[p + "mlp.down"])
            if tap is not None:
                self._add(x, pending, None)
                pending = None
                tap.append(x.clone())
        self._add(x, pending, None)
        xs = x.index_select(0, md.logits_indices)
        return seqmix.resid_update(xs, None, self.eps, norm_w=w["final.norm"], out_dtype=self.dtype)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """fp32 logits, soft-capped when the config says so."""
        return seqmix.softcap(ops.linear(hidden, self.w["head"]), self.softcap)
