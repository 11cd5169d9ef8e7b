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

from dataclasses import dataclass, field
from typing import Optional

import torch
import torch.nn.functional as F

from .. import ops
from ..ops import seqmix
from ..parallel.comm import get_tp
from .config import ModelConfig
from .mixers import Mixer, StepContext, build_mixer


@dataclass
class LayerRun:
    """One execution of a layer: the looped span's layers appear once per pass."""
    layer: int
    loop_pass: Optional[int]  # pass number inside the looped span, None outside it
    first_of_pass: bool
    kv_heads: int = 0
    dk: int = 0
    dv: int = 0
    koff: int = 0  # element offsets inside a cache block
    voff: int = 0
    soff: int = 0  # float offset inside a state slot


@dataclass
class LayerPlan:
    runs: list = field(default_factory=list)
    block_elems: int = 0  # K/V elements one block holds over all runs
    state_floats: int = 0

    @property
    def attn_runs(self) -> list:
        return [r for r in self.runs if r.kv_heads]


def _mixers(ac: dict) -> list:
    return [build_mixer(l["type"], f"l{i}.mix.", int(ac["width"]), l["mixer"]) for i, l in enumerate(ac["layers"])]


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
    plan = LayerPlan()
    for i, t, first in order:
        m: Mixer = mixers[i]
        r = LayerRun(i, t, first, m.kv_heads, m.dk, m.dv)
        if m.kv_heads:
            r.koff = plan.block_elems
            r.voff = r.koff + m.kv_heads * block_size * m.dk
            plan.block_elems = r.voff + m.kv_heads * block_size * m.dv
        r.soff = plan.state_floats
        plan.state_floats += m.state_floats
        plan.runs.append(r)
    return plan


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


class VoletarLM:
    """Same surface as TransformerLM for the model runner: weights in a flat dict, forward() over a
    step's batch, compute_logits()."""

    is_recurrent = True

    def __init__(self, cfg: ModelConfig, device, dtype: torch.dtype = torch.bfloat16, block_size: int = 16):
        if cfg.arch_config is None:
            raise ValueError("VoletarLM needs the checkpoint's layer list (ModelConfig.arch_config)")
        tp = get_tp()
        if tp.tp_size != 1:
            raise ValueError("Voletar runs on one GPU per replica (its recurrent state is not sharded)")
        self.cfg, self.ac = cfg, cfg.arch_config
        self.device, self.dtype = torch.device(device), dtype
        self.tp_rank, self.tp_size = 0, 1
        self.block_size = block_size
        self.width = int(self.ac["width"])
        self.eps = float(self.ac.get("norm", {}).get("eps", 1e-5))
        self.softcap = float(self.ac.get("logit_softcap") or 0.0)
        self.mixers = _mixers(self.ac)
        self.plan = layer_plan(self.ac, block_size, self.mixers)
        self.state_floats = self.plan.state_floats
        self.vocab_local = cfg.vocab_size
        self.w: dict[str, torch.Tensor] = {}
        self.kv_scales = [{"k_scale": 1.0, "v_scale": 1.0}]
        self.pf_chain = False
        # debugging tap: a list here receives the residual stream after every layer run (fp32 copies)
        self.layer_tap: Optional[list] = None

    # ------------------------------------------------------------------ cache / state geometry
    def kv_cache_shape(self, num_blocks: int, block_size: int) -> tuple:
        if block_size != self.block_size:
            self.block_size = block_size
            self.plan = layer_plan(self.ac, block_size, self.mixers)
        return (num_blocks, max(self.plan.block_elems, 1))

    # ------------------------------------------------------------------ weights
    def init_random(self, seed: int = 0, std: float = 0.02) -> None:
        self.load_full_state(random_state(self.ac, seed, device=self.device))

    def load_full_state(self, full: dict) -> None:
        """Checkpoint tensors (any float dtype; integer tables stay integers) -> this model's dtype, the
        mixers' input projections concatenated into one weight per layer."""
        shapes = weight_shapes(self.ac, self.mixers)
        missing = [k for k in shapes if k not in full]
        if missing:
            raise KeyError(f"checkpoint lacks {missing[:4]}{' ...' if len(missing) > 4 else ''}")
        w = {}
        for name, shape in shapes.items():
            t = full[name]
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name}: shape {tuple(t.shape)}, the config gives {tuple(shape)}")
            w[name] = t.to(device=self.device, dtype=self.dtype if t.is_floating_point() else t.dtype).contiguous()
        for i, m in enumerate(self.mixers):
            rows = m.proj_rows()
            w[f"l{i}.mix._in"] = torch.cat([w.pop(name) for name, _ in rows]).contiguous()
            if hasattr(m, "finish_weights"):
                m.finish_weights(w)
        self.w = w

    def prepare_fused_prefill(self, tuning: bool = True, max_rows: int = 8192) -> bool:
        return False

    def calibrate_kv_scales(self, block_size: int = 16, n: int = 256, headroom: float = 2.0) -> None:
        raise ValueError("Voletar keeps its K/V pages in the model dtype (no fp8 KV cache)")

    def lm_head_weight(self) -> torch.Tensor:
        return self.w["head"]

    def tunable_shapes(self) -> dict:
        """Decode-GEMM shapes for the start-up tuner: none, the projections run hipBLASLt's own choice."""
        return {}

    # ------------------------------------------------------------------ forward
    def _split(self, y: torch.Tensor, mixer: Mixer) -> list:
        parts, c = [], 0
        for _, rows in mixer.proj_rows():
            parts.append(y[:, c:c + rows])
            c += rows
        return parts

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
