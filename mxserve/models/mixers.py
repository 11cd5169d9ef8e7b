"""Token mixers that a layer can be built from, beside the rotary softmax attention of
mxserve/models/llama.py.  Each takes its sizes and constants as parameters, names the rows it wants
from the layer's fused input projection, says what it keeps per sequence (paged K/V, or fp32 state
in a slot) and computes its output from a step's flattened token batch.

  WindowAttention       softmax attention without positions over a sliding window plus the
                        sequence's first tokens, grouped kv heads, separate key and value sizes
  DecayLinearAttention  "lightning" linear attention: S = a_h S + k v^T, o = S^T q on SiLU(q, k, v),
                        one RMSNorm over all heads, sigmoid output gate
  MLSTM                 xLSTM's matrix memory with capped exponential gates and a running maximum,
                        per-head unit norm, sigmoid output gate
  ParallelPair          two mixers reading the same input; the layer averages their outputs after
                        an RMSNorm of each over the model width

The kernels are in mxserve/ops/seqmix.py (csrc/mixers/*.hip on the GPU).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from .. import ops
from ..ops import seqmix


@dataclass
class StepContext:
    """What a mixer needs of one engine step."""
    md: object  # AttnMetadata
    cache: Optional[torch.Tensor]  # [num_blocks, block_elems] paged K/V pool
    state: Optional[torch.Tensor]  # [slots, state_floats] fp32
    block_size: int
    eps: float


class Mixer:
    kv_heads = dk = dv = 0  # paged K/V per token (0: none)
    state_floats = 0  # fp32 state per sequence

    def proj_rows(self) -> list:
        """[(tensor name, rows)] of the fused input projection, in the order forward() reads them."""
        raise NotImplementedError

    def extra_shapes(self) -> dict:
        return {}


class WindowAttention(Mixer):
    def __init__(self, prefix: str, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float,
                 window: int, keep_first: int):
        if heads % kv_heads:
            raise ValueError(f"{prefix}: {heads} query heads do not divide over {kv_heads} kv heads")
        self.p, self.width = prefix, width
        self.heads, self.kv_heads, self.dk, self.dv = heads, kv_heads, dim, vdim
        self.scale, self.window, self.keep_first = float(scale), int(window), int(keep_first)

    def proj_rows(self) -> list:
        return [(self.p + "q", self.heads * self.dk), (self.p + "k", self.kv_heads * self.dk),
                (self.p + "v", self.kv_heads * self.dv)]

    def extra_shapes(self) -> dict:
        return {self.p + "o": (self.width, self.heads * self.dv)}

    def forward(self, parts: list, h: torch.Tensor, w: dict, ctx: StepContext, koff: int, voff: int, soff: int):
        q, k, v = parts
        md = ctx.md
        seqmix.kv_write(ctx.cache, k, v, md.slot_mapping, koff, voff, self.kv_heads, self.dk, self.dv, ctx.block_size)
        o = seqmix.window_attention(q, ctx.cache, md.block_tables, md.query_start_loc, md.seq_lens, koff, voff,
                                    self.heads, self.kv_heads, self.dk, self.dv, ctx.block_size, self.scale,
                                    self.window, self.keep_first, md.max_query_len)
        return ops.linear(o, w[self.p + "o"])


class DecayLinearAttention(Mixer):
    def __init__(self, prefix: str, width: int, heads: int, dim: int, vdim: int, decay: list):
        if len(decay) != heads:
            raise ValueError(f"{prefix}: {len(decay)} decays for {heads} heads")
        self.p, self.width, self.heads, self.qk, self.vd = prefix, width, heads, dim, vdim
        self.decay = [float(a) for a in decay]
        self.state_floats = heads * dim * vdim
        self._decay_dev: dict = {}

    def decay_on(self, device) -> torch.Tensor:
        """The per-head decays as an fp32 device tensor (made when the weights are loaded, so that no
        host-to-device copy falls into a graph capture)."""
        a = self._decay_dev.get(device)
        if a is None:
            a = self._decay_dev[device] = torch.tensor(self.decay, dtype=torch.float32, device=device)
        return a

    def finish_weights(self, w: dict) -> None:
        self.decay_on(w[self.p + "o"].device)

    def proj_rows(self) -> list:
        n, m = self.heads * self.qk, self.heads * self.vd
        return [(self.p + "q", n), (self.p + "k", n), (self.p + "v", m), (self.p + "g", m)]

    def extra_shapes(self) -> dict:
        return {self.p + "o": (self.width, self.heads * self.vd), self.p + "norm": (self.heads * self.vd,)}

    def forward(self, parts: list, h: torch.Tensor, w: dict, ctx: StepContext, koff: int, voff: int, soff: int):
        q, k, v, g = parts
        md = ctx.md
        a = self.decay_on(h.device)
        o = seqmix.decay_scan(q, k, v, a, ctx.state, md.state_rows, soff, md.query_start_loc, md.seq_lens,
                              self.heads, self.qk, self.vd, silu=True, max_query_len=md.max_query_len)
        y = seqmix.gated_rms_norm(o, g, w[self.p + "norm"], ctx.eps, 1, h.dtype)
        return ops.linear(y, w[self.p + "o"])


class MLSTM(Mixer):
    def __init__(self, prefix: str, width: int, heads: int, dim: int, vdim: int, gate_cap: float):
        self.p, self.width, self.heads, self.qk, self.vd = prefix, width, heads, dim, vdim
        self.gate_cap = float(gate_cap)
        self.state_floats = seqmix.mlstm_state_floats(heads, dim, vdim)

    def proj_rows(self) -> list:
        n, m = self.heads * self.qk, self.heads * self.vd
        return [(self.p + "q", n), (self.p + "k", n), (self.p + "v", m), (self.p + "g", m)]

    def extra_shapes(self) -> dict:
        H = self.heads
        return {self.p + "o": (self.width, H * self.vd), self.p + "norm": (H * self.vd,),
                self.p + "i": (H, self.width), self.p + "i.b": (H,), self.p + "f": (H, self.width),
                self.p + "f.b": (H,)}

    def finish_weights(self, w: dict) -> None:
        """Input and forget gate rows as one [2H, width] projection with its bias."""
        p = self.p
        w[p + "_if"] = torch.cat([w.pop(p + "i"), w.pop(p + "f")]).contiguous()
        w[p + "_if.b"] = torch.cat([w.pop(p + "i.b"), w.pop(p + "f.b")]).contiguous()

    def forward(self, parts: list, h: torch.Tensor, w: dict, ctx: StepContext, koff: int, voff: int, soff: int):
        q, k, v, g = parts
        md = ctx.md
        gates = seqmix.gate_linear(h, w[self.p + "_if"], w[self.p + "_if.b"])
        o = seqmix.mlstm_scan(q, k, v, gates, ctx.state, md.state_rows, soff, md.query_start_loc, md.seq_lens,
                              self.heads, self.qk, self.vd, self.gate_cap, self.qk ** -0.5,
                              max_query_len=md.max_query_len)
        y = seqmix.gated_rms_norm(o, g, w[self.p + "norm"], ctx.eps, self.heads, h.dtype)
        return ops.linear(y, w[self.p + "o"])


class ParallelPair(Mixer):
    """Two mixers over the same input.  forward() returns both outputs; the layer norms each over
    the width with `<prefix>left.out` / `<prefix>right.out` and adds half their sum to the stream."""

    def __init__(self, prefix: str, width: int, left: Mixer, right: Mixer):
        self.p, self.width, self.left, self.right = prefix, width, left, right
        self.kv_heads, self.dk, self.dv = left.kv_heads, left.dk, left.dv
        if right.kv_heads:
            raise ValueError("ParallelPair: only the left mixer may keep paged K/V")
        if left.state_floats:
            raise ValueError("ParallelPair: only the right mixer may keep a recurrent state")
        self.state_floats = right.state_floats

    def proj_rows(self) -> list:
        return self.left.proj_rows() + self.right.proj_rows()

    def extra_shapes(self) -> dict:
        return {**self.left.extra_shapes(), **self.right.extra_shapes(),
                self.p + "left.out": (self.width,), self.p + "right.out": (self.width,)}

    def finish_weights(self, w: dict) -> None:
        for m in (self.left, self.right):
            if hasattr(m, "finish_weights"):
                m.finish_weights(w)

    def forward(self, parts: list, h: torch.Tensor, w: dict, ctx: StepContext, koff: int, voff: int, soff: int):
        nl = len(self.left.proj_rows())
        a = self.left.forward(parts[:nl], h, w, ctx, koff, voff, soff)
        b = self.right.forward(parts[nl:], h, w, ctx, koff, voff, soff)
        return a, b


def build_mixer(kind: str, prefix: str, width: int, mc: dict) -> Mixer:
    """A layer's mixer from its config entry (`type` and `mixer` of a Voletar layer)."""
    if kind == "lightning":
        return DecayLinearAttention(prefix, width, int(mc["heads"]), int(mc["dim"]), int(mc["vdim"]), mc["decay"])
    if kind == "parallel":
        l, r = mc["left"], mc["right"]
        mask = l.get("mask") or {}
        left = WindowAttention(prefix + "left.", width, int(l["heads"]), int(l.get("kv_heads", l["heads"])),
                               int(l["dim"]), int(l["vdim"]), float(l["scale"]), int(mask.get("size", 0) or 0),
                               int(mask.get("keep_first", 0) or 0))
        right = MLSTM(prefix + "right.", width, int(r["heads"]), int(r["dim"]), int(r["vdim"]), float(r["gate_cap"]))
        return ParallelPair(prefix, width, left, right)
    raise ValueError(f"unknown mixer type {kind!r}")
