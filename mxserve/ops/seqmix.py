"""Sequence-mixer ops beyond rotary softmax attention: a 32-bit residual stream with fused norms,
paged attention with a sliding window and kept first tokens, decayed linear attention, the mLSTM
matrix memory, gated output norms, squared ReLU and logit soft-capping.

Like mxserve.ops: GPU tensors run the gfx950 kernels of the in-tree extension `mxserve/_M*.so`
(csrc/mixers/*.hip, activations bf16 or fp32; built by `python setup_ext.py --only M` or on first
use), CPU tensors the PyTorch forms below.  Everything the recurrences touch is fp32: the state
pools, decays, gates, scores and the residual stream.

Batch layout (shared with the attention ops): sequence s owns rows qsl[s]:qsl[s+1] of a step's
flattened tokens; they are the LAST rows of its seq_lens[s] tokens.  A sequence whose first row is
position 0 starts from a zero state, whatever its slot held before.

Paged cache of one attention layer inside the block-major pool `cache` [num_blocks, block_elems]:
K at `koff` as [Hkv, BS, dk], V at `voff` as [Hkv, BS, dv], both token-major.
Recurrent state of one layer inside the slot pool `state` [slots, state_floats] (fp32): decayed
linear attention S [H, dk, dv] at `off`; mLSTM S [H, dk, dv], then n [H, dk], then m [H].
"""
from __future__ import annotations

import importlib
import os
import threading
from typing import Optional

import torch
import torch.nn.functional as F

_EXT = None
_LOCK = threading.Lock()


def ext():
    """The mixer kernels' extension; built in-tree on first use when it is missing (hipcc)."""
    global _EXT
    if _EXT is None:
        with _LOCK:
            if _EXT is None:
                try:
                    _EXT = importlib.import_module("mxserve._M")
                except ImportError:
                    import sys
                    root = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
                    if root not in sys.path:
                        sys.path.insert(0, root)
                    import setup_ext
                    setup_ext.build_M()
                    importlib.invalidate_caches()
                    _EXT = importlib.import_module("mxserve._M")
    return _EXT


def _gpu(t: torch.Tensor) -> bool:
    return t.is_cuda and os.environ.get("MXS_FORCE_REFERENCE_OPS", "0") != "1"


def _rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)


# ----------------------------------------------------------------------------- residual stream
def resid_update(x: torch.Tensor, a: Optional[torch.Tensor], eps: float, *, wa: Optional[torch.Tensor] = None,
                 b: Optional[torch.Tensor] = None, wb: Optional[torch.Tensor] = None,
                 bias: Optional[torch.Tensor] = None, assign: bool = False,
                 norm_w: Optional[torch.Tensor] = None, out_dtype: Optional[torch.dtype] = None):
    """One pass over the fp32 residual stream x [T, W], in place:
        d = a                      (wa: RMSNorm(a) * wa)
        d = (d + RMSNorm(b) * wb) / 2      when b is given (two branches, each normed over the width)
        d += bias                  (a [W] vector)
        x = d if assign else x + d
    and, when norm_w is given, returns RMSNorm(x) * norm_w in out_dtype (the next sublayer's input).
    a = None leaves x as it is (norm only).  All sums and norms in fp32."""
    if _gpu(x):
        h = None
        if norm_w is not None:
            h = torch.empty(x.shape, dtype=out_dtype or norm_w.dtype, device=x.device)
        ext().resid_update(x, a, wa, b, wb, bias, bool(assign), norm_w, h, float(eps))
        return h
    if a is not None:
        d = a.float()
        if wa is not None:
            d = _rms(d, eps) * wa.float()
        if b is not None:
            d = 0.5 * (d + _rms(b.float(), eps) * wb.float())
        if bias is not None:
            d = d + bias.float()
        if assign:
            x.copy_(d)
        else:
            x.add_(d)
    if norm_w is None:
        return None
    return (_rms(x, eps) * norm_w.float()).to(out_dtype or norm_w.dtype)


def cast_into(dst: torch.Tensor, x: torch.Tensor) -> None:
    """dst[:, :W] = x (fp32 -> dst's dtype); dst may be a wider row-strided buffer."""
    if _gpu(x):
        ext().cast_into(dst, x)
    else:
        dst[:, :x.shape[1]].copy_(x)


def relu_sq(x: torch.Tensor) -> torch.Tensor:
    """max(x, 0)^2, computed in fp32."""
    if _gpu(x):
        out = torch.empty_like(x)
        ext().relu_sq(out, x)
        return out
    return F.relu(x.float()).square().to(x.dtype)


def softcap(x: torch.Tensor, cap: float) -> torch.Tensor:
    """cap * tanh(x / cap) as fp32 (cap <= 0: a plain fp32 copy)."""
    if _gpu(x):
        out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
        ext().softcap(out, x, float(cap))
        return out
    xf = x.float()
    return cap * torch.tanh(xf / cap) if cap > 0 else xf


def gated_rms_norm(o: torch.Tensor, gate: torch.Tensor, w: torch.Tensor, eps: float, groups: int,
                   out_dtype: torch.dtype) -> torch.Tensor:
    """RMSNorm(o) * w * sigmoid(gate).  o fp32 [T, N]; the norm runs over each of `groups` equal
    slices of a row (1: the whole row; H: per head).  gate [T, N] may be a row-strided view."""
    if _gpu(o):
        out = torch.empty(o.shape, dtype=out_dtype, device=o.device)
        ext().gated_rms_norm(out, o, gate, w, float(eps), int(groups))
        return out
    T, N = o.shape
    y = _rms(o.view(T, groups, N // groups), eps).reshape(T, N)
    return (y * w.float() * torch.sigmoid(gate.float())).to(out_dtype)


def gate_linear(h: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    """fp32 h @ w.T + bias for a handful of output columns (recurrence gates): inputs of any float
    dtype, products and sums in fp32, fp32 out."""
    if _gpu(h):
        out = torch.empty(h.shape[0], w.shape[0], dtype=torch.float32, device=h.device)
        ext().gate_linear(out, h, w, bias)
        return out
    return F.linear(h.float(), w.float(), None if bias is None else bias.float())


# ----------------------------------------------------------------------------- windowed attention
def kv_write(cache: torch.Tensor, k: torch.Tensor, v: torch.Tensor, slot_mapping: torch.Tensor, koff: int,
             voff: int, num_kv_heads: int, dk: int, dv: int, block_size: int) -> None:
    """k [T, Hkv*dk], v [T, Hkv*dv] (row-strided views) into the paged cache; slot -1 writes nothing."""
    if _gpu(k):
        ext().kv_write(cache, k, v, slot_mapping, int(koff), int(voff), num_kv_heads, dk, dv, block_size)
        return
    ok = slot_mapping >= 0
    slots = slot_mapping[ok]
    blk, off = slots // block_size, slots % block_size
    T = int(slots.numel())
    kc = cache[:, koff:koff + num_kv_heads * block_size * dk].view(-1, num_kv_heads, block_size, dk)
    vc = cache[:, voff:voff + num_kv_heads * block_size * dv].view(-1, num_kv_heads, block_size, dv)
    kc[blk, :, off] = k[ok].reshape(T, num_kv_heads, dk).to(cache.dtype)
    vc[blk, :, off] = v[ok].reshape(T, num_kv_heads, dv).to(cache.dtype)


def window_attention(q: torch.Tensor, cache: torch.Tensor, block_tables: torch.Tensor, qsl: torch.Tensor,
                     seq_lens: torch.Tensor, koff: int, voff: int, num_heads: int, num_kv_heads: int, dk: int,
                     dv: int, block_size: int, scale: float, window: int, keep_first: int,
                     max_query_len: int = 0) -> torch.Tensor:
    """Softmax attention over the paged cache (this step's keys already written).  The query at
    position i sees key j <= i when i - j < window or j < keep_first (window <= 0: every j <= i).
    q [T, H*dk] (row-strided view) -> [T, H*dv] in q's dtype; scores and weights in fp32.
    Query head h reads kv head h // (H / Hkv).  max_query_len: the longest chunk of the step (host
    int); from 16 rows a bf16 step with head sizes that are multiples of 16 runs the MFMA kernel."""
    T = q.shape[0]
    if _gpu(q):
        out = torch.empty(T, num_heads * dv, dtype=q.dtype, device=q.device)
        ext().window_attention(out, q, cache, block_tables, qsl, seq_lens, int(koff), int(voff), num_heads,
                               num_kv_heads, dk, dv, block_size, float(scale), int(window), int(keep_first),
                               int(max_query_len))
        return out
    out = torch.zeros(T, num_heads, dv, dtype=torch.float32)
    kc = cache[:, koff:koff + num_kv_heads * block_size * dk].view(-1, num_kv_heads, block_size, dk)
    vc = cache[:, voff:voff + num_kv_heads * block_size * dv].view(-1, num_kv_heads, block_size, dv)
    g = num_heads // num_kv_heads
    ql, sl = qsl.tolist(), seq_lens.tolist()
    for s in range(len(sl)):
        a, e = ql[s], ql[s + 1]
        n = sl[s]
        if e <= a:
            continue
        nb = -(-n // block_size)
        blocks = block_tables[s, :nb].long()
        K = kc[blocks].permute(0, 2, 1, 3).reshape(nb * block_size, num_kv_heads, dk)[:n].float()
        V = vc[blocks].permute(0, 2, 1, 3).reshape(nb * block_size, num_kv_heads, dv)[:n].float()
        qs = q[a:e].reshape(e - a, num_heads, dk).float()
        sc = torch.einsum("mhd,nhd->hmn", qs, K.repeat_interleave(g, dim=1)) * scale
        i = torch.arange(n - (e - a), n).unsqueeze(1)
        j = torch.arange(n).unsqueeze(0)
        seen = j <= i
        if window > 0:
            seen = seen & ((i - j < window) | (j < keep_first))
        p = torch.softmax(sc.masked_fill(~seen.unsqueeze(0), float("-inf")), dim=-1)
        out[a:e] = torch.einsum("hmn,nhd->mhd", p, V.repeat_interleave(g, dim=1))
    return out.reshape(T, num_heads * dv).to(q.dtype)


# ----------------------------------------------------------------------------- recurrences
SCAN_PIECE = int(os.environ.get("MXS_SCAN_PIECE", "0"))  # tokens per piece of a time-split scan; 0: by the launch's size
SCAN_SCRATCH_BYTES = 512 << 20
SCAN_TARGET_BLOCKS = 1024  # workgroups that fill the 256 CUs four deep


def _scan_split(S: int, T: int, max_query_len: int, floats: int, heads: int, dv: int, device) -> tuple:
    """(piece, npieces, scratch pool, scratch pool) of a scan launch: chunks of 2 pieces or more are cut
    into pieces that run side by side (two passes and a chaining step, csrc/mixers/scan.hip).  Pieces
    are 64 to 256 tokens, as short as it takes to reach SCAN_TARGET_BLOCKS workgroups over the long
    chunks of the step, and grow until both scratch pools [S, npieces, state] fit SCAN_SCRATCH_BYTES."""
    max_query_len = min(max_query_len, T)
    if max_query_len < 128:
        return 1, 1, None, None
    piece = SCAN_PIECE
    if piece <= 0:
        per_piece = heads * -(-dv // 64) * max(1, T // max_query_len)  # workgroups one piece index adds
        want = -(-SCAN_TARGET_BLOCKS // per_piece)
        piece = 256
        while piece > 64 and -(-max_query_len // piece) < want:
            piece //= 2
    while max_query_len >= 2 * piece:
        n = -(-max_query_len // piece)
        if 2 * S * n * floats * 4 <= SCAN_SCRATCH_BYTES:
            pool = torch.empty(2, S * n * floats, dtype=torch.float32, device=device)
            return piece, n, pool[0], pool[1]
        piece *= 2
    return 1, 1, None, None


def decay_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, state: torch.Tensor,
               state_rows: torch.Tensor, off: int, qsl: torch.Tensor, seq_lens: torch.Tensor, num_heads: int,
               dk: int, dv: int, silu: bool = True, max_query_len: int = 0) -> torch.Tensor:
    """Decayed linear attention, token by token per head: S = decay_h S + k v^T, o = S^T q, with q, k, v
    passed through SiLU first when `silu`.  q, k [T, H*dk], v [T, H*dv] (row-strided views); decay
    fp32 [H]; returns o fp32 [T, H*dv] and leaves each sequence's S in its slot.  max_query_len: the
    step's longest chunk (host int); long chunks are cut into pieces that run side by side."""
    T = q.shape[0]
    if _gpu(q):
        out = torch.empty(T, num_heads * dv, dtype=torch.float32, device=q.device)
        plan = _scan_split(seq_lens.numel(), T, max_query_len, num_heads * dk * dv, num_heads, dv, q.device)
        ext().decay_scan(out, q, k, v, decay, state, state_rows, int(off), qsl, seq_lens, num_heads, dk, dv,
                         bool(silu), *plan)
        return out
    out = torch.zeros(T, num_heads, dv, dtype=torch.float32)
    qf, kf, vf = (t.float().reshape(T, num_heads, -1) for t in (q, k, v))
    if silu:
        qf, kf, vf = F.silu(qf), F.silu(kf), F.silu(vf)
    ql, sl, rows = qsl.tolist(), seq_lens.tolist(), state_rows.tolist()
    n = num_heads * dk * dv
    for s in range(len(sl)):
        a, e = ql[s], ql[s + 1]
        if e <= a:
            continue
        S = state[rows[s], off:off + n].view(num_heads, dk, dv)
        if sl[s] - (e - a) == 0:
            S.zero_()
        for t in range(a, e):
            S.mul_(decay.view(-1, 1, 1)).add_(kf[t].unsqueeze(2) * vf[t].unsqueeze(1))
            out[t] = torch.einsum("hdv,hd->hv", S, qf[t])
    return out.reshape(T, num_heads * dv)


def mlstm_state_floats(num_heads: int, dk: int, dv: int) -> int:
    return num_heads * (dk * dv + dk + 1)


def mlstm_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, gates: torch.Tensor, state: torch.Tensor,
               state_rows: torch.Tensor, off: int, qsl: torch.Tensor, seq_lens: torch.Tensor, num_heads: int,
               dk: int, dv: int, gate_cap: float, q_scale: float, max_query_len: int = 0) -> torch.Tensor:
    """mLSTM matrix memory, token by token per head.  gates fp32 [T, 2H]: the input gates' then the
    forget gates' pre-activations.  With i = cap tanh(pre_i / cap), f = logsigmoid(cap tanh(pre_f / cap))
    and a running maximum m (0 at the start):
        m' = max(f + m, i);  S = e^(f + m - m') S + e^(i - m') k v^T;  n likewise with k;
        o = S^T q~ / (max(|n . q~|, e^(-m')) + 1e-6),   q~ = q_scale q.
    Returns o fp32 [T, H*dv] (before any norm)."""
    T = q.shape[0]
    if _gpu(q):
        out = torch.empty(T, num_heads * dv, dtype=torch.float32, device=q.device)
        plan = _scan_split(seq_lens.numel(), T, max_query_len, mlstm_state_floats(num_heads, dk, dv) + num_heads,
                           num_heads, dv, q.device)
        ext().mlstm_scan(out, q, k, v, gates, state, state_rows, int(off), qsl, seq_lens, num_heads, dk, dv,
                         float(gate_cap), float(q_scale), *plan)
        return out
    H = num_heads
    out = torch.zeros(T, H, dv, dtype=torch.float32)
    qf = q.float().reshape(T, H, dk) * q_scale
    kf, vf = k.float().reshape(T, H, dk), v.float().reshape(T, H, dv)
    ig = gate_cap * torch.tanh(gates[:, :H] / gate_cap)
    fg = F.logsigmoid(gate_cap * torch.tanh(gates[:, H:] / gate_cap))
    ql, sl, rows = qsl.tolist(), seq_lens.tolist(), state_rows.tolist()
    nS, nn = H * dk * dv, H * dk
    for s in range(len(sl)):
        a, e = ql[s], ql[s + 1]
        if e <= a:
            continue
        st = state[rows[s]]
        S = st[off:off + nS].view(H, dk, dv)
        n = st[off + nS:off + nS + nn].view(H, dk)
        m = st[off + nS + nn:off + nS + nn + H]
        if sl[s] - (e - a) == 0:
            S.zero_(), n.zero_(), m.zero_()
        for t in range(a, e):
            m_new = torch.maximum(fg[t] + m, ig[t])
            fa, ia = torch.exp(fg[t] + m - m_new), torch.exp(ig[t] - m_new)
            S.mul_(fa.view(H, 1, 1)).add_(ia.view(H, 1, 1) * kf[t].unsqueeze(2) * vf[t].unsqueeze(1))
            n.mul_(fa.view(H, 1)).add_(ia.view(H, 1) * kf[t])
            m.copy_(m_new)
            den = torch.maximum((n * qf[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
            out[t] = torch.einsum("hdv,hd->hv", S, qf[t]) / den.unsqueeze(1)
    return out.reshape(T, H * dv)
