"""Mixer kernels (csrc/mixers, mxserve/_M) against the PyTorch forms of the same ops in
mxserve/ops/seqmix.py, in bf16 and fp32: random chunked batches over paged K/V and state slots,
sizes that are not multiples of the tile sizes, windows' edges, kept first tokens, slot reuse."""
import random

import pytest
import torch

from mxserve.ops import seqmix

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


def _tol(dt):
    return dict(rtol=2e-2, atol=2e-2) if dt == torch.bfloat16 else dict(rtol=2e-4, atol=2e-5)


def _batch(lens_before, lens_new, bs, nblocks, seed=0):
    """Block tables, qsl, seq_lens and slot mapping of a step: sequence s has lens_before[s] tokens
    in the cache and gets lens_new[s] more; blocks are dealt out shuffled."""
    rng = random.Random(seed)
    free = list(range(nblocks))
    rng.shuffle(free)
    S = len(lens_new)
    maxb = max(-(-(a + b) // bs) for a, b in zip(lens_before, lens_new))
    bt = torch.zeros(S, maxb, dtype=torch.int32)
    for s in range(S):
        for i in range(-(-(lens_before[s] + lens_new[s]) // bs)):
            bt[s, i] = free.pop()
    qsl = [0]
    for n in lens_new:
        qsl.append(qsl[-1] + n)
    seq = [a + b for a, b in zip(lens_before, lens_new)]
    return bt, torch.tensor(qsl, dtype=torch.int32), torch.tensor(seq, dtype=torch.int32)


def _slots(bt, before, new, bs):
    out = []
    for s in range(len(new)):
        for p in range(before[s], before[s] + new[s]):
            out.append(int(bt[s, p // bs]) * bs + p % bs)
    return torch.tensor(out, dtype=torch.int64)


@pytest.mark.parametrize("dt", DTYPES)
def test_resid_update_forms(gpu, dt):
    torch.manual_seed(0)
    T, W = 37, 328
    x = torch.randn(T, W)
    a, b = torch.randn(T, 2 * W).to(dt)[:, 3:3 + W], torch.randn(T, W).to(dt)
    wa, wb, nw, bias = (torch.randn(W).to(dt) for _ in range(4))
    cases = [dict(a=None, norm_w=nw), dict(a=a, norm_w=nw), dict(a=a, norm_w=None), dict(a=a, wa=wa, b=b, wb=wb, norm_w=nw),
             dict(a=a, bias=bias, assign=True, norm_w=nw), dict(a=a, wa=wa, b=b, wb=wb, norm_w=None)]
    for kw in cases:
        xa = kw.pop("a")
        xc, xg = x.clone(), x.clone().to(gpu)
        hc = seqmix.resid_update(xc, xa, 1e-5, out_dtype=dt, **kw)
        kg = {k: (v.to(gpu) if torch.is_tensor(v) else v) for k, v in kw.items()}
        hg = seqmix.resid_update(xg, None if xa is None else xa.to(gpu), 1e-5, out_dtype=dt, **kg)
        torch.testing.assert_close(xg.cpu(), xc, rtol=1e-5, atol=1e-5)
        if hc is not None:
            torch.testing.assert_close(hg.cpu().float(), hc.float(), **_tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
def test_small_ops(gpu, dt):
    torch.manual_seed(1)
    T, N = 19, 6 * 40
    x = torch.randn(T, N).to(dt)
    torch.testing.assert_close(seqmix.relu_sq(x.to(gpu)).cpu().float(), seqmix.relu_sq(x).float(), **_tol(dt))
    big = (20 * torch.randn(T, 2 * N)).to(dt)[:, 5:5 + N]
    for cap in (12.5, 0.0):
        torch.testing.assert_close(seqmix.softcap(big.to(gpu), cap).cpu(), seqmix.softcap(big, cap), **_tol(dt))
    o = torch.randn(T, N) * 3
    g = torch.randn(T, 3 * N).to(dt)[:, N:2 * N]
    w = torch.randn(N).to(dt)
    for groups in (1, 6, 3):
        torch.testing.assert_close(seqmix.gated_rms_norm(o.to(gpu), g.to(gpu), w.to(gpu), 1e-5, groups, dt).cpu().float(),
                                   seqmix.gated_rms_norm(o, g, w, 1e-5, groups, dt).float(), **_tol(dt))
    h = torch.randn(T, 330).to(dt)
    gw, gb = torch.randn(10, 330).to(dt), torch.randn(10).to(dt)
    torch.testing.assert_close(seqmix.gate_linear(h.to(gpu), gw.to(gpu), gb.to(gpu)).cpu(), seqmix.gate_linear(h, gw, gb),
                               rtol=1e-4, atol=1e-4)
    dst = torch.zeros(T, 2 * N, dtype=dt, device=gpu)
    seqmix.cast_into(dst, o.to(gpu))
    torch.testing.assert_close(dst[:, :N].cpu().float(), o.to(dt).float())
    assert float(dst[:, N:].abs().max()) == 0.0


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,dk,dv,window,keep", [(5, 5, 80, 96, 50, 12), (4, 2, 40, 72, 9, 3), (8, 2, 64, 128, 300, 0),
                                                    (3, 1, 24, 200, 0, 0), (2, 2, 128, 64, 5, 11), (2, 1, 10, 6, 30, 2), (4, 2, 20, 36, 7, 1)])
def test_window_attention_paged(gpu, dt, H, G, dk, dv, window, keep):
    """Two rounds over the same pool: prompt chunks, then mixed single tokens and chunks."""
    torch.manual_seed(2)
    bs, nblocks = 16, 80
    other = 7 * 16  # another layer's elements in each block, before and after this one's
    koff, voff = other, other + G * bs * dk
    elems = voff + G * bs * dv + other
    cache_c = torch.randn(nblocks, elems).to(dt)
    cache_g = cache_c.to(gpu)
    before, new = [0, 0, 0, 0], [1, 330, 75, 18]
    bt = None
    for rnd in range(3):
        if rnd == 0:
            bt, qsl, seq = _batch(before, new, bs, nblocks, seed=3)
        else:
            before = [a + b for a, b in zip(before, new)]
            new = [1, 1, 40, 2] if rnd == 1 else [3, 1, 1, 1]
            nbt = torch.zeros(4, max(bt.shape[1], 40), dtype=torch.int32)
            nbt[:, :bt.shape[1]] = bt
            used = set(bt.flatten().tolist())
            free = [b for b in range(nblocks) if b not in used]
            for s in range(4):
                for i in range(-(-before[s] // bs), -(-(before[s] + new[s]) // bs)):
                    nbt[s, i] = free.pop()
            bt = nbt
            qsl = torch.tensor([0] + list(torch.tensor(new).cumsum(0)), dtype=torch.int32)
            seq = torch.tensor([a + b for a, b in zip(before, new)], dtype=torch.int32)
        T = sum(new)
        slots = _slots(bt, before, new, bs)
        proj = torch.randn(T, H * dk + G * dk + G * dv + 8).to(dt)
        q, k, v = proj[:, :H * dk], proj[:, H * dk:H * dk + G * dk], proj[:, H * dk + G * dk:H * dk + G * dk + G * dv]
        seqmix.kv_write(cache_c, k, v, slots, koff, voff, G, dk, dv, bs)
        pg = proj.to(gpu)
        qg, kg, vg = pg[:, :H * dk], pg[:, H * dk:H * dk + G * dk], pg[:, H * dk + G * dk:H * dk + G * dk + G * dv]
        sg = slots.to(gpu)
        seqmix.kv_write(cache_g, kg, vg, sg, koff, voff, G, dk, dv, bs)
        assert torch.equal(cache_g.cpu(), cache_c)
        oc = seqmix.window_attention(q, cache_c, bt, qsl, seq, koff, voff, H, G, dk, dv, bs, 0.13, window, keep)
        og = seqmix.window_attention(qg, cache_g, bt.to(gpu), qsl.to(gpu), seq.to(gpu), koff, voff, H, G, dk, dv, bs, 0.13,
                                     window, keep)
        torch.testing.assert_close(og.cpu().float(), oc.float(), **_tol(dt))
        # told the longest chunk, a bf16 step with MFMA-shaped heads takes the matrix-core kernel
        om = seqmix.window_attention(qg, cache_g, bt.to(gpu), qsl.to(gpu), seq.to(gpu), koff, voff, H, G, dk, dv, bs, 0.13,
                                     window, keep, max_query_len=max(new))
        torch.testing.assert_close(om.cpu().float(), oc.float(), **_tol(dt))


def test_kv_write_skips_padding(gpu):
    cache = torch.zeros(4, 2 * 16 * (8 + 8), device=gpu)
    k = torch.ones(3, 16, device=gpu)
    seqmix.kv_write(cache, k, k, torch.tensor([-1, 5, -1], device=gpu), 0, 2 * 16 * 8, 2, 8, 8, 16)
    assert float(cache.sum()) == 32.0


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,dk,dv", [(4, 64, 48), (3, 40, 64), (2, 20, 100), (2, 128, 128), (1, 160, 72)])
def test_scans_chunked_with_slot_reuse(gpu, dt, H, dk, dv):
    """Several steps over a state pool: fresh sequences in used slots, chunks of 1, 2, 17, ... tokens."""
    torch.manual_seed(4)
    slots_n, pad = 5, 11
    nl, nm = H * dk * dv, seqmix.mlstm_state_floats(H, dk, dv)
    st_c = torch.randn(slots_n, pad + nl + nm + 3)  # garbage: a fresh sequence must not read it
    st_g = st_c.to(gpu)
    decay = torch.tensor([0.6, 0.97, 0.999, 0.9, 0.8, 0.99][:H])
    steps = [([0, 0, 0], [33, 1, 2], [4, 0, 2]), ([33, 1, 2], [1, 17, 2], [4, 0, 2]), ([0, 18, 4], [5, 1, 1], [1, 0, 2]),
             ([5, 19, 5], [1, 1, 40], [1, 0, 2])]
    for before, new, rows in steps:
        T = sum(new)
        qsl = torch.tensor([0] + list(torch.tensor(new).cumsum(0)), dtype=torch.int32)
        seq = torch.tensor([a + b for a, b in zip(before, new)], dtype=torch.int32)
        rows_t = torch.tensor(rows, dtype=torch.int32)
        proj = torch.randn(T, 2 * H * dk + H * dv + 3).to(dt)
        q, k, v = proj[:, :H * dk], proj[:, H * dk:2 * H * dk], proj[:, 2 * H * dk:2 * H * dk + H * dv]
        gates = torch.randn(T, 2 * H) * 4
        pg = proj.to(gpu)
        qg, kg, vg = pg[:, :H * dk], pg[:, H * dk:2 * H * dk], pg[:, 2 * H * dk:2 * H * dk + H * dv]
        args_g = (st_g, rows_t.to(gpu)), (qsl.to(gpu), seq.to(gpu))
        oc = seqmix.decay_scan(q, k, v, decay, st_c, rows_t, pad, qsl, seq, H, dk, dv, silu=True)
        og = seqmix.decay_scan(qg, kg, vg, decay.to(gpu), *args_g[0], pad, *args_g[1], H, dk, dv, silu=True)
        torch.testing.assert_close(og.cpu(), oc, rtol=2e-4, atol=2e-4)
        oc = seqmix.mlstm_scan(q, k, v, gates, st_c, rows_t, pad + nl, qsl, seq, H, dk, dv, 11.0, dk ** -0.5)
        og = seqmix.mlstm_scan(qg, kg, vg, gates.to(gpu), *args_g[0], pad + nl, *args_g[1], H, dk, dv, 11.0, dk ** -0.5)
        torch.testing.assert_close(og.cpu(), oc, rtol=2e-4, atol=2e-4)
        live = sorted(set(rows))
        torch.testing.assert_close(st_g.cpu()[live, pad:pad + nl + nm], st_c[live, pad:pad + nl + nm], rtol=2e-4, atol=2e-4)
        assert torch.equal(st_g.cpu()[:, :pad], st_c[:, :pad]) and torch.equal(st_g.cpu()[:, pad + nl + nm:], st_c[:, pad + nl + nm:])


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,dk,dv", [(3, 40, 64), (2, 128, 72)])
def test_scans_split_over_time(gpu, dt, H, dk, dv):
    """Chunks of two pieces or more run as pieces side by side (end states chained): same outputs and
    end state as the serial walk, for fresh and continued sequences, next to a single-token row."""
    torch.manual_seed(6)
    nl, nm = H * dk * dv, seqmix.mlstm_state_floats(H, dk, dv)
    st_c = torch.randn(4, nl + nm)
    st_g = st_c.to(gpu)
    decay = torch.tensor([0.9, 0.99, 0.999][:H])
    for before, new, rows in (([0, 0, 0], [700, 1, 1300], [3, 1, 0]), ([700, 1, 1300], [513, 1, 1], [3, 1, 0])):
        T = sum(new)
        qsl = torch.tensor([0] + list(torch.tensor(new).cumsum(0)), dtype=torch.int32)
        seq = torch.tensor([a + b for a, b in zip(before, new)], dtype=torch.int32)
        rows_t = torch.tensor(rows, dtype=torch.int32)
        proj = (0.5 * torch.randn(T, 2 * H * dk + H * dv)).to(dt)
        q, k, v = proj[:, :H * dk], proj[:, H * dk:2 * H * dk], proj[:, 2 * H * dk:]
        gates = torch.randn(T, 2 * H) * 3 + torch.tensor([0.0] * H + [3.0] * H)
        pg = proj.to(gpu)
        qg, kg, vg = pg[:, :H * dk], pg[:, H * dk:2 * H * dk], pg[:, 2 * H * dk:]
        mq = max(new)
        oc = seqmix.decay_scan(q, k, v, decay, st_c, rows_t, 0, qsl, seq, H, dk, dv)
        og = seqmix.decay_scan(qg, kg, vg, decay.to(gpu), st_g, rows_t.to(gpu), 0, qsl.to(gpu), seq.to(gpu), H, dk, dv,
                               max_query_len=mq)
        torch.testing.assert_close(og.cpu(), oc, rtol=5e-4, atol=5e-4)
        oc = seqmix.mlstm_scan(q, k, v, gates, st_c, rows_t, nl, qsl, seq, H, dk, dv, 9.0, dk ** -0.5)
        og = seqmix.mlstm_scan(qg, kg, vg, gates.to(gpu), st_g, rows_t.to(gpu), nl, qsl.to(gpu), seq.to(gpu), H, dk, dv, 9.0,
                               dk ** -0.5, max_query_len=mq)
        torch.testing.assert_close(og.cpu(), oc, rtol=5e-4, atol=5e-4)
        live = sorted(set(rows))
        torch.testing.assert_close(st_g.cpu()[live], st_c[live], rtol=5e-4, atol=5e-4)
