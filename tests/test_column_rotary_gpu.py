"""The kernels of csrc/mixers/rotary_conv.hip and column_scan.hip against the PyTorch forms of the
same ops in mxserve/ops/seqmix.py, in bf16 and fp32: chunked batches over pages and state slots,
row-strided views that are not 16-byte aligned, sizes that are no multiples of the lane runs, steps
of single tokens (their own kernel form) and chunks long enough to be cut into pieces."""
import pytest
import torch

from mxserve.ops import seqmix
from tests.test_seqmix_gpu import _batch, _slots

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16]


def _tol(dt):
    return dict(rtol=2e-2, atol=2e-2) if dt == torch.bfloat16 else dict(rtol=3e-4, atol=3e-5)


def _view(T, n, dt, pad=3):
    """A [T, n] view at an odd column offset of a wider buffer."""
    return torch.randn(T, n + 2 * pad + 1).to(dt)[:, pad:pad + n]


STEPS = [([0, 5, 40], [33, 1, 7]), ([9, 0, 77, 3], [1, 1, 1, 1]), ([0], [2]), ([200], [1])]


@pytest.mark.parametrize("dt", DTYPES)
def test_embed_scaled_and_silu_mul(gpu, dt):
    torch.manual_seed(0)
    table = torch.randn(50, 72).to(dt)
    ids = torch.randint(0, 50, (19,))
    torch.testing.assert_close(seqmix.embed_scaled(ids.to(gpu), table.to(gpu), 3.5).cpu(), seqmix.embed_scaled(ids, table, 3.5))
    gu = _view(23, 2 * 88, dt)
    torch.testing.assert_close(seqmix.silu_mul(gu.to(gpu)[:, :]).cpu(), seqmix.silu_mul(gu), **_tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,dk,dv,nf,nvf,norm", [(6, 3, 24, 40, 8, 0, True), (4, 1, 64, 32, 32, 16, False), (2, 2, 16, 16, 1, 8, True),
                                                    (3, 1, 136, 72, 20, 36, True)])
def test_rope_qkv_cache_and_rows(gpu, dt, H, G, dk, dv, nf, nvf, norm):
    torch.manual_seed(1)
    bs, before, new = 16, [0, 21, 130], [35, 1, 6]
    bt, qsl, seq = _batch(before, new, bs, 24)
    slots = _slots(bt, before, new, bs)
    slots[-1] = -1  # a padding row writes nothing
    T = sum(new)
    pos = torch.cat([torch.arange(b, b + n) for b, n in zip(before, new)])
    fr = torch.rand(nf) + 0.01
    vfr = (torch.rand(nvf) + 0.01) if nvf else None
    qn, kn = (torch.randn(dk).to(dt), torch.randn(dk).to(dt)) if norm else (None, None)
    koff, voff = 8, 8 + G * bs * dk
    cache = torch.randn(24, voff + G * bs * dv + 5).to(dt)
    q, k, v = _view(T, H * dk, dt), _view(T, G * dk, dt), _view(T, G * dv, dt)
    g = lambda t: None if t is None else t.to(gpu)  # noqa: E731
    qc, cc = q.clone(), cache.clone()
    qg, cg = q.to(gpu).clone(), cache.to(gpu)
    seqmix.rope_qkv_cache(qc, k, v, pos, slots, cc, koff, voff, H, G, dk, dv, bs, fr, qn, kn, 1e-5, vfr)
    seqmix.rope_qkv_cache(qg, g(k), g(v), g(pos), g(slots), cg, koff, voff, H, G, dk, dv, bs, g(fr), g(qn), g(kn), 1e-5, g(vfr))
    torch.testing.assert_close(qg.cpu(), qc, **_tol(dt))
    torch.testing.assert_close(cg.cpu(), cc, **_tol(dt))
    # queries alone (a layer that reads another layer's pages)
    q2c, q2g = q.clone(), q.to(gpu).clone()
    seqmix.rope_qkv_cache(q2c, None, None, pos, slots, cc, koff, voff, H, G, dk, dv, bs, fr, qn, None, 1e-5, None)
    seqmix.rope_qkv_cache(q2g, None, None, g(pos), g(slots), cg, koff, voff, H, G, dk, dv, bs, g(fr), g(qn), None, 1e-5, None)
    torch.testing.assert_close(q2g.cpu(), q2c, **_tol(dt))
    # turning back, scaled, into a slice of a wider buffer
    if nvf:
        o = _view(T, H * dv, dt)
        bc, bg = torch.zeros(T, H * dv + 11, dtype=dt), torch.zeros(T, H * dv + 11, dtype=dt, device=gpu)
        seqmix.rope_rows(o, pos, H, dv, vfr, -1.0, 0.7, bc[:, 5:5 + H * dv])
        seqmix.rope_rows(g(o), g(pos), H, dv, g(vfr), -1.0, 0.7, bg[:, 5:5 + H * dv])
        torch.testing.assert_close(bg.cpu(), bc, **_tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("C,taps,aligned", [(200, 4, False), (256, 3, True), (72, 1, True), (40, 6, False)])
def test_causal_conv_carries_its_inputs(gpu, dt, C, taps, aligned):
    """Every step's outputs and the slot's carried inputs, over steps that start sequences, continue
    them with fewer tokens than the filter has taps, and reuse a slot that holds another's inputs."""
    torch.manual_seed(2)
    w, bias = torch.randn(taps, C).to(dt), torch.randn(C).to(dt)
    off = 8 if aligned else 5
    st_c = torch.randn(6, off + (taps - 1) * C + 3)
    st_g = st_c.to(gpu)
    rows = torch.tensor([4, 0, 2, 5], dtype=torch.int32)
    for before, new in STEPS + [([33, 6, 47, 0], [2, 1, 40, 9])]:
        S = len(new)
        _, qsl, seq = _batch(before, new, 16, 64)
        T = sum(new)
        x = torch.randn(T, C).to(dt) if aligned else _view(T, C, dt)
        for b in (bias, None):
            yc = seqmix.causal_conv(x, w, b, st_c, rows[:S], off, qsl, seq)
            yg = seqmix.causal_conv(x.to(gpu), w.to(gpu), None if b is None else b.to(gpu), st_g, rows[:S].to(gpu), off,
                                    qsl.to(gpu), seq.to(gpu))
            torch.testing.assert_close(yg.cpu(), yc, **_tol(dt))
            torch.testing.assert_close(st_g.cpu(), st_c, rtol=0, atol=0)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("groups,silu,first,wn", [(1, True, True, 192), (4, True, True, 192), (6, False, False, 32), (3, False, False, 192)])
def test_gated_norm_forms(gpu, dt, groups, silu, first, wn):
    torch.manual_seed(3)
    T, N = 29, 192
    o, gate, w = torch.randn(T, N), _view(T, N, dt), torch.randn(wn).to(dt)
    act = "silu" if silu else "sigmoid"
    bc, bg = torch.zeros(T, N + 9, dtype=dt), torch.zeros(T, N + 9, dtype=dt, device=gpu)
    seqmix.gated_norm(o, gate, w, 1e-5, groups, act, first, dt, 1.3, bc[:, 4:4 + N])
    seqmix.gated_norm(o.to(gpu), gate.to(gpu), w.to(gpu), 1e-5, groups, act, first, dt, 1.3, bg[:, 4:4 + N])
    torch.testing.assert_close(bg.cpu(), bc, **_tol(dt))


def _scan_steps():
    return STEPS + [([0, 31], [300, 150]), ([300, 181, 0], [140, 1, 129])]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,N,P,aligned", [(4, 2, 40, 24, False), (2, 1, 128, 64, True), (3, 3, 16, 8, True), (2, 2, 200, 72, True)])
def test_ssd_scan(gpu, dt, H, G, N, P, aligned):
    torch.manual_seed(4)
    off = 8 if aligned else 3
    st_c = torch.randn(5, off + H * N * P + 2)
    st_g = st_c.to(gpu)
    rows = torch.tensor([3, 1, 4, 0], dtype=torch.int32)
    dtb, A, D = torch.randn(H) - 1.0, torch.randn(H) * 0.5 - 1.5, torch.randn(H)
    for before, new in _scan_steps():
        S = len(new)
        _, qsl, seq = _batch(before, new, 16, 64)
        T = sum(new)
        mk = (lambda n: torch.randn(T, n).to(dt)) if aligned else (lambda n: _view(T, n, dt))
        x, B, C, d = mk(H * P), mk(G * N) * 0.3, mk(G * N) * 0.3, mk(H)
        g = lambda t: t.to(gpu)  # noqa: E731
        yc = seqmix.ssd_scan(x, B, C, d, dtb, A, D, st_c, rows[:S], off, qsl, seq, H, G, N, P)
        yg = seqmix.ssd_scan(g(x), g(B), g(C), g(d), g(dtb), g(A), g(D), st_g, g(rows[:S]), off, g(qsl), g(seq), H, G, N, P,
                             max_query_len=max(new))
        torch.testing.assert_close(yg.cpu(), yc, rtol=2e-4, atol=2e-4)
        torch.testing.assert_close(st_g[rows[:S].long()].cpu(), st_c[rows[:S].long()], rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,dk,dv,aligned", [(4, 2, 24, 40, False), (2, 2, 128, 128, True), (3, 1, 16, 8, True), (2, 1, 72, 200, True)])
def test_delta_scan(gpu, dt, H, G, dk, dv, aligned):
    torch.manual_seed(5)
    off = 8 if aligned else 3
    st_c = torch.randn(5, off + H * dk * dv + 2)
    st_g = st_c.to(gpu)
    rows = torch.tensor([3, 1, 4, 0], dtype=torch.int32)
    dtb, A = torch.randn(H * dk) - 1.0, torch.randn(H) * 0.5 - 2.0
    for before, new in _scan_steps():
        S = len(new)
        _, qsl, seq = _batch(before, new, 16, 64)
        T = sum(new)
        mk = (lambda n: torch.randn(T, n).to(dt)) if aligned else (lambda n: _view(T, n, dt))
        q, k, v, b, a = mk(G * dk), mk(G * dk), mk(H * dv), mk(H), mk(H * dk)
        g = lambda t: t.to(gpu)  # noqa: E731
        yc = seqmix.delta_scan(q, k, v, b, a, dtb, A, st_c, rows[:S], off, qsl, seq, H, G, dk, dv, dk ** -0.5)
        yg = seqmix.delta_scan(g(q), g(k), g(v), g(b), g(a), g(dtb), g(A), st_g, g(rows[:S]), off, g(qsl), g(seq), H, G, dk, dv,
                               dk ** -0.5, max_query_len=max(new))
        torch.testing.assert_close(yg.cpu(), yc, rtol=5e-4, atol=5e-4)
        torch.testing.assert_close(st_g[rows[:S].long()].cpu(), st_c[rows[:S].long()], rtol=5e-4, atol=5e-4)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,dk,dv", [(4, 2, 24, 40), (8, 2, 64, 64), (4, 1, 64, 32), (2, 2, 128, 128)])
def test_attention_sink_in_every_kernel_form(gpu, dt, H, G, dk, dv):
    """Generic, 16-byte-row and (bf16, MFMA-shaped heads, chunks of 16 rows or more) matrix-core forms with
    a per-head sink, against the PyTorch form.  The block tables are exactly as long as the longest
    sequence needs and its chunk ends in a partial tile of five rows: the tile must sit at its own
    positions although the table ends less than 16 tokens after its first."""
    torch.manual_seed(6)
    bs, before, new = 16, [0, 37, 130], [50, 1, 21]
    bt, qsl, seq = _batch(before, new, bs, 32)
    T = sum(new)
    koff, voff = 0, G * bs * dk
    cache = (torch.randn(32, voff + G * bs * dv) * 0.5).to(dt)
    q = torch.randn(T, H * dk).to(dt)
    sink = torch.randn(H) * 2.0
    oc = seqmix.window_attention(q, cache, bt, qsl, seq, koff, voff, H, G, dk, dv, bs, dk ** -0.5, 0, 0, max(new), sink=sink)
    og = seqmix.window_attention(q.to(gpu), cache.to(gpu), bt.to(gpu), qsl.to(gpu), seq.to(gpu), koff, voff, H, G, dk, dv, bs,
                                 dk ** -0.5, 0, 0, max(new), sink=sink.to(gpu))
    torch.testing.assert_close(og.cpu(), oc, **_tol(dt))
    # single tokens only (the row kernels)
    bt, qsl, seq = _batch([5, 99, 16], [1, 1, 1], bs, 32)
    q1 = torch.randn(3, H * dk).to(dt)
    oc = seqmix.window_attention(q1, cache, bt, qsl, seq, koff, voff, H, G, dk, dv, bs, dk ** -0.5, 0, 0, 1, sink=sink)
    og = seqmix.window_attention(q1.to(gpu), cache.to(gpu), bt.to(gpu), qsl.to(gpu), seq.to(gpu), koff, voff, H, G, dk, dv, bs,
                                 dk ** -0.5, 0, 0, 1, sink=sink.to(gpu))
    torch.testing.assert_close(og.cpu(), oc, **_tol(dt))
