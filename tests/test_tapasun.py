"""Tapasun through the engine (paged K/V, shared pages, state slots, forced and scheduled steps)
against the plain float64 oracle of tests/tapasun_oracle.py: on the PyTorch forms of the ops here, on
the HIP kernels under `-m gpu`.  Every test makes its own small configuration and random weights."""
import types

import numpy as np
import pytest
import torch

from tests import tapasun_oracle as to
from tests.tapasun_utils import (BANDS, BASE, attention, config, cut, engine, mamba2, parallel, rel_err, replay,
                                 write_checkpoint)

DEVS = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
DEV_DTYPE_TOL = [("cpu", "float32", 1e-4), pytest.param("cuda", "float32", 1e-4, marks=pytest.mark.gpu),
                 pytest.param("cuda", "bfloat16", 0.12, marks=pytest.mark.gpu)]
EPS = 1e-5


def _skip(dev):
    if dev == "cuda" and not torch.cuda.is_available():
        pytest.skip("no GPU")


def _tokens(n, vocab, seed):
    return np.random.default_rng(seed).integers(0, vocab, n).tolist()


def _row_errors(got, want):
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)) / np.sqrt((want ** 2).mean())


def _check(got, want, tol):
    """fp32 (tol well below 1e-2): every row within tol.  bf16: rounding leaves a few per cent on a
    typical row and several times that on a row where a sublayer's output is small before its norm,
    whatever the schedule; so the mean over the rows (of eight or more) is held to tol / 4 and the worst
    row to 2.5 tol."""
    if tol < 1e-2:
        e = rel_err(got, want)
        assert e < tol, f"relative error {e:.3g} >= {tol}"
        return
    e = _row_errors(got, want)
    assert (len(e) < 8 or e.mean() < tol / 4) and e.max() < 2.5 * tol, f"row errors: mean {e.mean():.3g}, worst {e.max():.3g} (tol {tol})"


def _oracle_model(cfg, w, tokens):
    return to.Oracle(cfg, w).run(tokens)[0]


# ----------------------------------------------------------------------------- mechanisms alone
def _mixer_setup(kind, mc, width, seed=0):
    from mxserve.models.tapasun import build_mixer
    m = build_mixer(kind, "m.", width, mc)
    g = torch.Generator().manual_seed(seed)
    shapes = {name: (rows, width) for name, rows in m.proj_rows()}
    shapes.update(m.extra_shapes())
    w = {k: torch.randn(s, generator=g) * (s[-1] ** -0.5 if len(s) > 1 else 1.0) for k, s in shapes.items()}
    for k in w:
        if k.endswith("A_log") or k.endswith("dt_bias"):
            w[k] = w[k] * 0.7 - 0.5
    return m, w


class _Pages:
    """One sequence's pages and state slot, scattered over a pool that holds stale numbers."""

    def __init__(self, T, elems, state_floats, dev, bs=16, slot=2):
        nb = -(-T // bs) + 3
        self.bs, self.dev, self.slot = bs, dev, slot
        self.cache = torch.randn(nb, elems + 16, device=dev)
        self.state = torch.randn(4, state_floats + 7, device=dev)
        self.blocks = torch.randperm(nb, generator=torch.Generator().manual_seed(3))[:-(-T // bs)].to(torch.int32)

    def ctx(self, at, n):
        from mxserve.models.mixers import StepContext
        dev, bs = self.dev, self.bs
        pos = torch.arange(at, at + n)
        md = types.SimpleNamespace(
            positions=pos.to(dev), slot_mapping=(self.blocks[pos // bs].long() * bs + pos % bs).to(dev),
            block_tables=self.blocks[None].to(dev), query_start_loc=torch.tensor([0, n], dtype=torch.int32, device=dev),
            seq_lens=torch.tensor([at + n], dtype=torch.int32, device=dev), max_query_len=n,
            state_rows=torch.tensor([self.slot], dtype=torch.int32, device=dev))
        return StepContext(md=md, cache=self.cache, state=self.state, block_size=bs, eps=EPS)


def _run_mixers(ms, ws, h, dev, portions, offs=None):
    """The mixers, one after the other on the same input, over one sequence cut into portions, through
    paged K/V and a state slot.  offs: (koff, voff) per mixer (a mixer that reads another's pages gets
    that one's)."""
    T = h.shape[0]
    wts, w_ins = [], []
    for m, w in zip(ms, ws):
        wt = {k: v.to(dev) for k, v in w.items()}
        w_ins.append(torch.cat([wt[name] for name, _ in m.proj_rows()]))
        m.finish_weights(wt)
        wts.append(wt)
    bs = 16
    if offs is None:
        offs, at = [], 0
        for m in ms:
            offs.append((at, at + m.kv_heads * bs * m.dk))
            at += m.kv_heads * bs * (m.dk + m.dv)
    elems = max([v + m.kv_heads * bs * m.dv for m, (_, v) in zip(ms, offs)] + [1])
    soffs, sf = [], 5
    for m in ms:
        soffs.append(sf)
        sf += m.state_floats
    pg = _Pages(T, elems, sf, dev, bs)
    outs, at, i = [[] for _ in ms], 0, 0
    while at < T:
        n = min(portions[min(i, len(portions) - 1)], T - at)
        i += 1
        ctx = pg.ctx(at, n)
        hp = h[at:at + n].to(dev)
        for j, m in enumerate(ms):
            y = hp @ w_ins[j].T
            parts, c = [], 0
            for _, rows in m.proj_rows():
                parts.append(y[:, c:c + rows])
                c += rows
            outs[j].append(m.forward(parts, hp, wts[j], ctx, offs[j][0], offs[j][1], soffs[j]))
        at += n
    return [torch.cat(o).double().cpu().numpy() for o in outs]


def _oracle_steps(mixer, h):
    caches = {}
    return np.stack([mixer.step(h[t], t, caches) for t in range(h.shape[0])])


PORTIONS = [[1000], [1], [2], [5, 1, 9, 2, 30]]


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("portions", PORTIONS)
def test_state_space_mixer(dev, portions):
    _skip(dev)
    width, T = 80, 70
    h = torch.randn(T, width, generator=torch.Generator().manual_seed(1))
    for mc in (mamba2(heads=4, vdim=24, state=40, groups=2, conv=4, norm_groups=2)["mixer"],
               mamba2(heads=3, vdim=40, state=72, groups=3, conv=1, norm_groups=1)["mixer"],
               mamba2(heads=2, vdim=8, state=16, groups=1, conv=5, norm_groups=4)["mixer"]):
        m, w = _mixer_setup("mamba2", mc, width)
        wn = {k: v.double().numpy() for k, v in w.items()}
        want = _oracle_steps(to.Mamba2(mc, wn, "m.", EPS), h.double().numpy())
        _check(_run_mixers([m], [w], h, dev, portions)[0], want, 1e-4)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("portions", [[300], [129, 171], [7, 290, 3], [150, 1, 149]])
def test_state_space_long_chunks(dev, portions):
    """Chunks long enough that the GPU scan cuts them into pieces that run side by side: a piece's
    start state is chained from the pieces before it, and from the slot when the chunk is not the
    sequence's first."""
    _skip(dev)
    width, T = 64, 300
    h = torch.randn(T, width, generator=torch.Generator().manual_seed(4))
    mc = mamba2(heads=4, vdim=24, state=40, groups=2, conv=3, norm_groups=1)["mixer"]
    m, w = _mixer_setup("mamba2", mc, width)
    w["m.A_log"] = w["m.A_log"] - 2.0  # slow decays: what a piece inherits matters to its end
    wn = {k: v.double().numpy() for k, v in w.items()}
    want = _oracle_steps(to.Mamba2(mc, wn, "m.", EPS), h.double().numpy())
    _check(_run_mixers([m], [w], h, dev, portions)[0], want, 1e-4)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("portions", [[300], [129, 171], [7, 290, 3], [150, 1, 149]])
def test_delta_rule_long_chunks(dev, portions):
    """The same for the delta rule, whose pieces are chained through their transition matrices."""
    _skip(dev)
    from mxserve.models.tapasun import build_mixer
    width, T = 64, 300
    h = torch.randn(T, width, generator=torch.Generator().manual_seed(6))
    mc = parallel(rheads=4, rkv=2, rdim=24, rvdim=40, conv=3)["mixer"]
    m = build_mixer("parallel", "m.", width, mc).right
    g = torch.Generator().manual_seed(7)
    shapes = {name: (rows, width) for name, rows in m.proj_rows()}
    shapes.update(m.extra_shapes())
    w = {k: torch.randn(s, generator=g) * (s[-1] ** -0.5 if len(s) > 1 else 1.0) for k, s in shapes.items()}
    w["m.right.A_log"] = w["m.right.A_log"] - 3.0  # slow decays: what a piece inherits matters to its end
    w["m.right.dt_bias"] = w["m.right.dt_bias"] - 1.0
    wn = {k: v.double().numpy() for k, v in w.items()}
    want = _oracle_steps(to.GatedDeltaRule(mc["right"], wn, "m.right.", EPS), h.double().numpy())
    _check(_run_mixers([m], [w], h, dev, portions)[0], want, 1e-4)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("portions", PORTIONS)
def test_rotary_attention_mixer_and_shared_pages(dev, portions):
    """An attention layer with keys of its own and a second one that reads the first one's pages with
    its own queries; full and partial rotation, band-scaled, linearly scaled and plain frequencies."""
    _skip(dev)
    width, T = 80, 70
    h = torch.randn(T, width, generator=torch.Generator().manual_seed(2))
    hn = h.double().numpy()
    for kw in (dict(heads=6, kv_heads=3, dim=24, vdim=40, dims=16, scaling=BANDS), dict(heads=2, kv_heads=2, dim=16, vdim=8, dims=16, scaling=None),
               dict(heads=4, kv_heads=1, dim=40, vdim=72, dims=2, scaling={"factor": 3.0}, base=50.0)):
        a, b = attention(**kw)["mixer"], attention(kv_from=0, **kw)["mixer"]
        ma, wa = _mixer_setup("attention", a, width, seed=1)
        mb, wb = _mixer_setup("attention", b, width, seed=2)
        assert [n for n, _ in mb.proj_rows()] == ["m.q"] and "m.k.norm" not in mb.extra_shapes()
        wan, wbn = ({k: v.double().numpy() for k, v in w.items()} for w in (wa, wb))
        oa = to.Attention(a, wan, "m.", EPS, 0, True, False, False)
        ob = to.Attention(b, wbn, "m.", EPS, 1, True, False, False)
        caches, wa_, wb_ = {}, [], []
        for t in range(T):
            wa_.append(oa.step(hn[t], t, caches))
            wb_.append(ob.step(hn[t], t, caches))
        bs = 16
        off = (0, ma.kv_heads * bs * ma.dk)
        ga, gb = _run_mixers([ma, mb], [wa, wb], h, dev, portions, offs=[off, off])
        _check(ga, np.stack(wa_), 1e-4)
        _check(gb, np.stack(wb_), 1e-4)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("portions", PORTIONS)
@pytest.mark.parametrize("scales", [(0.7, 1.2), (1.0, 0.0), (0.0, 1.0)])
def test_parallel_mixer(dev, portions, scales):
    """Both branches together and each alone (the other's scale zero): learned sink, turned values and
    their turning back on the left; convolutions, unit norms, channel decays and the delta rule on the right."""
    _skip(dev)
    width, T = 80, 70
    h = torch.randn(T, width, generator=torch.Generator().manual_seed(3))
    for kw in (dict(), dict(heads=2, kv_heads=1, dim=16, vdim=40, dims=16, rheads=3, rkv=3, rdim=40, rvdim=16, conv=4),
               dict(heads=3, kv_heads=3, dim=8, vdim=8, dims=2, rheads=2, rkv=1, rdim=72, rvdim=24, conv=2, factor=1.0)):
        mc = parallel(ls=scales[0], rs=scales[1], **kw)["mixer"]
        m, w = _mixer_setup("parallel", mc, width)
        w["m.left.sink"] = w["m.left.sink"] * 2.0
        wn = {k: v.double().numpy() for k, v in w.items()}
        want = _oracle_steps(to.Parallel(mc, wn, "m.", EPS, 0), h.double().numpy())
        _check(_run_mixers([m], [w], h, dev, portions)[0], want, 1e-4)


def _one_head(width, sink, dims=2, qk_norm=False):
    from mxserve.models.mixers import RotaryAttention
    return RotaryAttention("m.", width, 1, 1, width, width, 1.0, {"dims": dims, "base": 100.0}, qk_norm=qk_norm, sink=sink)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("target", [0, 1, 15, 16, 17, 31, 32, 47, 48, 200, 255, 256, 299])
def test_one_far_key_stands_out(dev, target):
    """One key among three hundred matches the last query so strongly that the output is that key's
    value: the first token, both sides of page borders and keys far back, in a whole prompt, when the
    last token is decoded alone, and in uneven portions."""
    _skip(dev)
    T, width = 301, 16
    m = _one_head(width, "zero")
    eye = torch.eye(width)
    wq = eye.clone()
    wq[[3, 5]] = wq[[5, 3]]  # the query reads coordinate 3 as 5: the last token does not match itself
    w = {"m.q": wq, "m.k": eye, "m.v": eye, "m.o": eye}
    g = torch.Generator().manual_seed(5)
    h = 0.1 * torch.randn(T, width, generator=g)
    h[:, :2] = 0.0  # the turned pair stays out of the scores
    h[target, 5] += 8.0
    h[T - 1] = 0.0
    h[T - 1, 3] = 8.0
    mc = {"heads": 1, "kv_heads": 1, "dim": width, "vdim": width, "scale": 1.0, "rot": {"dims": 2, "base": 100.0}}
    wn = {k: v.double().numpy() for k, v in w.items()}
    want = _oracle_steps(to.Attention(mc, wn, "m.", EPS, 0, False, False, False), h.double().numpy())
    assert np.abs(want[T - 1] - h[target].double().numpy()).max() < 0.05  # the oracle itself shows the case
    for portions in ([T], [T - 1, 1], [7, 2, 160, 3, 100, 1]):
        got = _run_mixers([m], [dict(w)], h, dev, portions)[0]
        assert np.abs(got - want).max() < 1e-4


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("kind,level,weight", [(None, 0.0, 1.0), ("zero", 0.0, 0.5), ("learned", 2.0, 1.0 / (1.0 + np.e ** 2)),
                                               ("learned", -30.0, 1.0)])
def test_sink_takes_its_share(dev, kind, level, weight):
    """A single key whose score is exactly 0: the output is the value times 1 / (1 + exp(sink)); without
    a sink it is the value.  Left out, the sink would show as a factor of two."""
    _skip(dev)
    width = 16
    m = _one_head(width, kind)
    eye = torch.eye(width)
    w = {"m.q": torch.zeros(width, width), "m.k": eye, "m.v": eye, "m.o": eye}
    if kind == "learned":
        w["m.sink"] = torch.tensor([level])
    h = torch.randn(1, width, generator=torch.Generator().manual_seed(1))
    h[:, :2] = 0.0
    got = _run_mixers([m], [w], h, dev, [1])[0]
    assert np.abs(got - weight * h.double().numpy()).max() < 1e-5
    # and with many keys of score 0: the sink counts once, not once per key
    h = torch.randn(40, width, generator=torch.Generator().manual_seed(2))
    h[:, :2] = 0.0
    got = _run_mixers([m], [w], h, dev, [33, 1])[0]
    z = 0.0 if kind is None else np.exp(level)
    want = np.cumsum(h.double().numpy(), 0) / (np.arange(1, 41)[:, None] + z)
    assert np.abs(got - want).max() < 1e-5


@pytest.mark.parametrize("dev", DEVS)
def test_positions_turn_keys_values_and_outputs(dev):
    """With identity projections and a query that sees one key only, the output is that key's value
    turned forward by its own position and back by the query's: the difference of positions shows."""
    _skip(dev)
    from mxserve.models.mixers import RotaryAttention
    width, T = 8, 37
    m = RotaryAttention("m.", width, 1, 1, width, width, 1.0, {"dims": 2, "base": 100.0}, qk_norm=False, sink="learned",
                        rotate_values=True)
    eye = torch.eye(width)
    wq = eye.clone()
    wq[[3, 5]] = wq[[5, 3]]
    w = {"m.q": wq, "m.k": eye, "m.v": eye, "m.o": eye, "m.sink": torch.tensor([-40.0])}
    h = torch.zeros(T, width)
    h[4, 5] = 9.0
    h[4, 6], h[4, 7] = 1.0, 0.5
    h[T - 1, 3] = 9.0
    mc = {"heads": 1, "kv_heads": 1, "dim": width, "vdim": width, "scale": 1.0, "rot": {"dims": 2, "base": 100.0}}
    wn = {k: v.double().numpy() for k, v in w.items()}
    want = _oracle_steps(to.Attention(mc, wn, "m.", EPS, 0, False, True, True), h.double().numpy())
    ang = -(T - 1 - 4) * 100.0 ** (-6.0 / 8)  # pair (6, 7) turns by the distance times its frequency
    assert abs(want[T - 1, 6] - (np.cos(ang) * 1.0 - np.sin(ang) * 0.5)) < 1e-3
    for portions in ([T], [T - 1, 1], [3, 2]):
        assert np.abs(_run_mixers([m], [dict(w)], h, dev, portions)[0] - want).max() < 1e-4


@pytest.mark.parametrize("dev", DEVS)
def test_delta_rule_overwrites_a_key(dev):
    """Writing twice under the same unit key with full strength and no decay leaves the second value
    only: the delta rule's correction, which a plain linear attention would not make."""
    _skip(dev)
    from mxserve.ops import seqmix
    H, dk, dv, T = 1, 8, 4, 3
    q = torch.zeros(T, dk)
    k = torch.zeros(T, dk)
    k[0, 2] = k[1, 2] = 3.0   # unit-normed inside
    q[2, 2] = 5.0
    k[2, 5] = 1.0             # the last token writes elsewhere
    v = torch.tensor([[1.0, 2.0, 3.0, 4.0], [-1.0, 0.5, 0.0, 2.0], [0.0, 0.0, 0.0, 0.0]])
    beta = torch.full((T, H), 40.0)      # sigmoid -> 1
    a = torch.full((T, H * dk), -60.0)   # softplus -> 0: no decay
    args = dict(dt_bias=torch.zeros(H * dk), A_log=torch.zeros(H))
    state = torch.randn(2, H * dk * dv + 3)
    dv_ = torch.device(dev)
    o = seqmix.delta_scan(q.to(dv_), k.to(dv_), v.to(dv_), beta.to(dv_), a.to(dv_), args["dt_bias"].to(dv_), args["A_log"].to(dv_),
                          state.to(dv_), torch.tensor([1], dtype=torch.int32, device=dv_), 2,
                          torch.tensor([0, T], dtype=torch.int32, device=dv_), torch.tensor([T], dtype=torch.int32, device=dv_),
                          H, 1, dk, dv, 1.0, 1e-6)
    assert np.abs(o[2].cpu().numpy() - v[1].numpy()).max() < 1e-4


# ----------------------------------------------------------------------------- whole models, schedules
@pytest.fixture(scope="module")
def base(tmp_path_factory):
    path = tmp_path_factory.mktemp("tapasun_base")
    w = write_checkpoint(path, BASE, seed=11)
    toks = {f"r{i}": _tokens(n, BASE["vocab"], 20 + i) for i, n in enumerate([90, 37, 1, 64, 130, 16])}
    want = {rid: _oracle_model(BASE, w, t) for rid, t in toks.items()}
    return path, w, toks, want


@pytest.mark.parametrize("dev,dtype,tol", DEV_DTYPE_TOL)
def test_portions_and_decoding(base, dev, dtype, tol):
    """Whole prompt, token by token, and portions of several sizes down to two tokens."""
    _skip(dev)
    path, _, toks, want = base
    eng = engine(path, dev, dtype, max_tokens=256)
    for sizes in ([1000], [1], [2], [40, 1], [3, 16, 2, 17, 1, 32, 5]):
        steps = [[("a", p, False)] for p in cut(toks["r0"], sizes)]
        steps[-1] = [("a", steps[-1][0][1], True)]
        _check(replay(eng, steps)["a"], want["r0"], tol)
    assert eng.kv.num_free() == eng.kv.num_blocks


@pytest.mark.parametrize("dev,dtype,tol", DEV_DTYPE_TOL)
def test_long_decoding(base, dev, dtype, tol):
    """A short prompt, then well over a hundred tokens one by one (through the decode graphs on the
    GPU): pages fill and new ones start, recurrent and convolution states are carried all the way."""
    _skip(dev)
    path, _, toks, want = base
    eng = engine(path, dev, dtype, max_tokens=192, eager=(dev == "cpu"))
    steps = [[("a", p, False)] for p in cut(toks["r4"], [10, 1])]
    steps[-1] = [("a", steps[-1][0][1], True)]
    _check(replay(eng, steps)["a"], want["r4"], tol)
    assert eng.kv.num_free() == eng.kv.num_blocks


@pytest.mark.parametrize("dev,dtype,tol", DEV_DTYPE_TOL)
@pytest.mark.parametrize("eager", [True, False])
def test_mixed_batches_reuse_pages_and_slots(base, dev, dtype, tol, eager):
    """Six unequal requests through four slots and a pool that cannot hold them all at once: portions of
    some beside single tokens of others; each must equal the request run alone (the oracle)."""
    _skip(dev)
    if dev == "cpu" and not eager:
        pytest.skip("graphs are a GPU path")
    path, _, toks, want = base
    eng = engine(path, dev, dtype, max_tokens=384, eager=eager)
    rng = np.random.default_rng(3)
    at = {r: 0 for r in toks}
    waiting, live, steps = list(toks), [], []
    while waiting or live:
        while waiting and len(live) < 4 and sum(-(-len(toks[r]) // 64) * 64 for r in live + waiting[:1]) <= 384:
            live.append(waiting.pop(0))
        step = []
        for r in list(live):
            if rng.random() < 0.2 and len(live) > 1:
                continue  # left out of this step
            left = len(toks[r]) - at[r]
            n = min(left, int(rng.choice([1, 1, 2, 3, 16, 29])))
            end = n == left
            step.append((r, toks[r][at[r]:at[r] + n], end))
            at[r] += n
            if end:
                live.remove(r)
        if step:
            steps.append(step)
    got = replay(eng, steps)
    for r in toks:
        _check(got[r], want[r], tol)
    assert eng.kv.num_free() == eng.kv.num_blocks and not eng.runner._row_of


@pytest.mark.parametrize("dev,dtype,tol", DEV_DTYPE_TOL)
def test_request_that_fills_the_pool(tmp_path, dev, dtype, tol):
    """A request three tokens short of the pool and of the longest sequence the engine admits, with head
    sizes that take the matrix-core attention in bf16: its last portions end in partial tiles on the
    last page of the block table."""
    _skip(dev)
    cfg = config([attention(heads=4, kv_heads=2, dim=64, vdim=64, dims=32, scale=0.125, mlp=128),
                  parallel(heads=4, kv_heads=1, dim=32, vdim=32, dims=16, scale=0.18, rheads=2, rkv=2, rdim=32, rvdim=32,
                           conv=4, mlp=None),
                  attention(heads=4, kv_heads=2, dim=64, vdim=64, dims=32, scale=0.125, kv_from=0, mlp=128)],
                 width=128, vocab=200)
    w = write_checkpoint(tmp_path, cfg, seed=8)
    t = _tokens(125, cfg["vocab"], 9)
    want = _oracle_model(cfg, w, t)
    eng = engine(tmp_path, dev, dtype, max_tokens=128)
    for sizes in ([1000], [90, 35], [100, 19, 1], [64, 40, 21]):
        steps = [[("a", p, False)] for p in cut(t, sizes)]
        steps[-1] = [("a", steps[-1][0][1], True)]
        _check(replay(eng, steps)["a"], want, tol)
    assert eng.kv.num_free() == eng.kv.num_blocks


VARIANTS = {
    "every_head_its_own_kv_and_group": config([attention(heads=3, kv_heads=3, dim=16, vdim=16, dims=16, scaling=None, mlp=64),
                                               mamba2(heads=2, vdim=16, state=16, groups=2, conv=2, norm_groups=2, mlp=None),
                                               parallel(heads=2, kv_heads=2, dim=16, vdim=16, dims=16, rheads=2, rkv=2, rdim=16,
                                                        rvdim=16, conv=2, ls=1.0, rs=1.0, mlp=None)], width=48, vocab=96,
                                              embed_scale=1.0),
    "one_head_one_group_filter_of_one": config([mamba2(heads=1, vdim=40, state=8, groups=1, conv=1, norm_groups=1, mlp=64),
                                                attention(heads=1, kv_heads=1, dim=8, vdim=24, dims=2, scale=1.0,
                                                          scaling={"factor": 1.0}, mlp=None),
                                                parallel(heads=1, kv_heads=1, dim=8, vdim=2, dims=4, rheads=1, rkv=1, rdim=8,
                                                         rvdim=8, conv=1, ls=0.5, rs=2.0, mlp=32)], width=40, vocab=50, eps=1e-3),
    "pages_shared_by_three_layers": config([attention(heads=8, kv_heads=2, dim=8, vdim=8, dims=4, mlp=None),
                                            attention(heads=8, kv_heads=2, dim=8, vdim=8, dims=4, kv_from=0, mlp=32),
                                            parallel(mlp=None), attention(heads=8, kv_heads=2, dim=8, vdim=8, dims=4, kv_from=0,
                                                                          mlp=None)], width=64, vocab=70, embed_scale=7.5),
    "wide_state_and_long_filter": config([mamba2(heads=2, vdim=72, state=136, groups=1, conv=6, norm_groups=3, mlp=None),
                                          parallel(heads=2, kv_heads=1, dim=72, vdim=136, dims=36, rheads=2, rkv=1, rdim=136,
                                                   rvdim=72, conv=5, mlp=None)], width=72, vocab=60),
}


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("name", list(VARIANTS))
def test_other_sizes(tmp_path, dev, name):
    _skip(dev)
    cfg = VARIANTS[name]
    w = write_checkpoint(tmp_path, cfg, seed=5, ranks=(1, 9) if "one_head" in name else (24, 8))
    t = _tokens(45, cfg["vocab"], 6)
    want = _oracle_model(cfg, w, t)
    eng = engine(tmp_path, dev, "float32", max_tokens=128)
    for sizes in ([1000], [20, 2, 1, 7, 1]):
        steps = [[("a", p, False)] for p in cut(t, sizes)]
        steps[-1] = [("a", steps[-1][0][1], True)]
        _check(replay(eng, steps)["a"], want, 1e-4)


@pytest.mark.parametrize("dev", DEVS)
def test_layer_tap_matches_oracle_streams(base, dev):
    _skip(dev)
    path, w, toks, _ = base
    eng = engine(path, dev, "float32", max_tokens=128)
    tap = eng.runner.model.layer_tap = []
    replay(eng, [[("a", toks["r1"], True)]])
    ref = to.Oracle(BASE, w).run(toks["r1"])[1]
    assert len(tap) == len(ref) == len(BASE["layers"])
    for a, b in zip(tap, ref):
        assert np.abs(a.double().cpu().numpy() - b).max() < 1e-3 * max(1.0, np.abs(b).max())


def test_pages_and_state_of_the_plan():
    """Layers that read another layer's pages keep none of their own; every recurrent layer has its
    place in the slot, with the filters' carried inputs behind the matrix state."""
    from mxserve.models.config import tapasun_config
    from mxserve.models.tapasun import layer_plan, mixers_of
    plan = layer_plan(BASE, 16)
    ms = mixers_of(BASE)
    assert [r.owns_kv for r in plan.runs] == [True, True, True, False, True, True]
    assert (plan.runs[3].koff, plan.runs[3].voff) == (plan.runs[1].koff, plan.runs[1].voff)
    own = [r for r in plan.runs if r.kv_heads and r.owns_kv]
    assert plan.block_elems == sum(r.kv_heads * 16 * (r.dk + r.dv) for r in own)
    assert plan.state_floats == sum(m.state_floats for m in ms)
    m0 = ms[0]
    assert m0.state_floats == m0.heads * m0.P * m0.N + (m0.taps - 1) * (m0.inner + 2 * m0.G * m0.N)
    cfg = tapasun_config("t", BASE)
    assert cfg.has_recurrent_state and cfg.kv_bytes_per_token(2) == 2 * plan.block_elems // 16
    bad = config([attention(), attention(kv_from=2), attention()])
    with pytest.raises(ValueError):
        layer_plan(bad, 16)


@pytest.mark.parametrize("dev,dtype", [("cpu", "float32"), pytest.param("cuda", "float32", marks=pytest.mark.gpu),
                                       pytest.param("cuda", "bfloat16", marks=pytest.mark.gpu)])
def test_greedy_generation_through_the_scheduler(base, dev, dtype):
    """LLMEngine.generate: the scheduler chunks the prompts (a small token budget), batches the
    requests and decodes; every generated token must be the oracle's choice given the same prefix
    (or within its near-ties)."""
    _skip(dev)
    from mxserve.config import EngineArgs
    from mxserve.engine.engine import LLMEngine
    from mxserve.engine.request import SamplingParams
    path, w, toks, _ = base
    args = EngineArgs(model=str(path), device=dev, dtype=dtype, num_gpu_blocks=40, cpu_num_blocks=40, max_model_len=256,
                      max_num_seqs=3, max_num_batched_tokens=48, load_format="safetensors", cuda_graph_max_bs=2)
    eng = LLMEngine(args)
    assert not eng.kv.caching  # recurrent layers: no prefix reuse
    prompts = [toks["r1"], toks["r3"], toks["r2"], toks["r5"]]
    outs = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    margin = 1e-3 if dtype == "float32" else 0.25
    for p, o in zip(prompts, outs):
        assert len(o) == 12
        lg = _oracle_model(BASE, w, p + o[:-1])[len(p) - 1:]
        for row, tok in zip(lg, o):
            assert row[tok] >= row.max() - margin * (row.max() - row.min())
    assert eng.kv.num_free() == eng.kv.num_blocks


def test_registered_small_model_runs():
    """The registry's small Tapasun with random weights, by name, as a served model would start."""
    from mxserve.config import EngineArgs
    from mxserve.engine.engine import LLMEngine
    from mxserve.engine.request import SamplingParams
    eng = LLMEngine(EngineArgs(model="tiny-tapasun", device="cpu", dtype="float32", num_gpu_blocks=16, cpu_num_blocks=16,
                               max_model_len=128, max_num_seqs=2, max_num_batched_tokens=64))
    outs = eng.generate([[1, 2, 3, 4, 5], [7] * 20], SamplingParams(max_tokens=5, temperature=0.0, ignore_eos=True))
    assert [len(o) for o in outs] == [5, 5]


def test_trace_runner_command_line(base, tmp_path):
    """bin/trace_run as a user starts it: steps on stdin, `done <step>` after each, logits files for the
    steps that want some, pages and slots given back under --max-tokens."""
    import json
    import os
    import subprocess
    import sys
    path, _, toks, want = base
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    t = toks["r1"]
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": t[:20], "want": [0, 19]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": t[20:22], "want": []}, {"id": "y", "tokens": toks["r2"], "want": [0]}],
              "end": ["y"]},
             {"step": 2, "entries": [{"id": "x", "tokens": t[22:], "want": [len(t) - 23]}], "end": ["x"]}]
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(path), "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "128", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    V = BASE["vocab"]
    a = np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, V)
    b = np.fromfile(out / "1.f32", dtype="<f4").reshape(-1, V)
    c = np.fromfile(out / "2.f32", dtype="<f4").reshape(-1, V)
    _check(a.astype(np.float64), want["r1"][[0, 19]], 1e-4)
    _check(b.astype(np.float64), want["r2"][[0]], 1e-4)
    _check(c.astype(np.float64), want["r1"][[len(t) - 1]], 1e-4)
