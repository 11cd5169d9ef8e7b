"""Voletar through the engine (paged K/V, state slots, forced and scheduled steps) against the plain
float64 oracle of tests/voletar_oracle.py: on the CPU forms of the ops here, on the HIP kernels
under `-m gpu`.  Every test makes its own small configuration and random checkpoint."""
import types

import numpy as np
import pytest
import torch

from tests import voletar_oracle as vo
from tests.voletar_utils import BASE, config, cut, engine, lightning, parallel, rel_err, replay, write_checkpoint

DEVS = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


def _skip(dev):
    if dev == "cuda" and not torch.cuda.is_available():
        pytest.skip("no GPU")


def _tokens(n, vocab, seed):
    return np.random.default_rng(seed).integers(0, vocab, n).tolist()


def _check(got, want, tol):
    e = rel_err(got, want)
    assert e < tol, f"relative error {e:.3g} >= {tol}"


# ----------------------------------------------------------------------------- mechanisms alone
def _mixer_setup(kind, mc, width, dev, seed=0):
    from mxserve.models.mixers import build_mixer
    m = build_mixer(kind, "m.", width, mc)
    g = torch.Generator().manual_seed(seed)
    shapes = {name: (rows, width) for name, rows in m.proj_rows()}
    shapes.update(m.extra_shapes())
    w = {k: torch.randn(s, generator=g) * (s[-1] ** -0.5 if len(s) > 1 else 1.0) for k, s in shapes.items()}
    return m, w


def _run_mixer(m, w, h, dev, portions, bs=16, slot=2):
    """The mixer over one sequence cut into portions, through paged K/V and a state slot."""
    from mxserve.models.mixers import StepContext
    wt = {k: v.to(dev) for k, v in w.items()}
    w_in = torch.cat([wt[name] for name, _ in m.proj_rows()])
    if hasattr(m, "finish_weights"):
        m.finish_weights(wt)
    T = h.shape[0]
    nb = -(-T // bs) + 3
    voff = m.kv_heads * bs * m.dk
    cache = torch.randn(nb, voff + m.kv_heads * bs * m.dv + 16, device=dev)
    state = torch.randn(4, m.state_floats + 7, device=dev)
    blocks = torch.randperm(nb)[:-(-T // bs)].to(torch.int32)
    outs, at, i = [], 0, 0
    while at < T:
        n = min(portions[min(i, len(portions) - 1)], T - at)
        i += 1
        pos = torch.arange(at, at + n)
        md = types.SimpleNamespace(
            slot_mapping=(blocks[pos // bs].long() * bs + pos % bs).to(dev), block_tables=blocks[None].to(dev),
            query_start_loc=torch.tensor([0, n], dtype=torch.int32, device=dev),
            seq_lens=torch.tensor([at + n], dtype=torch.int32, device=dev), max_query_len=n,
            state_rows=torch.tensor([slot], dtype=torch.int32, device=dev))
        ctx = StepContext(md=md, cache=cache, state=state, block_size=bs, eps=1e-5)
        hp = h[at:at + n].to(dev)
        y = hp @ w_in.T
        parts, c = [], 0
        for _, rows in m.proj_rows():
            parts.append(y[:, c:c + rows])
            c += rows
        out = m.forward(parts, hp, wt, ctx, 0, voff, 5)
        outs.append(out if isinstance(out, tuple) else (out,))
        at += n
    return [torch.cat([o[i] for o in outs]).double().cpu().numpy() for i in range(len(outs[0]))]


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("portions", [[1000], [1], [2], [5, 1, 9, 2, 30]])
def test_each_mixer_alone(dev, portions):
    _skip(dev)
    width, T = 96, 70
    h = torch.randn(T, width, generator=torch.Generator().manual_seed(1))
    hn = h.double().numpy()
    eps = 1e-5
    lc = lightning(heads=3, dim=24, vdim=40)["mixer"]
    m, w = _mixer_setup("lightning", lc, width, dev)
    wn = {k: v.double().numpy() for k, v in w.items()}
    _check(_run_mixer(m, w, h, dev, portions)[0], vo.lightning_mixer(hn, wn, "m.", lc, eps), 1e-4)
    pc = parallel(heads=4, kv_heads=2, dim=24, vdim=40, size=11, keep=3, rheads=2, rdim=40, rvdim=24)["mixer"]
    m, w = _mixer_setup("parallel", pc, width, dev)
    w["m.right.i.b"] += 1.0
    wn = {k: v.double().numpy() for k, v in w.items()}
    a, b = _run_mixer(m, w, h, dev, portions)
    _check(a, vo.window_attention(hn, wn, "m.left.", pc["left"]), 1e-4)
    _check(b, vo.mlstm_mixer(hn, wn, "m.right.", pc["right"], eps), 1e-4)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("size,keep,target,seen", [(8, 0, 33, True), (8, 0, 32, False), (8, 4, 3, True), (8, 4, 4, False),
                                                   (1000, 0, 1, True), (1, 0, 39, False), (1, 2, 1, True),
                                                   # the window's first key is a page's first token; the one before it is the previous page's last
                                                   (9, 0, 32, True), (9, 0, 31, False), (1000, 0, 15, True), (1000, 0, 16, True)])
def test_one_key_stands_out(dev, size, keep, target, seen):
    """One key far back matches the last query so strongly that the output is that key's value when
    the mask lets it through: the window's edge, the kept first tokens and a far key each decide the
    result, in a whole prompt and when the last token is decoded alone."""
    _skip(dev)
    T, width = 41, 16
    mc = {"heads": 1, "kv_heads": 1, "dim": width, "vdim": width, "scale": 1.0, "mask": {"size": size, "keep_first": keep}}
    from mxserve.models.mixers import build_mixer
    m = build_mixer("parallel", "m.", width, {"left": mc, "right": {"heads": 1, "dim": 8, "vdim": 8, "gate_cap": 5.0}}).left
    eye = torch.eye(width)
    wq = eye.clone()
    wq[[3, 5]] = wq[[5, 3]]  # the query reads coordinate 3 as 5: the last token does not match itself
    w = {"m.left.q": wq, "m.left.k": eye, "m.left.v": eye, "m.left.o": eye}
    g = torch.Generator().manual_seed(5)
    h = 0.1 * torch.randn(T, width, generator=g)
    h[target, 5] += 6.0
    h[T - 1] = 0.0
    h[T - 1, 3] = 6.0
    want = vo.window_attention(h.double().numpy(), {k: v.double().numpy() for k, v in w.items()}, "m.left.", mc)
    hit = np.abs(want[T - 1] - h[target].double().numpy()).max() < 0.05
    assert hit == seen  # the oracle itself shows the case
    for portions in ([T], [T - 1, 1], [7, 2, 16, 3, 1]):
        got = _run_mixer(m, dict(w), h, dev, portions)[0]
        assert np.abs(got - want).max() < 1e-4


# ----------------------------------------------------------------------------- whole models, schedules
@pytest.fixture(scope="module")
def base(tmp_path_factory):
    path = tmp_path_factory.mktemp("voletar_base")
    w = write_checkpoint(path, BASE, seed=11)
    toks = {f"r{i}": _tokens(n, BASE["vocab"], 20 + i) for i, n in enumerate([90, 37, 1, 64, 130, 16])}
    want = {rid: vo.forward(BASE, w, t) for rid, t in toks.items()}
    return path, w, toks, want


@pytest.mark.parametrize("dev,dtype,tol", [("cpu", "float32", 1e-4), pytest.param("cuda", "float32", 1e-4, marks=pytest.mark.gpu),
                                           pytest.param("cuda", "bfloat16", 0.12, marks=pytest.mark.gpu)])
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


@pytest.mark.parametrize("dev,dtype,tol", [("cpu", "float32", 1e-4), pytest.param("cuda", "float32", 1e-4, marks=pytest.mark.gpu),
                                           pytest.param("cuda", "bfloat16", 0.12, marks=pytest.mark.gpu)])
def test_long_decoding(base, dev, dtype, tol):
    """A short prompt, then well over a hundred tokens one by one: the windows slide off the prompt and
    over decoded tokens, pages fill and new ones start, the recurrent state is carried all the way."""
    _skip(dev)
    path, _, toks, want = base
    eng = engine(path, dev, dtype, max_tokens=192, eager=(dev == "cpu"))
    steps = [[("a", p, False)] for p in cut(toks["r4"], [10, 1])]
    steps[-1] = [("a", steps[-1][0][1], True)]
    got = replay(eng, steps)["a"]
    _check(got[8:], want["r4"][8:], tol)
    assert eng.kv.num_free() == eng.kv.num_blocks


@pytest.mark.parametrize("dev,dtype,tol", [("cpu", "float32", 1e-4), pytest.param("cuda", "float32", 1e-4, marks=pytest.mark.gpu),
                                           pytest.param("cuda", "bfloat16", 0.12, marks=pytest.mark.gpu)])
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
    for r in toks:  # bf16: a sequence's very first tokens round coarsely (one key, near-ties in the mLSTM's max)
        if len(toks[r]) > 8:
            _check(got[r][8:], want[r][8:], tol)
        _check(got[r][:8], want[r][:8], tol if dtype == "float32" else 0.6)
    assert eng.kv.num_free() == eng.kv.num_blocks and not eng.runner._row_of


VARIANTS = {
    "one_kv_head_no_loop": config([parallel(heads=4, kv_heads=1, dim=32, vdim=32, size=9, keep=2, rheads=1, rdim=16, rvdim=16),
                                   lightning(heads=1, dim=16, vdim=16, ff=64)], width=64, vocab=96, softcap=None),
    "window_of_one_loop_from_zero": config([parallel(heads=2, kv_heads=2, dim=8, vdim=24, size=1, keep=0, rheads=2, rdim=8,
                                                     rvdim=8, ff=None), lightning(heads=2, dim=8, vdim=8)],
                                           width=48, vocab=80, loop=(0, 2, 2)),
    "single_pass_loop_at_the_end": config([lightning(heads=2, dim=40, vdim=8, ff=96), parallel(size=1000, keep=7)],
                                          width=80, vocab=64, loop=(1, 2, 1), softcap=3.0),
    "keeps_more_than_the_window": config([parallel(heads=6, kv_heads=3, dim=16, vdim=8, size=3, keep=12, ff=48)], width=72,
                                         vocab=50),
}


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("name", list(VARIANTS))
def test_other_sizes(tmp_path, dev, name):
    _skip(dev)
    cfg = VARIANTS[name]
    w = write_checkpoint(tmp_path, cfg, seed=5)
    t = _tokens(45, cfg["vocab"], 6)
    want = vo.forward(cfg, w, t)
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
    ref = []
    vo.forward(BASE, w, toks["r1"], ref)
    assert len(tap) == len(ref) == 2 + 2 * 3
    for a, b in zip(tap, ref):
        assert np.abs(a.double().cpu().numpy() - b).max() < 1e-3 * max(1.0, np.abs(b).max())


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
        lg = vo.forward(BASE, w, p + o[:-1])[len(p) - 1:]
        for row, tok in zip(lg, o):
            assert row[tok] >= row.max() - margin * (row.max() - row.min())
    assert eng.kv.num_free() == eng.kv.num_blocks


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
