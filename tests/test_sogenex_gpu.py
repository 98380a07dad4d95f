"""The Sogenex decoder on the GPU against the plain implementation (tests/plain_sogenex.py): every mechanism
alone at the level of its kernels, then whole models of three tiny configurations through the engine's step
function (whole prompts, tails decoded one by one, portions down to two tokens, mixed batches with pages and
slots used again), standout keys at the window's edge and far away, long memory of the recurrence across
portions, long decoding through recorded steps, and greedy generation through the entry point."""
import copy
import math
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import helpers
import plain_sogenex as plain
import schedules
import sogenex_cases as cases

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {"float32": 2e-5, "bfloat16": 3e-2}
LENGTHS = [5, 17, 33, 70, 150, 41, 64, 2, 1]
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def row_errs(got, ref):
    return np.abs(got.astype(np.float64) - ref).max(axis=-1) / np.abs(ref).max()


def check_rows(out, ref, dt, what):
    """float32: every row within the limit.  bfloat16: nine rows in ten (a router's choice between two experts whose
    logits differ by less than the rounding may fall the other way, and moves that token's rows)."""
    e = np.concatenate([row_errs(out[r], ref[r]) for r in ref])
    worst, q90 = float(e.max()), float(np.quantile(e, 0.9))
    print(f"[observed] {what} {dt}: worst {worst:.3e}, nine in ten below {q90:.3e}")
    assert (worst if dt == "float32" else q90) < TOL[dt], (what, dt, worst, q90)
    assert np.isfinite(e).all()


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, (cfg, page, seed) in cases.CASES.items():
        w = cases.draw_weights(cfg, seed)
        for dt in ("float32", "bfloat16"):
            d = cases.write_model(tmp_path_factory.mktemp(f"s{name}{dt}"), cfg, w, DT[dt])
            reqs = helpers.random_requests(cfg["vocab"], LENGTHS, seed + 10)
            wd = cases.stored(w, DT[dt])
            out[(name, dt)] = (d, reqs, {r: plain.forward(cfg, wd, t) for r, t in reqs.items()})
    return out


def _engine(d, dt, page, max_tokens, **kw):
    from litinfer_amd.engine import Engine
    return Engine.from_dir(d, dtype=dt, device=DEV, page_size=page, max_tokens=max_tokens, max_seqs=4,
                           page_order_seed=5, **kw)


# ------------------------------------------------------------------------------------------ whole models
@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(cases.CASES))
@pytest.mark.parametrize("kind", ["whole", "tail", "chunks", "mixed"])
def test_schedules_match_the_plain_implementation(models, name, dt, kind):
    cfg, page, _ = cases.CASES[name]
    d, reqs, ref = models[(name, dt)]
    steps = getattr(schedules, kind)(reqs)
    eng = _engine(d, dt, page, schedules.max_live_tokens(reqs, steps, page if kind == "mixed" else 64))
    out = schedules.run(eng, reqs, steps)
    eng.cache.check_invariants()
    assert all(f == g.pool.capacity for f, g in zip(eng.cache.free_pages(), eng.cache.groups))
    assert eng.cache.free_slots() == 4
    if kind == "mixed":
        assert all(g.pool.total_allocations > g.pool.capacity for g in eng.cache.groups), "no page was used again"
    check_rows(out, ref, dt, f"{name} {kind}")


@pytest.mark.parametrize("name", list(cases.CASES))
def test_float32_logits_do_not_depend_on_the_schedule(models, name):
    cfg, page, _ = cases.CASES[name]
    d, reqs, _ = models[(name, "float32")]
    outs = {}
    for kind in ("whole", "tail", "chunks", "mixed"):
        steps = getattr(schedules, kind)(reqs)
        outs[kind] = schedules.run(_engine(d, "float32", page, schedules.max_live_tokens(reqs, steps)), reqs, steps)
    for kind in ("tail", "chunks", "mixed"):
        for r in reqs:
            assert schedules.rel_err(outs[kind][r], outs["whole"][r].astype(np.float64)) < 2e-5, (kind, r)


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["recurrent only", "attention only"])
def test_models_of_one_kind_of_mixer(tmp_path, dt, kind):
    """No page group at all (every layer keeps state of fixed size only), and no state at all (recorded steps are then
    filled up with copies of their last entry): the mixed schedule with eight requests on four slots, and decoding."""
    if kind == "recurrent only":
        layers = [cases.mamba_layer(2, 20, 12, 2, 3, 1, cases.moe(3, 2, 24, 0)), cases.mamba_layer(4, 8, 40, 1, 1, 2, None),
                  cases.mamba_layer(2, 20, 12, 2, 3, 1, cases.moe(3, 2, 24, 0), weights_of=0)]
    else:
        layers = [cases.attention_layer(2, 1, 8, 24, 9, 0.0, 0.3, cases.moe(2, 1, 16, 8)), cases.attention_layer(3, 3, 10, 6, 1, 0.5, 0.3, None)]
    cfg = {"architecture": "Sogenex", "vocab": 50, "width": 40, "norm": {"eps": 1e-6}, "logit_softcap": 5.0, "layers": layers}
    w32 = cases.draw_weights(cfg, 12)
    d = cases.write_model(tmp_path / "m", cfg, w32, DT[dt])
    w = cases.stored(w32, DT[dt])
    reqs = helpers.random_requests(50, [9, 30, 70, 3, 1, 25, 12, 40], 6)
    ref = {r: plain.forward(cfg, w, t) for r, t in reqs.items()}
    for name in ("mixed", "tail"):
        steps = getattr(schedules, name)(reqs)
        eng = _engine(d, dt, 8, schedules.max_live_tokens(reqs, steps, 8 if name == "mixed" else 64))
        assert len(eng.cache.groups) == (0 if kind == "recurrent only" else 2) and eng.cache.has_state == (kind == "recurrent only")
        out = schedules.run(eng, reqs, steps)
        eng.cache.check_invariants()
        check_rows(out, ref, dt, f"{kind} {name}")
    from litinfer_amd.engine import Engine, StepEntry
    # six requests decoding together: recorded steps of six, filled to eight where no mixer keeps state
    eng = Engine.from_dir(d, dtype=dt, device=DEV, page_size=8, max_tokens=512, max_seqs=8)
    rids = list(reqs)[:6]
    for r in rids:
        eng.step([StepEntry(r, reqs[r][:1], [])])
    got = {r: [] for r in rids}
    for i in range(1, 9):
        live = [r for r in rids if len(reqs[r]) > i]
        if not live:
            break
        out = eng.step([StepEntry(r, [reqs[r][i]], [0]) for r in live]).float().cpu().numpy()
        for r, row in zip(live, out):
            got[r].append(row.copy())
    for r in rids:
        if got[r]:
            check_rows({r: np.stack(got[r])}, {r: ref[r][1:1 + len(got[r])]}, dt, f"{kind} decoding together {r}")


def test_layers_that_share_tensors_keep_caches_and_states_of_their_own(models):
    from litinfer_amd.config import load_config
    d, _, _ = models[("A", "float32")]
    _, cfg, spec = load_config(d)
    assert [e.layer for e in spec.order] == [0, 1, 2, 0, 1] and len(spec.layers) == 3
    eng = _engine(d, "float32", 8, 256)
    views = [eng.cache.view(i) for i in range(5)]
    assert views[0].states["ssm"].data_ptr() != views[3].states["ssm"].data_ptr()
    assert views[1].tensors["k1"].data_ptr() != views[4].tensors["k1"].data_ptr()
    assert views[1].group == views[4].group and views[2].states["ssm"].shape[1:] == (3, 8, 40)


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_long_decoding_through_recorded_steps(models, dt):
    """A short prompt, then 150 tokens one by one, now with and now without wanted logits (two shapes of recorded
    steps): the window passes, pages go back, the states move once a step."""
    cfg, page, _ = cases.CASES["A"]
    d, _, _ = models[("A", dt)]
    toks = helpers.random_requests(cfg["vocab"], [160], 77)["r0"]
    w = cases.stored(cases.draw_weights(cfg, cases.CASES["A"][2]), DT[dt])
    ref = plain.forward(cfg, w, toks)
    from litinfer_amd.engine import StepEntry
    eng = _engine(d, dt, page, 256)
    eng.step([StepEntry("a", toks[:10], [])])
    rows, at = [], []
    for i in range(10, 160):
        r = eng.step([StepEntry("a", [toks[i]], [0] if i % 3 else [])])
        if r is not None:
            rows.append(r.float().cpu().numpy().copy())
            at.append(i)
        held = [g.pool.capacity - f for g, f in zip(eng.cache.groups, eng.cache.free_pages())]
        assert all(h <= -(-g.need.window // page) + 1 for g, h in zip(eng.cache.groups, held))
    assert eng.graph_replays > 100 and eng.graphs_recorded >= 2
    check_rows({"a": np.concatenate(rows)}, {"a": ref[at]}, dt, "long decoding")
    eng.finish("a")
    eng.cache.check_invariants()


def test_a_state_slot_that_is_used_again_starts_from_zero(models):
    cfg, page, _ = cases.CASES["B"]
    d, reqs, ref = models[("B", "float32")]
    from litinfer_amd.engine import StepEntry
    eng = _engine(d, "float32", page, 512)
    for rid in ("r3", "r4", "r2", "r3"):                           # the one slot in use is the same every time
        t = reqs[rid]
        out = eng.step([StepEntry("x", t, list(range(len(t))))]).float().cpu().numpy()
        eng.finish("x")
        assert schedules.rel_err(out, ref[rid]) < TOL["float32"]


def test_greedy_generation_through_the_entry_point(models):
    from litinfer_amd import models as entry
    cfg, page, seed = cases.CASES["A"]
    d, reqs, _ = models[("A", "float32")]
    w = cases.stored(cases.draw_weights(cfg, seed), torch.float32)
    lm = entry.load(d, dtype="float32", device=DEV, page_size=page, max_tokens=512, max_seqs=4)
    prompt = reqs["r1"]
    new = list(lm.generate(prompt, max_new_tokens=12, top_k=1, top_p=1.0, temperature=1.0))
    assert len(new) == 12
    seq = list(prompt)
    for t in new:
        logits = plain.forward(cfg, w, seq)[-1]
        top = np.argsort(logits)[::-1]
        assert t == top[0] or logits[top[0]] - logits[t] < 1e-4 * np.abs(logits).max(), (len(seq), t, top[:3])
        seq.append(int(t))


def test_several_requests_through_the_scheduler(models):
    """Continuous batching of five prompts on four state slots: each request's greedy tokens are those of the
    request alone."""
    from litinfer_amd import models as entry
    cfg, page, seed = cases.CASES["B"]
    d, reqs, _ = models[("B", "float32")]
    lm = entry.load(d, dtype="float32", device=DEV, page_size=page, max_tokens=1024, max_seqs=4)
    prompts = [reqs[r] for r in ("r0", "r1", "r2", "r5", "r7")]
    alone = [list(lm.generate(p, max_new_tokens=8)) for p in prompts]
    lm.engine_start()
    ids = [lm.engine_add_request(p, 8) for p in prompts]
    while lm.engine_has_unfinished():
        lm.engine_step()
    got = {i: list(lm.engine_get_output(i)) for i in ids}
    assert [got[i] for i in ids] == alone


# --------------------------------------------------------------------------- standout keys and long memory
def _standout_model(tmp, window, dt, page_tokens=8):
    """One attention layer (and a recurrent one behind it) whose weights make ONE key win: token A's key of map 1
    scores e^14 with token B's query, and A's value is large.  Whether B sees A decides B's logits."""
    cfg = {"architecture": "Sogenex", "vocab": 64, "width": 64, "norm": {"eps": 1e-6}, "logit_scale": 1.0,
           "layers": [cases.attention_layer(4, 2, 16, 24, window, 0.2, 0.25, None),
                      cases.mamba_layer(2, 16, 16, 1, 2, 1, None)]}
    w = cases.draw_weights(cfg, 5)
    A, B, W = 63, 62, 64
    w["embed"][:, :2] = 0.0
    w["embed"][A] = 0.0
    w["embed"][B] = 0.0
    amp = 8.0                                                       # (not larger: the attention's output must weigh against it)
    w["embed"][A, 0] = amp
    w["embed"][B, 1] = amp
    w["l0.norm1"][:2] = 0.0
    rng = np.random.default_rng(1)
    normed = amp / math.sqrt((amp * amp + W / 2) / W)               # the standout column behind the norm (the position vector's squares add W / 2)
    c = math.sqrt(14.0 / (normed * normed * 0.25))
    dirs = rng.normal(size=(2, 16))
    dirs /= np.linalg.norm(dirs, axis=1, keepdims=True)
    for g in range(2):
        w["l0.mix.k"][(2 * g) * 16:(2 * g + 1) * 16, 0] = c * dirs[g]               # map 1 of kv head g
        for h in (2 * g, 2 * g + 1):
            w["l0.mix.q"][(2 * h) * 16:(2 * h + 1) * 16, 1] = c * dirs[g]
    w["l0.mix.v"][:, 0] = rng.normal(0.0, 3.0, w["l0.mix.v"].shape[0])
    d = cases.write_model(tmp, cfg, w, DT[dt])
    return cfg, cases.stored(w, DT[dt]), d, A, B


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("how", ["prompt", "portions", "decoded"])
def test_a_key_just_inside_and_just_outside_the_window(tmp_path, dt, how):
    window, page = 21, 8
    cfg, w, d, A, B = _standout_model(tmp_path / "m", window, dt)
    from litinfer_amd.engine import StepEntry
    rng = np.random.default_rng(3)
    seen = []
    for pa in (7, 8, 15, 16, 30):                                    # the key at the last and first row of a page, and elsewhere
        for gap in (window - 1, window):                             # the last position that sees it, the first that does not
            toks = rng.integers(0, 60, pa + gap + 4).tolist()
            toks[pa], toks[pa + gap] = A, B
            ref = plain.forward(cfg, w, toks)
            eng = _engine(d, dt, page, 128)
            n = len(toks)
            if how == "prompt":
                out = eng.step([StepEntry("a", toks, list(range(n)))]).float().cpu().numpy()
            elif how == "portions":                                  # a cut between the key and the query, and one right at the query
                cuts = [0, pa + 1, pa + gap, pa + gap + 2, n]
                out = np.concatenate([eng.step([StepEntry("a", toks[a:b], list(range(b - a)))]).float().cpu().numpy()
                                      for a, b in zip(cuts, cuts[1:]) if b > a])
            else:
                head = pa + 3
                rows = [eng.step([StepEntry("a", toks[:head], list(range(head)))]).float().cpu().numpy()]
                rows += [eng.step([StepEntry("a", [toks[i]], [0])]).float().cpu().numpy().copy() for i in range(head, n)]
                out = np.concatenate(rows)
            e = schedules.rel_err(out, ref)
            assert e < TOL[dt], (pa, gap, e)
            seen.append(ref[pa + gap])
    # the test has teeth: whether the key is seen moves the query's logits by far more than the tolerance
    for inside, outside in zip(seen[::2], seen[1::2]):
        assert np.abs(inside - outside).max() > 0.1 * np.abs(inside).max()


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_a_far_key_among_hundreds(tmp_path, dt):
    cfg, w, d, A, B = _standout_model(tmp_path / "m", 0, dt)
    from litinfer_amd.engine import StepEntry
    rng = np.random.default_rng(4)
    toks = rng.integers(0, 60, 420).tolist()
    toks[3], toks[400] = A, B
    ref = plain.forward(cfg, w, toks)
    other = list(toks)
    other[3] = 5
    assert np.abs(plain.forward(cfg, w, other)[400] - ref[400]).max() > 0.1 * np.abs(ref[400]).max()
    for cuts in ([0, 420], [0, 390, 420], [0, 2, 5, 399, 401, 420]):
        eng = _engine(d, dt, 16, 512)
        out = np.concatenate([eng.step([StepEntry("a", toks[a:b], list(range(b - a)))]).float().cpu().numpy()
                              for a, b in zip(cuts, cuts[1:])])
        assert schedules.rel_err(out[395:], ref[395:]) < TOL[dt], cuts
    eng = _engine(d, dt, 16, 512)
    eng.step([StepEntry("a", toks[:398], [])])
    out = np.concatenate([eng.step([StepEntry("a", [toks[i]], [0])]).float().cpu().numpy().copy() for i in range(398, 404)])
    assert schedules.rel_err(out, ref[398:404]) < TOL[dt]


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_the_recurrence_remembers_across_portions_and_chunks(tmp_path, dt):
    """Half of the heads forget less than a hundredth a token: what a token did 300 positions back still shows, so a
    state that is lost or doubled at the edge of a portion, of a chunk of 64 tokens or at the first decoded token
    moves every later row."""
    cfg = {"architecture": "Sogenex", "vocab": 97, "width": 64, "norm": {"eps": 1e-6},
           "layers": [cases.mamba_layer(4, 16, 32, 2, 4, 2, cases.moe(4, 2, 32, 32)), cases.mamba_layer(2, 48, 20, 2, 3, 1, None)]}
    w32 = cases.draw_weights(cfg, 9, long_memory=True)
    d = cases.write_model(tmp_path / "m", cfg, w32, DT[dt])
    w = cases.stored(w32, DT[dt])
    from litinfer_amd.engine import StepEntry
    toks = np.random.default_rng(8).integers(0, 97, 330).tolist()
    ref = plain.forward(cfg, w, toks)
    changed = list(toks)
    changed[2] = (toks[2] + 1) % 97
    assert np.abs(plain.forward(cfg, w, changed)[320:] - ref[320:]).max() > 1e-3 * np.abs(ref).max()
    for cuts in ([0, 330], [0, 64, 128, 330], [0, 63, 65, 129, 130, 132, 300, 330], [0, 1, 3, 200, 330]):
        eng = _engine(d, dt, 16, 512)
        out = np.concatenate([eng.step([StepEntry("a", toks[a:b], list(range(b - a)))]).float().cpu().numpy()
                              for a, b in zip(cuts, cuts[1:])])
        check_rows({"a": out}, {"a": ref}, dt, f"portions {cuts}")
    eng = _engine(d, dt, 16, 512)
    rows = [eng.step([StepEntry("a", toks[:290], list(range(290)))]).float().cpu().numpy()]
    rows += [eng.step([StepEntry("a", [toks[i]], [0])]).float().cpu().numpy().copy() for i in range(290, 330)]
    check_rows({"a": np.concatenate(rows)}, {"a": ref}, dt, "decoded behind a long prompt")


# ------------------------------------------------------------------------------------------ mechanisms alone
def _ctx(q_lens, slots):
    q_len = np.asarray(q_lens, dtype=np.int32)
    q_start = np.concatenate([[0], np.cumsum(q_len)[:-1]]).astype(np.int32)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.int32)).to(DEV)
    return SimpleNamespace(num_tokens=int(q_len.sum()), num_segments=len(q_len), host_state_slots=np.asarray(slots, dtype=np.int32),
                           seg_of_token=dev(np.repeat(np.arange(len(q_len)), q_len)), q_start=dev(q_start), q_len=dev(q_len),
                           state_slots=dev(slots), max_q_len=int(q_len.max()))


@pytest.mark.parametrize("taps,C", [(4, 37), (2, 300), (7, 64), (4, 128), (3, 72)])
def test_causal_convolution_with_its_tail_across_steps(taps, C):
    from litinfer_amd.kernels import ops
    rng = np.random.default_rng(taps)
    w, b = rng.normal(size=(C, taps)), rng.normal(size=C)
    seqs = {0: rng.normal(size=(140, C)), 2: rng.normal(size=(124, C))}            # by state slot
    ref = {s: plain.silu(plain.causal_conv(u, w, b)) for s, u in seqs.items()}
    tail = torch.zeros(3, taps - 1, C, device=DEV)
    tail[1] = 7.0                                                                  # a slot nobody uses stays as it is
    wd, bd = torch.tensor(w, dtype=torch.float32, device=DEV), torch.tensor(b, dtype=torch.float32, device=DEV)
    at = {0: 0, 2: 0}
    # (slot, tokens); the last step has rows enough for the form with four channels a thread, where the sizes allow it
    for k, step in enumerate(([(0, 1), (2, 5)], [(2, 1), (0, 2)], [(0, 1)], [(0, 20), (2, 2)], [(2, 15), (0, 16)], [(2, 100), (0, 1), ], [(0, 99), (2, 1)])):
        u = np.concatenate([seqs[s][at[s]:at[s] + n] for s, n in step])
        lead, extra = (4, 8) if k >= 5 else (3, 5)                                  # the rows are a view with a stride
        wide = torch.zeros(len(u), C + extra, device=DEV)
        wide[:, lead:lead + C] = torch.tensor(u, dtype=torch.float32)
        out = torch.empty(len(u), C, device=DEV)
        ops.causal_conv_silu(wide[:, lead:lead + C], wd, bd, tail, _ctx([n for _, n in step], [s for s, _ in step]), out)
        o = 0
        for s, n in step:
            np.testing.assert_allclose(out[o:o + n].cpu().numpy(), ref[s][at[s]:at[s] + n], rtol=2e-5, atol=2e-5)
            at[s] += n
            o += n
    assert bool((tail[1] == 7.0).all())


@pytest.mark.parametrize("heads,vdim,N,G", [(4, 16, 24, 2), (2, 64, 128, 1), (3, 40, 8, 3), (2, 32, 160, 2), (8, 32, 32, 2), (1, 8, 256, 1),
                                            (2, 30, 20, 1), (4, 7, 130, 2), (1, 128, 64, 1)])     # (head sizes that are no multiple of 4: one column a lane)
def test_state_space_recurrence_in_one_pass_in_chunks_and_across_steps(heads, vdim, N, G):
    from litinfer_amd.kernels import ops
    rng = np.random.default_rng(N + vdim)
    inner = heads * vdim
    A_log, D, dt_bias = rng.uniform(-5, 0.5, heads), rng.normal(1, 0.3, heads), rng.normal(0, 0.5, heads)
    L = {0: 200, 1: 70}
    raw = {s: (rng.normal(size=(n, inner)), rng.normal(size=(n, G * N)), rng.normal(size=(n, G * N)), rng.normal(size=(n, heads)))
           for s, n in L.items()}
    ref = {s: plain.ssm_scan(x, B, C, plain.softplus(dt + dt_bias), A_log, D, heads, vdim, G, N) for s, (x, B, C, dt) in raw.items()}
    f32 = lambda a: torch.tensor(a, dtype=torch.float32, device=DEV)
    state = torch.zeros(2, heads, N, vdim, device=DEV)
    from litinfer_amd.engine.workspace import Workspace
    ws = Workspace(DEV)
    at = {0: 0, 1: 0}
    # a decoded token beside a portion of three chunks; a portion that ends inside a chunk; single tokens; the rest
    for step in ([(0, 1), (1, 3)], [(1, 1), (0, 130)], [(0, 64)], [(1, 1)], [(1, 65), (0, 5)]):
        xbc = np.concatenate([np.concatenate([raw[s][0], raw[s][1], raw[s][2]], axis=1)[at[s]:at[s] + n] for s, n in step])
        dt = np.concatenate([raw[s][3][at[s]:at[s] + n] for s, n in step])
        y = torch.empty(len(xbc), inner, device=DEV)
        ops.ssm_scan(f32(xbc), f32(dt), f32(dt_bias), f32(A_log), f32(D), state, _ctx([n for _, n in step], [s for s, _ in step]),
                     y, heads, vdim, N, G, ws)
        o = 0
        for s, n in step:
            r = ref[s][at[s]:at[s] + n]
            assert np.abs(y[o:o + n].cpu().numpy() - r).max() < 3e-5 * max(1.0, np.abs(ref[s]).max()), (step, s)
            at[s] += n
            o += n


def test_gated_norm_in_groups():
    from litinfer_amd.kernels import ops
    rng = np.random.default_rng(0)
    for n, groups in ((96, 2), (120, 3), (4608, 2), (64, 1)):
        y, z, w = rng.normal(size=(5, n)), rng.normal(size=(5, n)), rng.normal(1, 0.2, n)
        ref = plain.grouped_rms(y * plain.silu(z), groups, 1e-5) * w
        for dt, tol in ((torch.float32, 1e-5), (torch.bfloat16, 1e-2)):
            out = torch.empty(5, n, dtype=dt, device=DEV)
            ops.gated_group_norm(torch.tensor(y, dtype=torch.float32, device=DEV), torch.tensor(z, dtype=torch.float32, device=DEV),
                                 torch.tensor(w, dtype=torch.float32, device=DEV), 1e-5, groups, out)
            assert np.abs(out.float().cpu().numpy() - ref).max() < tol * np.abs(ref).max()


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,K,E,top,ff,shared", [(1, 96, 5, 2, 40, 56), (70, 128, 8, 2, 64, 128), (300, 64, 3, 3, 48, 0),
                                                 (33, 256, 64, 6, 96, 0), (9, 128, 4, 1, 72, 24), (2200, 256, 4, 2, 160, 0),
                                                 (40, 512, 6, 2, 48, 0), (1500, 128, 4, 2, 192, 64), (600, 128, 8, 2, 96, 0)])
def test_routed_feed_forward(dt, T, K, E, top, ff, shared):
    """The part itself (router, plan, products by tile, weighted sum, gated shared expert) against the plain one, on
    tokens whose choice of experts is not a close call for the rounding of the engine's dtype."""
    from litinfer_amd.config.spec import PartSpec
    from litinfer_amd.engine.workspace import Workspace
    from litinfer_amd.parts.base import Runtime, build_part
    from litinfer_amd.parts.stream import ResidualStream
    rng = np.random.default_rng(T + E)
    tdt = DT[dt]
    rnd = lambda a: torch.tensor(a, dtype=torch.float32).to(tdt)
    w = {"router": rng.normal(0, 1 / math.sqrt(K), (E, K)), "router.b": rng.normal(0, 0.1, E)}
    for e in range(E):
        w[f"e{e}.up"], w[f"e{e}.down"] = rng.normal(0, 1 / math.sqrt(K), (ff, K)), rng.normal(0, 1 / math.sqrt(ff), (K, ff))
    if shared:
        w["shared.up"], w["shared.down"] = rng.normal(0, 1 / math.sqrt(K), (shared, K)), rng.normal(0, 1 / math.sqrt(shared), (K, shared))
        w["shared.sg"] = rng.normal(0, 1 / math.sqrt(K), (1, K))
    wt = {n: rnd(a) for n, a in w.items()}
    # tokens whose choice is clear: the top-th and the next logit lie further apart than the dtype's rounding moves them
    cand = rnd(rng.normal(size=(8 * T + 8, K)))
    z = np.sort(cand.double().numpy() @ wt["router"].double().numpy().T + wt["router.b"].double().numpy(), axis=-1)[:, ::-1]
    ok = np.ones(len(cand), bool) if top == E else (z[:, top - 1] - z[:, top]) > (1e-4 if dt == "float32" else 3e-2)
    assert ok.sum() >= T
    h = cand[np.nonzero(ok)[0][:T]]
    clear = np.ones(T, bool)
    part = build_part("feed_forward", PartSpec("routed_relu2", "", {"hidden_size": K, "experts": E, "top": top, "intermediate_size": ff,
                                                                     "shared_intermediate_size": shared}),
                      Runtime(torch.device(DEV), tdt))
    part.load_params(lambda n: wt[n])
    x0 = rng.normal(size=(T, K))
    x = torch.tensor(x0, dtype=torch.float32, device=DEV)
    ws = Workspace(DEV)
    part.forward(h.to(DEV), ResidualStream(x, ws), SimpleNamespace(ws=ws))
    w64 = {n: a.double().numpy() for n, a in wt.items()}
    h64 = h.double().numpy()
    ref = x0 + plain.moe(h64, w64, "", {"router": {"top": top}, "shared": {"ff": shared} if shared else None})
    err = np.abs(x.cpu().numpy() - ref)[clear].max() / np.abs(ref - x0).max()
    print(f"[observed] routed feed-forward {dt} {T, K, E, top, ff, shared}: {err:.3e}")
    assert err < (1e-5 if dt == "float32" else 2e-2)
    # the router's own outputs: the chosen experts and their weights
    idx = ws.buffer("moe.idx", (T, top), torch.int32).cpu().numpy()
    wts = ws.buffer("moe.wt", (T, top), torch.float32).cpu().numpy()
    pidx, pw = plain.route(h64, w64["router"], w64["router.b"], top)
    assert (np.sort(idx[clear], axis=1) == np.sort(pidx[clear], axis=1)).all()
    assert np.abs(np.sort(wts[clear], axis=1) - np.sort(pw[clear], axis=1)).max() < (1e-5 if dt == "float32" else 2e-2)


def test_equal_router_logits_take_the_lower_expert():
    from litinfer_amd.kernels import ops
    x = torch.ones(3, 32, device=DEV)
    router = torch.zeros(6, 32, device=DEV)
    router[4] = 0.5                                                 # expert 4 wins; the others tie at their bias
    bias = torch.tensor([0.0, 1.0, 1.0, 0.0, 0.0, 1.0], device=DEV)
    idx = torch.empty(3, 3, dtype=torch.int32, device=DEV)
    wt = torch.empty(3, 3, device=DEV)
    ops.moe_route(x, router, bias, None, idx, wt, None)
    assert idx.cpu().tolist() == [[4, 1, 2]] * 3
    e = np.exp(np.array([16.0, 1.0, 1.0]) - 16.0)
    assert np.allclose(wt.cpu().numpy(), e / e.sum(), atol=1e-6)


def test_difference_of_two_maps_and_its_norm():
    from litinfer_amd.kernels import ops
    rng = np.random.default_rng(2)
    for dv in (16, 96, 200):
        a1, a2 = rng.normal(size=(7, 3 * dv)), rng.normal(size=(7, 3 * dv))
        o = (a1 - 0.37 * a2).reshape(7, 3, dv)
        ref = (plain.rms(o, 1e-5) * 0.8).reshape(7, 3 * dv)
        out = torch.empty(7, 3 * dv, device=DEV)
        ops.diff_combine(torch.tensor(a1, dtype=torch.float32, device=DEV), torch.tensor(a2, dtype=torch.float32, device=DEV),
                         0.37, 1e-5, 0.8, out, dv)
        assert np.abs(out.cpu().numpy() - ref).max() < 1e-5


def test_position_vector_and_capped_logits():
    from litinfer_amd.kernels import ops
    for H in (96, 7):
        pos = np.array([0, 1, 5, 1000, 70000], dtype=np.int32)
        freq = torch.pow(torch.tensor(10000.0, dtype=torch.float64), -2.0 * torch.arange((H + 1) // 2, dtype=torch.float64) / H)
        x = torch.zeros(len(pos), H, device=DEV)
        ops.sinusoid_add(x, torch.from_numpy(pos).to(DEV), freq.float().to(DEV))
        ref = plain.sinusoid(pos, H)
        # (the angle is a float32 product: at position 70000 its rounding alone moves sin and cos by some 1e-3)
        assert np.abs(x.cpu().numpy()[:3] - ref[:3]).max() < 1e-6 and np.abs(x.cpu().numpy() - ref).max() < 5e-3
    v = torch.linspace(-80, 80, 1001, device=DEV)
    ref = 15.0 * np.tanh(v.cpu().numpy().astype(np.float64) * 0.5 / 15.0)
    ops.scale_softcap(v, 0.5, 15.0)
    assert np.abs(v.cpu().numpy() - ref).max() < 1e-5
    u = torch.linspace(-3, 3, 11, device=DEV)
    ops.scale_softcap(u, 2.0, 0.0)
    assert torch.allclose(u, torch.linspace(-6, 6, 11, device=DEV))
