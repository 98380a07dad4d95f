"""The Tovasun decoder on the GPU against the plain implementation (tests/plain_tovasun.py): every
mechanism alone at the level of its kernel, then whole models of several tiny configurations through the
engine's step function (whole prompts, tails decoded one by one, portions down to two tokens, mixed batches
with pages and slots used again), long decoding past every window, and greedy generation through the entry
point and the scheduler."""
import math

import numpy as np
import pytest
import torch

import helpers
import plain_impl
import plain_tovasun as plain
import schedules

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {"float32": 5e-6, "bfloat16": 2.5e-2}


def yarn(factor, original, fast=32.0, slow=1.0):
    return {"factor": factor, "original": original, "fast": fast, "slow": slow}


def attention_layer(heads, kv_heads, dim, vdim, rot_dims, size, keep_first, softcap, scale, ff, scaling=None, base=10000.0):
    rot = {"base": base, "dims": rot_dims}
    if scaling:
        rot["scaling"] = scaling
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": rot, "scale": scale,
         "mask": {"size": size, "keep_first": keep_first}}
    if softcap:
        m["softcap"] = softcap
    return {"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def latent_layer(heads, dim, rot_dim, vdim, rank, size, scale, ff, scaling=None, base=10000.0):
    rot = {"base": base, "dims": rot_dim}
    if scaling:
        rot["scaling"] = scaling
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "rot": rot,
                      "scale": scale, "mask": {"size": size}},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


# P: small odd sizes; the loop starts at layer 0; a layer without feed-forward; value sizes that differ from the key sizes
CONFIG_P = {"architecture": "Tovasun", "vocab": 211, "width": 96, "norm": {"eps": 1e-6},
            "layers": [attention_layer(4, 2, 24, 16, 8, 12, 3, 20.0, 0.2, 136),
                       latent_layer(3, 16, 8, 24, 40, 9, 0.25, 0, scaling=yarn(4.0, 16)),
                       attention_layer(2, 2, 32, 32, 32, 50, 0, 0.0, 0.17, 64, scaling=yarn(2.0, 32, 4.0, 1.0))],
            "loop": {"start": 0, "stop": 2, "times": 2}, "token_side": {"dim": 8}}
PAGE_P = 8
# Q: no loop, no token input; one kv head; a window longer than any request; keep_first larger than a page
CONFIG_Q = {"architecture": "Tovasun", "vocab": 300, "width": 128, "norm": {"eps": 1e-5},
            "layers": [latent_layer(2, 32, 16, 32, 48, 500, 0.144, 256),
                       attention_layer(6, 1, 16, 48, 4, 7, 20, 5.0, 0.25, 192, base=500.0)]}
PAGE_Q = 16
# R: the loop is the whole middle, passed three times; head sizes 64 and 128; one pass-through layer behind it
CONFIG_R = {"architecture": "Tovasun", "vocab": 384, "width": 256, "norm": {"eps": 1e-5},
            "layers": [attention_layer(4, 4, 64, 64, 64, 33, 1, 50.0, 0.125, 512),
                       latent_layer(8, 64, 64, 128, 192, 17, 0.0884, 320, scaling=yarn(16.0, 64)),
                       attention_layer(8, 2, 128, 64, 32, 16, 2, 0.0, 0.0884, 0),
                       latent_layer(1, 128, 32, 64, 64, 64, 0.079, 256)],
            "loop": {"start": 1, "stop": 3, "times": 3}, "token_side": {"dim": 24}}
PAGE_R = 32
CASES = {"P": (CONFIG_P, PAGE_P, 21), "Q": (CONFIG_Q, PAGE_Q, 22), "R": (CONFIG_R, PAGE_R, 23)}
LENGTHS = [5, 17, 33, 70, 100, 41, 64, 2, 1]


def plain_logits(model_dir, requests):
    cfg, w = plain_impl.load_folder(model_dir, np.float64)
    return {rid: plain.forward(toks, w, cfg) for rid, toks in requests.items()}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, (cfg, page, seed) in CASES.items():
        for dt in ("float32", "bfloat16"):
            stored = torch.float32 if dt == "float32" else torch.bfloat16
            d = helpers.make_model(tmp_path_factory.mktemp(f"t{name}{dt}"), cfg, seed, stored)
            reqs = helpers.random_requests(cfg["vocab"], LENGTHS, seed + 10)
            out[(name, dt)] = (d, reqs, plain_logits(d, reqs))
    return out


def _engine(d, dt, page, max_tokens, **kw):
    from litinfer_amd.engine import Engine
    return Engine.from_dir(d, dtype=dt, device=DEV, page_size=page, max_tokens=max_tokens, max_seqs=4,
                           page_order_seed=5, **kw)


# ------------------------------------------------------------------------------------------ whole models
@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CASES))
@pytest.mark.parametrize("kind", ["whole", "tail", "chunks", "mixed"])
def test_schedules_match_the_plain_implementation(models, name, dt, kind):
    cfg, page, _ = CASES[name]
    d, reqs, ref = models[(name, dt)]
    steps = getattr(schedules, kind)(reqs)
    eng = _engine(d, dt, page, schedules.max_live_tokens(reqs, steps, page if kind == "mixed" else 64))
    out = schedules.run(eng, reqs, steps)
    eng.cache.check_invariants()
    assert all(f == g.pool.capacity for f, g in zip(eng.cache.free_pages(), eng.cache.groups))
    assert eng.cache.free_slots() == 4
    if kind == "mixed":
        assert all(g.pool.total_allocations > g.pool.capacity for g in eng.cache.groups), "no page was used again"
    worst = max(schedules.rel_err(out[r], ref[r]) for r in reqs)
    print(f"[observed] {name} {dt} {kind}: {worst:.3e}")
    assert worst < TOL[dt], f"{name} {dt} {kind}: {worst}"


@pytest.mark.parametrize("name", list(CASES))
def test_float32_logits_do_not_depend_on_the_schedule(models, name):
    cfg, page, _ = CASES[name]
    d, reqs, _ = models[(name, "float32")]
    outs = {}
    for kind in ("whole", "tail", "chunks", "mixed"):
        steps = getattr(schedules, kind)(reqs)
        outs[kind] = schedules.run(_engine(d, "float32", page, schedules.max_live_tokens(reqs, steps)), reqs, steps)
    for kind in ("tail", "chunks", "mixed"):
        for r in reqs:
            assert schedules.rel_err(outs[kind][r], outs["whole"][r].astype(np.float64)) < 5e-6


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_long_decoding_passes_every_window_and_gives_pages_back(models, dt):
    """A short prompt, then 150 tokens one by one (recorded steps): the windows (7 to 50 keys) and several pages
    pass; windowed groups hold a bounded number of pages while the kept first positions stay readable."""
    cfg, page, _ = CASES["P"]
    d, _, _ = models[("P", dt)]
    toks = helpers.random_requests(cfg["vocab"], [160], 77)["r0"]
    ref = plain_logits(d, {"a": toks})["a"]
    from litinfer_amd.engine import StepEntry
    eng = _engine(d, dt, page, 256)
    rows = [eng.step([StepEntry("a", toks[:10], list(range(10)))]).float().cpu().numpy()]
    held = []
    for i in range(10, 160):
        rows.append(eng.step([StepEntry("a", [toks[i]], [0])]).float().cpu().numpy().copy())
        held.append([g.pool.capacity - f for g, f in zip(eng.cache.groups, eng.cache.free_pages())])
    got = np.concatenate(rows)
    assert eng.graph_replays > 100
    for g, h in zip(eng.cache.groups, np.array(held).max(axis=0)):
        assert h <= -(-g.need.window // page) + 1 + -(-g.need.keep_first // page), (g.need, h)
    err = schedules.rel_err(got, ref)
    print(f"[observed] long decoding {dt}: {err:.3e}")
    assert err < TOL[dt]
    eng.finish("a")
    eng.cache.check_invariants()


def test_greedy_generation_through_the_entry_point(models):
    """`models.load(folder).generate`: the scheduler, the sampler and the engine; every new token is the argmax
    of the plain logits of the sequence so far."""
    from litinfer_amd import models as entry
    cfg, page, _ = CASES["Q"]
    d, reqs, _ = models[("Q", "float32")]
    _, w = plain_impl.load_folder(d, np.float64)
    lm = entry.load(d, dtype="float32", device=DEV, page_size=page, max_tokens=512, max_seqs=4)
    prompt = reqs["r1"]
    out = lm.generate(prompt, max_new_tokens=12, top_k=1, top_p=1.0, temperature=1.0)
    new = list(out)
    assert len(new) == 12
    seq = list(prompt)
    for t in new:
        logits = plain.forward(seq, w, cfg)[-1]
        top = np.argsort(logits)[::-1]
        assert t == top[0] or logits[top[0]] - logits[t] < 1e-4 * np.abs(logits).max(), (len(seq), t, top[:3])
        seq.append(int(t))


def test_unknown_mixer_and_bad_sizes_are_refused():
    from litinfer_amd.config import TovasunConfig
    from litinfer_amd.config.qwen2 import ConfigError
    import copy
    bad = copy.deepcopy(CONFIG_P)
    bad["layers"][0]["type"] = "convolution"
    with pytest.raises(ConfigError):
        TovasunConfig.from_dict(bad)
    bad = copy.deepcopy(CONFIG_P)
    bad["layers"][1]["mixer"]["rot"]["dims"] = 6            # must equal rot_dim
    with pytest.raises(ConfigError):
        TovasunConfig.from_dict(bad)
    bad = copy.deepcopy(CONFIG_P)
    bad["loop"]["stop"] = 9
    with pytest.raises(ConfigError):
        TovasunConfig.from_dict(bad)


# ------------------------------------------------------------------------------------------ mechanisms alone
def _meta(seg_specs, page, tables):
    from litinfer_amd.engine.batch import AttentionMeta
    q_len = np.array([q for _, q in seg_specs], dtype=np.int32)
    ctx_len = np.array([c for c, _ in seg_specs], dtype=np.int32)
    q_start = np.concatenate([[0], np.cumsum(q_len)[:-1]]).astype(np.int32)
    seg_of = np.repeat(np.arange(len(seg_specs), dtype=np.int32), q_len)
    dev = lambda a: torch.from_numpy(a).to(DEV)
    single = np.nonzero(q_len[seg_of] == 1)[0].astype(np.int32)
    multi = np.nonzero(q_len[seg_of] != 1)[0].astype(np.int32)
    tiles = np.asarray([(i, int(q_start[i]) + a, min(32, int(q_len[i]) - a), 0) for i in range(len(seg_specs))
                        if q_len[i] > 1 for a in range(0, int(q_len[i]), 32)], dtype=np.int32).reshape(-1, 4)
    return AttentionMeta(block_table=dev(tables), max_blocks=tables.shape[1], seg_of_token=dev(seg_of),
                         q_start=dev(q_start), q_len=dev(q_len), ctx_len=dev(ctx_len), num_segments=len(seg_specs),
                         num_tokens=int(q_len.sum()), max_q_len=int(q_len.max()), max_ctx_len=int(ctx_len.max()),
                         host_q_start=q_start, host_q_len=q_len, host_ctx_len=ctx_len,
                         single_tokens=dev(single) if len(multi) else None, num_single=len(single),
                         multi_tokens=dev(multi) if len(single) else None, num_multi=len(multi),
                         tiles=dev(tiles), num_tiles=len(tiles), tile_rows=32)


def _masked_case(dtype, seg_specs, nh, nkv, dk, dv, page, window, keep_first, softcap, seed, standout=None,
                 shared_rows=False, return_values=False, heads_kernel=None):
    """Random queries, keys and values for segments (context, queries); pages in shuffled order with garbage
    in every slot that no key owns (and -1 in the table where a windowed cache would have given a page back).
    `standout` = (key position, query row): that key's score is made to win by e^12.  `shared_rows`: values are
    the first dv columns of the keys' rows (one cached tensor)."""
    from litinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(seed)
    blocks = [-(-c // page) for c, _ in seg_specs]
    num_pages = sum(blocks) + 2
    perm = torch.randperm(num_pages, generator=g).tolist()
    kc = torch.randn(num_pages, nkv, page, dk, generator=g).to(dtype)
    vc = kc if shared_rows else torch.randn(num_pages, nkv, page, dv, generator=g).to(dtype)
    tab = np.full((len(seg_specs), max(blocks)), -1, dtype=np.int32)
    T = sum(q for _, q in seg_specs)
    q = torch.randn(T, nh, dk, generator=g)
    scale = 1.0 / math.sqrt(dk)
    ks, vs, o = [], [], 0
    for s, (c, ql) in enumerate(seg_specs):
        k = torch.randn(c, nkv, dk, generator=g).to(dtype)
        v = k[..., :dv].clone() if shared_rows else torch.randn(c, nkv, dv, generator=g).to(dtype)
        if standout is not None:
            far, row = standout
            big = math.sqrt(12.0 / scale)
            k[far] = 0
            k[far, :, dk - 1] = big
            if shared_rows:
                v = k[..., :dv].clone()
            q[o + (ql - 1 if row is None else row)] = 0
            q[o + (ql - 1 if row is None else row), :, dk - 1] = big
        first_query = c - ql
        lo_block = max(0, first_query - window + 1) // page if window else 0
        kept_blocks = -(-keep_first // page)
        for b in range(blocks[s]):
            if window and kept_blocks <= b < lo_block:
                continue                                           # a page that the window has passed: given back
            tab[s, b] = perm.pop()
            n = min(page, c - b * page)
            kc[tab[s, b], :, :n] = k[b * page:b * page + n].transpose(0, 1)
            if not shared_rows:
                vc[tab[s, b], :, :n] = v[b * page:b * page + n].transpose(0, 1)
        ks.append(k)
        vs.append(v)
        o += ql
    meta = _meta(seg_specs, page, tab)
    out = torch.empty(T, nh * dv, dtype=dtype, device=DEV)
    qd = q.to(DEV).contiguous()
    kd = kc.to(DEV)
    vd = kd if shared_rows else vc.to(DEV)
    from litinfer_amd.engine.workspace import Workspace
    was = ops._heads_kernel_pays
    if heads_kernel is not None:                         # single tokens on the matrix cores, or not, whatever their number
        ops._heads_kernel_pays = lambda *a: bool(heads_kernel)
    try:
        ops.masked_attention(qd, nh * dk, dk, out, kd, vd, meta, nh, nkv, dk, dv, page, window, keep_first, softcap, scale,
                             ws=Workspace(DEV))
    finally:
        ops._heads_kernel_pays = was
    refs, o = [], 0
    rep = nh // nkv
    for s, (c, ql) in enumerate(seg_specs):
        kk = np.repeat(ks[s].double().numpy(), rep, axis=1)
        vv = np.repeat(vs[s].double().numpy(), rep, axis=1)
        refs.append(plain.masked_softmax_attention(q[o:o + ql].double().numpy(), kk, vv, scale, window, keep_first,
                                                   softcap or None, q_pos=np.arange(c - ql, c), k_pos=np.arange(c))
                    .reshape(ql, -1))
        o += ql
    if return_values:
        return out.float().cpu().numpy(), np.concatenate(refs), [np.repeat(v.double().numpy(), rep, axis=1) for v in vs]
    return out.float().cpu().numpy(), np.concatenate(refs)


def _close(got, ref, dtype):
    err = float(np.abs(got - ref).max() / np.abs(ref).max())
    assert err < (2e-5 if dtype is torch.float32 else 1.2e-2), err


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("segs,nh,nkv,dk,dv,page,window,keep,cap", [
    ([(2, 2)], 1, 1, 4, 4, 16, 0, 0, 0.0),
    ([(11, 5), (20, 1)], 4, 2, 8, 6, 16, 0, 0, 0.0),                  # no window: all keys
    ([(100, 37), (33, 2), (300, 1), (70, 70)], 6, 3, 24, 40, 8, 20, 0, 0.0),    # window crosses pages, value wider than key
    ([(100, 37), (33, 2), (300, 1), (70, 70)], 6, 3, 24, 40, 8, 20, 5, 3.0),    # kept first positions and a cap
    ([(200, 8), (64, 64), (65, 1)], 8, 1, 72, 64, 16, 64, 17, 30.0),  # kept positions over two pages
    ([(130, 130), (257, 3)], 4, 4, 128, 128, 32, 40, 4, 0.0),
    ([(500, 1), (90, 1), (3, 1), (41, 1)], 5, 5, 20, 12, 8, 40, 4, 7.5),         # decoding only
    ([(90, 30)], 3, 1, 300, 260, 16, 50, 2, 0.0),                      # long rows: several value columns a lane
    # sizes that the matrix-core kernel for portions takes in bfloat16; single tokens beside the portions
    ([(100, 37), (33, 2), (300, 1), (70, 70), (64, 64), (1, 1)], 6, 3, 64, 64, 8, 20, 5, 3.0),
    ([(257, 100), (90, 90), (64, 33), (700, 1)], 10, 2, 128, 64, 16, 50, 0, 0.0),       # five heads a group: two turns of waves
    ([(200, 130), (40, 40)], 7, 1, 96, 64, 16, 0, 0, 10.0),            # seven heads on one kv head, no window
    ([(300, 200)], 4, 2, 64, 128, 32, 100, 33, 0.0),
    ([(150, 150), (500, 35)], 3, 1, 320, 256, 16, 64, 1, 0.0),
    ([(130, 100), (40, 1)], 2, 1, 192, 128, 16, 70, 0, 0.0),
    ([(100, 100), (300, 40), (90, 1)], 2, 2, 256, 256, 16, 64, 2, 20.0),
    ([(140, 75)], 5, 1, 288, 256, 8, 0, 0, 0.0),
    ([(700, 300), (64, 1), (400, 33)], 4, 2, 64, 64, 16, 0, 0, 0.0),            # few tiles against many keys: splits of a tile's keys
    ([(900, 200), (300, 1)], 6, 1, 128, 128, 16, 512, 7, 25.0),
    # decoding steps at sizes that the kernel for single tokens takes in bfloat16 (1, 2 and 4 heads a block)
    ([(700, 1), (90, 1), (3, 1), (41, 1), (1, 1)], 12, 2, 128, 128, 16, 200, 4, 30.0),
    ([(700, 1), (33, 1)], 7, 1, 64, 64, 8, 0, 0, 0.0),
    ([(300, 1), (130, 1), (64, 1)], 3, 3, 96, 64, 16, 40, 2, 0.0),
    ([(1500, 1), (100, 1)], 5, 1, 320, 256, 16, 1024, 0, 0.0),
    ([(260, 1), (17, 1)], 8, 2, 192, 128, 32, 100, 40, 5.0),
    ([(3000, 1), (5, 1), (129, 1)], 4, 2, 128, 128, 16, 0, 0, 0.0),           # many splits of the keys, some of them empty
    ([(2500, 1), (300, 1)], 6, 1, 160, 128, 16, 2000, 3, 0.0),
    ([(400, 1), (30, 1)], 3, 1, 256, 192, 16, 300, 0, 0.0),
    ([(400, 1), (30, 1)], 4, 4, 72, 136, 16, 300, 5, 0.0),
    # many heads on one kv head: single tokens on the matrix cores, the heads as a tile's columns
    ([(700, 1), (90, 1), (3, 1), (41, 1), (1, 1)], 12, 1, 128, 128, 16, 200, 4, 30.0),
    ([(1500, 1), (100, 1), (64, 1)], 40, 1, 320, 256, 16, 1024, 0, 0.0),            # two chunks of 32 heads
    ([(300, 1), (33, 1), (200, 60)], 18, 2, 64, 64, 8, 0, 0, 0.0),                 # beside a portion
])
def test_masked_attention_against_the_plain_attention(dtype, segs, nh, nkv, dk, dv, page, window, keep, cap):
    got, ref = _masked_case(dtype, segs, nh, nkv, dk, dv, page, window, keep, cap, seed=3)
    _close(got, ref, dtype)
    for heads_kernel in (False, True):                   # single tokens on the vector ALU and on the matrix cores
        got, ref = _masked_case(dtype, segs, nh, nkv, dk, dv, page, window, keep, cap, seed=3, heads_kernel=heads_kernel)
        _close(got, ref, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_values_that_are_the_first_columns_of_the_keys_rows(dtype):
    got, ref = _masked_case(dtype, [(120, 50), (77, 1)], 6, 1, 56, 40, 16, 30, 0, 0.0, seed=4, shared_rows=True)
    _close(got, ref, dtype)
    got, ref = _masked_case(dtype, [(400, 70), (77, 1), (33, 33)], 6, 1, 160, 128, 16, 90, 0, 0.0, seed=5, shared_rows=True)
    _close(got, ref, dtype)
    got, ref = _masked_case(dtype, [(400, 1), (77, 1), (1, 1)], 4, 1, 160, 128, 16, 90, 0, 0.0, seed=6, shared_rows=True)
    _close(got, ref, dtype)
    for heads_kernel in (False, True):
        got, ref = _masked_case(dtype, [(900, 1), (77, 1), (1, 1)], 10, 1, 160, 128, 16, 500, 0, 0.0, seed=7, shared_rows=True,
                                heads_kernel=heads_kernel)
        _close(got, ref, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ql", [1, 40])
@pytest.mark.parametrize("where", ["edge_in", "edge_out", "kept_in", "kept_out", "page_border", "self"])
def test_one_standout_key_at_the_edges_of_window_and_kept_positions(where, ql, dtype):
    """Context 400, window 64, 3 kept positions, pages of 16.  One key is given a score that wins by e^12: just
    inside the window's edge it must dominate the output of the last query, just outside it must not; the same
    for the last kept position and the first one that is not kept."""
    c, window, keep, page = 400, 64, 3, 16
    p = c - 1
    key = {"edge_in": p - window + 1, "edge_out": p - window, "kept_in": keep - 1, "kept_out": keep,
           "page_border": p - (p % page), "self": p}[where]
    got, ref, values = _masked_case(dtype, [(c, ql)], 4, 2, 64, 64, page, window, keep, 0.0, seed=9,
                                    standout=(key, None), return_values=True)
    _close(got, ref, dtype)
    # the last query's output is the standout key's value exactly when that key is visible
    dominated = np.abs(got[-1].reshape(4, 64) - values[0][key]).max() < 0.05
    assert dominated == (where not in ("edge_out", "kept_out"))


def test_rotation_of_neighbouring_pairs_and_its_scaling():
    from litinfer_amd.config.spec import PartSpec
    from litinfer_amd.kernels import ops
    from litinfer_amd.parts.position import pair_frequencies
    for dims, base, sc in ((8, 10000.0, None), (32, 500.0, yarn(8.0, 512)), (16, 10000.0, yarn(4.0, 16, 8.0, 2.0)),
                           (64, 1e6, yarn(1.0, 4096))):
        f, amp = pair_frequencies(dims, base, sc)
        rf, ramp = plain.rotary_frequencies(dims, base, sc)
        assert np.allclose(f, rf, rtol=1e-12) and abs(amp - ramp) < 1e-12
        heads, d, t = 3, dims + 6, 50
        g = torch.Generator().manual_seed(1)
        x = torch.randn(t, heads * d, generator=g)
        pos = torch.arange(1000, 1000 + t, dtype=torch.int32)
        cos = torch.empty(t, dims // 2, device=DEV)
        sin = torch.empty(t, dims // 2, device=DEV)
        ops.rope_freq_table(pos.to(DEV), torch.tensor(f, dtype=torch.float32, device=DEV), amp, cos, sin)
        xd = x.to(DEV).clone()
        ops.rope_pairs_apply(xd, heads, d, dims, cos, sin)
        ref = plain.rotate_pairs(x.double().numpy().reshape(t, heads, d), pos.numpy(), dims, base, sc).reshape(t, -1)
        assert np.abs(xd.cpu().numpy() - ref).max() < 3e-4          # float32 angles near position 1000


def test_norm_behind_a_sublayer_and_the_next_norm_in_one_kernel():
    from litinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(2)
    for t, h in ((1, 96), (7, 1000), (300, 260), (3, 5000)):
        x, y = torch.randn(t, h, generator=g), torch.randn(t, h, generator=g) * 3
        w, w2 = torch.randn(h, generator=g), torch.randn(h, generator=g)
        ref = x.double().numpy() + plain.rms_norm(y.double().numpy(), w.double().numpy(), 1e-5)
        ref2 = plain.rms_norm(ref, w2.double().numpy(), 1e-6)
        for out_dtype in (torch.float32, torch.bfloat16):
            xd, xn = x.to(DEV).clone(), torch.empty(t, h, dtype=out_dtype, device=DEV)
            ops.rmsnorm_add(y.to(DEV), w.to(DEV), 1e-5, xd, w2.to(DEV), 1e-6, xn)
            assert np.abs(xd.cpu().numpy() - ref).max() < 1e-5
            assert np.abs(xn.float().cpu().numpy() - ref2).max() < (1e-5 if out_dtype is torch.float32 else 4e-2)
        xd = x.to(DEV).clone()
        ops.rmsnorm_add(y.to(DEV), w.to(DEV), 1e-5, xd)
        assert np.abs(xd.cpu().numpy() - ref).max() < 1e-5


def test_squared_relu_gelu_gate_and_the_stream_additions():
    from litinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(3)
    x = torch.randn(37, 130, generator=g)
    out = torch.empty(37, 130, device=DEV)
    ops.relu_squared(x.to(DEV), out)
    assert np.abs(out.cpu().numpy() - plain.relu_squared(x.double().numpy())).max() < 1e-6
    table = torch.randn(50, 48, generator=g)
    ids = torch.randint(0, 50, (37,), generator=g, dtype=torch.int32)
    a = torch.randn(37, 12, generator=g) * 2
    gg = torch.empty(37, 12, device=DEV)
    ops.gelu_gate_rows(a.to(DEV), ids.to(DEV), table.to(DEV), 24, gg)
    ref = plain.gelu_tanh(a.double().numpy()) * table.double().numpy()[ids.numpy()][:, 24:36]
    assert np.abs(gg.cpu().numpy() - ref).max() < 1e-6
    emb = torch.randn(50, 130, generator=g)
    vec = torch.randn(130, generator=g)
    xs = x.to(DEV).clone()
    ops.embedding_add(xs, ids.to(DEV), emb.to(DEV), vec.to(DEV))
    assert np.abs(xs.cpu().numpy() - (x + emb[ids.long()] + vec).numpy()).max() < 1e-6
    xs = x.to(DEV).clone()
    ops.embedding_add(xs, None, None, vec.to(DEV))                  # the first pass: the vector alone
    assert np.abs(xs.cpu().numpy() - (x + vec).numpy()).max() < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_products_with_a_matrix_of_its_own_for_every_head(dtype):
    from litinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(4)
    # (the last three: sizes that go to the matrix cores in bfloat16, 32 tokens a tile)
    for t, nh, n_out, n_in, pad, opad in ((1, 3, 40, 16, 8, 3), (19, 5, 300, 72, 0, 3), (64, 2, 24, 130, 6, 3),
                                          (40, 3, 128, 64, 8, 4), (100, 4, 64, 160, 0, 0), (33, 2, 256, 48, 16, 8)):
        m = torch.randn(nh, n_out, n_in, generator=g).to(dtype)
        x = torch.randn(t, nh, n_in + pad, generator=g)              # a head's inputs lie inside a wider row
        out = torch.zeros(t, nh, n_out + opad, dtype=dtype, device=DEV)
        ops.headwise_linear(x.to(DEV), nh * (n_in + pad), n_in + pad, m.to(DEV), out, nh * (n_out + opad), n_out + opad, t)
        ref = np.einsum("hjk,thk->thj", m.double().numpy(), x[..., :n_in].double().numpy())
        got = out.float().cpu().numpy()
        assert np.abs(got[..., :n_out] - ref).max() / np.abs(ref).max() < (1e-5 if dtype is torch.float32 else 1e-2)
        assert opad == 0 or np.abs(got[..., n_out:]).max() == 0      # nothing written beside a head's outputs


def test_mixers_alone_against_their_plain_forms(models):
    """One layer's mixer through the engine's parts and cache (a prompt in two portions, then two single tokens)
    against the plain mixer on the whole sequence: the latent attention's reordered products give what the
    expansion of every key and value gives."""
    from litinfer_amd.engine import Engine, StepEntry
    cfg, page, _ = CASES["R"]
    d, _, _ = models[("R", "float32")]
    _, w = plain_impl.load_folder(d, np.float64)
    eng = Engine.from_dir(d, dtype="float32", device=DEV, page_size=page, max_tokens=256, max_seqs=2,
                          use_graphs=False)              # (the tap reads the stream on the host)
    toks = helpers.random_requests(cfg["vocab"], [75], 5)["r0"]
    taps = {}

    def tap(i, x):
        taps.setdefault(i, []).append(x.detach().cpu().numpy().copy())
    eng.model.tap = tap
    for a, b in ((0, 40), (40, 73), (73, 74), (74, 75)):
        eng.step([StepEntry("a", toks[a:b], [])])
    runs = []
    plain.forward(toks, w, cfg, runs)
    for i, ref in enumerate(runs):
        got = np.concatenate(taps[i])
        assert np.abs(got - ref).max() / np.abs(ref).max() < 2e-5, i
