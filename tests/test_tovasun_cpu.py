"""Tovasun without a GPU: the configuration reader and the model as data, the cache's kept first positions,
the rotary frequencies, and pins of the plain implementation (tests/plain_tovasun.py)."""
import copy
import math

import numpy as np
import pytest
import torch

import plain_tovasun as plain
from litinfer_amd.cache import CacheManager
from litinfer_amd.config import TovasunConfig, architecture_name, lookup, tovasun_model_spec
from litinfer_amd.config.qwen2 import ConfigError
from litinfer_amd.engine.model import Model, expected_params_of_spec
from litinfer_amd.parts.base import PagedNeed, PagedTensor, Runtime
from litinfer_amd.parts.position import pair_frequencies

CONFIG = {
    "architecture": "Tovasun", "vocab": 97, "width": 48, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "attention", "mlp": {"kind": "dense", "ff": 80},
         "mixer": {"heads": 4, "kv_heads": 2, "dim": 12, "vdim": 10, "scale": 0.3, "softcap": 15.0,
                   "mask": {"size": 9, "keep_first": 2}, "rot": {"base": 100.0, "dims": 6}}},
        {"type": "latent_attention", "mlp": None,
         "mixer": {"heads": 3, "dim": 8, "rot_dim": 4, "vdim": 6, "kv_rank": 20, "scale": 0.29, "mask": {"size": 5},
                   "rot": {"base": 10000.0, "dims": 4, "scaling": {"factor": 4.0, "original": 8, "fast": 4.0, "slow": 1.0}}}},
        {"type": "attention", "mlp": {"kind": "dense", "ff": 64},
         "mixer": {"heads": 4, "kv_heads": 2, "dim": 12, "vdim": 10, "scale": 0.3, "softcap": 15.0,
                   "mask": {"size": 9, "keep_first": 2}, "rot": {"base": 100.0, "dims": 6}}},
    ],
    "loop": {"start": 1, "stop": 3, "times": 3}, "token_side": {"dim": 5},
}


def test_the_architecture_is_found_under_its_key_and_read_into_a_spec():
    assert architecture_name(CONFIG) == "Tovasun"
    arch = lookup("Tovasun")
    cfg = arch.config_from_dict(CONFIG)
    assert isinstance(cfg, TovasunConfig) and cfg.loop == (1, 3, 3) and cfg.side_dim == 5
    spec = arch.model_spec(cfg)
    spec.validate()
    # layer 0 once, layers 1..2 three times, each pass entered through the injection with its number
    assert [(e.layer, e.inject) for e in spec.order] == [(0, None), (1, (0, 0)), (2, None), (1, (0, 1)), (2, None),
                                                         (1, (0, 2)), (2, None)]
    names = expected_params_of_spec(spec)
    assert names["loop.step"].shape == (3, 48) and names["side.embed"].shape == (97, 15)
    assert names["l0.mix.q.norm"].shape == (48,) and names["l0.mix.k.norm"].shape == (24,)
    assert names["l0.mix.v"].shape == (20, 48) and names["l0.mix.o"].shape == (48, 40)
    assert names["l1.mix.dkv"].shape == (24, 48) and names["l1.mix.uk"].shape == (24, 20) and names["l1.mix.uv"].shape == (18, 20)
    assert "l1.mlp.up" not in names and "l1.norm2" not in names and "l1.norm1b" in names
    assert names["l2.side.gate"].shape == (5, 48) and names["l2.side.proj"].shape == (48, 5)
    assert names["embed"].shape == (97, 48) and names["head"].shape == (97, 48) and names["final.norm"].shape == (48,)


def test_every_pass_of_the_loop_has_a_cache_of_its_own_in_the_group_of_its_need():
    spec = tovasun_model_spec(TovasunConfig.from_dict(CONFIG))
    model = Model(spec, Runtime(torch.device("cpu"), torch.float32))
    needs, sources = model.cache_needs()
    assert sources == [None] * 7
    cache = CacheManager(needs, sources, page_size=4, num_pages=16, max_seqs=2, dtype=torch.float32, device="cpu")
    # two groups: the windowed attention with its kept positions (layers 0 and 2: 1 + 3 entries) and the latent rows
    assert [(g.need.window, g.need.keep_first, len(g.entries)) for g in cache.groups] == [(9, 2, 4), (5, 0, 3)]
    assert cache.groups[0].data["k"].shape == (4, 16, 2, 4, 12) and cache.groups[0].data["v"].shape == (4, 16, 2, 4, 10)
    assert cache.groups[1].data["latent"].shape == (3, 16, 1, 4, 24)


@pytest.mark.parametrize("change,text", [
    (lambda c: c["layers"][0].update(type="state_space"), "unknown mixer"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=6), "rot_dim"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "dense"),
    (lambda c: c["loop"].update(stop=5), "loop"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=14), "exceeds"),
])
def test_configurations_that_cannot_be_built_are_refused_with_a_reason(change, text):
    bad = copy.deepcopy(CONFIG)
    change(bad)
    with pytest.raises(ConfigError, match=text):
        TovasunConfig.from_dict(bad)


def test_optional_keys_may_be_absent():
    c = copy.deepcopy(CONFIG)
    del c["loop"], c["token_side"]
    del c["layers"][0]["mixer"]["softcap"], c["layers"][0]["mixer"]["mask"]["keep_first"], c["layers"][0]["mixer"]["kv_heads"]
    cfg = TovasunConfig.from_dict(c)
    spec = tovasun_model_spec(cfg)
    assert [e.layer for e in spec.order] == [0, 1, 2] and not spec.injections
    m = cfg.layers[0].mixer
    assert m.softcap == 0.0 and m.keep_first == 0 and m.kv_heads == 4
    assert "side.embed" not in expected_params_of_spec(spec)


def test_kept_first_positions_keep_their_pages_while_the_window_gives_the_others_back():
    need = PagedNeed((PagedTensor("k", (1, 4)),), window=6, keep_first=5)
    plain_need = PagedNeed((PagedTensor("k", (1, 4)),), window=6)
    cache = CacheManager([need, plain_need], [None, None], page_size=4, num_pages=12, max_seqs=2,
                         dtype=torch.float32, device="cpu")
    cache.admit("a")
    for _ in range(10):
        cache.reserve("a", 3)
        cache.commit("a", 3)
        cache.check_invariants()
    # 30 tokens cached: a query at 30 sees 25..30, block 6 on; positions 0..4 lie in blocks 0 and 1
    kept, windowed = cache.block_table("a", 0), cache.block_table("a", 1)
    assert [p >= 0 for p in kept] == [True, True, False, False, False, False, True, True]
    assert [p >= 0 for p in windowed] == [False] * 6 + [True, True]
    cache.release("a")
    assert cache.free_pages() == [12, 12]
    cache.check_invariants()


def test_pair_frequencies_follow_the_scaling_rule():
    f, amp = pair_frequencies(8, 10000.0)
    assert amp == 1.0 and np.allclose(f, [1.0, 0.1, 0.01, 0.001])
    sc = {"factor": 8.0, "original": 512, "fast": 32.0, "slow": 1.0}
    f, amp = pair_frequencies(32, 10000.0, sc)
    rf, ramp = plain.rotary_frequencies(32, 10000.0, sc)
    assert np.allclose(f, rf, rtol=1e-13) and amp == pytest.approx(0.1 * math.log(8.0) + 1.0) and ramp == pytest.approx(amp)
    base = [10000.0 ** (-2.0 * i / 32) for i in range(16)]
    assert f[0] == base[0] and f[-1] == pytest.approx(base[-1] / 8.0)          # fast pairs untouched, slow ones divided
    assert all(b / 8.0 - 1e-15 <= x <= b + 1e-15 for x, b in zip(f, base))


# ------------------------------------------------------------------------------- pins of the plain implementation
def test_plain_visibility():
    see = [[plain.visible(i, j, 3, 2) for j in range(7)] for i in range(7)]
    assert see[6] == [True, True, False, False, True, True, True]
    assert see[2] == [True, True, True, False, False, False, False]
    assert [plain.visible(5, j, 0) for j in range(7)] == [True] * 6 + [False]


def test_plain_rotation_is_a_rotation_by_the_relative_position():
    rng = np.random.default_rng(0)
    q, k = rng.normal(size=(1, 1, 6)), rng.normal(size=(1, 1, 6))
    def score(pq, pk):
        a = plain.rotate_pairs(q, np.array([pq]), 4, 50.0)
        b = plain.rotate_pairs(k, np.array([pk]), 4, 50.0)
        return float((a * b).sum())
    assert score(7, 3) == pytest.approx(score(104, 100)) and score(7, 3) != pytest.approx(score(7, 4))
    out = plain.rotate_pairs(q, np.array([9]), 4, 50.0)
    assert np.array_equal(out[..., 4:], q[..., 4:])                                  # columns beyond `dims` pass
    c, s = math.cos(9.0), math.sin(9.0)                                             # the first pair turns by p * 1
    assert out[0, 0, 0] == pytest.approx(q[0, 0, 0] * c - q[0, 0, 1] * s) and out[0, 0, 1] == pytest.approx(q[0, 0, 1] * c + q[0, 0, 0] * s)


def test_plain_latent_attention_equals_attention_over_the_latent_rows():
    """The reordering the engine relies on: scores through Wuk^T q and values through Wuv (sum p c) give what
    expanding every key and value gives."""
    rng = np.random.default_rng(1)
    T, H, d, dr, dv, r, W = 9, 2, 4, 2, 3, 5, 12
    m = {"heads": H, "dim": d, "rot_dim": dr, "vdim": dv, "kv_rank": r, "scale": 0.4, "mask": {"size": 4},
         "rot": {"base": 30.0, "dims": dr}}
    w = {"q": rng.normal(size=(H * (d + dr), W)), "dkv": rng.normal(size=(r + dr, W)), "dkv.norm": rng.normal(size=r),
         "uk": rng.normal(size=(H * d, r)), "uv": rng.normal(size=(H * dv, r)), "o": rng.normal(size=(W, H * dv))}
    h = rng.normal(size=(T, W))
    pos = np.arange(T)
    ref = plain.latent_attention_mixer(h, w, "", m, 1e-6, pos)
    q = (h @ w["q"].T).reshape(T, H, d + dr)
    down = h @ w["dkv"].T
    c = plain.rms_norm(down[:, :r], w["dkv.norm"], 1e-6)
    kr = plain.rotate_pairs(down[:, None, r:], pos, dr, 30.0)
    qr = plain.rotate_pairs(q[..., d:], pos, dr, 30.0)
    uk, uv = w["uk"].reshape(H, d, r), w["uv"].reshape(H, dv, r)
    q_lat = np.einsum("thd,hdr->thr", q[..., :d], uk)
    rows = np.concatenate([c[:, None, :], kr], axis=-1)                             # one row a token, shared by the heads
    o_lat = plain.masked_softmax_attention(np.concatenate([q_lat, qr], axis=-1), np.repeat(rows, H, axis=1),
                                           np.repeat(c[:, None, :], H, axis=1), 0.4, 4)
    out = np.einsum("thr,hvr->thv", o_lat, uv).reshape(T, H * dv) @ w["o"].T
    assert np.allclose(out, ref, rtol=1e-10, atol=1e-10)
