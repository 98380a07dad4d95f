"""The Sogenex decoder without a GPU: pins of the plain implementation (tests/plain_sogenex.py; these import nothing
from the package), the configuration and its errors, the model as data (layers that run with another layer's
tensors), the tensors it expects and what its entries ask of the cache."""
import copy
import math

import numpy as np
import pytest

import plain_sogenex as plain
import sogenex_cases as cases


# ------------------------------------------------------------------------------------ the plain implementation
def test_causal_convolution_is_a_convolution_with_zeros_before_the_start():
    rng = np.random.default_rng(0)
    u, w, b = rng.normal(size=(9, 3)), rng.normal(size=(3, 4)), rng.normal(size=3)
    out = plain.causal_conv(u, w, b)
    for c in range(3):
        full = np.convolve(u[:, c], w[c, ::-1])[:9]               # the last tap multiplies the current token
        assert np.allclose(out[:, c], full + b[c])
    assert np.allclose(out[0], w[:, -1] * u[0] + b)


def test_recurrence_against_its_closed_form():
    """With one head and one group: y_t = sum_{s <= t} (prod_{r = s+1..t} a_r) dt_s (B_s . C_t) x_s + D x_t."""
    rng = np.random.default_rng(1)
    T, N, P = 7, 5, 3
    x, B, C = rng.normal(size=(T, P)), rng.normal(size=(T, N)), rng.normal(size=(T, N))
    dt, A_log, D = rng.uniform(0.1, 1.0, (T, 1)), np.array([-0.3]), np.array([0.7])
    a = np.exp(-math.exp(A_log[0]) * dt[:, 0])
    y = plain.ssm_scan(x, B, C, dt, A_log, D, 1, P, 1, N)
    for t in range(T):
        acc = D[0] * x[t]
        for s in range(t + 1):
            acc = acc + np.prod(a[s + 1:t + 1]) * dt[s, 0] * (B[s] @ C[t]) * x[s]
        assert np.allclose(y[t], acc)


def test_heads_use_their_group():
    rng = np.random.default_rng(2)
    T, N, P = 4, 3, 2
    x, dt = rng.normal(size=(T, 4 * P)), rng.uniform(0.1, 1, (T, 4))
    B, C = rng.normal(size=(T, 2 * N)), rng.normal(size=(T, 2 * N))
    A_log, D = rng.normal(size=4), rng.normal(size=4)
    y = plain.ssm_scan(x, B, C, dt, A_log, D, 4, P, 2, N)
    for h in range(4):
        g = h // 2
        alone = plain.ssm_scan(x[:, h * P:(h + 1) * P], B[:, g * N:(g + 1) * N], C[:, g * N:(g + 1) * N], dt[:, h:h + 1],
                               A_log[h:h + 1], D[h:h + 1], 1, P, 1, N)
        assert np.allclose(y[:, h * P:(h + 1) * P], alone)


def test_window_and_softmax():
    assert [plain.visible(10, j, 4) for j in (6, 7, 10, 11)] == [False, True, True, False]
    assert plain.visible(10, 0, 0)
    rng = np.random.default_rng(3)
    q, k, v = rng.normal(size=(6, 4)), rng.normal(size=(6, 4)), rng.normal(size=(6, 2))
    out = plain.softmax_attention(q, k, v, 0.5, 3)
    s = np.exp(np.array([q[5] @ k[j] for j in (3, 4, 5)]) * 0.5)
    assert np.allclose(out[5], (s / s.sum()) @ v[3:6])
    assert np.allclose(out[0], v[0])


def test_router_takes_the_largest_and_weighs_the_chosen_alone():
    h = np.eye(3)
    router = np.array([[1.0, 0, 0], [3.0, 0, 0], [2.0, 5, 0], [0.0, 5, 0]])
    idx, wt = plain.route(h, router, np.zeros(4), 2)
    assert idx[0].tolist() == [1, 2] and idx[1].tolist() == [2, 3]           # equal logits: the lower expert first
    assert np.allclose(wt[0], np.exp([3.0, 2.0]) / np.exp([3.0, 2.0]).sum()) and np.allclose(wt[1], [0.5, 0.5])


def test_position_vector_norm_and_cap():
    s = plain.sinusoid([0, 3], 6)
    assert np.allclose(s[0], [0, 1, 0, 1, 0, 1])
    assert np.allclose(s[1, 2:4], [math.sin(3 * 10000 ** (-2 / 6)), math.cos(3 * 10000 ** (-2 / 6))])
    x = np.array([[3.0, 4.0]])
    assert np.allclose(plain.offset_norm(x, np.zeros(2), 0.0), x / math.sqrt(12.5))
    assert np.allclose(plain.offset_norm(x, np.array([1.0, -1.0]), 0.0), [[6 / math.sqrt(12.5), 0.0]])
    cfg = {"norm": {"eps": 0.0}, "logit_scale": 2.0, "logit_softcap": 4.0}
    w = {"final.norm": np.zeros(2), "head": np.eye(2)}
    assert np.allclose(plain.head(cfg, w, x), 4.0 * np.tanh(2.0 * x / math.sqrt(12.5) / 4.0))


def test_the_plain_model_decodes_as_it_prefills():
    """A whole sequence against the same sequence fed token by token with carried states is the engine's job; here only
    that a prefix's logits do not depend on what follows (causality of every mechanism)."""
    cfg = cases.CONFIG_A
    w = {n: a.astype(np.float64) for n, a in cases.draw_weights(cfg, 4).items()}
    toks = np.random.default_rng(5).integers(0, cfg["vocab"], 30).tolist()
    full = plain.forward(cfg, w, toks)
    assert np.allclose(plain.forward(cfg, w, toks[:17]), full[:17], atol=1e-9)
    assert np.isfinite(full).all() and np.abs(full).max() <= cfg["logit_softcap"]


# ------------------------------------------------------------------------------------ configuration and model as data
def test_config_and_execution_order():
    from litinfer_amd.config import SogenexConfig, sogenex_model_spec
    c = SogenexConfig.from_dict(cases.CONFIG_A)
    assert (c.vocab, c.width, c.eps, c.logit_scale, c.logit_softcap) == (211, 96, 1e-6, 0.7, 9.0)
    assert [L.weights_of for L in c.layers] == [None, None, None, 0, 1] and c.layers[2].mlp is None
    assert c.layers[1].mixer.window == 12 and c.layers[0].mixer.norm_groups == 2
    spec = sogenex_model_spec(c)
    assert len(spec.layers) == 3 and [e.layer for e in spec.order] == [0, 1, 2, 0, 1]
    assert "feed_forward" not in spec.layers[2].parts
    b = SogenexConfig.from_dict(cases.CONFIG_B)
    assert b.logit_scale == 1.0 and b.logit_softcap == 0.0 and b.layers[0].mixer.window == 0 and b.layers[0].mlp.shared_ff == 0


def test_a_layer_with_tensors_of_its_own_behind_sharing_ones_keeps_its_number():
    from litinfer_amd.config import SogenexConfig, sogenex_model_spec
    from litinfer_amd.engine.model import expected_params_of_spec
    cfg = copy.deepcopy(cases.CONFIG_A)
    cfg["layers"].append(cases.mamba_layer(2, 8, 4, 1, 2, 1, None))              # layer 5, its own tensors
    spec = sogenex_model_spec(SogenexConfig.from_dict(cfg))
    names = set(expected_params_of_spec(spec))
    assert "l5.mix.A_log" in names and "l5.norm1" in names and not any(n.startswith(("l3.", "l4.")) for n in names)
    assert [e.layer for e in spec.order] == [0, 1, 2, 0, 1, 3]
    assert {"embed", "head", "final.norm", "l0.mix.in", "l0.mix.conv", "l0.mix.conv.b", "l0.mix.dt_bias", "l0.mix.D", "l0.mix.norm",
            "l0.mix.o", "l1.mix.q", "l1.mix.lq1", "l1.mix.lk2", "l0.mlp.router", "l0.mlp.router.b", "l0.mlp.e4.up", "l0.mlp.e0.down",
            "l0.mlp.shared.up", "l0.mlp.shared.sg"} <= names
    assert "l2.norm2" not in names and "l0.mlp.e5.up" not in names
    p = expected_params_of_spec(spec)
    assert p["l0.mix.in"].shape == (2 * 96 + 2 * 3 * 24 + 6, 96) and p["l0.mix.conv"].shape == (96 + 2 * 72, 4)
    assert p["l1.mix.q"].shape == (4 * 2 * 24, 96) and p["l1.mix.k"].shape == (2 * 2 * 24, 96) and p["l1.mix.v"].shape == (2 * 16, 96)
    assert p["l0.mlp.shared.sg"].shape == (1, 96)


@pytest.mark.parametrize("change,where", [
    (lambda c: c["layers"][0].update(type="convolution"), "unknown mixer"),
    (lambda c: c["layers"][3].update(weights_of=4), "has no tensors of its own"),
    (lambda c: c["layers"][3].update(weights_of=1), "differs"),
    (lambda c: c["layers"][3].update(weights_of=9), "weights_of"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "not supported"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][0]["mixer"].update(groups=4), "multiple"),
    (lambda c: c["layers"][2]["mixer"].update(norm_groups=7), "norm groups"),
    (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda c: c.update(logit_softcap=-1.0), "logit_softcap"),
])
def test_bad_configurations_are_refused(change, where):
    from litinfer_amd.config import ConfigError, SogenexConfig
    cfg = copy.deepcopy(cases.CONFIG_A)
    cfg["layers"][0]["mlp"] = copy.deepcopy(cfg["layers"][0]["mlp"])
    change(cfg)
    with pytest.raises(ConfigError, match=where):
        SogenexConfig.from_dict(cfg)


def test_top_above_the_number_of_experts_is_refused():
    from litinfer_amd.config import ConfigError, SogenexConfig
    cfg = copy.deepcopy(cases.CONFIG_B)
    cfg["layers"][1]["mlp"]["router"]["top"] = 5
    with pytest.raises(ConfigError):
        SogenexConfig.from_dict(cfg)


def test_what_the_entries_ask_of_the_cache():
    import torch
    from litinfer_amd.cache import group_needs
    from litinfer_amd.config import SogenexConfig, sogenex_model_spec
    from litinfer_amd.engine.model import Model
    from litinfer_amd.parts import PagedNeed, Runtime, StateNeed, needs_of
    model = Model(sogenex_model_spec(SogenexConfig.from_dict(cases.CONFIG_A)), Runtime(torch.device("cpu"), torch.float32))
    needs, sources = model.cache_needs()
    assert sources == [None] * 5
    paged0, states0 = needs_of(needs[0])
    assert paged0 is None and {s.name: s.shape for s in states0} == {"ssm": (6, 24, 16), "conv": (3, 96 + 2 * 72)}
    assert all(s.dtype is torch.float32 for s in states0)
    paged1, states1 = needs_of(needs[1])
    assert not states1 and paged1.window == 12 and [(t.name, t.shape) for t in paged1.tensors] == [("k1", (2, 24)), ("k2", (2, 24)), ("v", (2, 16))]
    assert len(group_needs(needs, sources)) == 1                                  # the two attention entries share pages ids, not pages
    assert {s.name: s.shape for s in needs_of(needs[2])[1]} == {"ssm": (3, 8, 40), "conv": (1, 120 + 16)}
    assert model.graph_safe


def test_the_command_line_knows_the_architecture(tmp_path):
    """`random` writes a model folder for the configuration; its tensors are those the model expects."""
    import json
    from litinfer_amd.__main__ import main
    from litinfer_amd.weights.safetensors_io import SafetensorsFile
    (tmp_path / "c.json").write_text(json.dumps(cases.CONFIG_B))
    assert main(["random", "--config", str(tmp_path / "c.json"), "--seed", "3", "--out", str(tmp_path / "m")]) == 0
    names = set(SafetensorsFile(tmp_path / "m" / "model.safetensors").entries)
    assert {"embed", "l0.mix.lq1", "l1.mix.A_log", "l1.mlp.e3.down", "l1.mlp.shared.sg"} <= names and "l0.mlp.shared.up" not in names
