"""Plain, slow implementation of the Tovasun decoder: NumPy float64, whole sequences,
no cache, one function per mechanism.  Shares no code with the package.

Notation: x [T, W] is the residual stream of one sequence, positions 0..T-1;
weights are a dict name -> array, matrices stored [out, in] and applied as x @ W.T.
"""
from __future__ import annotations

import math

import numpy as np


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def rms_norm(x, w, eps):
    return rms(x, eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def relu_squared(z):
    return np.maximum(z, 0.0) ** 2


def rotary_frequencies(dims, base, scaling=None):
    """(f [dims/2], amplitude): f_i = base^(-2i/dims); with YaRN scaling the
    low frequencies are divided by `factor`, blended by a linear ramp between the
    dimensions whose wavelengths fit `fast` and `slow` times into `original` positions,
    and cos/sin are multiplied by 0.1 ln(factor) + 1."""
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def dim_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(scaling["slow"]))), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    f = f / factor * ramp + f * (1.0 - ramp)
    return f, 0.1 * math.log(factor) + 1.0


def rotate_pairs(v, positions, dims, base, scaling=None):
    """v [T, heads, d]: the first `dims` of d are rotated, neighbours (2i, 2i+1) forming a pair."""
    f, amp = rotary_frequencies(dims, base, scaling)
    a = positions[:, None].astype(np.float64) * f[None, :]                 # [T, dims/2]
    cos, sin = (np.cos(a) * amp)[:, None, :], (np.sin(a) * amp)[:, None, :]
    out = v.copy()
    u, w = v[..., 0:dims:2], v[..., 1:dims:2]
    out[..., 0:dims:2] = u * cos - w * sin
    out[..., 1:dims:2] = w * cos + u * sin
    return out


def visible(i, j, size, keep_first=0):
    """Whether the query at position i sees the key at position j."""
    if j > i:
        return False
    if not size or i - j < size:
        return True
    return j < keep_first


def masked_softmax_attention(q, k, v, scale, size, keep_first=0, softcap=None, q_pos=None, k_pos=None):
    """q [Tq, H, dk], k [Tk, H, dk], v [Tk, H, dv] (keys already expanded to the query heads); positions
    default to 0..T-1 on both sides.  Returns [Tq, H, dv]."""
    Tq, H, _ = q.shape
    q_pos = np.arange(Tq) if q_pos is None else np.asarray(q_pos)
    k_pos = np.arange(k.shape[0]) if k_pos is None else np.asarray(k_pos)
    see = np.array([[visible(int(i), int(j), size, keep_first) for j in k_pos] for i in q_pos])
    out = np.zeros((Tq, H, v.shape[-1]))
    for h in range(H):
        s = (q[:, h] @ k[:, h].T) * scale
        if softcap:
            s = softcap * np.tanh(s / softcap)
        s = np.where(see, s, -np.inf)
        s = s - s.max(axis=1, keepdims=True)
        p = np.exp(s)
        p /= p.sum(axis=1, keepdims=True)
        out[:, h] = p @ v[:, h]
    return out


def attention_mixer(h, w, pre, m, eps, positions):
    """Grouped-query attention with an RMS norm over the whole query and the whole key
    projection, partial pair rotation, capped scores, a window and kept first tokens."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_norm(h @ w[pre + "q"].T, w[pre + "q.norm"], eps).reshape(T, H, d)
    k = rms_norm(h @ w[pre + "k"].T, w[pre + "k.norm"], eps).reshape(T, G, d)
    v = (h @ w[pre + "v"].T).reshape(T, G, dv)
    rot = m["rot"]
    q = rotate_pairs(q, positions, rot["dims"], rot["base"], rot.get("scaling"))
    k = rotate_pairs(k, positions, rot["dims"], rot["base"], rot.get("scaling"))
    rep = H // G
    k, v = np.repeat(k, rep, axis=1), np.repeat(v, rep, axis=1)
    mask = m.get("mask") or {}
    o = masked_softmax_attention(q, k, v, m["scale"], mask.get("size", 0), mask.get("keep_first", 0), m.get("softcap"))
    return o.reshape(T, H * dv) @ w[pre + "o"].T


def latent_attention_mixer(h, w, pre, m, eps, positions):
    """Attention whose keys and values are expanded from one normed latent vector per token;
    beside it one rotated key part that all heads share."""
    T = h.shape[0]
    H, d, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = (h @ w[pre + "q"].T).reshape(T, H, d + dr)
    down = h @ w[pre + "dkv"].T
    c = rms_norm(down[:, :r], w[pre + "dkv.norm"], eps)
    rot = m["rot"]
    kr = rotate_pairs(down[:, None, r:], positions, dr, rot["base"], rot.get("scaling"))       # [T, 1, dr]
    qr = rotate_pairs(q[..., d:], positions, dr, rot["base"], rot.get("scaling"))
    k_plain = (c @ w[pre + "uk"].T).reshape(T, H, d)
    v = (c @ w[pre + "uv"].T).reshape(T, H, dv)
    qq = np.concatenate([q[..., :d], qr], axis=-1)
    kk = np.concatenate([k_plain, np.repeat(kr, H, axis=1)], axis=-1)
    mask = m.get("mask") or {}
    o = masked_softmax_attention(qq, kk, v, m["scale"], mask.get("size", 0), mask.get("keep_first", 0), m.get("softcap"))
    return o.reshape(T, H * dv) @ w[pre + "o"].T


def dense_mlp(h, w, pre):
    return relu_squared(h @ w[pre + "up"].T) @ w[pre + "down"].T


def token_side_input(x, tokens, w, layer, dim, eps):
    """The layer's slice of a second embedding table, gated by the stream, projected,
    normed and added."""
    pre = f"l{layer}.side."
    e = w["side.embed"][tokens][:, layer * dim:(layer + 1) * dim]
    g = gelu_tanh(x @ w[pre + "gate"].T) * e
    y = g @ w[pre + "proj"].T
    return x + rms_norm(y, w[pre + "norm"], eps)


MIXERS = {"attention": attention_mixer, "latent_attention": latent_attention_mixer}


def layer_forward(x, tokens, positions, w, cfg, i):
    L = cfg["layers"][i]
    eps = cfg["norm"]["eps"]
    p = f"l{i}."
    mixed = MIXERS[L["type"]](rms_norm(x, w[p + "norm1"], eps), w, p + "mix.", L["mixer"], eps, positions)
    x = x + rms_norm(mixed, w[p + "norm1b"], eps)
    if L.get("mlp"):
        if L["mlp"]["kind"] != "dense":
            raise ValueError(L["mlp"]["kind"])
        x = x + rms_norm(dense_mlp(rms_norm(x, w[p + "norm2"], eps), w, p + "mlp."), w[p + "norm2b"], eps)
    side = cfg.get("token_side")
    if side:
        x = token_side_input(x, tokens, w, i, side["dim"], eps)
    return x


def layer_runs(cfg):
    """[(layer, pass number or None, first of its pass)] in the order they run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None, False) for i in range(n)]
    runs = [(i, None, False) for i in range(loop["start"])]
    for t in range(loop["times"]):
        runs += [(i, t, i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, None, False) for i in range(loop["stop"], n)]


def forward(tokens, w, cfg, collect=None):
    """Logits [T, vocab] of one sequence; `collect` (a list) receives the stream after every layer run."""
    tokens = np.asarray(tokens)
    w = {k: (v.astype(np.float64) if v.dtype.kind == "f" else v) for k, v in w.items()}
    positions = np.arange(len(tokens))
    x0 = w["embed"][tokens]
    x = x0.copy()
    for i, t, first in layer_runs(cfg):
        if first:
            if t > 0:
                x = x + x0
            x = x + w["loop.step"][t]
        x = layer_forward(x, tokens, positions, w, cfg, i)
        if collect is not None:
            collect.append(x.copy())
    return rms_norm(x, w["final.norm"], cfg["norm"]["eps"]) @ w["head"].T
