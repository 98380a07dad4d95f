"""The Sogenex decoder written plainly: NumPy float64, whole sequences, no cache, no batches, one
function per mechanism, each from its equations.  It shares no code with the package; the tests compare
the engine with it.

Notation: T tokens, W the model's width.  Weights are a dict name -> array, linear weights [out, in],
applied as y = x @ w.T.  `cfg` is the parsed config.json.
"""
import math

import numpy as np


def silu(z):
    return z / (1.0 + np.exp(-z))


def softplus(z):
    return np.logaddexp(0.0, z)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def offset_norm(x, w, eps):
    """The layers' norm: the weight is stored around zero, y = rms(x) * (1 + w)."""
    return rms(x, eps) * (1.0 + w)


def sinusoid(positions, width):
    """Row p: entry 2i = sin(p * 10000^(-2i/width)), entry 2i+1 = cos of the same angle."""
    out = np.zeros((len(positions), width))
    for r, p in enumerate(positions):
        for i in range((width + 1) // 2):
            a = p * 10000.0 ** (-2.0 * i / width)
            out[r, 2 * i] = math.sin(a)
            if 2 * i + 1 < width:
                out[r, 2 * i + 1] = math.cos(a)
    return out


def embed(ids, table, first_position=0):
    ids = np.asarray(ids)
    return table[ids] + sinusoid(np.arange(first_position, first_position + len(ids)), table.shape[1])


# ------------------------------------------------------------------------------------------ mamba2
def causal_conv(u, w, b):
    """u [T, C]; w [C, taps], the last column multiplies the current token; zeros before the start."""
    T, C = u.shape
    taps = w.shape[1]
    out = np.zeros((T, C))
    for t in range(T):
        acc = b.copy()
        for j in range(taps):
            s = t - (taps - 1 - j)
            if s >= 0:
                acc = acc + w[:, j] * u[s]
        out[t] = acc
    return out


def ssm_scan(x, B, C, dt, A_log, D, heads, vdim, groups, state):
    """x [T, heads*vdim], B and C [T, groups*state], dt [T, heads] (after the softplus).
    S_t = exp(-exp(A_log_h) dt) S_{t-1} + dt B_t x_t^T (S: state x vdim); y_t = S_t^T C_t + D_h x_t."""
    T = x.shape[0]
    y = np.zeros((T, heads * vdim))
    per = heads // groups
    for h in range(heads):
        g = h // per
        S = np.zeros((state, vdim))
        a = math.exp(A_log[h])
        for t in range(T):
            xt = x[t, h * vdim:(h + 1) * vdim]
            Bt, Ct = B[t, g * state:(g + 1) * state], C[t, g * state:(g + 1) * state]
            S = math.exp(-a * dt[t, h]) * S + dt[t, h] * np.outer(Bt, xt)
            y[t, h * vdim:(h + 1) * vdim] = S.T @ Ct + D[h] * xt
    return y


def grouped_rms(y, parts, eps):
    T, n = y.shape
    return rms(y.reshape(T, parts, n // parts), eps).reshape(T, n)


def mamba2(h, w, p, m, eps):
    """The whole mixer for a sequence from its start.  m: the layer's 'mixer' object of config.json."""
    heads, vdim, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = heads * vdim
    proj = h @ w[p + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[p + "conv"], w[p + "conv.b"]))
    x, B, C = xbc[:, :inner], xbc[:, inner:inner + G * N], xbc[:, inner + G * N:]
    dt = softplus(dt + w[p + "dt_bias"])
    y = ssm_scan(x, B, C, dt, w[p + "A_log"], w[p + "D"], heads, vdim, G, N)
    y = grouped_rms(y * silu(z), m["norm_groups"], eps) * w[p + "norm"]
    return y @ w[p + "o"].T


# ------------------------------------------------------------------------------ differential attention
def visible(i, j, window):
    return 0 <= i - j and (window <= 0 or i - j < window)


def softmax_attention(q, k, v, scale, window):
    """q [T, d], k [T, d], v [T, dv]: one head, causal, position i sees j with 0 <= i - j < window."""
    T = q.shape[0]
    out = np.zeros((T, v.shape[1]))
    for i in range(T):
        js = [j for j in range(T) if visible(i, j, window)]
        s = np.array([q[i] @ k[j] for j in js]) * scale
        s = np.exp(s - s.max())
        s = s / s.sum()
        out[i] = s @ v[js]
    return out


def diff_lambda(w, p, diff):
    return math.exp(float(np.sum(w[p + "lq1"] * w[p + "lk1"]))) - math.exp(float(np.sum(w[p + "lq2"] * w[p + "lk2"]))) + diff


def diff_attention(h, w, p, m, eps):
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    window = (m.get("mask") or {}).get("size") or 0
    q, k, v = h @ w[p + "q"].T, h @ w[p + "k"].T, h @ w[p + "v"].T
    lam = diff_lambda(w, p, m["diff"])
    T = h.shape[0]
    out = np.zeros((T, H * dv))
    for hd in range(H):
        g = hd // (H // G)
        vh = v[:, g * dv:(g + 1) * dv]
        maps = []
        for part in range(2):
            qh = q[:, (2 * hd + part) * d:(2 * hd + part + 1) * d]
            kh = k[:, (2 * g + part) * d:(2 * g + part + 1) * d]
            maps.append(softmax_attention(qh, kh, vh, m["scale"], window))
        o = maps[0] - lam * maps[1]
        out[:, hd * dv:(hd + 1) * dv] = rms(o, eps) * (1.0 - m["diff"])
    return out @ w[p + "o"].T


# ------------------------------------------------------------------------------------- feed-forward
def relu2_expert(h, up, down):
    return np.maximum(h @ up.T, 0.0) ** 2 @ down.T


def route(h, router, bias, top):
    """(chosen experts [T, top], their weights [T, top]): the largest logits, softmax over the chosen ones."""
    z = h @ router.T + bias
    idx = np.argsort(-z, axis=-1, kind="stable")[:, :top]
    zc = np.take_along_axis(z, idx, axis=-1)
    e = np.exp(zc - zc.max(axis=-1, keepdims=True))
    return idx, e / e.sum(axis=-1, keepdims=True)


def moe(h, w, p, mlp):
    T = h.shape[0]
    out = np.zeros((T, w[p + "e0.down"].shape[0]))
    idx, wt = route(h, w[p + "router"], w[p + "router.b"], mlp["router"]["top"])
    for t in range(T):
        for e, a in zip(idx[t], wt[t]):
            out[t] += a * relu2_expert(h[t:t + 1], w[p + f"e{e}.up"], w[p + f"e{e}.down"])[0]
    if mlp.get("shared"):
        gate = sigmoid(h @ w[p + "shared.sg"].T)                 # [T, 1]
        out = out + gate * relu2_expert(h, w[p + "shared.up"], w[p + "shared.down"])
    return out


# ------------------------------------------------------------------------------------------- model
def layer_prefix(cfg, i):
    """Layer i's tensors: its own, or those of the layer it names with 'weights_of'."""
    j = cfg["layers"][i].get("weights_of")
    return f"l{i if j is None else j}."


def forward(cfg, w, ids, taps=None):
    """Logits [T, vocab] of a whole sequence.  `taps`, a list, receives the stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = embed(ids, w["embed"])
    for i, L in enumerate(cfg["layers"]):
        p = layer_prefix(cfg, i)
        hn = offset_norm(x, w[p + "norm1"], eps)
        if L["type"] == "mamba2":
            x = x + mamba2(hn, w, p + "mix.", L["mixer"], eps)
        elif L["type"] == "attention":
            x = x + diff_attention(hn, w, p + "mix.", L["mixer"], eps)
        else:
            raise ValueError(L["type"])
        if L.get("mlp") is not None:
            x = x + moe(offset_norm(x, w[p + "norm2"], eps), w, p + "mlp.", L["mlp"])
        if taps is not None:
            taps.append(x.copy())
    return head(cfg, w, x)


def head(cfg, w, x):
    logits = offset_norm(x, w["final.norm"], cfg["norm"]["eps"]) @ w["head"].T * cfg.get("logit_scale", 1.0)
    cap = cfg.get("logit_softcap") or 0.0
    return cap * np.tanh(logits / cap) if cap else logits
