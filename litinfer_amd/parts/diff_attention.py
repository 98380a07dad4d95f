"""Differential attention over the paged cache: every head has TWO attention maps over the same values,
and puts out their difference.

q has heads * 2 * dim columns and k has kv_heads * 2 * dim, stored head by head as [map 1, map 2]; v has
kv_heads * vdim.  Each map is an attention of its own (score = (q . k) * scale, a window, softmax) with the
head's one value; with a1, a2 the two results and
    lambda = exp(sum(lq1 * lk1)) - exp(sum(lq2 * lk2)) + diff        (one number a layer),
o = a1 - lambda * a2, then o / sqrt(mean(o^2) + eps) over the head's vdim columns, times (1 - diff); the
output projection follows.  No position encoding enters the scores unless one is given.

The rows of Wq and Wk are sorted by map when they are bound, so that each map is an ordinary grouped-query
attention with `heads` query heads on `kv_heads` key heads; the cache keeps three tensors a token (the keys
of map 1, the keys of map 2, the values), and the two maps are two calls of the masked attention kernels
against the same values.  lambda is worked out once, in float32, when the weights are bound.
"""
from __future__ import annotations

import math

import torch

from ..kernels import ops
from ..weights.loader import ParamSpec
from .base import BatchNeeds, Mixer, PagedNeed, PagedTensor, register_part
from .linear import Linear


class DiffAttention(Mixer):
    graph_safe = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        a = spec.args
        self.hidden = int(a["hidden_size"])
        self.nh = int(a["num_heads"])
        self.nkv = int(a.get("num_kv_heads") or self.nh)
        self.dk = int(a["head_dim"])
        self.dv = int(a.get("value_dim") or self.dk)
        self.window = int(a.get("window") or 0)
        self.keep_first = int(a.get("keep_first") or 0) if self.window else 0
        self.softcap = float(a.get("softcap") or 0.0)
        self.scale = float(a["scale"]) if a.get("scale") is not None else self.dk ** -0.5
        self.diff = float(a["diff"])
        self.eps = float(a.get("eps", 1e-6))
        if min(self.nh, self.nkv, self.dk, self.dv) <= 0 or self.nh % self.nkv:
            raise ValueError(f"differential attention: {self.nh} heads are not a multiple of {self.nkv} kv heads")
        if self.window < 0:
            raise ValueError("differential attention: the window must not be negative")
        self.names = {"q": "q", "k": "k", "v": "v", "o": "o", "lq1": "lq1", "lk1": "lk1", "lq2": "lq2", "lk2": "lk2",
                      **(a.get("names") or {})}
        self.n_q, self.n_k, self.n_v = self.nh * self.dk, self.nkv * self.dk, self.nkv * self.dv      # of ONE map
        self.qkv = self.out = None
        self.lam = None

    def cache_need(self):
        return PagedNeed((PagedTensor("k1", (self.nkv, self.dk)), PagedTensor("k2", (self.nkv, self.dk)),
                          PagedTensor("v", (self.nkv, self.dv))), self.window, self.keep_first)

    def batch_needs(self):
        return BatchNeeds(tile_rows=ops.MASKED_TILE_ROWS, token_kinds=True,
                          row_tile=self.qkv.row_tile() if self.qkv is not None else 1)

    def expected_params(self):
        p, n = self.prefix, self.names
        e = {p + n["q"]: ParamSpec((2 * self.n_q, self.hidden)), p + n["k"]: ParamSpec((2 * self.n_k, self.hidden)),
             p + n["v"]: ParamSpec((self.n_v, self.hidden)), p + n["o"]: ParamSpec((self.hidden, self.nh * self.dv))}
        for x in ("lq1", "lk1", "lq2", "lk2"):
            e[p + n[x]] = ParamSpec((self.dk,))
        return e

    @staticmethod
    def _by_map(w: torch.Tensor, heads: int, dim: int) -> torch.Tensor:
        """Rows [head][map][dim] -> [map][head][dim]."""
        return w.reshape(heads, 2, dim, w.shape[1]).transpose(0, 1).reshape(2 * heads * dim, w.shape[1])

    def load_params(self, get):
        p, n = self.prefix, self.names
        wq, wk, wv = get(p + n["q"]), get(p + n["k"]), get(p + n["v"])
        dt = torch.float32 if any(w.dtype is torch.float32 for w in (wq, wk, wv)) else wq.dtype
        packed = torch.cat([self._by_map(wq.to(dt), self.nh, self.dk), self._by_map(wk.to(dt), self.nkv, self.dk), wv.to(dt)], dim=0)
        self.qkv = Linear(self.rt, packed)
        self.out = Linear(self.rt, get(p + n["o"]))
        l = {x: get(p + n[x]).to(torch.float32) for x in ("lq1", "lk1", "lq2", "lk2")}
        s1, s2 = torch.sum(l["lq1"] * l["lk1"]), torch.sum(l["lq2"] * l["lk2"])
        self.lam = float(torch.exp(s1) - torch.exp(s2) + torch.tensor(self.diff, dtype=torch.float32))
        if not math.isfinite(self.lam):
            raise ValueError("differential attention: lambda is not finite")

    def forward(self, xn, residual, ctx, cache):
        t, nq, nk = xn.shape[0], self.n_q, self.n_k
        width = 2 * nq + 2 * nk + self.n_v
        qkv = ctx.ws.buffer("diff_attn.qkv32", (t, width), torch.float32)
        self.qkv(xn, qkv, ws=ctx.ws)
        k1, k2, v = cache.tensors["k1"], cache.tensors["k2"], cache.tensors["v"]
        if cache.owned:
            ops.paged_store(qkv, [(2 * nq, self.nkv, self.dk, k1), (2 * nq + nk, self.nkv, self.dk, k2),
                                  (2 * nq + 2 * nk, self.nkv, self.dv, v)], ctx.slot_map(cache.group), cache.page_size)
        meta = ctx.attention_meta(cache.group)
        flat = qkv.view(-1)
        maps = []
        for m, keys in enumerate((k1, k2)):
            a = ctx.ws.buffer(f"diff_attn.map{m}", (t, self.nh * self.dv), self.rt.dtype)
            ops.masked_attention(flat[m * nq:], width, self.dk, a, keys, v, meta, self.nh, self.nkv, self.dk, self.dv,
                                 cache.page_size, self.window, self.keep_first, self.softcap, self.scale, ws=ctx.ws)
            maps.append(a)
        o = ctx.ws.buffer("attn.out", (t, self.nh * self.dv), self.rt.dtype)
        ops.diff_combine(maps[0], maps[1], self.lam, self.eps, 1.0 - self.diff, o, self.dv)
        residual.add_linear(self.out, o)


register_part("mixer", "diff_attention", DiffAttention)
