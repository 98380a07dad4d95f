"""A selective state-space mixer (the state-space-duality form) whose state has a fixed size per request.

With inner = heads * vdim, N = state values a column, G groups (head h uses group h // (heads / G)):
the input projection gives [z: inner | x: inner | B: G N | C: G N | dt: heads] a token.  x, B and C pass a
causal convolution per channel over the last `conv` tokens (bias, then silu).  dt <- softplus(dt + dt_bias).
Per head:  S_t = exp(-exp(A_log_h) dt_t) S_{t-1} + dt_t B_t x_t^T  (S: N x vdim),  y_t = S_t^T C_t + D_h x_t.
y is gated by silu(z), RMS-normed in `norm_groups` equal runs of columns (each by its own mean) times a
weight, and projected back.

A request keeps two states in its slot, both float32 and zero at admission: the N x vdim matrices of all
heads, and the last conv - 1 inputs of the convolution.  The projection's result, the convolution, the
decays and step sizes, the recurrence and the norm are float32 in both engine dtypes; the projections
themselves run in the engine's dtype.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import ParamSpec
from .base import BatchNeeds, Mixer, StateNeed, register_part
from .linear import Linear


class Mamba2Mixer(Mixer):
    graph_safe = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        a = spec.args
        self.hidden = int(a["hidden_size"])
        self.heads = int(a["num_heads"])
        self.vdim = int(a["value_dim"])
        self.n_state = int(a["state_size"])
        self.groups = int(a.get("groups") or 1)
        self.taps = int(a.get("conv") or 1)
        self.norm_groups = int(a.get("norm_groups") or 1)
        self.eps = float(a.get("eps", 1e-6))
        self.inner = self.heads * self.vdim
        self.n_bc = self.groups * self.n_state
        self.channels = self.inner + 2 * self.n_bc               # what passes the convolution
        self.n_proj = 2 * self.inner + 2 * self.n_bc + self.heads
        if min(self.heads, self.vdim, self.n_state, self.groups, self.taps, self.norm_groups) <= 0:
            raise ValueError("mamba2: sizes must be positive")
        if self.heads % self.groups:
            raise ValueError(f"mamba2: {self.heads} heads are not a multiple of {self.groups} groups")
        if self.inner % self.norm_groups:
            raise ValueError(f"mamba2: {self.inner} columns do not split into {self.norm_groups} equal norm groups")
        if self.n_state > 256 or self.taps > 64:
            raise ValueError("mamba2: the kernels take states of at most 256 values a column and at most 64 taps")
        self.names = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias", "a_log": "A_log", "d": "D",
                      "norm": "norm", "out": "o", **(a.get("names") or {})}
        self.proj = self.out = self.conv_w = self.conv_b = self.dt_bias = self.a_log = self.d = self.norm_w = None

    def cache_need(self):
        need = [StateNeed((self.heads, self.n_state, self.vdim), torch.float32, name="ssm")]
        if self.taps > 1:
            need.append(StateNeed((self.taps - 1, self.channels), torch.float32, name="conv"))
        return tuple(need)

    def batch_needs(self):
        return BatchNeeds(row_tile=self.proj.row_tile() if self.proj is not None else 1)

    def expected_params(self):
        p, n = self.prefix, self.names
        return {p + n["in"]: ParamSpec((self.n_proj, self.hidden)),
                p + n["conv"]: ParamSpec((self.channels, self.taps)),
                p + n["conv_bias"]: ParamSpec((self.channels,), init="zeros"),
                p + n["dt_bias"]: ParamSpec((self.heads,)),
                p + n["a_log"]: ParamSpec((self.heads,)),
                p + n["d"]: ParamSpec((self.heads,), init="ones"),
                p + n["norm"]: ParamSpec((self.inner,), init="one_plus_normal"),
                p + n["out"]: ParamSpec((self.hidden, self.inner))}

    def load_params(self, get):
        p, n = self.prefix, self.names
        self.proj = Linear(self.rt, get(p + n["in"]))
        self.out = Linear(self.rt, get(p + n["out"]))
        self.conv_w = self.rt.vector(get(p + n["conv"]))
        self.conv_b = self.rt.vector(get(p + n["conv_bias"]))
        self.dt_bias = self.rt.vector(get(p + n["dt_bias"]))
        self.a_log = self.rt.vector(get(p + n["a_log"]))
        self.d = self.rt.vector(get(p + n["d"]))
        self.norm_w = self.rt.vector(get(p + n["norm"]))

    def forward(self, xn, residual, ctx, cache):
        t, inner = xn.shape[0], self.inner
        proj = ctx.ws.buffer("mamba2.proj32", (t, self.n_proj), torch.float32)
        self.proj(xn, proj, ws=ctx.ws)
        z, dt = proj[:, :inner], proj[:, inner + self.channels:]
        xbc = ctx.ws.buffer("mamba2.xbc", (t, self.channels), torch.float32)
        tail = cache.states["conv"] if self.taps > 1 else cache.states["ssm"].view(cache.states["ssm"].shape[0], 1, -1)
        ops.causal_conv_silu(proj[:, inner:inner + self.channels], self.conv_w, self.conv_b, tail, ctx, xbc)
        y = ctx.ws.buffer("mamba2.y", (t, inner), torch.float32)
        ops.ssm_scan(xbc, dt, self.dt_bias, self.a_log, self.d, cache.states["ssm"], ctx, y, self.heads, self.vdim,
                     self.n_state, self.groups, ctx.ws)
        g = ctx.ws.buffer("mamba2.gated", (t, inner), self.rt.dtype)
        ops.gated_group_norm(y, z, self.norm_w, self.eps, self.norm_groups, g)
        residual.add_linear(self.out, g)


register_part("mixer", "mamba2", Mamba2Mixer)
