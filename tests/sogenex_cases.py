"""Tiny Sogenex configurations and weights for the tests, made here: sizes that differ in everything from each
other, and weights with gains near one, so that every mechanism moves the logits (the framework's own random
weights are N(0, 0.02): a mixer's fault would hardly show through them)."""
import json
from pathlib import Path

import numpy as np
import torch


def mamba_layer(heads, vdim, state, groups, conv, norm_groups, mlp, weights_of=None):
    L = {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                                     "norm_groups": norm_groups}, "mlp": mlp}
    if weights_of is not None:
        L["weights_of"] = weights_of
    return L


def attention_layer(heads, kv_heads, dim, vdim, window, diff, scale, mlp, weights_of=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": diff, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    L = {"type": "attention", "mixer": m, "mlp": mlp}
    if weights_of is not None:
        L["weights_of"] = weights_of
    return L


def moe(experts, top, ff, shared_ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top},
            "shared": {"ff": shared_ff} if shared_ff else None}


# A: small odd sizes; a state that is no multiple of 16; a layer without feed-forward; two layers that run with
# another layer's tensors; groups, norm groups, kv heads all different from 1 and from each other
MOE_A = moe(5, 2, 40, 56)
CONFIG_A = {"architecture": "Sogenex", "vocab": 211, "width": 96, "norm": {"eps": 1e-6}, "logit_scale": 0.7, "logit_softcap": 9.0,
            "layers": [mamba_layer(6, 16, 24, 3, 4, 2, MOE_A),
                       attention_layer(4, 2, 24, 16, 12, 0.25, 0.2, MOE_A),
                       mamba_layer(3, 40, 8, 1, 2, 3, None),
                       mamba_layer(6, 16, 24, 3, 4, 2, MOE_A, weights_of=0),
                       attention_layer(4, 2, 24, 16, 12, 0.25, 0.2, MOE_A, weights_of=1)]}
# B: attention first and without a window; one kv head; one group, one norm group; every expert chosen in one layer,
# one of them in the other; no shared expert; no cap and no scale of the logits
CONFIG_B = {"architecture": "Sogenex", "vocab": 300, "width": 128, "norm": {"eps": 1e-5},
            "layers": [attention_layer(6, 1, 16, 48, 0, 0.4, 0.25, moe(3, 3, 48, 0)),
                       mamba_layer(4, 32, 16, 1, 2, 1, moe(4, 1, 72, 24)),
                       attention_layer(2, 2, 32, 32, 50, 0.1, 0.17, None)]}
# C: sizes that reach the matrix-core kernels (head size 64, widths in multiples of 32), a state of 128 and one of 160
# values a column, values of 64 and of 32 columns a head
MOE_C = moe(8, 2, 64, 128)
CONFIG_C = {"architecture": "Sogenex", "vocab": 384, "width": 256, "norm": {"eps": 1e-5}, "logit_scale": 1.5, "logit_softcap": 30.0,
            "layers": [mamba_layer(4, 64, 128, 2, 4, 4, MOE_C),
                       attention_layer(8, 2, 64, 64, 33, 0.3, 0.125, MOE_C),
                       mamba_layer(8, 32, 160, 1, 3, 2, moe(6, 4, 96, 0)),
                       attention_layer(8, 2, 64, 64, 33, 0.3, 0.125, MOE_C, weights_of=1)]}
CASES = {"A": (CONFIG_A, 8, 31), "B": (CONFIG_B, 16, 32), "C": (CONFIG_C, 32, 33)}


def draw_weights(config, seed, long_memory=False):
    """name -> float32 array for every tensor of the configuration's model, gains near one.  `long_memory`: half of the
    state-space heads decay by less than a hundredth a token."""
    from litinfer_amd.config import lookup, architecture_name
    from litinfer_amd.engine.model import expected_params_of_spec
    arch = lookup(architecture_name(config))
    spec = arch.model_spec(arch.config_from_dict(config))
    rng = np.random.default_rng(seed)
    out = {}
    for name, p in sorted(expected_params_of_spec(spec).items()):
        shape, leaf = tuple(p.shape), name.split(".")[-1]
        if name.endswith("A_log"):
            a = rng.uniform(-2.0, 0.5, shape)
            if long_memory:
                a[::2] = rng.uniform(-6.0, -5.0, a[::2].shape)
        elif name.endswith("dt_bias"):
            a = rng.normal(0.0, 0.5, shape)
        elif name.endswith(".D"):
            a = rng.normal(1.0, 0.3, shape)
        elif name.endswith("mix.norm"):
            a = rng.normal(1.0, 0.1, shape)
        elif leaf in ("norm1", "norm2") or name == "final.norm":
            a = rng.normal(0.0, 0.1, shape)
        elif name.endswith("conv"):
            a = rng.normal(0.0, 0.5, shape)
        elif name.endswith("conv.b") or name.endswith("router.b"):
            a = rng.normal(0.0, 0.1, shape)
        elif leaf in ("lq1", "lk1", "lq2", "lk2"):
            a = rng.normal(0.0, 0.6 / np.sqrt(shape[0]), shape)
        elif name == "embed":
            a = rng.normal(0.0, 1.0, shape)
        elif leaf == "down" and ".e" in name:
            a = rng.normal(0.0, 0.7 / np.sqrt(shape[1]), shape)
        else:                                       # a matrix [out, in]
            a = rng.normal(0.0, 1.0 / np.sqrt(shape[-1]), shape)
        out[name] = a.astype(np.float32)
    return out


def write_model(folder, config, weights, dtype=torch.float32):
    """config.json and model.safetensors with these weights, stored in `dtype`."""
    from litinfer_amd.weights.safetensors_io import write_safetensors
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(config))
    write_safetensors(folder / "model.safetensors", ((n, torch.from_numpy(a).to(dtype)) for n, a in sorted(weights.items())),
                      metadata={"format": "pt"})
    return folder


def stored(weights, dtype):
    """The weights as a checkpoint of `dtype` holds them, float64."""
    return {n: torch.from_numpy(a).to(dtype).to(torch.float64).numpy() for n, a in weights.items()}
