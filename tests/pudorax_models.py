"""Small Pudorax configurations and random weights for the tests: the tensor list is derived here from the
configuration alone (not from the package's manifest), the weights are drawn so that every mechanism moves the logits
(norm weights and biases away from one and zero, convolution taps of order one, decays that neither vanish nor stay, a
router whose choices vary), and model folders are written with the package's safetensors writer."""

from __future__ import annotations

import json
import os

import numpy as np
import torch


def attention(heads, kv_heads, dim, vdim, conv, scale, rot_dims, base=10000.0, mlp=None):
    return {"type": "attention", "mlp": mlp,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv, "scale": scale,
                      "rot": {"base": base, "dims": rot_dims}}}


def mamba2(heads, vdim, state, groups, norm_groups, conv, mlp=None):
    return {"type": "mamba2", "mlp": mlp,
            "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "norm_groups": norm_groups, "conv": conv}}


def moe(experts, top, ff, limit, shared_ff=None, shared_limit=None):
    mlp = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}
    if shared_ff:
        mlp["shared"] = {"ff": shared_ff, "limit": shared_limit}
    return mlp


# Key and value sizes differ (40 and 24: padded to one cached head of 64), a rotation over part of a head, the loop over
# both kinds of layers three times, five experts of which two are used, no shared expert in one layer, a layer without
# a feed-forward.
MIXED = {
    "architecture": "Pudorax", "vocab": 97, "width": 64, "embedding": {"scale": 2.5}, "logit_softcap": 9.0, "norm": {"eps": 1e-5},
    "token_side": {"dim": 8}, "loop": {"start": 0, "stop": 2, "times": 3},
    "layers": [attention(4, 2, 40, 24, 4, 0.2, 12, base=500.0, mlp=moe(5, 2, 48, 1.2)),
               mamba2(4, 16, 12, 2, 2, 3, mlp=moe(4, 1, 40, 3.0, shared_ff=56, shared_limit=0.8)),
               attention(3, 3, 16, 48, 2, 0.3, 16, mlp=None)],
}
# No loop, no token side input, no cap on the logits, an embedding scale of one; one head, one group, one norm part, one
# expert to choose from; the rotation over a whole head; a head of 128; a convolution of one tap; a state of one row.
PLAIN = {
    "architecture": "Pudorax", "vocab": 131, "width": 96, "norm": {"eps": 1e-6},
    "layers": [attention(1, 1, 128, 128, 1, 0.09, 128, base=20000.0, mlp=moe(1, 1, 64, 2.0)),
               mamba2(1, 64, 1, 1, 1, 2, mlp=None),
               mamba2(6, 8, 40, 3, 1, 5, mlp=moe(3, 3, 32, 1.0, shared_ff=32, shared_limit=1.0))],
}
# A loop that runs once, another that is empty in a copy; eight query heads on one key/value head; no rotation at all;
# a cached head beyond the matrix-core kernels' sizes; a vocabulary smaller than the width.
SINGLE = {
    "architecture": "Pudorax", "vocab": 53, "width": 72, "embedding": {"scale": 0.5}, "logit_softcap": 30.0, "norm": {"eps": 1e-3},
    "token_side": {"dim": 5}, "loop": {"start": 1, "stop": 2, "times": 1},
    "layers": [attention(8, 1, 12, 20, 3, 0.4, 0, mlp=moe(6, 3, 24, 1.5, shared_ff=20, shared_limit=2.5)),
               mamba2(3, 24, 16, 1, 3, 4, mlp=moe(2, 2, 36, 0.7)),
               attention(2, 2, 272, 16, 2, 0.05, 64, base=1e6, mlp=None)],
}
# A long loop over three layers in the middle, twice.
DEEP = {
    "architecture": "Pudorax", "vocab": 211, "width": 128, "embedding": {"scale": 3.0}, "logit_softcap": 12.0, "norm": {"eps": 1e-5},
    "token_side": {"dim": 16}, "loop": {"start": 1, "stop": 4, "times": 2},
    "layers": [mamba2(8, 16, 32, 4, 4, 4, mlp=moe(8, 2, 64, 2.0, shared_ff=96, shared_limit=1.5)),
               attention(8, 2, 32, 32, 3, 0.18, 8, base=1000.0, mlp=moe(8, 4, 32, 1.0, shared_ff=64, shared_limit=2.0)),
               mamba2(4, 32, 16, 1, 2, 2, mlp=None),
               attention(4, 4, 64, 32, 4, 0.125, 32, mlp=moe(16, 3, 48, 2.0)),
               attention(2, 1, 96, 96, 2, 0.1, 48, base=1e5, mlp=moe(4, 2, 80, 4.0, shared_ff=32, shared_limit=1.0))],
}
CONFIGS = {"mixed": MIXED, "plain": PLAIN, "single": SINGLE, "deep": DEEP}


def tensor_shapes(config):
    """{name: shape} of a configuration's checkpoint."""
    width, vocab = config["width"], config["vocab"]
    shapes = {"embed": (vocab, width), "final.norm": (width,), "final.norm.b": (width,), "head": (vocab, width)}
    if config.get("loop"):
        shapes["loop.in"] = (width, 2 * width)
    side = (config.get("token_side") or {}).get("dim", 0)
    if side:
        shapes["side.embed"] = (vocab, len(config["layers"]) * side)
    for index, layer in enumerate(config["layers"]):
        p, m = f"l{index}.", layer["mixer"]
        for q in (1, 2) if layer["mlp"] else (1,):
            shapes[f"{p}norm{q}"] = (width,)
            shapes[f"{p}norm{q}.b"] = (width,)
        if layer["type"] == "attention":
            q_width, k_width, v_width = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            shapes.update({p + "mix.q": (q_width, width), p + "mix.k": (k_width, width), p + "mix.v": (v_width, width),
                           p + "mix.g": (m["heads"] * m["vdim"], width), p + "mix.o": (width, m["heads"] * m["vdim"]),
                           p + "mix.q.norm": (q_width,), p + "mix.k.norm": (k_width,), p + "mix.q.conv": (q_width, m["conv"]),
                           p + "mix.k.conv": (k_width, m["conv"]), p + "mix.v.conv": (v_width, m["conv"])})
        else:
            inner, bc = m["heads"] * m["vdim"], 2 * m["groups"] * m["state"]
            shapes.update({p + "mix.in": (2 * inner + bc + m["heads"], width), p + "mix.conv": (inner + bc, m["conv"]),
                           p + "mix.conv.b": (inner + bc,), p + "mix.dt_bias": (m["heads"],), p + "mix.A_log": (m["heads"],),
                           p + "mix.D": (m["heads"],), p + "mix.norm": (inner,), p + "mix.o": (width, inner)})
        if layer["mlp"]:
            mlp = layer["mlp"]
            shapes.update({p + "mlp.router": (mlp["router"]["experts"], width), p + "mlp.router.b": (mlp["router"]["experts"],)})
            kinds = [(f"e{e}", mlp["expert"]["ff"]) for e in range(mlp["router"]["experts"])]
            if mlp.get("shared"):
                kinds.append(("shared", mlp["shared"]["ff"]))
            for name, ff in kinds:
                shapes.update({f"{p}mlp.{name}.gate": (ff, width), f"{p}mlp.{name}.up": (ff, width), f"{p}mlp.{name}.down": (width, ff)})
        if side:
            shapes.update({p + "side.gate": (side, width), p + "side.proj": (width, side), p + "side.norm": (width,)})
    return shapes


def random_weights(config, seed, gain=1.0):
    """float32 arrays that are exact in bfloat16.  Matrices N(0, gain / sqrt(inputs)), so that activations stay of order
    one; norm weights 1 + N(0, 0.3) with biases N(0, 0.3); convolution taps N(0, 0.6) with the present one near 1;
    A_log in [-2.5, 0.5] (decays from slow to fast), dt_bias in [-3, 1]; router matrices four times the others, so that
    the choice varies from token to token."""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(config).items():
        last = name.split(".")[-1]
        if name in ("embed", "side.embed"):
            values = rng.standard_normal(shape)
        elif last == "conv":
            values = 0.6 * rng.standard_normal(shape)
            values[:, -1] += 1.0
        elif last == "router":
            values = rng.standard_normal(shape) * 4.0 / np.sqrt(shape[1])
        elif len(shape) == 2:
            values = rng.standard_normal(shape) * gain / np.sqrt(shape[1])
        elif last == "A_log":
            values = rng.uniform(-2.5, 0.5, shape)
        elif last == "dt_bias":
            values = rng.uniform(-3.0, 1.0, shape)
        elif last == "b":
            values = 0.3 * rng.standard_normal(shape)
        else:       # norm weights, D
            values = 1.0 + 0.3 * rng.standard_normal(shape)
        out[name] = torch.from_numpy(values.astype(np.float32)).to(torch.bfloat16).to(torch.float32).numpy()
    return out


def write_model(folder, config, weights):
    from beholdd.weights import write_safetensors

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(config, handle)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      {name: torch.from_numpy(np.ascontiguousarray(value)).to(torch.bfloat16) for name, value in weights.items()})
    return str(folder)


def drawn_config(seed):
    """A configuration whose every size, count, constant and layer order is drawn: widths and head sizes that are no
    multiples of 8 among them, key and value sizes that differ, a loop anywhere (also empty, also over everything), with
    and without the token side input, the cap and a shared expert."""
    rng = np.random.default_rng(seed)
    pick = lambda *values: values[int(rng.integers(len(values)))]
    width = int(pick(24, 40, 52, 64, 72, 96, 130))
    n_layers = int(rng.integers(1, 5))
    layers = []
    for _ in range(n_layers):
        mlp = None
        if rng.random() < 0.75:
            experts = int(pick(1, 2, 4, 7, 12))
            shared = int(pick(0, 16, 40))
            mlp = moe(experts, int(rng.integers(1, min(experts, 4) + 1)), int(pick(12, 32, 50)), float(pick(0.5, 1.5, 7.0)),
                      shared_ff=shared, shared_limit=float(pick(0.6, 2.0)))
        if rng.random() < 0.55:
            kv_heads = int(pick(1, 2, 3))
            dim = int(pick(4, 8, 20, 32, 48, 64))
            turned = int(pick(*[d for d in (0, 2, 4, 8, 20, 32, 64) if d <= dim]))
            layers.append(attention(kv_heads * int(pick(1, 2, 4)), kv_heads, dim, int(pick(4, 12, 16, 36, 64)), int(pick(1, 2, 3, 4)),
                                    float(pick(0.1, 0.2, 0.35)), turned, base=float(pick(100.0, 10000.0, 500000.0)), mlp=mlp))
        else:
            groups = int(pick(1, 2, 3))
            heads = groups * int(pick(1, 2, 3))
            vdim = int(pick(4, 8, 12, 32))
            norm_groups = int(pick(*[g for g in (1, 2, 3, 4) if (heads * vdim) % g == 0]))
            layers.append(mamba2(heads, vdim, int(pick(1, 8, 16, 24, 64)), groups, norm_groups, int(pick(2, 3, 4)), mlp=mlp))
    config = {"architecture": "Pudorax", "vocab": int(pick(37, 64, 150, 301)), "width": width,
              "embedding": {"scale": float(pick(0.5, 1.0, 3.0))}, "norm": {"eps": float(pick(1e-6, 1e-5, 1e-3))}, "layers": layers}
    if rng.random() < 0.7:
        config["logit_softcap"] = float(pick(5.0, 15.0, 50.0))
    if rng.random() < 0.7:
        config["token_side"] = {"dim": int(pick(3, 8, 16))}
    if rng.random() < 0.8:
        start = int(rng.integers(0, n_layers + 1))
        config["loop"] = {"start": start, "stop": int(rng.integers(start, n_layers + 1)), "times": int(pick(1, 2, 3))}
    return config
