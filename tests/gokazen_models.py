"""Small Gokazen configurations and random weights for the tests: the tensor list is derived here from the
configuration alone (not from the package's manifest), the weights are drawn so that every mechanism moves the
logits (norm weights away from zero, channel scales and stream matrices away from one and the identity, sharp
attention), and model folders are written with the package's safetensors writer."""

from __future__ import annotations

import json
import os

import numpy as np
import torch


def lightning(heads, dim, vdim, decay, ff=None):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, base=10000.0, dims=None, ff=None):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
                      "rot": {"base": base, "dims": dims or rot_dim}},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


# Three streams; the looped stretch starts at the first layer; a rotation that turns half of the rotated part; one
# cached head of 64 (the matrix-core attention's sizes) and one of 48 (not a multiple of 32); key and value sizes differ.
MIXED = {
    "architecture": "Gokazen", "vocab": 97, "width": 64, "streams": 3, "logit_scale": 1.7, "norm": {"eps": 1e-5},
    "loop": {"start": 0, "stop": 2, "times": 2},
    "layers": [lightning(2, 16, 24, [0.9, 0.999], ff=80),
               latent(3, 16, 16, 24, 48, 0.9, base=500.0, dims=8),
               latent(2, 24, 8, 16, 40, 0.6, base=10000.0, ff=72)],
}
# No streams and no loop at all, a logit scale of one, one lightning head, a cached head of 128.
PLAIN = {
    "architecture": "Gokazen", "vocab": 131, "width": 96, "logit_scale": 1.0, "norm": {"eps": 1e-6},
    "layers": [latent(4, 32, 32, 32, 96, 0.5, base=20000.0, ff=128),
               lightning(1, 64, 64, [0.97]),
               latent(1, 8, 4, 40, 28, 1.3, base=100.0, ff=64)],
}
# One stream with hyper-connections of its own, a loop that runs once, and one that is empty in another copy.
SINGLE = {
    "architecture": "Gokazen", "vocab": 53, "width": 32, "streams": 1, "logit_scale": 0.4, "norm": {"eps": 1e-5},
    "loop": {"start": 1, "stop": 2, "times": 1},
    "layers": [lightning(4, 8, 8, [0.5, 0.8, 0.95, 1.0], ff=48),
               latent(2, 16, 16, 8, 16, 0.7, ff=40),
               lightning(3, 20, 12, [0.99, 0.9, 0.7])],
}
# Four streams and a long loop over both kinds of layers.
DEEP = {
    "architecture": "Gokazen", "vocab": 211, "width": 128, "streams": 4, "logit_scale": 0.5, "norm": {"eps": 1e-6},
    "loop": {"start": 1, "stop": 3, "times": 3},
    "layers": [latent(4, 32, 32, 32, 96, 0.4, ff=160), lightning(2, 64, 32, [0.98, 0.9995]),
               latent(8, 16, 16, 16, 48, 0.5, base=1000.0, ff=96), lightning(4, 32, 48, [0.6, 0.9, 0.99, 0.999], ff=144)],
}
CONFIGS = {"mixed": MIXED, "plain": PLAIN, "single": SINGLE, "deep": DEEP}
# The gain of a configuration's matrices in the tests.  PLAIN has two squared feed-forwards, a sharp attention and no
# logit scale below one: at unit gain the rounding of bfloat16 activations alone (exact sums, the torch double of
# the kernels) moves its logits by 3 %, more than the tests allow the kernels.
GAIN = {"plain": 0.6}


def tensor_shapes(config):
    """{name: shape} of a configuration's checkpoint, and which names hold what kind of numbers."""
    width, streams = config["width"], config.get("streams")
    shapes = {"embed": (config["vocab"], width), "final.norm": (width,), "head": (config["vocab"], width)}
    for index, layer in enumerate(config["layers"]):
        p, m = f"l{index}.", layer["mixer"]
        subs = [1] + ([2] if layer["mlp"] else [])
        for q in subs:
            shapes[f"{p}norm{q}"] = (width,)
            shapes[f"{p}ls{q}"] = (width,)
            if streams:
                shapes[f"{p}hc{q}.in"] = (streams,)
                shapes[f"{p}hc{q}.out"] = (streams,)
                shapes[f"{p}hc{q}.mix"] = (streams, streams)
        if layer["type"] == "lightning":
            keys, values = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            shapes.update({p + "mix.q": (keys, width), p + "mix.k": (keys, width), p + "mix.v": (values, width),
                           p + "mix.g": (values, width), p + "mix.norm": (values,), p + "mix.o": (width, values)})
        else:
            shapes.update({p + "mix.q": (m["heads"] * (m["dim"] + m["rot_dim"]), width),
                           p + "mix.dkv": (m["kv_rank"] + m["rot_dim"], width), p + "mix.dkv.norm": (m["kv_rank"],),
                           p + "mix.uk": (m["heads"] * m["dim"], m["kv_rank"]), p + "mix.uv": (m["heads"] * m["vdim"], m["kv_rank"]),
                           p + "mix.o": (width, m["heads"] * m["vdim"])})
        if layer["mlp"]:
            shapes.update({p + "mlp.up": (layer["mlp"]["ff"], width), p + "mlp.down": (width, layer["mlp"]["ff"])})
    return shapes


def random_weights(config, seed, gain=1.0):
    """float32 arrays that are exact in bfloat16.  Matrices N(0, gain / sqrt(inputs)), so that activations stay of
    order one; zero-centred norm weights N(0, 0.3); plain norm weights and channel scales 1 + N(0, 0.3); stream
    readers and writers around one, stream matrices the identity + N(0, 0.3)."""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(config).items():
        last = name.split(".")[-1]
        if name == "embed":
            values = rng.standard_normal(shape)
        elif len(shape) == 2 and ".hc" not in name:
            values = rng.standard_normal(shape) * gain / np.sqrt(shape[1])
        elif len(shape) == 2:       # a stream matrix
            values = np.eye(shape[0]) + 0.3 * rng.standard_normal(shape)
        elif last in ("norm1", "norm2") or name == "final.norm":
            values = 0.3 * rng.standard_normal(shape)
        else:       # plain norm weights, channel scales, the streams' readers and writers
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
    multiples of 8 among them, one to four streams or none, a loop anywhere (also empty, also over everything)."""
    rng = np.random.default_rng(seed)
    pick = lambda *values: values[int(rng.integers(len(values)))]
    width = int(pick(24, 40, 52, 64, 72, 96, 130))
    n_layers = int(rng.integers(1, 5))
    layers = []
    for index in range(n_layers):
        ff = int(pick(0, 36, 64, 100))
        if rng.random() < 0.5 or (index == n_layers - 1 and not any(l["type"] == "lightning" for l in layers) and rng.random() < 0.7):
            heads = int(pick(1, 2, 3, 5))
            layers.append(lightning(heads, int(pick(4, 12, 16, 33, 64)), int(pick(4, 10, 16, 40, 64, 72)),
                                    [float(pick(0.3, 0.6, 0.9, 0.97, 0.999, 1.0)) for _ in range(heads)], ff=ff))
        else:
            rot_dim = int(pick(2, 4, 8, 16, 24))
            dims = int(pick(*[d for d in (2, 4, 8, 16, 24) if d <= rot_dim]))
            layers.append(latent(int(pick(1, 2, 3, 6)), int(pick(4, 8, 20, 32)), rot_dim, int(pick(4, 12, 16, 36)),
                                 int(pick(8, 24, 30, 40, 56, 112)), float(pick(0.2, 0.35, 0.5, 1.0)),
                                 base=float(pick(100.0, 10000.0, 500000.0)), dims=dims, ff=ff))
    config = {"architecture": "Gokazen", "vocab": int(pick(37, 64, 150, 301)), "width": width,
              "logit_scale": float(pick(0.25, 0.7, 1.0, 3.0)), "norm": {"eps": float(pick(1e-6, 1e-5, 1e-3))}, "layers": layers}
    if rng.random() < 0.8:
        config["streams"] = int(pick(1, 2, 3, 4))
    if rng.random() < 0.8:
        start = int(rng.integers(0, n_layers + 1))
        config["loop"] = {"start": start, "stop": int(rng.integers(start, n_layers + 1)), "times": int(pick(1, 2, 3))}
    return config
