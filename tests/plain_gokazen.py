"""A plain, slow implementation of the Gokazen decoder in NumPy: whole sequences, no cache, no batches, one
function per mechanism, float64 sums rounded to float32 where the design says 32-bit.  It shares no code with
the package and is the oracle of the tests.

The design in this file's notation (T tokens, width D, residual streams s = 1..S):
  embedding            X_s = E[token] for every stream s
  sublayer q of a layer   u = sum_s a_q[s] X_s;  y = F_q(norm(u)) * ls_q;  X_t <- sum_s M_q[s, t] X_s + b_q[t] y
  norm                 n(x) = x / sqrt(mean(x^2) + eps) * (1 + w)          (the stored weight lies around zero)
  lightning mixer      q = silu(Wq h), k = silu(Wk h), v = silu(Wv h);  S_t = lambda_h S_(t-1) + k_t v_t^T;
                       o_t = S_t^T q_t;  out = Wo (rms(o) * g_norm * sigmoid(Wg h))
  latent attention     q = Wq h = per head [q_c (dim), q_r (rot)];  Wdkv h = [c_raw (rank), k_r (rot)];
                       c = rms(c_raw) * w_c;  score_ij = (q_c,i . (Wuk c_j) + R_i q_r,i . R_j k_r,j) * scale;
                       causal softmax;  out = Wo concat_h sum_j p_ij (Wuv c_j)
  feed-forward         Wdown relu(Wup h)^2
  output               logits = H n_final(sum_s X_s) * logit_scale
  loop                 layers start..stop-1 run `times` times in a row, every pass with its own memory
"""

from __future__ import annotations

import json
import os

import numpy as np

F32 = np.float32


def load(folder):
    """(config dictionary, {name: float32 array}) of a model folder."""
    import torch
    from safetensors import safe_open

    with open(os.path.join(folder, "config.json")) as handle:
        config = json.load(handle)
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as handle:
        weights = {name: handle.get_tensor(name).to(torch.float32).numpy() for name in handle.keys()}
    return config, weights


def linear(x, w):
    """W x for every row of x, summed in float64."""
    return (x.astype(np.float64) @ w.astype(np.float64).T).astype(F32)


def rms(x, eps):
    x = x.astype(np.float64)
    return (x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)).astype(F32)


def zero_centred_norm(x, w, eps):
    return (rms(x, eps).astype(np.float64) * (1.0 + w.astype(np.float64))).astype(F32)


def plain_weight_norm(x, w, eps):
    return (rms(x, eps).astype(np.float64) * w.astype(np.float64)).astype(F32)


def silu(x):
    x = x.astype(np.float64)
    return (x / (1.0 + np.exp(-x))).astype(F32)


def sigmoid(x):
    return (1.0 / (1.0 + np.exp(-x.astype(np.float64)))).astype(F32)


def squared_relu(x):
    r = np.maximum(x.astype(np.float64), 0.0)
    return (r * r).astype(F32)


def rotate(x, positions, dims, base):
    """x [T, ..., n]: the first `dims` of the last axis are turned, dimension i with i + dims/2, by
    position * base^(-2i/dims); the rest passes."""
    half = dims // 2
    freqs = np.array([base ** (-2.0 * i / dims) for i in range(half)], dtype=np.float64).astype(F32)
    angles = (np.asarray(positions, dtype=F32)[:, None] * freqs[None, :]).astype(F32).astype(np.float64)   # the angle is a float32
    shape = (len(positions),) + (1,) * (x.ndim - 2) + (half,)
    cos, sin = np.cos(angles).reshape(shape), np.sin(angles).reshape(shape)
    out = x.astype(np.float64).copy()
    u, v = x[..., :half].astype(np.float64), x[..., half:dims].astype(np.float64)
    out[..., :half] = u * cos - v * sin
    out[..., half:dims] = v * cos + u * sin
    return out.astype(F32)


def lightning_mixer(h, w, prefix, sizes, eps, state=None):
    """h [T, D] -> (mixer output [T, D], state [heads, dim, vdim] after the last token)."""
    heads, dim, vdim, decay = sizes["heads"], sizes["dim"], sizes["vdim"], sizes["decay"]
    t_len = h.shape[0]
    q = silu(linear(h, w[prefix + "q"])).reshape(t_len, heads, dim).astype(np.float64)
    k = silu(linear(h, w[prefix + "k"])).reshape(t_len, heads, dim).astype(np.float64)
    v = silu(linear(h, w[prefix + "v"])).reshape(t_len, heads, vdim).astype(np.float64)
    s = np.zeros((heads, dim, vdim), np.float64) if state is None else state.astype(np.float64)
    o = np.zeros((t_len, heads, vdim), F32)
    for t in range(t_len):
        for head in range(heads):
            s[head] = (np.float64(decay[head]) * s[head] + np.outer(k[t, head], v[t, head])).astype(F32)   # the state is a float32
            o[t, head] = (s[head].T @ q[t, head]).astype(F32)
    normed = plain_weight_norm(o.reshape(t_len, heads * vdim), w[prefix + "norm"], eps)
    gated = (normed.astype(np.float64) * sigmoid(linear(h, w[prefix + "g"])).astype(np.float64)).astype(F32)
    return linear(gated, w[prefix + "o"]), s.astype(F32)


def latent_attention(h, w, prefix, sizes, eps, first_position=0):
    """h [T, D] -> mixer output [T, D]; every position sees itself and what came before."""
    heads, dim, rot_dim, vdim, rank = sizes["heads"], sizes["dim"], sizes["rot_dim"], sizes["vdim"], sizes["kv_rank"]
    turned, base, scale = sizes["rot"]["dims"], sizes["rot"]["base"], sizes["scale"]
    t_len = h.shape[0]
    positions = np.arange(first_position, first_position + t_len)
    q = linear(h, w[prefix + "q"]).reshape(t_len, heads, dim + rot_dim)
    q_plain, q_turned = q[..., :dim], rotate(q[..., dim:], positions, turned, base)
    down = linear(h, w[prefix + "dkv"])
    latent = plain_weight_norm(down[:, :rank], w[prefix + "dkv.norm"], eps)
    k_turned = rotate(down[:, rank:], positions, turned, base)                      # one for all heads
    k_plain = linear(latent, w[prefix + "uk"]).reshape(t_len, heads, dim)
    values = linear(latent, w[prefix + "uv"]).reshape(t_len, heads, vdim)
    out = np.zeros((t_len, heads, vdim), F32)
    for head in range(heads):
        scores = (q_plain[:, head].astype(np.float64) @ k_plain[:, head].astype(np.float64).T
                  + q_turned[:, head].astype(np.float64) @ k_turned.astype(np.float64).T) * np.float64(scale)
        scores = scores.astype(F32).astype(np.float64)
        scores[np.triu_indices(t_len, 1)] = -np.inf
        weights = np.exp(scores - scores.max(axis=-1, keepdims=True))
        weights = (weights / weights.sum(axis=-1, keepdims=True)).astype(F32)
        out[:, head] = (weights.astype(np.float64) @ values[:, head].astype(np.float64)).astype(F32)
    return linear(out.reshape(t_len, heads * vdim), w[prefix + "o"])


def feed_forward(h, w, prefix):
    return linear(squared_relu(linear(h, w[prefix + "up"])), w[prefix + "down"])


def run_order(config):
    """The layer indices in the order in which they run."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n))
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    return list(range(start)) + list(range(start, stop)) * times + list(range(stop, n))


def mix_streams(streams, w, prefix, y):
    """The hyper-connection's write: every new stream from all the old ones, plus its share of y."""
    mix, out = w[prefix + "mix"].astype(np.float64), w[prefix + "out"].astype(np.float64)
    old = [x.astype(np.float64) for x in streams]
    return [(sum(mix[s, t] * old[s] for s in range(len(old))) + out[t] * y.astype(np.float64)).astype(F32)
            for t in range(len(old))]


def forward(config, w, tokens, layer_outputs=None):
    """Logits [T, vocab] of one whole sequence.  `layer_outputs` (a list) receives the sum of the streams after
    every layer run."""
    eps = config["norm"]["eps"]
    n_streams = config.get("streams")
    x = w["embed"][np.asarray(tokens)].astype(F32)
    streams = [x.copy() for _ in range(n_streams or 1)]
    for index in run_order(config):
        layer, prefix = config["layers"][index], f"l{index}."
        for q, kind in ((1, "mixer"), (2, "mlp")):
            if kind == "mlp" and layer["mlp"] is None:
                continue
            if n_streams:
                take = w[f"{prefix}hc{q}.in"].astype(np.float64)
                u = sum(take[s] * streams[s].astype(np.float64) for s in range(n_streams)).astype(F32)
            else:
                u = streams[0]
            h = zero_centred_norm(u, w[f"{prefix}norm{q}"], eps)
            if kind == "mlp":
                if layer["mlp"]["kind"] != "dense":
                    raise ValueError(layer["mlp"]["kind"])
                y = feed_forward(h, w, prefix + "mlp.")
            elif layer["type"] == "lightning":
                y, _ = lightning_mixer(h, w, prefix + "mix.", layer["mixer"], eps)
            elif layer["type"] == "latent_attention":
                y = latent_attention(h, w, prefix + "mix.", layer["mixer"], eps)
            else:
                raise ValueError(layer["type"])
            y = (y.astype(np.float64) * w[f"{prefix}ls{q}"].astype(np.float64)).astype(F32)
            if n_streams:
                streams = mix_streams(streams, w, f"{prefix}hc{q}.", y)
            else:
                streams = [(streams[0].astype(np.float64) + y).astype(F32)]
        if layer_outputs is not None:
            layer_outputs.append(sum(s.astype(np.float64) for s in streams).astype(F32))
    total = sum(s.astype(np.float64) for s in streams).astype(F32)
    return (linear(zero_centred_norm(total, w["final.norm"], eps), w["head"]).astype(np.float64)
            * np.float64(config["logit_scale"])).astype(F32)


def greedy(config, w, prompt, n_new):
    tokens = list(prompt)
    for _ in range(n_new):
        tokens.append(int(np.argmax(forward(config, w, tokens)[-1])))
    return tokens[len(prompt):]
