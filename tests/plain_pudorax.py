"""A plain, slow implementation of the Pudorax decoder in NumPy: whole sequences, no cache, no batches, one
function per mechanism, float64 sums rounded to float32 where the design says 32-bit.  It shares no code with
the package and is the oracle of the tests.

The design in this file's notation (T tokens, width D, position t counted from 0):
  embedding        X = E[token] * embedding.scale;  X0 = X is kept for the loop
  layer            X <- X + mixer(ln1(X));  X <- X + ff(ln2(X)) where the layer has a feed-forward;
                   X <- X + rms(P (gelu_tanh(Gs X) * side[token, layer's slice])) * w_side where the model has a side table
  ln               (x - mean) / sqrt(var + eps) * w + b
  rms              x / sqrt(mean(x^2) + eps)
  short conv       y_t = sum_j c[:, j] u_(t - taps + 1 + j), zeros before the sequence (c's last column is the present)
  attention        q, k, v = conv(Wq h), conv(Wk h), conv(Wv h);  q <- rms(q over ALL its channels) * wq, k likewise;
                   the first rot.dims of each head turned in neighbouring pairs (2i, 2i+1) by t * base^(-2i/dims);
                   causal softmax of q.k * scale, query head a on key head a // (H/G);
                   out = Wo (heads * sigmoid(Wg h))
  mamba2           [z | x | B | C | dt] = Win h;  (x, B, C) <- silu(conv(x, B, C) + bias);  dt <- softplus(dt + dt_bias);
                   S_t = exp(-exp(A_log) dt) S_(t-1) + dt B_t x_t^T;  y_t = S_t^T C_t + D x_t;
                   out = Wo (rms in norm_groups parts of (y * silu(z)) * w)
  feed-forward     z = Wr h + br; the `top` largest, weights softmax over those;  expert(h) = Wd (g' sigmoid(1.702 g') (u' + 1))
                   with g' = min(Wg h, limit), u' = clamp(Wu h, -limit, limit);  plus a shared expert for every token
  loop             layers start..stop-1 run `times` times; before a pass's first layer X <- Win [X; X0]; memory per pass
  output           logits = cap tanh(H ln_final(X) / cap)
"""

from __future__ import annotations

import json
import math
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


def layer_norm(x, w, b, eps):
    x = x.astype(np.float64)
    centred = x - x.mean(axis=-1, keepdims=True)
    var = (centred * centred).mean(axis=-1, keepdims=True)
    return (centred / np.sqrt(var + eps) * w.astype(np.float64) + b.astype(np.float64)).astype(F32)


def sigmoid(x):
    return (1.0 / (1.0 + np.exp(-x.astype(np.float64)))).astype(F32)


def silu(x):
    x = x.astype(np.float64)
    return (x / (1.0 + np.exp(-x))).astype(F32)


def softplus(x):
    x = x.astype(np.float64)
    return np.logaddexp(0.0, x).astype(F32)


def gelu_tanh(x):
    x = x.astype(np.float64)
    return (0.5 * x * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x ** 3)))).astype(F32)


def short_conv(u, taps_weight, bias=None, before=None):
    """u [T, C], taps_weight [C, taps]: every channel filtered over time, the last column on the present row.
    `before` [taps - 1, C] stands ahead of the first row (zeros when a sequence starts)."""
    t_len, channels = u.shape
    taps = taps_weight.shape[1]
    lead = np.zeros((taps - 1, channels), np.float64) if before is None else before.astype(np.float64)
    padded = np.concatenate([lead, u.astype(np.float64)], axis=0)
    out = np.zeros((t_len, channels), np.float64)
    for j in range(taps):
        out += padded[j:j + t_len] * taps_weight[:, j].astype(np.float64)[None, :]
    if bias is not None:
        out += bias.astype(np.float64)[None, :]
    return out.astype(F32)


def rotate_pairs(x, positions, dims, base):
    """x [T, heads, n]: dimensions 2i and 2i+1 (i < dims/2) of every head turned by position * base^(-2i/dims)."""
    half = dims // 2
    freqs = np.array([base ** (-2.0 * i / dims) for i in range(half)], dtype=np.float64).astype(F32)
    angles = (np.asarray(positions, dtype=F32)[:, None] * freqs[None, :]).astype(F32).astype(np.float64)
    cos, sin = np.cos(angles)[:, None, :], np.sin(angles)[:, None, :]
    out = x.astype(np.float64).copy()
    u, v = out[..., 0:dims:2].copy(), out[..., 1:dims:2].copy()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out.astype(F32)


def attention_scores_softmax(q, k, v, scale, first_position=0):
    """q [T, H, d], k [S, G, d], v [S, G, e] with S = first_position + T: causal softmax attention, [T, H, e]."""
    t_len, heads, _ = q.shape
    groups = k.shape[1]
    per = heads // groups
    out = np.zeros((t_len, heads, v.shape[2]), F32)
    for head in range(heads):
        g = head // per
        scores = (q[:, head].astype(np.float64) @ k[:, g].astype(np.float64).T) * scale
        for t in range(t_len):
            row = scores[t, :first_position + t + 1]
            p = np.exp(row - row.max())
            p /= p.sum()
            out[t, head] = (p @ v[:first_position + t + 1, g].astype(np.float64)).astype(F32)
    return out


def gated_attention(h, w, prefix, sizes, eps):
    """h [T, D] from position 0 -> mixer output [T, D]."""
    heads, groups, dim, vdim = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"]
    t_len = h.shape[0]
    q = short_conv(linear(h, w[prefix + "q"]), w[prefix + "q.conv"])
    k = short_conv(linear(h, w[prefix + "k"]), w[prefix + "k.conv"])
    v = short_conv(linear(h, w[prefix + "v"]), w[prefix + "v.conv"])
    q = (rms(q, eps).astype(np.float64) * w[prefix + "q.norm"].astype(np.float64)).astype(F32)
    k = (rms(k, eps).astype(np.float64) * w[prefix + "k.norm"].astype(np.float64)).astype(F32)
    positions = np.arange(t_len)
    q = rotate_pairs(q.reshape(t_len, heads, dim), positions, sizes["rot"]["dims"], sizes["rot"]["base"])
    k = rotate_pairs(k.reshape(t_len, groups, dim), positions, sizes["rot"]["dims"], sizes["rot"]["base"])
    o = attention_scores_softmax(q, k, v.reshape(t_len, groups, vdim), sizes["scale"])
    gate = sigmoid(linear(h, w[prefix + "g"]))
    gated = (o.reshape(t_len, heads * vdim).astype(np.float64) * gate.astype(np.float64)).astype(F32)
    return linear(gated, w[prefix + "o"])


def mamba2(h, w, prefix, sizes, eps):
    """h [T, D] from position 0 -> (mixer output [T, D], state [heads, N, vdim] after the last token)."""
    heads, vdim, n, groups, parts = sizes["heads"], sizes["vdim"], sizes["state"], sizes["groups"], sizes["norm_groups"]
    inner = heads * vdim
    t_len = h.shape[0]
    proj = linear(h, w[prefix + "in"])
    z = proj[:, :inner]
    xbc = silu(short_conv(proj[:, inner:2 * inner + 2 * groups * n], w[prefix + "conv"], w[prefix + "conv.b"]))
    x = xbc[:, :inner].reshape(t_len, heads, vdim).astype(np.float64)
    b = xbc[:, inner:inner + groups * n].reshape(t_len, groups, n).astype(np.float64)
    c = xbc[:, inner + groups * n:].reshape(t_len, groups, n).astype(np.float64)
    dt = softplus(proj[:, 2 * inner + 2 * groups * n:].astype(np.float64) + w[prefix + "dt_bias"].astype(np.float64)).astype(np.float64)
    rate = np.exp(w[prefix + "A_log"].astype(np.float64))
    skip = w[prefix + "D"].astype(np.float64)
    state = np.zeros((heads, n, vdim), np.float64)
    y = np.zeros((t_len, heads, vdim), F32)
    per = heads // groups
    for t in range(t_len):
        for head in range(heads):
            g = head // per
            decay = np.exp(-rate[head] * dt[t, head])
            state[head] = (decay * state[head] + dt[t, head] * np.outer(b[t, g], x[t, head])).astype(F32)   # a float32 state
            y[t, head] = (state[head].T @ c[t, g] + skip[head] * x[t, head]).astype(F32)
    gated = (y.reshape(t_len, inner).astype(np.float64) * silu(z).astype(np.float64)).astype(F32)
    normed = rms(gated.reshape(t_len, parts, inner // parts), eps).reshape(t_len, inner)
    normed = (normed.astype(np.float64) * w[prefix + "norm"].astype(np.float64)).astype(F32)
    return linear(normed, w[prefix + "o"]), state.astype(F32)


def clamped_expert(h, w, prefix, limit):
    g = np.minimum(linear(h, w[prefix + "gate"]).astype(np.float64), limit)
    u = np.clip(linear(h, w[prefix + "up"]).astype(np.float64), -limit, limit)
    y = g / (1.0 + np.exp(-1.702 * g)) * (u + 1.0)
    return linear(y.astype(F32), w[prefix + "down"])


def route(h, w, prefix, top):
    """(chosen experts [T, top], their weights [T, top]): the largest logits, softmax over those alone."""
    logits = linear(h, w[prefix + "router"]).astype(np.float64) + w[prefix + "router.b"].astype(np.float64)
    chosen = np.argsort(-logits, axis=-1, kind="stable")[:, :top]
    picked = np.take_along_axis(logits, chosen, axis=-1)
    p = np.exp(picked - picked.max(axis=-1, keepdims=True))
    return chosen, (p / p.sum(axis=-1, keepdims=True)).astype(F32)


def routed_experts(h, w, prefix, mlp):
    chosen, weights = route(h, w, prefix, mlp["router"]["top"])
    out = np.zeros((h.shape[0], w[prefix + "e0.down"].shape[0]), np.float64)
    for t in range(h.shape[0]):
        for e, share in zip(chosen[t], weights[t]):
            out[t] += float(share) * clamped_expert(h[t:t + 1], w, f"{prefix}e{int(e)}.", mlp["expert"]["limit"])[0].astype(np.float64)
    if mlp.get("shared"):
        out += clamped_expert(h, w, prefix + "shared.", mlp["shared"]["limit"]).astype(np.float64)
    return out.astype(F32)


def token_side(x, tokens, w, prefix, layer, dim, eps):
    """What the per-layer token table adds to the residual x [T, D]."""
    e = w["side.embed"][np.asarray(tokens)][:, layer * dim:(layer + 1) * dim]
    g = (gelu_tanh(linear(x, w[prefix + "side.gate"])).astype(np.float64) * e.astype(np.float64)).astype(F32)
    y = linear(g, w[prefix + "side.proj"])
    return (rms(y, eps).astype(np.float64) * w[prefix + "side.norm"].astype(np.float64)).astype(F32)


def run_order(config):
    """Layer indices in the order they run."""
    count = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(count)), set()
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    order = list(range(start)) + list(range(start, stop)) * times + list(range(stop, count))
    firsts, at = set(), start
    for _ in range(times):
        if stop > start:
            firsts.add(at)
        at += stop - start
    return order, firsts


def forward(config, w, tokens, residual_after_runs=None):
    """Logits [T, vocab] of one whole sequence from position 0; `residual_after_runs` collects X after every layer run."""
    eps = config["norm"]["eps"]
    tokens = np.asarray(tokens)
    x = (w["embed"][tokens].astype(np.float64) * (config.get("embedding") or {}).get("scale", 1.0)).astype(F32)
    x0 = x.copy()
    order, firsts = run_order(config)
    side = config.get("token_side")
    for run, index in enumerate(order):
        layer, p = config["layers"][index], f"l{index}."
        if run in firsts:
            x = linear(np.concatenate([x, x0], axis=1), w["loop.in"])
        h = layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps)
        if layer["type"] == "attention":
            mixed = gated_attention(h, w, p + "mix.", layer["mixer"], eps)
        elif layer["type"] == "mamba2":
            mixed, _ = mamba2(h, w, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = (x.astype(np.float64) + mixed.astype(np.float64)).astype(F32)
        if layer.get("mlp"):
            h = layer_norm(x, w[p + "norm2"], w[p + "norm2.b"], eps)
            x = (x.astype(np.float64) + routed_experts(h, w, p + "mlp.", layer["mlp"]).astype(np.float64)).astype(F32)
        if side:
            x = (x.astype(np.float64) + token_side(x, tokens, w, p, index, side["dim"], eps).astype(np.float64)).astype(F32)
        if residual_after_runs is not None:
            residual_after_runs.append(x.copy())
    h = layer_norm(x, w["final.norm"], w["final.norm.b"], eps)
    logits = linear(h, w["head"]).astype(np.float64)
    cap = config.get("logit_softcap")
    if cap:
        logits = cap * np.tanh(logits / cap)
    return logits.astype(F32)


def greedy(config, w, prompt, n_new):
    """The tokens that greedy decoding adds to `prompt` (the whole sequence run again for every token; ties to the lower id)."""
    fed, out = list(prompt), []
    for _ in range(n_new):
        token = int(np.argmax(forward(config, w, fed)[-1]))
        out.append(token)
        fed.append(token)
    return out
