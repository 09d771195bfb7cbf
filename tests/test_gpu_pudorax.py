"""Pudorax on the GPU: every new kernel alone against the plain implementation's function of the same mechanism, and the
engine over every cut of the work (whole prompts, token by token, portions down to two tokens, batches of unequal
requests, slots and pages used again) in float32 and bfloat16 on configurations that differ in every size, with a key
hundreds of positions back that decides the logits, keys at page borders, the first tokens of a sequence under the
convolutions, long decoding through the captured steps, greedy generation through the entry point and the trace replay
program."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_pudorax as plain
import pudorax_models as pm
import schedules

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOLERANCE = {"float32": 1e-4, "bfloat16": 2e-2}      # max |difference| / max |logit|
DTYPES = [torch.float32, torch.bfloat16]
PAGE = 64


@pytest.fixture(scope="module")
def K():
    from beholdd.kernels import HipKernels
    return HipKernels("cuda:0")


def dev(t, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(t)) if isinstance(t, np.ndarray) else t
    return (t if dtype is None else t.to(dtype)).to("cuda:0")


def rel(got, want):
    got = got.double().cpu().numpy() if isinstance(got, torch.Tensor) else np.asarray(got, np.float64)
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))


def tol(dtype, f32=2e-5, bf16=1.6e-2):
    return f32 if dtype == torch.float32 else bf16


def rounded(values, dtype):
    """Random inputs as the kernel's element type holds them, and the same numbers as float32 for the plain side."""
    t = torch.from_numpy(np.asarray(values, np.float32)).to(dtype)
    return t, t.to(torch.float32).numpy()


def ragged(lengths, slots):
    """The step's integer tensors for sequences of these row counts in these slots."""
    starts = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    row_seq = np.concatenate([np.full(n, i, np.int32) for i, n in enumerate(lengths)])
    return dev(starts), dev(np.asarray(slots, np.int32)), dev(row_seq), starts


# ---- kernels alone ------------------------------------------------------------------------------------------

@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("rows,width,eps", [(1, 48, 1e-6), (33, 1000, 1e-5), (4, 5120, 1e-6), (70, 260, 1e-2), (3, 9001, 1e-6)])
def test_layernorm(K, out_dtype, rows, width, eps):
    rng = np.random.default_rng(width)
    x = (rng.standard_normal((2 * rows, width)) * 3 + 40).astype(np.float32)            # a mean far larger than the spread
    w, b = (1 + 0.3 * rng.standard_normal(width)).astype(np.float32), rng.standard_normal(width).astype(np.float32)
    out = torch.empty(2 * rows, width, dtype=out_dtype, device="cuda:0")
    K.layernorm(dev(x), dev(w), dev(b), eps, out)
    assert rel(out, plain.layer_norm(x, w, b, eps)) < tol(out_dtype, f32=1e-4, bf16=8e-3)
    picked = rng.permutation(2 * rows)[:rows].astype(np.int32)
    out = torch.empty(rows, width, dtype=out_dtype, device="cuda:0")
    K.layernorm(dev(x), dev(w), None, eps, out, rows=dev(picked))
    assert rel(out, plain.layer_norm(x[picked], w, np.zeros(width, np.float32), eps)) < tol(out_dtype, f32=1e-4, bf16=8e-3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_small_row_kernels(K, dtype):
    rng = np.random.default_rng(0)
    a, b = rng.standard_normal((7, 333)).astype(np.float32), rng.standard_normal((7, 333)).astype(np.float32)
    out = torch.empty(7, 666, dtype=dtype, device="cuda:0")
    K.cast_concat(dev(a), dev(b), out)
    assert torch.equal(out.cpu(), torch.from_numpy(np.concatenate([a, b], 1)).to(dtype))
    out = torch.empty(7, 333, dtype=dtype, device="cuda:0")
    K.cast_concat(dev(a), None, out)
    assert torch.equal(out.cpu(), torch.from_numpy(a).to(dtype))
    logits = (rng.standard_normal((5, 77)) * 20).astype(np.float32)
    on_device = dev(logits)
    K.softcap(on_device, 15.0)
    assert rel(on_device, 15.0 * np.tanh(logits.astype(np.float64) / 15.0)) < 1e-6
    hidden, y, w = rng.standard_normal((9, 130)).astype(np.float32), rng.standard_normal((9, 130)).astype(np.float32) * 5, rng.standard_normal(130).astype(np.float32)
    on_device = dev(hidden)
    K.rms_scale_add(on_device, dev(y), dev(w), 1e-5)
    assert rel(on_device, hidden + plain.rms(y, 1e-5).astype(np.float64) * w) < 2e-6
    gate_t, gate = rounded(rng.standard_normal((9, 12)) * 2, dtype)
    table_t, table = rounded(rng.standard_normal((50, 40)), dtype)
    tokens = rng.integers(0, 50, 9).astype(np.int32)
    out = torch.empty(9, 12, dtype=dtype, device="cuda:0")
    K.gelu_gate_table(dev(gate_t), dev(tokens), dev(table_t), 24, out)
    assert rel(out, plain.gelu_tanh(gate).astype(np.float64) * table[tokens][:, 24:36]) < tol(dtype, bf16=8e-3)
    fed = rng.integers(0, 50, 20).astype(np.int32)                    # tokens chosen on the device stand in for some rows'
    src = np.array([-1, 3, -1, 0, 19, -1, -1, 7, 2], np.int32)
    K.gelu_gate_table(dev(gate_t), dev(tokens), dev(table_t), 24, out, token_src=dev(src), fed_tokens=dev(fed))
    actual = np.where(src >= 0, fed[np.maximum(src, 0)], tokens)
    assert rel(out, plain.gelu_tanh(gate).astype(np.float64) * table[actual][:, 24:36]) < tol(dtype, bf16=8e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("channels,taps,lengths,silu", [(70, 4, [5, 1, 31], True), (300, 2, [1, 1, 1], False), (33, 5, [2, 3, 1, 40], True),
                                                        (8, 1, [4, 9], False), (520, 3, [130], True),
                                                        (70, 4, [100, 3, 60, 1, 40], True),      # many rows: the walk down the rows, sequences starting inside a stretch
                                                        (300, 2, [33, 31, 64, 1, 1, 70], False)])
def test_short_conv_and_its_state(K, dtype, channels, taps, lengths, silu):
    """A step's rows after a past of the same length: the state left by the past's step is what the present's rows read,
    also where a sequence brings fewer rows than the state holds."""
    rng = np.random.default_rng(channels + taps)
    first, stride = 11, channels + 20
    w, b = rng.standard_normal((channels, taps)).astype(np.float32), rng.standard_normal(channels).astype(np.float32)
    slots = list(rng.permutation(len(lengths) + 2)[:len(lengths)])
    seq_start, seq_slot, row_seq, starts = ragged(lengths, slots)
    offset = 7
    state = torch.zeros(len(lengths) + 2, offset + (taps - 1) * channels + 3, device="cuda:0")
    past_t, past = rounded(rng.standard_normal((sum(lengths), stride)), dtype)
    now_t, now = rounded(rng.standard_normal((sum(lengths), stride)), dtype)
    out = torch.empty(sum(lengths), channels, device="cuda:0")
    for step_t in (past_t, now_t):
        K.short_conv(dev(step_t), first, dev(w), dev(b), state, offset, row_seq, seq_start, seq_slot, out, silu=silu)
        K.short_conv_state(dev(step_t), first, channels, taps, state, offset, seq_start, seq_slot)
    for i, n in enumerate(lengths):
        lo = starts[i]
        both = np.concatenate([past[lo:lo + n, first:first + channels], now[lo:lo + n, first:first + channels]])
        want = plain.short_conv(both, w, b)
        want = plain.silu(want) if silu else want
        assert rel(out[lo:lo + n], want[n:]) < 1e-5, i
        if taps > 1:
            kept = state[slots[i], offset:offset + (taps - 1) * channels].reshape(taps - 1, channels).cpu().numpy()
            padded = np.concatenate([np.zeros((taps - 1, channels), np.float32), both])
            assert np.array_equal(kept, padded[-(taps - 1):]), i
    assert float(state[:, :offset].abs().max()) == 0 and float(state[:, offset + (taps - 1) * channels:].abs().max()) == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,pad,turned,base", [(6, 2, 24, 40, 64, 8, 1e4), (4, 4, 64, 64, 64, 64, 500.0), (8, 1, 12, 20, 32, 0, 1.0),
                                                                    (2, 2, 272, 16, 272, 64, 1e6), (3, 1, 128, 128, 128, 32, 1e6)])
def test_norm_rotation_cache_write_and_attention(K, dtype, heads, kv_heads, dim, vdim, pad, turned, base):
    """From the convolved rows to the attended heads: norm over the whole projection, rotation in neighbouring pairs, keys and
    values of different sizes through one padded head, a prompt that ends inside its third page and decode rows after it."""
    rng = np.random.default_rng(dim + vdim)
    t_len, eps, scale = 150, 1e-5, 0.2
    q_width, k_width, v_width = heads * dim, kv_heads * dim, kv_heads * vdim
    qkv = rng.standard_normal((t_len, q_width + k_width + v_width)).astype(np.float32)
    wq, wk = (1 + 0.3 * rng.standard_normal(q_width)).astype(np.float32), (1 + 0.3 * rng.standard_normal(k_width)).astype(np.float32)
    positions = np.arange(t_len)
    q = plain.rotate_pairs((plain.rms(qkv[:, :q_width], eps) * wq).reshape(t_len, heads, dim), positions, turned, base)
    k = plain.rotate_pairs((plain.rms(qkv[:, q_width:q_width + k_width], eps) * wk).reshape(t_len, kv_heads, dim), positions, turned, base)
    want = plain.attention_scores_softmax(q, k, qkv[:, q_width + k_width:].reshape(t_len, kv_heads, vdim), scale)
    freq = dev(np.array([base ** (-2.0 * i / turned) for i in range(turned // 2)], np.float32)) if turned else None
    k_pages = torch.zeros(5, kv_heads, PAGE, pad, dtype=dtype, device="cuda:0")
    v_pages = torch.zeros(5, kv_heads, pad, PAGE, dtype=dtype, device="cuda:0")
    table = dev(np.array([[3, 0, 4, 1]], np.int32))

    class Layout:
        n_seqs, seq_start = 1, None
    got = []
    for lo, hi in [(0, 140)] + [(t, t + 1) for t in range(140, t_len)]:
        n = hi - lo
        pos = dev(np.arange(lo, hi, dtype=np.int32))
        q_out = torch.empty(n, heads * pad, dtype=dtype, device="cuda:0")
        K.whole_norm_rope_write(dev(qkv[lo:hi]), dev(wq), dev(wk), eps, freq, turned, pos, dev(np.zeros(n, np.int32)), q_out, k_pages, v_pages,
                                table, heads, kv_heads, dim, vdim, pad, True)
        layout = Layout()
        layout.seq_start, layout.max_rows_per_seq, layout.max_position = dev(np.array([0, n], np.int32)), n, hi - 1
        attended = torch.empty(n, heads * pad, dtype=dtype, device="cuda:0")
        K.attention(q_out, attended, k_pages, v_pages, table, dev(np.zeros(n, np.int32)), pos, heads, kv_heads, pad, scale, 0, layout=layout)
        got.append(attended.float().reshape(n, heads, pad)[..., :vdim].cpu().numpy())
        if pad > vdim:
            assert float(attended.float().reshape(n, heads, pad)[..., vdim:].abs().max()) == 0
    assert rel(np.concatenate(got), want) < tol(dtype, f32=3e-5, bf16=2e-2)
    gate_t, gate = rounded(rng.standard_normal((t_len, 5 + heads * vdim)), dtype)
    att_t, att = rounded(rng.standard_normal((t_len, heads * pad)), dtype)
    out = torch.empty(t_len, heads * vdim, dtype=dtype, device="cuda:0")
    K.gate_heads(dev(att_t), pad, dev(gate_t), 5, out, heads, vdim)
    picked = att.reshape(t_len, heads, pad)[..., :vdim].reshape(t_len, heads * vdim)
    assert rel(out, picked.astype(np.float64) * plain.sigmoid(gate[:, 5:])) < tol(dtype, bf16=8e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,vdim,n_state,groups,lengths", [(6, 32, 24, 2, [5, 1, 31]), (1, 64, 1, 1, [70]), (4, 8, 128, 4, [3, 17, 2]),
                                                               (8, 64, 128, 1, [40]), (3, 12, 40, 3, [1, 1, 1, 1]), (2, 256, 16, 2, [9]),
                                                               (2, 16, 24, 2, [700, 3, 130]),      # long enough to be cut into chunks that run side by side
                                                               (4, 64, 128, 2, [333]),             # chunks whose last one is not full
                                                               (3, 40, 40, 3, [129, 64, 65, 128]), # sequences that end at, before and after a chunk's end
                                                               (1, 48, 200, 1, [150]),             # a state too tall for registers: the walk with the state in LDS
                                                               ])
def test_state_space_scan(K, dtype, heads, vdim, n_state, groups, lengths):
    """The recurrence over ragged rows of several sequences, into slots in another order than the batch's, and then a second
    step that continues from the states the first one left."""
    rng = np.random.default_rng(heads * vdim + n_state)
    inner, bc = heads * vdim, 2 * groups * n_state
    names = {"dt_bias": rng.uniform(-3, 1, heads), "A_log": rng.uniform(-2.5, 0.5, heads), "D": 1 + 0.3 * rng.standard_normal(heads)}
    names = {k: v.astype(np.float32) for k, v in names.items()}
    slots = list(rng.permutation(len(lengths) + 1)[:len(lengths)])
    seq_start, seq_slot, _, starts = ragged(lengths, slots)
    offset = 5
    state = torch.zeros(len(lengths) + 1, offset + heads * n_state * vdim + 2, device="cuda:0")
    total = sum(lengths)
    steps = []
    for _ in range(2):
        xbc = rng.standard_normal((total, inner + bc)).astype(np.float32)
        proj_t, proj = rounded(rng.standard_normal((total, 9 + heads)), dtype)
        out = torch.empty(total, inner, device="cuda:0")
        K.ssm_scan(dev(xbc), dev(proj_t), 9, dev(names["dt_bias"]), dev(names["A_log"]), dev(names["D"]), state, offset, seq_start, seq_slot,
                   out, heads, vdim, n_state, groups, max_rows_per_seq=max(lengths))
        steps.append((xbc, proj, out.cpu().numpy()))
    per = heads // groups
    for i, n in enumerate(lengths):
        lo = starts[i]
        s = np.zeros((heads, n_state, vdim))
        for xbc, proj, got in steps:
            for row in range(lo, lo + n):
                x = xbc[row, :inner].reshape(heads, vdim).astype(np.float64)
                b = xbc[row, inner:inner + groups * n_state].reshape(groups, n_state).astype(np.float64)
                c = xbc[row, inner + groups * n_state:].reshape(groups, n_state).astype(np.float64)
                dt = plain.softplus(proj[row, 9:].astype(np.float64) + names["dt_bias"]).astype(np.float64)
                for h in range(heads):
                    s[h] = np.exp(-np.exp(np.float64(names["A_log"][h])) * dt[h]) * s[h] + dt[h] * np.outer(b[h // per], x[h])
                    want = s[h].T @ c[h // per] + names["D"][h] * x[h]
                    assert np.abs(got[row, h * vdim:(h + 1) * vdim] - want).max() < 2e-4 * max(np.abs(want).max(), 1.0), (i, row, h)
        kept = state[slots[i], offset:offset + heads * n_state * vdim].reshape(heads, n_state, vdim).cpu().numpy()
        assert rel(kept, s) < 2e-5
    assert float(state[:, :offset].abs().max()) == 0 and float(state[:, -2:].abs().max()) == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,pad,turned,taps,lengths", [(6, 2, 24, 40, 64, 8, 4, [5, 1, 31]), (2, 2, 64, 64, 64, 64, 2, [2, 1]),
                                                                            (4, 1, 12, 20, 32, 0, 0, [9]), (3, 3, 32, 16, 32, 16, 1, [3, 3, 3]),
                                                                            (32, 8, 128, 128, 128, 64, 4, [40])])
def test_convolution_norm_rotation_and_write_in_one_launch(K, dtype, heads, kv_heads, dim, vdim, pad, turned, taps, lengths):
    """The one launch against the two it stands for (the convolution, then norm, rotation and write), from a state that an earlier
    step left: the same queries and the same pages."""
    rng = np.random.default_rng(heads * dim + taps)
    channels = (heads + kv_heads) * dim + kv_heads * vdim
    first, total = 6, sum(lengths)
    slots = list(rng.permutation(len(lengths) + 1)[:len(lengths)])
    seq_start, seq_slot, row_seq, starts = ragged(lengths, slots)
    positions = dev(np.concatenate([np.arange(n, dtype=np.int32) + 60 for n in lengths]))
    proj = dev(rounded(rng.standard_normal((total, first + channels + 3)), dtype)[0])
    conv_w = dev(rng.standard_normal((channels, max(taps, 1))).astype(np.float32)) if taps else None
    state = dev((rng.standard_normal((len(lengths) + 1, 4 + max(taps - 1, 0) * channels))).astype(np.float32))
    wq, wk = dev((1 + 0.3 * rng.standard_normal(heads * dim)).astype(np.float32)), dev((1 + 0.3 * rng.standard_normal(kv_heads * dim)).astype(np.float32))
    freq = dev(np.array([1e4 ** (-2.0 * i / turned) for i in range(turned // 2)], np.float32)) if turned else None
    table = dev(rng.permutation(8)[:2 * len(lengths)].reshape(len(lengths), 2).astype(np.int32))      # pages of their own
    outs = []
    for fused in (False, True):
        k_pages = torch.zeros(8, kv_heads, PAGE, pad, dtype=dtype, device="cuda:0")
        v_pages = torch.zeros(8, kv_heads, pad, PAGE, dtype=dtype, device="cuda:0")
        q_out = torch.empty(total, heads * pad, dtype=dtype, device="cuda:0")
        if fused:
            K.conv_norm_rope_write(proj, first, conv_w, state, 4, seq_start, seq_slot, wq, wk, 1e-5, freq, turned, positions, row_seq, q_out,
                                   k_pages, v_pages, table, heads, kv_heads, dim, vdim, pad, True)
        else:
            conv = torch.empty(total, channels, device="cuda:0")
            K.short_conv(proj, first, conv_w if taps else torch.ones(channels, 1, device="cuda:0"), None, state if taps > 1 else None, 4,
                         row_seq, seq_start, seq_slot, conv)
            K.whole_norm_rope_write(conv, wq, wk, 1e-5, freq, turned, positions, row_seq, q_out, k_pages, v_pages, table, heads, kv_heads,
                                    dim, vdim, pad, True)
        outs.append((q_out.float().cpu(), k_pages.float().cpu(), v_pages.float().cpu()))
    for a, b in zip(*outs):
        assert float((a - b).abs().max()) <= (2e-6 if dtype == torch.float32 else 1.6e-2) * max(float(a.abs().max()), 1.0)
    assert float(outs[0][1].abs().max()) > 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,width,groups,eps", [(1, 48, 1, 1e-6), (9, 512, 4, 1e-5), (40, 3000, 3, 1e-6), (5, 192, 2, 1e-3)])
def test_gated_group_rmsnorm(K, dtype, rows, width, groups, eps):
    rng = np.random.default_rng(width)
    y = rng.standard_normal((rows, width)).astype(np.float32) * 4
    z_t, z = rounded(rng.standard_normal((rows, 6 + width)) * 2, dtype)
    w = (1 + 0.3 * rng.standard_normal(width)).astype(np.float32)
    out = torch.empty(rows, width, dtype=dtype, device="cuda:0")
    K.gated_group_rmsnorm(dev(y), dev(z_t), 6, dev(w), eps, out, groups)
    gated = (y.astype(np.float64) * plain.silu(z[:, 6:]).astype(np.float64)).astype(np.float32)
    want = plain.rms(gated.reshape(rows, groups, width // groups), eps).reshape(rows, width).astype(np.float64) * w
    assert rel(out, want) < tol(dtype, bf16=8e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,width,experts,top,ff,limit", [(1, 64, 4, 1, 40, 1.0), (37, 192, 8, 3, 96, 2.0), (5, 130, 5, 5, 33, 0.5), (130, 256, 64, 8, 64, 7.0)])
def test_routed_experts_kernels(K, dtype, rows, width, experts, top, ff, limit):
    rng = np.random.default_rng(rows + experts)
    h_t, h = rounded(rng.standard_normal((rows, width)), dtype)
    names = {"m.router": (rng.standard_normal((experts, width)) * 4 / np.sqrt(width)), "m.router.b": rng.standard_normal(experts)}
    for e in range(experts):
        names.update({f"m.e{e}.gate": rng.standard_normal((ff, width)) / np.sqrt(width) * 2, f"m.e{e}.up": rng.standard_normal((ff, width)) / np.sqrt(width) * 2,
                      f"m.e{e}.down": rng.standard_normal((width, ff)) / np.sqrt(ff)})
    names = {k: rounded(v, dtype)[1] for k, v in names.items()}
    logits = plain.linear(h, names["m.router"])
    chosen = torch.empty(rows, top, dtype=torch.int32, device="cuda:0")
    weights = torch.empty(rows, top, device="cuda:0")
    K.route_top_k(dev(logits), dev(names["m.router.b"]), chosen, weights)
    want_chosen, want_weights = plain.route(h, names, "m.", top)
    assert np.array_equal(chosen.cpu().numpy(), want_chosen) and rel(weights, want_weights) < 1e-5
    w_gu = dev(np.stack([np.concatenate([names[f"m.e{e}.gate"], names[f"m.e{e}.up"]]) for e in range(experts)]), dtype)
    w_d = dev(np.stack([names[f"m.e{e}.down"] for e in range(experts)]), dtype)
    inner = torch.empty(rows * top, ff, dtype=dtype, device="cuda:0")
    K.experts_gate_up(dev(h_t), chosen, w_gu, inner, limit, 1.702)
    hidden = rng.standard_normal((rows, width)).astype(np.float32)
    on_device = dev(hidden)
    K.experts_down(inner, chosen, weights, w_d, on_device)
    mlp = {"router": {"top": top}, "expert": {"limit": limit}}
    assert rel(on_device, hidden.astype(np.float64) + plain.routed_experts(h, names, "m.", mlp)) < tol(dtype, f32=3e-5, bf16=1.2e-2)
    both_t, both = rounded(rng.standard_normal((rows, 2 * ff)) * 3, dtype)
    out = torch.empty(rows, ff, dtype=dtype, device="cuda:0")
    K.clamped_glu(dev(both_t), out, limit, 1.702)
    g, u = np.minimum(both[:, :ff].astype(np.float64), limit), np.clip(both[:, ff:].astype(np.float64), -limit, limit)
    assert rel(out, g / (1 + np.exp(-1.702 * g)) * (u + 1)) < tol(dtype, bf16=8e-3)


@pytest.mark.parametrize("inputs,outputs,counts", [(64, 40, [0, 5, 130, 128, 1, 257]), (128, 64, [3, 0, 0, 70]), (192, 200, [129, 127, 256]),
                                                   (1024, 384, [300, 1, 60, 0, 515])])
def test_all_experts_products_in_one_launch(K, inputs, outputs, counts):
    """Stretches of rows that end at, before and after a tile's end, experts without rows, outputs that fill no whole block."""
    rng = np.random.default_rng(inputs + outputs)
    experts, total, limit = len(counts), sum(counts), 1.5
    rows_t, rows = rounded(rng.standard_normal((total, inputs)), torch.bfloat16)
    gate_up_t, gate_up = rounded(rng.standard_normal((experts, 2 * outputs, inputs)) / np.sqrt(inputs) * 2, torch.bfloat16)
    plain_t, plain_w = rounded(rng.standard_normal((experts, outputs, inputs)) / np.sqrt(inputs), torch.bfloat16)
    starts = np.concatenate([[0], np.cumsum(counts)])
    tiles = dev(np.array([(e, starts[e] + at, min(128, c - at)) for e, c in enumerate(counts) for at in range(0, c, 128)], np.int32))
    gated = torch.full((total, outputs), 7.0, dtype=torch.bfloat16, device="cuda:0")
    K.experts_products(dev(rows_t), dev(gate_up_t), tiles, gated, gated=True, limit=limit, alpha=1.702)
    sums = torch.full((total, outputs), 7.0, device="cuda:0")
    K.experts_products(dev(rows_t), dev(plain_t), tiles, sums)
    for e, c in enumerate(counts):
        if not c:
            continue
        x = rows[starts[e]:starts[e + 1]].astype(np.float64)
        both = x @ gate_up[e].astype(np.float64).T
        g, u = np.minimum(both[:, :outputs], limit), np.clip(both[:, outputs:], -limit, limit)
        assert rel(gated[starts[e]:starts[e + 1]], g / (1 + np.exp(-1.702 * g)) * (u + 1)) < 1e-2, e
        assert rel(sums[starts[e]:starts[e + 1]], x @ plain_w[e].astype(np.float64).T) < 2e-5, e


# ---- the engine over every cut ------------------------------------------------------------------------------------

@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}

    def get(name, seed=5):
        if (name, seed) not in made:
            config = pm.CONFIGS[name]
            weights = pm.random_weights(config, seed)
            made[(name, seed)] = (pm.write_model(tmp_path_factory.mktemp(f"pudorax_{name}_{seed}"), config, weights), config, weights)
        return made[(name, seed)]

    return get


def engine_for(folder, dtype, max_tokens=4096, **kw):
    from beholdd.engine import Engine
    return Engine(folder, dtype=dtype, max_tokens=max_tokens, **kw)


def check(label, got, want, tolerance, stray=0.0):
    """Every position within `tolerance` (max |difference| of its logits over the request's largest |logit|).  With `stray`, the
    median position within it and at most that share of a request's positions beyond it: where a router's two candidates lie
    closer than the rounding of bfloat16 activations, two correct computations choose differently, that position differs by
    more than any rounding, and so does, less and less, whatever later positions read of it through the mixers.  Float32 runs
    allow none; the kernels alone are held to strict bounds in bfloat16 too (the tests above, and the model without experts
    below)."""
    for index, (g, e) in enumerate(zip(got, want)):
        assert g.shape == e.shape, (label, index, g.shape, e.shape)
        assert np.isfinite(g).all(), (label, index)
        per_row = np.abs(g.astype(np.float64) - e).max(axis=1) / np.abs(e).max()
        over = int((per_row >= tolerance).sum())
        if over > stray * len(per_row) or (stray and np.median(per_row) >= tolerance):
            pytest.fail(f"{label}: request {index} (length {len(g)}): {over} positions differ by {tolerance} or more (median "
                        f"{np.median(per_row):.3e}, worst {per_row.max():.3e}); first such position {int(np.argmax(per_row >= tolerance))}")


STRAY = {"float32": 0.0, "bfloat16": 0.35}


def tolerances_for(folder, dtype, requests, want, least=None):
    """A tolerance per request.  Float32: the one tolerance.  Bfloat16: how far the rounding of bfloat16 activations alone moves
    a model's logits depends on the model (sharp scores, small norms' eps, few channels), so a request is held to three times
    what that rounding does to nine in ten of its positions, measured with the torch double of the kernels (exact sums,
    bfloat16 storage), where that is more than the one tolerance."""
    least = TOLERANCE[dtype] if least is None else least
    if dtype == "float32":
        return [least] * len(requests)
    from beholdd.engine import Engine
    from kernel_emulation import TorchKernels
    double = Engine(folder, dtype=dtype, max_tokens=1024, device="cpu", kernels=TorchKernels())
    found = []
    for g, e in zip(schedules.whole(double, requests), want):
        per_row = np.abs(g.astype(np.float64) - e).max(axis=1) / np.abs(e).max()
        found.append(max(least, 3.0 * float(np.quantile(per_row, 0.9))))
    return found


def check_each(label, got, want, tolerances, stray):
    for index, tolerance in enumerate(tolerances):
        check(f"{label} (request {index})", got[index:index + 1], want[index:index + 1], tolerance, stray)


LENGTHS = {"mixed": [5, 11, 1, 70, 33, 128, 300], "plain": [1, 7, 23, 64, 90, 200], "single": [3, 65, 130, 2, 31], "deep": [2, 50, 129, 260]}


@pytest.fixture(scope="module")
def expected(folders):
    cache = {}

    def get(name):
        if name not in cache:
            folder, config, weights = folders(name)
            requests = schedules.random_requests(config["vocab"], LENGTHS[name], seed=11)
            cache[name] = (folder, requests, [plain.forward(config, weights, r) for r in requests])
        return cache[name]

    return get


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(LENGTHS))
def test_every_cut_matches_the_plain_implementation(expected, name, dtype):
    folder, requests, want = expected(name)
    engine = engine_for(folder, dtype)
    tolerances, stray = tolerances_for(folder, dtype, requests, want), STRAY[dtype]
    whole = schedules.whole(engine, requests)
    check_each("whole", whole, want, tolerances, stray)
    tail = schedules.tail_one_by_one(engine, requests, tail=32)
    check_each("last 32 one by one", tail, want, tolerances, stray)
    for batch_size in (3, len(requests)):
        batched = schedules.batches(engine, requests, batch_size=batch_size)
        check_each(f"batches of {batch_size}", batched, want, tolerances, stray)
    in_portions = schedules.portions(engine, requests)
    check_each("portions", in_portions, want, tolerances, stray)
    pairs = schedules.portions(engine, requests, sizes=(2, 2, 3, 2, 1, 2), rest_every=3)
    check_each("portions of two and three", pairs, want, tolerances, stray)
    between = [t / 2 for t in tolerances] if dtype == "float32" else tolerances
    check_each("tail vs whole", tail, whole, between, stray)
    check_each("batches vs whole", batched, whole, between, stray)
    check_each("portions vs whole", in_portions, whole, between, stray)
    engine.cache.check_invariants()
    assert engine.cache.live_slots() == [] and engine.cache.free_page_count() == engine.cache.n_pages


# Without experts nothing magnifies a rounding: both mixers, the token side input and the loop in bfloat16 too, every position.
NO_EXPERTS = {
    "architecture": "Pudorax", "vocab": 83, "width": 64, "embedding": {"scale": 2.0}, "logit_softcap": 20.0, "norm": {"eps": 1e-5},
    "token_side": {"dim": 8}, "loop": {"start": 0, "stop": 2, "times": 2},
    "layers": [pm.attention(4, 2, 32, 48, 3, 0.2, 16, base=1000.0, mlp=None), pm.mamba2(4, 16, 24, 2, 2, 4, mlp=None),
               pm.attention(2, 1, 64, 64, 4, 0.15, 64, mlp=None)],
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_cut_without_experts_holds_at_every_position(tmp_path, dtype):
    config = NO_EXPERTS
    weights = pm.random_weights(config, 7)
    folder = pm.write_model(tmp_path / "bare", config, weights)
    requests = schedules.random_requests(config["vocab"], [1, 9, 66, 130, 200], seed=21)
    want = [plain.forward(config, weights, r) for r in requests]
    engine = engine_for(folder, dtype)
    tolerances = tolerances_for(folder, dtype, requests, want, least=1e-4 if dtype == "float32" else 3e-2)
    for label, got in (("whole", schedules.whole(engine, requests)), ("tail", schedules.tail_one_by_one(engine, requests, tail=40)),
                       ("batches", schedules.batches(engine, requests, batch_size=3)), ("portions", schedules.portions(engine, requests)),
                       ("small portions", schedules.portions(engine, requests, sizes=(2, 2, 3, 2, 1, 2), rest_every=3))):
        check_each(label, got, want, tolerances, 0.0)
    engine.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_batch_changes_nothing_for_its_members(expected, dtype):
    """Rows depend on their batch by rounding alone: a step of many rows runs the experts as matrix products and cuts long
    sequences of the recurrence into chunks, which adds the same float32 terms up in another order."""
    folder, requests, _ = expected("mixed")
    engine = engine_for(folder, dtype)
    alone = schedules.whole(engine, requests)
    from beholdd.engine import StepEntry
    slots = [engine.alloc_slot() for _ in requests]
    together = engine.step([StepEntry(s, r, list(range(len(r)))) for s, r in zip(slots, requests)]).float().cpu().numpy()
    at = 0
    for r, a in zip(requests, alone):
        check("together", [together[at:at + len(r)]], [a], 2e-5 if dtype == "float32" else TOLERANCE[dtype], STRAY[dtype])
        at += len(r)


def far_key_model(tmp_path, seed=3):
    """One attention layer whose last query finds ONE key among hundreds: the token `needle` alone projects onto a key
    direction that the token `asker` alone asks for (sharply: the score stands out by far more than the others' spread), and
    the value behind that key is large, so the asker's logits hang on whether that one far position is read."""
    config = {"architecture": "Pudorax", "vocab": 40, "width": 32, "norm": {"eps": 1e-5},
              "layers": [pm.attention(2, 1, 32, 16, 2, 4.0, 8, base=1e4, mlp=None)]}
    weights = pm.random_weights(config, seed)
    needle, asker = 7, 9
    embed = weights["embed"]
    embed[:, :2] = 0.0                        # the other tokens have nothing in the two dimensions that needle and asker use,
    embed[:, 2:] -= embed[:, 2:].mean(axis=1, keepdims=True)      # and no mean that the layer norm would carry there
    embed[needle] = 0.0
    embed[needle, 0] = 8.0
    embed[asker] = 0.0
    embed[asker, 1] = 8.0
    for name in ("l0.norm1", "final.norm"):
        weights[name][:] = 1.0
        weights[name + ".b"][:] = 0.0
    weights["l0.mix.q"][:] *= 0.05
    weights["l0.mix.k"][:] *= 0.05
    weights["l0.mix.q"][20, 1] = 3.0          # the asker's query: dimension 20 of head 0 (beyond the turned dimensions)
    weights["l0.mix.q"][32 + 20, 1] = 3.0     # and of head 1
    weights["l0.mix.k"][20, 0] = 3.0          # the needle's key: the same dimension
    weights["l0.mix.v"][:, 0] = 2.0           # and a value that stands out
    for name in ("q", "k", "v"):
        weights[f"l0.mix.{name}.conv"][:] = 0.0
        weights[f"l0.mix.{name}.conv"][:, -1] = 1.0
        weights[f"l0.mix.{name}.conv"][:, 0] = 0.25
    weights = {k: torch.from_numpy(v).to(torch.bfloat16).to(torch.float32).numpy() for k, v in weights.items()}
    return pm.write_model(tmp_path / "far", config, weights), config, weights, needle, asker


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("needle_at", [0, 1, 63, 64, 65, 127, 128, 300])
def test_one_far_key_decides(tmp_path, dtype, needle_at):
    """The needle at the first positions, at page borders and hundreds of tokens back; the asker last, in the prompt and decoded."""
    folder, config, weights, needle, asker = far_key_model(tmp_path)
    rng = np.random.default_rng(needle_at)
    others = [t for t in range(config["vocab"]) if t not in (needle, asker)]
    tokens = [int(rng.choice(others)) for _ in range(420)]
    without = list(tokens) + [asker]
    tokens[needle_at] = needle
    tokens.append(asker)
    want, blind = plain.forward(config, weights, tokens)[-1], plain.forward(config, weights, without)[-1]
    assert np.abs(want - blind).max() > 0.2 * np.abs(want).max()                 # the one key moves the logits
    engine = engine_for(folder, dtype, max_tokens=1024)
    from beholdd.engine import StepEntry
    slot = engine.alloc_slot()
    in_prompt = engine.step([StepEntry(slot, tokens, [len(tokens) - 1])]).float().cpu().numpy()[0]
    engine.free_slot(slot)
    slot = engine.alloc_slot()
    engine.step([StepEntry(slot, tokens[:200], [])])
    engine.step([StepEntry(slot, tokens[200:-1], [])])
    decoded = engine.step([StepEntry(slot, tokens[-1:], [0])]).float().cpu().numpy()[0]
    engine.free_slot(slot)
    for got in (in_prompt, decoded):          # scores of order 100 and values of order 10: bfloat16 rounds them to four parts in a thousand
        assert np.abs(got - want).max() < (1e-4 if dtype == "float32" else 5e-2) * np.abs(want).max()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompts_in_portions_and_long_decoding(folders, dtype):
    """A request of 700 tokens: the prompt in portions that end at, before and after page borders, then 150 tokens one by one
    through the captured steps, in a cache whose pages and slots were used before by other requests."""
    folder, config, weights = folders("deep")
    long_one = schedules.random_requests(config["vocab"], [700], seed=31)[0]
    want = plain.forward(config, weights, long_one)
    engine = engine_for(folder, dtype, max_tokens=1024)
    schedules.whole(engine, schedules.random_requests(config["vocab"], [300, 90], seed=32))
    from beholdd.engine import StepEntry
    slot = engine.alloc_slot()
    rows, at = [], 0
    for size in (63, 1, 64, 65, 127, 2, 100, 128):
        rows.append(engine.step([StepEntry(slot, long_one[at:at + size], list(range(size)))]).float().cpu().numpy())
        at += size
    assert at == 550
    for token in long_one[at:]:
        rows.append(engine.step([StepEntry(slot, [token], [0])]).float().cpu().numpy().copy())
    engine.free_slot(slot)
    check("long", [np.concatenate(rows)], [want], TOLERANCE[dtype], STRAY[dtype])
    if engine.graphs is not None:
        assert len(engine.graphs.graphs) >= 1          # the one-token steps were captured and replayed


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_tall_state_through_the_captured_steps(tmp_path, dtype):
    """A state of 256 rows a head: the scan's stage needs more local memory than a kernel may use unasked, in the prompt's chunks
    and in decode steps that are captured and replayed."""
    config = {"architecture": "Pudorax", "vocab": 61, "width": 64, "norm": {"eps": 1e-5}, "token_side": {"dim": 8},
              "layers": [pm.mamba2(2, 64, 256, 1, 2, 3, mlp=None), pm.attention(2, 1, 32, 32, 2, 0.2, 8, mlp=None)]}
    weights = pm.random_weights(config, 13)
    folder = pm.write_model(tmp_path / "tall", config, weights)
    request = schedules.random_requests(config["vocab"], [300], seed=5)[0]
    want = [plain.forward(config, weights, request)]
    engine = engine_for(folder, dtype, max_tokens=512)
    tolerances = tolerances_for(folder, dtype, [request], want, least=1e-4 if dtype == "float32" else 3e-2)
    check_each("whole", schedules.whole(engine, [request]), want, tolerances, 0.0)
    check_each("last 60 one by one", schedules.tail_one_by_one(engine, [request], tail=60), want, tolerances, 0.0)
    if engine.graphs is not None:
        assert len(engine.graphs.graphs) >= 1


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(folders, dtype):
    import beholdd
    folder, config, weights = folders("mixed")
    prompts = schedules.random_requests(config["vocab"], [1, 9, 30, 70], seed=6)
    max_new = [12, 9, 12, 40]
    engine = beholdd.Engine(folder, dtype=dtype, max_tokens=1024)
    results = engine.generate(prompts, max_new_tokens=max_new)
    assert len({token for r in results for token in r.token_ids}) >= 6
    for prompt, result, n in zip(prompts, results, max_new):
        if dtype == "float32":
            assert result.token_ids == plain.greedy(config, weights, prompt, n)
            continue
        fed = list(prompt)
        for token in result.token_ids:          # as good as the plain choice within rounding
            row = plain.forward(config, weights, fed)[-1]
            assert row[token] >= row.max() - 3e-2 * np.abs(row).max(), (fed, token)
            fed.append(token)
    sampled = engine.generate(prompts, max_new_tokens=8, temperature=0.9, top_k=20, top_p=0.9, seed=4)
    again = engine.generate(prompts, max_new_tokens=8, temperature=0.9, top_k=20, top_p=0.9, seed=4)
    assert [r.token_ids for r in sampled] == [r.token_ids for r in again]
    engine.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_and_generate_programs(folders, tmp_path, dtype):
    folder, config, weights = folders("single")
    requests = schedules.random_requests(config["vocab"], [40, 7, 66], seed=9)
    want = [plain.forward(config, weights, r) for r in requests]
    tolerances = tolerances_for(folder, dtype, requests, want)
    steps = schedules.trace_of(schedules.batches, requests, batch_size=3)
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                          "--out", str(tmp_path / "out"), "--max-tokens", "256"],
                         input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    done = {f"r{i}": 0 for i in range(len(requests))}
    for record in steps:
        got = np.fromfile(tmp_path / "out" / f"{record['step']}.f32", dtype="<f4").reshape(-1, config["vocab"])
        rows = []
        for entry in record["entries"]:
            index = int(entry["id"][1:])
            rows.append(want[index][[done[entry["id"]] + w for w in entry["want"]]])
            done[entry["id"]] += len(entry["tokens"])
        check(f"step {record['step']}", [got], [np.concatenate(rows)], max(tolerances), STRAY[dtype])
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "beholdd"), "generate", "--model", folder, "--dtype", dtype,
                          "--prompt-ids", ",".join(str(t) for t in requests[1]), "--max-new-tokens", "5"],
                         capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    if dtype == "float32":
        expected_tokens = plain.greedy(config, weights, requests[1], 5)
        assert all(str(token) in run.stdout for token in expected_tokens), (run.stdout, expected_tokens)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(10))
def test_drawn_configurations(seed, dtype, tmp_path):
    """Sizes, counts, constants and layer orders that nobody picked, on the kernels: every cut against the plain implementation."""
    config = pm.drawn_config(100 + seed)
    folder = pm.write_model(tmp_path / "drawn", config, pm.random_weights(config, seed, gain=0.6))
    _, weights = plain.load(folder)
    requests = schedules.random_requests(config["vocab"], [1, 19, 70, 150], seed=seed)
    want = [plain.forward(config, weights, r) for r in requests]
    engine = engine_for(folder, dtype, max_tokens=1024)
    tolerances = tolerances_for(folder, dtype, requests, want, least=1e-4 if dtype == "float32" else 3e-2)
    for label, got in (("whole", schedules.whole(engine, requests)), ("tail", schedules.tail_one_by_one(engine, requests, tail=20)),
                       ("batches", schedules.batches(engine, requests, batch_size=4)), ("portions", schedules.portions(engine, requests))):
        check_each(f"{label} {config}", got, want, tolerances, STRAY[dtype])
    engine.cache.check_invariants()
