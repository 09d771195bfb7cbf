"""Gokazen on the CPU: the configuration and its manifest, the plain implementation's mechanisms against closed forms,
and the engine's own logic (schedule with a loop, state and pages per layer run, slots used again, portions, batches,
generation) with the kernel library replaced by the torch double, against the plain implementation."""

import copy

import numpy as np
import pytest
import torch

import beholdd
import gokazen_models as gm
import plain_gokazen as plain
import schedules
from beholdd.config import ConfigError, GokazenConfig
from beholdd.engine import Engine, StepEntry
from kernel_emulation import TorchKernels


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}

    def get(name, seed=5):
        gain = gm.GAIN.get(name, 1.0)
        key = (name, seed, gain)
        if key not in made:
            config = gm.CONFIGS[name]
            made[key] = (gm.write_model(tmp_path_factory.mktemp(f"gokazen_{name}_{seed}"), config, gm.random_weights(config, seed, gain)),
                         config)
        return made[key]

    return get


def make_engine(folder, dtype="float32", max_tokens=1024, **kw):
    return Engine(folder, dtype=dtype, max_tokens=max_tokens, device="cpu", kernels=TorchKernels(), **kw)


# ---- configuration -----------------------------------------------------------------------------------------

def test_the_loop_repeats_a_stretch_of_layers_with_an_entry_for_every_run():
    config = GokazenConfig.from_dict(gm.DEEP)
    assert config.run_order() == [0, 1, 2, 1, 2, 1, 2, 3]
    assert config.schedule() == [(layer, run) for run, layer in enumerate([0, 1, 2, 1, 2, 1, 2, 3])]
    assert GokazenConfig.from_dict(gm.PLAIN).run_order() == [0, 1, 2]                    # no loop at all
    empty = dict(gm.DEEP, loop={"start": 2, "stop": 2, "times": 5})
    assert GokazenConfig.from_dict(empty).run_order() == [0, 1, 2, 3]                    # an empty stretch
    whole = dict(gm.DEEP, loop={"start": 0, "stop": 4, "times": 2})
    assert GokazenConfig.from_dict(whole).run_order() == [0, 1, 2, 3, 0, 1, 2, 3]


def test_every_constant_comes_from_the_file():
    config = GokazenConfig.from_dict(gm.MIXED)
    assert (config.vocab, config.hidden, config.streams, config.logit_scale, config.rms_eps) == (97, 64, 3, 1.7, 1e-5)
    first, second = config.layers[0].mixer, config.layers[1].mixer
    assert (first.heads, first.dim, first.vdim, first.decay) == (2, 16, 24, (0.9, 0.999))
    assert (second.heads, second.dim, second.rot_dim, second.vdim, second.kv_rank) == (3, 16, 16, 24, 48)
    assert (second.rot_dims, second.rot_base, second.scale) == (8, 500.0, 0.9)
    assert [layer.ff for layer in config.layers] == [80, 0, 72]
    assert GokazenConfig.from_dict(gm.PLAIN).streams == 0 and config.max_position is None


@pytest.mark.parametrize("change,message", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c.pop("logit_scale"), "logit_scale"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][0].update(type="convolution"), "not implemented"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "not implemented"),
    (lambda c: c["layers"][0]["mixer"].update(decay=[0.5]), "decay"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=32), "dims"),
    (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["loop"].update(stop=7), "stop"),
    (lambda c: c.update(layers=[]), "layers"),
])
def test_a_configuration_that_lacks_or_overreaches_is_refused(change, message):
    config = copy.deepcopy(gm.MIXED)
    change(config)
    with pytest.raises(ConfigError, match=message):
        GokazenConfig.from_dict(config)


@pytest.mark.parametrize("name", sorted(gm.CONFIGS))
def test_the_manifest_is_what_the_configuration_implies(name):
    config = gm.CONFIGS[name]
    entry = beholdd.resolve_architecture(config)
    model = entry.build(entry.config_class.from_dict(config))
    assert {spec.name: tuple(spec.shape) for spec in model.tensor_specs()} == gm.tensor_shapes(config)


def test_a_checkpoint_with_other_tensors_is_refused(folders, tmp_path):
    config = gm.CONFIGS["single"]
    weights = gm.random_weights(config, 1)
    weights["l0.hc1.gate"] = weights.pop("l0.hc1.in")
    folder = gm.write_model(tmp_path / "odd", config, weights)
    with pytest.raises(beholdd.WeightError) as caught:
        make_engine(folder)
    assert caught.value.missing == ["l0.hc1.in"] and caught.value.unexpected == ["l0.hc1.gate"]


# ---- the plain implementation's mechanisms against closed forms --------------------------------------------

def test_plain_lightning_is_the_decayed_sum_over_the_past():
    rng = np.random.default_rng(0)
    sizes = {"heads": 2, "dim": 5, "vdim": 3, "decay": [0.8, 0.95]}
    width, t_len = 7, 9
    w = {"m.q": rng.standard_normal((10, width)), "m.k": rng.standard_normal((10, width)), "m.v": rng.standard_normal((6, width)),
         "m.g": rng.standard_normal((6, width)), "m.norm": rng.standard_normal(6), "m.o": np.eye(width, 6)}
    w = {k: v.astype(np.float32) for k, v in w.items()}
    h = rng.standard_normal((t_len, width)).astype(np.float32)
    got, state = plain.lightning_mixer(h, w, "m.", sizes, 1e-6)
    q = plain.silu(h @ w["m.q"].T).reshape(t_len, 2, 5).astype(np.float64)
    k = plain.silu(h @ w["m.k"].T).reshape(t_len, 2, 5).astype(np.float64)
    v = plain.silu(h @ w["m.v"].T).reshape(t_len, 2, 3).astype(np.float64)
    o = np.zeros((t_len, 2, 3))
    for t in range(t_len):
        for j in range(t + 1):
            for head in range(2):
                o[t, head] += sizes["decay"][head] ** (t - j) * (q[t, head] @ k[j, head]) * v[j, head]
    o = o.reshape(t_len, 6)
    want = o / np.sqrt((o * o).mean(-1, keepdims=True) + 1e-6) * w["m.norm"] / (1 + np.exp(-(h @ w["m.g"].T)))
    assert np.abs(got[:, :6] - want).max() < 1e-4 * np.abs(want).max()
    # the state after the last token continues a sequence exactly
    first, carried = plain.lightning_mixer(h[:4], w, "m.", sizes, 1e-6)
    second, _ = plain.lightning_mixer(h[4:], w, "m.", sizes, 1e-6, state=carried)
    assert np.abs(np.concatenate([first, second]) - got).max() < 1e-5 * np.abs(got).max()
    assert state.shape == (2, 5, 3)


def test_plain_latent_attention_depends_on_distances_only_and_on_one_key_as_a_closed_form():
    rng = np.random.default_rng(1)
    sizes = {"heads": 2, "dim": 4, "rot_dim": 6, "vdim": 3, "kv_rank": 5, "scale": 0.7, "rot": {"dims": 4, "base": 50.0}}
    width = 8
    shapes = {"m.q": (20, width), "m.dkv": (11, width), "m.dkv.norm": (5,), "m.uk": (8, 5), "m.uv": (6, 5), "m.o": (width, 6)}
    w = {k: rng.standard_normal(s).astype(np.float32) for k, s in shapes.items()}
    h = rng.standard_normal((6, width)).astype(np.float32)
    at_zero = plain.latent_attention(h, w, "m.", sizes, 1e-6)
    shifted = plain.latent_attention(h, w, "m.", sizes, 1e-6, first_position=37)
    assert np.abs(at_zero - shifted).max() < 2e-5 * np.abs(at_zero).max()
    # the first token sees itself only: its output is Wo Wuv c_0 whatever the query
    down = h[0] @ w["m.dkv"].T
    c = down[:5] / np.sqrt((down[:5] ** 2).mean() + 1e-6) * w["m.dkv.norm"]
    want = w["m.o"] @ (w["m.uv"] @ c)
    assert np.abs(at_zero[0] - want).max() < 1e-5 * np.abs(want).max()
    # the last two of the six rotated dimensions pass unturned: with queries and keys zero elsewhere the scores do
    # not depend on the positions
    still = {k: v.copy() for k, v in w.items()}
    still["m.q"].reshape(2, 10, width)[:, :8] = 0
    still["m.uk"][:] = 0
    still["m.dkv"][5:9] = 0
    near = plain.latent_attention(h, still, "m.", sizes, 1e-6)
    far = plain.latent_attention(h, still, "m.", sizes, 1e-6, first_position=1000)
    assert np.abs(near - far).max() < 1e-6 * np.abs(near).max()


def test_plain_rotation_turns_pairs_half_the_width_apart():
    x = np.zeros((1, 8), np.float32)
    x[0, 1], x[0, 7] = 1.0, 5.0
    out = plain.rotate(x, [3], 6, 100.0)
    angle = np.float32(3) * np.float32(100.0 ** (-2.0 / 6))
    want = np.zeros(8)
    want[1], want[4], want[7] = np.cos(angle), np.sin(angle), 5.0       # dimension 1 pairs with 1 + 3; 6 and 7 pass
    assert np.abs(out[0] - want).max() < 1e-6


def test_plain_streams_with_one_plain_stream_are_a_residual():
    rng = np.random.default_rng(2)
    x, y = rng.standard_normal((4, 6)).astype(np.float32), rng.standard_normal((4, 6)).astype(np.float32)
    w = {"c.mix": np.ones((1, 1), np.float32), "c.out": np.ones(1, np.float32)}
    assert np.array_equal(plain.mix_streams([x], w, "c.", y)[0], (x.astype(np.float64) + y).astype(np.float32))
    w = {"c.mix": np.array([[1, 2], [3, 4]], np.float32), "c.out": np.array([10, 20], np.float32)}
    a, b = plain.mix_streams([x, 2 * x], w, "c.", y)          # [from, to]: the first new stream is 1 * x + 3 * (2 x)
    assert np.allclose(a, 7 * x + 10 * y, atol=1e-5) and np.allclose(b, 10 * x + 20 * y, atol=1e-5)


# ---- the engine's logic with the torch double ----------------------------------------------------------------

@pytest.mark.parametrize("name,lengths", [("mixed", [5, 70, 17, 131]), ("plain", [1, 23, 66]), ("single", [3, 64, 65, 9]),
                                          ("deep", [40, 7, 90])])
def test_every_cut_matches_the_plain_implementation(folders, name, lengths):
    folder, _ = folders(name)
    config, weights = plain.load(folder)
    requests = schedules.random_requests(config["vocab"], lengths, seed=3)
    expected = [plain.forward(config, weights, r) for r in requests]
    engine = make_engine(folder)
    for label, got in (("whole", schedules.whole(engine, requests)),
                       ("tail", schedules.tail_one_by_one(engine, requests, tail=12)),
                       ("batches", schedules.batches(engine, requests, batch_size=3)),
                       ("portions", schedules.portions(engine, requests))):
        for i, (g, e) in enumerate(zip(got, expected)):
            assert g.shape == e.shape, (label, i)
            assert schedules.relative_error(g, e) < 1e-4, (label, i, schedules.relative_error(g, e))
    engine.cache.check_invariants()
    assert engine.cache.live_slots() == []
    assert engine.cache.free_page_count() == engine.cache.n_pages


def test_every_layer_run_has_memory_of_its_own(folders):
    folder, config = folders("deep")
    engine = make_engine(folder)
    needs = engine.model.entry_needs
    assert len(needs) == 8                                      # 4 layers, two of them run three times
    kinds = [needs[run].kind for run in range(8)]
    assert kinds == ["kv", "state", "kv", "state", "kv", "state", "kv", "state"]
    assert needs[1].state_shape == (2, 64, 32) and needs[7].state_shape == (4, 32, 48)
    assert (needs[0].kv_heads, needs[0].head_dim, needs[2].head_dim) == (1, 128, 64)     # the latent and the shared key part
    slot = engine.alloc_slot()
    engine.step([StepEntry(slot, [1, 2, 3, 4, 5], [])])
    states = [g.state for g in engine.cache.groups if g.need.kind == "state" and g.need.state_shape == (2, 64, 32)][0]
    assert states.shape[0] == 3                                 # the three passes of layer 1
    held = [states[run, slot].clone() for run in range(3)]
    assert all(float(h.abs().max()) > 0 for h in held)
    assert not torch.equal(held[0], held[1]) and not torch.equal(held[1], held[2])


def test_a_slot_that_is_used_again_starts_from_nothing(folders):
    folder, _ = folders("mixed")
    config, weights = plain.load(folder)
    first, second = schedules.random_requests(config["vocab"], [80, 30], seed=8)
    engine = make_engine(folder, max_tokens=128, max_slots=1)
    slot = engine.alloc_slot()
    engine.step([StepEntry(slot, first, [])])
    engine.free_slot(slot)
    again = engine.alloc_slot()
    assert again == slot
    got = engine.step([StepEntry(again, second, list(range(len(second))))]).numpy()
    assert schedules.relative_error(got, plain.forward(config, weights, second)) < 1e-4


def test_a_failed_step_puts_state_and_lengths_back(folders):
    folder, _ = folders("single")
    config, weights = plain.load(folder)
    tokens = schedules.random_requests(config["vocab"], [20], seed=4)[0]
    engine = make_engine(folder)
    slot = engine.alloc_slot()
    engine.step([StepEntry(slot, tokens[:10], [])])
    calls = {"n": 0}
    real = engine.kernels.gated_rmsnorm

    def failing(*args, **kw):
        calls["n"] += 1
        if calls["n"] == 2:                   # the second lightning layer of the step: the first has advanced its state
            raise RuntimeError("injected")
        return real(*args, **kw)

    engine.kernels.gated_rmsnorm = failing
    with pytest.raises(RuntimeError, match="injected"):
        engine.step([StepEntry(slot, tokens[10:15], [])])
    engine.kernels.gated_rmsnorm = real
    assert engine.cache.length(slot) == 10
    got = engine.step([StepEntry(slot, tokens[10:], list(range(10)))]).numpy()
    assert schedules.relative_error(got, plain.forward(config, weights, tokens)[10:]) < 1e-4


def test_far_tokens_decide_the_logits_of_the_test_models(folders):
    """The long requests of the tests would not notice a lost far key or state if far tokens did not matter: without
    its first 150 tokens the last position's logits are others, by far more than any tolerance."""
    for name in ("mixed", "deep"):
        folder, _ = folders(name)
        config, weights = plain.load(folder)
        tokens = schedules.random_requests(config["vocab"], [200], seed=21)[0]
        full = plain.forward(config, weights, tokens)[-1]
        cut = plain.forward(config, weights, tokens[150:])[-1]
        assert schedules.relative_error(cut, full) > 0.05, name


def test_greedy_generation_through_the_engine(folders):
    folder, _ = folders("mixed")
    config, weights = plain.load(folder)
    prompts = schedules.random_requests(config["vocab"], [1, 9, 30], seed=6)
    engine = make_engine(folder)
    results = engine.generate(prompts, max_new_tokens=[6, 8, 5])
    for prompt, result, n_new in zip(prompts, results, [6, 8, 5]):
        want = plain.greedy(config, weights, prompt, n_new)
        assert result.token_ids == want, (result.token_ids, want)
    assert len({token for r in results for token in r.token_ids}) >= 4       # the continuations vary
    engine.cache.check_invariants()
    assert engine.cache.live_slots() == []


def test_prompts_longer_than_a_step_go_through_in_portions(folders):
    folder, _ = folders("single")
    config, weights = plain.load(folder)
    prompts = schedules.random_requests(config["vocab"], [50, 3, 21], seed=9)
    engine = make_engine(folder, max_rows_per_step=8)
    results = engine.generate(prompts, max_new_tokens=4)
    for prompt, result in zip(prompts, results):
        assert result.token_ids == plain.greedy(config, weights, prompt, 4)


@pytest.mark.parametrize("seed", range(8))
def test_drawn_configurations_on_the_torch_double(seed, tmp_path):
    """Sizes, counts, constants and layer orders that nobody picked: whole prompts and a tail token by token."""
    config = gm.drawn_config(seed)
    folder = gm.write_model(tmp_path / "drawn", config, gm.random_weights(config, seed, gain=0.7))
    _, weights = plain.load(folder)
    requests = schedules.random_requests(config["vocab"], [1, 19, 70], seed=seed)
    expected = [plain.forward(config, weights, r) for r in requests]
    engine = make_engine(folder)
    for label, got in (("whole", schedules.whole(engine, requests)), ("tail", schedules.tail_one_by_one(engine, requests, tail=5)),
                       ("batches", schedules.batches(engine, requests, batch_size=3))):
        for i, (g, e) in enumerate(zip(got, expected)):
            assert schedules.relative_error(g, e) < 1e-4, (config, label, i, schedules.relative_error(g, e))


def test_the_command_line_plans_the_bytes_of_this_design_without_a_gpu(folders):
    import io
    from beholdd import cli
    folder, _ = folders("deep")
    out = io.StringIO()
    code = cli.main(["generate", "--model", folder, "--prompt-ids", "1,2,3", "--max-new-tokens", "70", "--dtype", "bfloat16",
                     "--plan-only"], out=out)
    text = out.getvalue()
    assert code == 0, text
    # four runs of latent layers (two kinds of cached head) and four of lightning layers (two kinds of state)
    assert "keys/values of 1 layers (1 heads x 128)" in text and "keys/values of 3 layers (1 heads x 64)" in text
    assert "state (2, 64, 32) of 3 layers" in text and "state (4, 32, 48) of 1 layers" in text
    assert "not counted" not in text          # every part says what a step of its allocates
