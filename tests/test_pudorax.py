"""Pudorax on the CPU: the configuration and its manifest, the plain implementation's mechanisms against closed forms,
and the engine's own logic (schedule with a loop entered through a matrix, pages with a state beside them, state
regions, slots used again, portions, batches, generation) with the kernel library replaced by the torch double,
against the plain implementation."""

import copy

import numpy as np
import pytest
import torch

import beholdd
import plain_pudorax as plain
import pudorax_models as pm
import schedules
from beholdd.config import ConfigError, PudoraxConfig
from beholdd.engine import Engine, StepEntry
from kernel_emulation import TorchKernels


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


def make_engine(folder, dtype="float32", max_tokens=1024, **kw):
    return Engine(folder, dtype=dtype, max_tokens=max_tokens, device="cpu", kernels=TorchKernels(), **kw)


# ---- configuration -----------------------------------------------------------------------------------------

def test_the_loop_repeats_a_stretch_and_names_where_its_passes_start():
    config = PudoraxConfig.from_dict(pm.DEEP)
    assert config.run_order() == [0, 1, 2, 3, 1, 2, 3, 4]
    assert config.schedule() == [(layer, run) for run, layer in enumerate([0, 1, 2, 3, 1, 2, 3, 4])]
    assert config.pass_starts() == [1, 4]
    assert PudoraxConfig.from_dict(pm.MIXED).pass_starts() == [0, 2, 4]
    plain_config = PudoraxConfig.from_dict(pm.PLAIN)
    assert plain_config.run_order() == [0, 1, 2] and plain_config.pass_starts() == [] and not plain_config.has_loop
    empty = PudoraxConfig.from_dict(dict(pm.DEEP, loop={"start": 2, "stop": 2, "times": 5}))
    assert empty.run_order() == [0, 1, 2, 3, 4] and empty.pass_starts() == [] and empty.has_loop


def test_every_constant_comes_from_the_file():
    config = PudoraxConfig.from_dict(pm.MIXED)
    assert (config.vocab, config.hidden, config.embedding_scale, config.logit_softcap, config.rms_eps, config.token_side_dim) == \
        (97, 64, 2.5, 9.0, 1e-5, 8)
    first, second = config.layers[0], config.layers[1]
    m = first.mixer
    assert (m.heads, m.kv_heads, m.dim, m.vdim, m.conv, m.rot_dims, m.rot_base, m.scale) == (4, 2, 40, 24, 4, 12, 500.0, 0.2)
    assert (first.mlp.experts, first.mlp.top, first.mlp.expert.ff, first.mlp.expert.limit, first.mlp.shared) == (5, 2, 48, 1.2, None)
    s = second.mixer
    assert (s.heads, s.vdim, s.state, s.groups, s.norm_groups, s.conv) == (4, 16, 12, 2, 2, 3)
    assert (second.mlp.shared.ff, second.mlp.shared.limit) == (56, 0.8) and config.layers[2].mlp is None
    bare = PudoraxConfig.from_dict(pm.PLAIN)
    assert (bare.embedding_scale, bare.logit_softcap, bare.token_side_dim, bare.max_position) == (1.0, 0.0, 0, None)


@pytest.mark.parametrize("change,message", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][0].update(type="convolution"), "not implemented"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "not implemented"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "kv_heads"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=42), "dims"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "dims"),
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][1]["mixer"].update(groups=3), "groups"),
    (lambda c: c["layers"][1]["mixer"].update(norm_groups=5), "norm_groups"),
    (lambda c: c["layers"][1]["mixer"].pop("state"), "state"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=6), "top"),
    (lambda c: c["layers"][0]["mlp"]["expert"].pop("limit"), "limit"),
    (lambda c: c["loop"].update(stop=7), "stop"),
    (lambda c: c.update(layers=[]), "layers"),
])
def test_a_configuration_that_lacks_or_overreaches_is_refused(change, message):
    config = copy.deepcopy(pm.MIXED)
    change(config)
    with pytest.raises(ConfigError, match=message):
        PudoraxConfig.from_dict(config)


@pytest.mark.parametrize("name", sorted(pm.CONFIGS))
def test_the_manifest_is_the_list_derived_from_the_configuration(name):
    config = pm.CONFIGS[name]
    model = beholdd.registry.resolve_architecture(config).build(PudoraxConfig.from_dict(config))
    assert {spec.name: tuple(spec.shape) for spec in model.tensor_specs()} == pm.tensor_shapes(config)


def test_the_cached_head_holds_keys_and_values_of_different_sizes():
    model = beholdd.registry.resolve_architecture(pm.MIXED).build(PudoraxConfig.from_dict(pm.MIXED))
    needs = model.entry_needs
    assert len(needs) == 7                                            # two layers in three passes, and the last layer: memory per run
    first = needs[0]
    assert (first.kind, first.kv_heads, first.head_dim) == ("kv", 2, 64)           # 40 and 24 under one size of 64
    assert first.state_shape == (3 * (4 * 40 + 2 * 40 + 2 * 24),)                  # the last three projected rows
    assert needs[1].kind == "state" and needs[1].state_shape == (4 * 12 * 16 + 2 * (64 + 2 * 2 * 12),)
    single = beholdd.registry.resolve_architecture(pm.SINGLE).build(PudoraxConfig.from_dict(pm.SINGLE))
    assert single.entry_needs[2].head_dim == 272                      # beyond 256: as large as the larger of the two


# ---- the plain implementation's mechanisms against closed forms -------------------------------------------------

def test_short_conv_is_a_causal_filter_that_can_be_continued():
    rng = np.random.default_rng(0)
    u, w, b = rng.standard_normal((9, 3)).astype(np.float32), rng.standard_normal((3, 4)).astype(np.float32), rng.standard_normal(3).astype(np.float32)
    got = plain.short_conv(u, w, b)
    for c in range(3):
        full = np.convolve(u[:, c].astype(np.float64), w[c, ::-1].astype(np.float64))[:9] + b[c]
        assert np.allclose(got[:, c], full, atol=1e-6)
    assert np.allclose(plain.short_conv(u[5:], w, b, before=u[2:5]), got[5:], atol=1e-6)      # continued from its last inputs
    assert np.allclose(plain.short_conv(u[:1], w), (u[:1] * w[:, -1]), atol=1e-7)             # the first token sees only itself


def test_rotation_turns_neighbouring_pairs_and_depends_on_the_distance_alone():
    rng = np.random.default_rng(1)
    q, k = rng.standard_normal((1, 1, 10)).astype(np.float32), rng.standard_normal((1, 1, 10)).astype(np.float32)
    turned = plain.rotate_pairs(q, [7], 6, 100.0)
    assert np.allclose(turned[..., 6:], q[..., 6:])                                           # what lies beyond `dims` passes
    angle = np.float32(7) * np.float32(100.0 ** (-2 / 6))
    assert np.allclose(turned[0, 0, 2], q[0, 0, 2] * np.cos(angle) - q[0, 0, 3] * np.sin(angle), atol=1e-6)
    assert np.allclose(turned[0, 0, 3], q[0, 0, 3] * np.cos(angle) + q[0, 0, 2] * np.sin(angle), atol=1e-6)
    score = lambda a, b: float((plain.rotate_pairs(q, [a], 6, 100.0) * plain.rotate_pairs(k, [b], 6, 100.0)).sum())
    assert abs(score(12, 5) - score(107, 100)) < 1e-4 and abs(score(12, 5) - score(12, 6)) > 1e-3


def test_the_state_space_recurrence_is_a_decaying_sum():
    """One head, one state row, constant inputs: S_t = a S_(t-1) + dt B x, so S_t = dt B x (1 - a^t) / (1 - a)."""
    sizes = {"heads": 1, "vdim": 2, "state": 1, "groups": 1, "norm_groups": 1}
    width, taps, t_len = 4, 2, 6
    w = {"m.in": np.zeros((2 * 2 + 2 + 1, width), np.float32), "m.conv": np.zeros((4, taps), np.float32), "m.conv.b": np.zeros(4, np.float32),
         "m.dt_bias": np.array([0.3], np.float32), "m.A_log": np.array([-0.5], np.float32), "m.D": np.array([0.0], np.float32),
         "m.norm": np.ones(2, np.float32), "m.o": np.eye(width, 2, dtype=np.float32)}
    w["m.conv.b"][:] = [1.0, 2.0, 0.7, 1.3]                       # x = silu(1), silu(2); B = silu(0.7); C = silu(1.3): the same in every row
    _, state = plain.mamba2(np.ones((t_len, width), np.float32), w, "m.", sizes, 1e-6)
    silu = lambda v: v / (1 + np.exp(-v))
    dt = np.log1p(np.exp(0.3))
    a = np.exp(-np.exp(-0.5) * dt)
    want = dt * silu(0.7) * np.array([silu(1.0), silu(2.0)]) * (1 - a ** t_len) / (1 - a)
    assert np.allclose(state[0, 0], want, rtol=1e-5)


def test_routing_takes_the_largest_logits_and_norms_over_them_alone():
    w = {"r.router": np.eye(4, dtype=np.float32), "r.router.b": np.array([0.0, 0.5, 0.0, -3.0], np.float32)}
    chosen, weights = plain.route(np.array([[1.0, 0.6, 0.2, 5.0]], np.float32), w, "r.", 2)
    assert chosen.tolist() == [[3, 1]]                                       # 5 - 3 = 2 and 0.6 + 0.5 = 1.1 beat 1.0
    assert np.allclose(weights[0], np.exp([2.0, 1.1]) / np.exp([2.0, 1.1]).sum(), atol=1e-6)


def test_the_expert_clamps_before_it_gates():
    w = {"e.gate": np.array([[1.0]], np.float32), "e.up": np.array([[1.0]], np.float32), "e.down": np.array([[1.0]], np.float32)}
    big = plain.clamped_expert(np.array([[10.0]], np.float32), w, "e.", 2.0)[0, 0]
    assert np.isclose(big, 2.0 / (1 + np.exp(-1.702 * 2.0)) * 3.0, atol=1e-6)                 # both at the limit
    low = plain.clamped_expert(np.array([[-10.0]], np.float32), w, "e.", 2.0)[0, 0]
    assert np.isclose(low, -10.0 / (1 + np.exp(17.02)) * (-2.0 + 1.0), atol=1e-9)             # the gate has no lower limit, the other side has


# ---- the engine's logic on the torch double -------------------------------------------------------------------

LENGTHS = {"mixed": [5, 11, 1, 70, 33, 130], "plain": [1, 7, 23, 64, 90], "single": [3, 65, 130, 2, 31], "deep": [2, 50, 129]}


@pytest.mark.parametrize("name", sorted(LENGTHS))
def test_every_cut_matches_the_plain_implementation(folders, name):
    folder, config, weights = folders(name)
    requests = schedules.random_requests(config["vocab"], LENGTHS[name], seed=11)
    want = [plain.forward(config, weights, r) for r in requests]
    engine = make_engine(folder)
    for label, got in (("whole", schedules.whole(engine, requests)), ("tail", schedules.tail_one_by_one(engine, requests, tail=12)),
                       ("batches", schedules.batches(engine, requests, batch_size=3)), ("portions", schedules.portions(engine, requests)),
                       ("small portions", schedules.portions(engine, requests, sizes=(2, 2, 3, 2, 1, 2), rest_every=3))):
        for index, (g, e) in enumerate(zip(got, want)):
            assert schedules.relative_error(g, e) < 1e-4, (label, index)
    engine.cache.check_invariants()
    assert engine.cache.live_slots() == [] and engine.cache.free_page_count() == engine.cache.n_pages


def test_a_slot_that_is_used_again_starts_from_nothing(folders):
    """The convolution's last inputs beside the pages and the recurrence's state are zero when a slot starts again."""
    folder, config, weights = folders("mixed")
    engine = make_engine(folder, max_slots=1)
    first, second = schedules.random_requests(config["vocab"], [40, 9], seed=3)
    for tokens in (first, second, first):
        slot = engine.alloc_slot()
        assert slot == 0
        got = engine.step([StepEntry(slot, tokens, list(range(len(tokens))))]).numpy()
        assert schedules.relative_error(got, plain.forward(config, weights, tokens)) < 1e-4
        engine.free_slot(slot)


def test_a_failed_step_puts_the_state_beside_the_pages_back(folders):
    folder, config, weights = folders("mixed")
    engine = make_engine(folder)
    tokens = schedules.random_requests(config["vocab"], [30], seed=8)[0]
    slot = engine.alloc_slot()
    engine.step([StepEntry(slot, tokens[:10], [])])
    boom = RuntimeError("the head fails")
    original = engine.model.head.forward
    engine.model.head.forward = lambda ctx, x: (_ for _ in ()).throw(boom)
    with pytest.raises(RuntimeError):
        engine.step([StepEntry(slot, tokens[10:20], [0])])
    engine.model.head.forward = original
    assert engine.cache.length(slot) == 10
    got = engine.step([StepEntry(slot, tokens[10:], list(range(20)))]).numpy()
    assert schedules.relative_error(got, plain.forward(config, weights, tokens)[10:]) < 1e-4


def test_greedy_generation_through_the_entry_point(folders):
    folder, config, weights = folders("single")
    prompts = schedules.random_requests(config["vocab"], [1, 9, 30], seed=6)
    engine = make_engine(folder)
    results = engine.generate(prompts, max_new_tokens=[6, 5, 6])
    for prompt, result, n in zip(prompts, results, [6, 5, 6]):
        assert result.token_ids == plain.greedy(config, weights, prompt, n)
    engine.cache.check_invariants()


def test_the_routing_is_left_for_the_caller(folders):
    folder, config, weights = folders("mixed")
    engine = make_engine(folder)
    slot = engine.alloc_slot()
    extras = {}
    engine.step([StepEntry(slot, [3, 4, 5], [2])], extras=extras)
    chosen, shares = extras["routing"]
    assert chosen.shape[0] == 3 and torch.allclose(shares.sum(-1), torch.ones(3), atol=1e-6)
