"""Dupidra on the CPU: the configuration and its manifest, the plain implementation's mechanisms against closed forms,
and the engine's own logic (layers that run another layer's tensors with memory of their own, pages that a chunk or a
window gives back, state regions, slots used again, portions, batches, generation) with the kernel library replaced by
the torch double, against the plain implementation."""

import copy
import math

import numpy as np
import pytest

import beholdd
import dupidra_models as dm
import plain_dupidra as plain
import schedules
from beholdd.config import ConfigError, DupidraConfig
from beholdd.engine import Engine, StepEntry
from kernel_emulation import TorchKernels


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}

    def get(name, seed=5):
        if (name, seed) not in made:
            config = dm.CONFIGS[name]
            weights = dm.random_weights(config, seed)
            made[(name, seed)] = (dm.write_model(tmp_path_factory.mktemp(f"dupidra_{name}_{seed}"), config, weights), config, weights)
        return made[(name, seed)]

    return get


def make_engine(folder, dtype="float32", max_tokens=1024, **kw):
    return Engine(folder, dtype=dtype, max_tokens=max_tokens, device="cpu", kernels=TorchKernels(), **kw)


# ---- configuration -----------------------------------------------------------------------------------------

def test_a_borrowing_layer_runs_its_owners_parts_with_memory_of_its_own():
    config = DupidraConfig.from_dict(dm.MIXED)
    assert config.schedule() == [(0, 0), (1, 1), (2, 2), (3, 3), (1, 4), (0, 5), (2, 6)]
    kinds = config.layer_kinds()
    assert [k is None for k in kinds] == [False, False, False, False, True, True, True]
    model = beholdd.registry.resolve_architecture(dm.MIXED).build(config)
    needs = model.entry_needs
    assert len(needs) == 7 and needs[4] == needs[1] and needs[5] == needs[0] and needs[6] == needs[2]
    bare = copy.deepcopy(dm.MIXED)
    bare["layers"][4].pop("mlp")                                            # the feed-forward is the owner's, named again or not
    assert DupidraConfig.from_dict(bare).layers[4].mlp == config.layers[1].mlp
    chained = copy.deepcopy(dm.MIXED)
    chained["layers"].append(dm.borrowed(chained["layers"], 7, 4))          # borrows from a borrower: runs the first owner's
    assert DupidraConfig.from_dict(chained).schedule()[-1] == (1, 7)


def test_every_constant_comes_from_the_file():
    config = DupidraConfig.from_dict(dm.MIXED)
    assert (config.vocab, config.hidden, config.postln_alpha, config.rms_eps, config.max_position) == (97, 64, 1.7, 1e-5, None)
    memory, attention, latent, bare = (config.layers[i] for i in range(4))
    assert (memory.mixer.heads, memory.mixer.dim, memory.mixer.vdim, memory.mixer.gate_cap, memory.mlp.ff) == (3, 8, 20, 9.0, 80)
    a = attention.mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.scale, a.chunk, a.rot_dims, a.rot_base) == (6, 2, 24, 40, 0.2, 20, 12, 500.0)
    assert (attention.mlp.experts, attention.mlp.top, attention.mlp.expert.ff, attention.mlp.expert.limit) == (5, 2, 24, 1.2)
    m = latent.mixer
    assert (m.heads, m.dim, m.vdim, m.kv_rank, m.scale, m.window) == (3, 16, 12, 32, 0.3, 27)
    assert bare.mlp is None and bare.mixer.rot_dims == 0 and bare.mixer.chunk == 50
    plain_config = DupidraConfig.from_dict(dm.PLAIN)
    assert plain_config.layers[0].mixer.chunk == 0 and plain_config.layers[1].mixer.window == 0


@pytest.mark.parametrize("change,message", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][0].update(type="convolution"), "not implemented"),
    (lambda c: c["layers"][0]["mlp"].update(kind="glu"), "not implemented"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=4), "kv_heads"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=26), "dims"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=7), "dims"),
    (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][1]["mixer"]["mask"].update(size=0), "size"),
    (lambda c: c["layers"][2]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][0]["mixer"].update(gate_cap=0.0), "gate_cap"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=6), "top"),
    (lambda c: c["layers"][1]["mlp"]["expert"].pop("limit"), "limit"),
    (lambda c: c["layers"][4].update(weights_of=9), "weights_of"),
    (lambda c: c["layers"][4].update(weights_of=2), "other sizes"),
    (lambda c: (c["layers"][4].update(weights_of=5), c["layers"][5].update(weights_of=4)), "circle"),
    (lambda c: c.update(layers=[]), "layers"),
])
def test_a_configuration_that_lacks_or_overreaches_is_refused(change, message):
    config = copy.deepcopy(dm.MIXED)
    change(config)
    with pytest.raises(ConfigError, match=message):
        DupidraConfig.from_dict(config)


@pytest.mark.parametrize("name", sorted(dm.CONFIGS))
def test_the_manifest_is_the_list_derived_from_the_configuration(name):
    config = dm.CONFIGS[name]
    model = beholdd.registry.resolve_architecture(config).build(DupidraConfig.from_dict(config))
    assert {spec.name: tuple(spec.shape) for spec in model.tensor_specs()} == dm.tensor_shapes(config)


def test_cache_needs_follow_the_mixers():
    model = beholdd.registry.resolve_architecture(dm.MIXED).build(DupidraConfig.from_dict(dm.MIXED))
    memory, attention, latent = model.entry_needs[0], model.entry_needs[1], model.entry_needs[2]
    assert memory.kind == "state" and memory.state_shape == (3 * ((20 + 1) * 8 + 1),)      # values' columns, n's, and m, a head
    assert (attention.kind, attention.kv_heads, attention.head_dim, attention.window) == ("kv", 2, 64, 20)      # 24 and 40 under 64
    assert (latent.kind, latent.kv_heads, latent.head_dim, latent.window) == ("kv", 1, 32, 27)                 # the latent alone


# ---- the plain implementation's mechanisms against closed forms -------------------------------------------------

def test_rotation_pairs_a_dimension_with_the_one_half_the_span_away_and_depends_on_the_distance_alone():
    rng = np.random.default_rng(1)
    q, k = rng.standard_normal((1, 1, 10)), rng.standard_normal((1, 1, 10))
    turned = plain.rotate_halves(q, [7], 6, 100.0)
    assert np.allclose(turned[..., 6:], q[..., 6:])                                           # what lies beyond `dims` passes
    angle = float(np.float32(7) * np.float32(100.0 ** (-2 / 6)))                               # pair 1: dimensions 1 and 4
    assert np.allclose(turned[0, 0, 1], q[0, 0, 1] * math.cos(angle) - q[0, 0, 4] * math.sin(angle), atol=1e-9)
    assert np.allclose(turned[0, 0, 4], q[0, 0, 4] * math.cos(angle) + q[0, 0, 1] * math.sin(angle), atol=1e-9)
    score = lambda a, b: float((plain.rotate_halves(q, [a], 6, 100.0) * plain.rotate_halves(k, [b], 6, 100.0)).sum())
    assert abs(score(12, 5) - score(107, 100)) < 1e-4 and abs(score(12, 5) - score(12, 6)) > 1e-3


def test_chunks_count_from_zero_and_windows_from_the_query():
    chunked = plain.visible(10, "chunk", 4)
    assert chunked[5].tolist() == [False] * 4 + [True, True] + [False] * 4                    # 4 and 5: the chunk 4..7 up to itself
    assert chunked[4].tolist() == [False] * 4 + [True] + [False] * 5 and chunked[3][:4].all()  # a chunk's first sees itself alone
    windowed = plain.visible(10, "window", 3)
    assert windowed[5].tolist() == [False] * 3 + [True] * 3 + [False] * 4                     # itself and the two before
    assert windowed[1].tolist() == [True, True] + [False] * 8
    assert (plain.visible(6) == np.tril(np.ones((6, 6), bool))).all()


def test_the_matrix_memory_with_constant_gates_is_a_weighted_sum():
    """One head, gates without inputs: every step forgets by sigmoid(cap tanh(bf / cap)) and takes in exp(i); with the running
    maximum taken out again, S_t = sum_j sigma^(t - j) e^i k_j v_j^T, and the read-out is divided by max(|n . q| e^m, 1) e^-m."""
    width, dim, vdim, cap, t_len = 4, 2, 3, 5.0, 9
    rng = np.random.default_rng(3)
    w = {"m.q": rng.standard_normal((dim, width)), "m.k": rng.standard_normal((dim, width)), "m.v": rng.standard_normal((vdim, width)),
         "m.g": np.zeros((vdim, width)), "m.o": np.eye(width, vdim), "m.norm": np.ones(vdim), "m.i": np.zeros((1, width)),
         "m.f": np.zeros((1, width)), "m.i.b": np.array([0.4]), "m.f.b": np.array([1.5])}
    h = rng.standard_normal((t_len, width))
    sizes = {"heads": 1, "dim": dim, "vdim": vdim, "gate_cap": cap}
    _, (memory, norm, top) = plain.matrix_memory(h, w, "m.", sizes, 1e-6)
    keep = 1.0 / (1.0 + math.exp(-cap * math.tanh(1.5 / cap)))
    take = math.exp(cap * math.tanh(0.4 / cap))
    k, v = h @ w["m.k"].T, h @ w["m.v"].T
    unscaled = sum(keep ** (t_len - 1 - j) * take * np.outer(k[j], v[j]) for j in range(t_len))
    assert np.allclose(memory[0] * math.exp(top[0]), unscaled, rtol=1e-9)
    assert np.allclose(norm[0] * math.exp(top[0]), sum(keep ** (t_len - 1 - j) * take * k[j] for j in range(t_len)), rtol=1e-9)
    # the maximum starts at 0, not below everything: a first step with a negative input gate keeps m at log(keep) or the gate
    w["m.i.b"] = np.array([-3.0])
    _, (_, _, top) = plain.matrix_memory(h[:1], w, "m.", sizes, 1e-6)
    assert np.isclose(top[0], max(math.log(keep), cap * math.tanh(-3.0 / cap)))
    # continued from its state, the second half is what the whole gives
    out_whole, _ = plain.matrix_memory(h, w, "m.", sizes, 1e-6)
    _, state = plain.matrix_memory(h[:4], w, "m.", sizes, 1e-6)
    out_rest, _ = plain.matrix_memory(h[4:], w, "m.", sizes, 1e-6, state=state)
    assert np.allclose(out_rest, out_whole[4:], rtol=1e-9)


def test_routing_norms_the_chosen_scores_of_a_softmax_over_all():
    w = {"r.router": np.eye(4, dtype=np.float32)}
    chosen, shares = plain.route(np.array([[1.0, 0.6, 0.2, 5.0]], np.float32), w, "r.", 2)
    assert chosen.tolist() == [[3, 0]]
    assert np.allclose(shares[0], np.exp([5.0, 1.0]) / np.exp([5.0, 1.0]).sum(), atol=1e-9)
    tied, _ = plain.route(np.array([[2.0, 2.0, 2.0, 1.0]], np.float32), w, "r.", 2)
    assert tied.tolist() == [[0, 1]]                                            # ties go to the lower index


def test_the_expert_clamps_before_it_gates():
    w = {"e.gate": np.array([[1.0]]), "e.up": np.array([[1.0]]), "e.down": np.array([[1.0]])}
    big = plain.clamped_expert(np.array([[10.0]]), w, "e.", 2.0)[0, 0]
    assert np.isclose(big, 2.0 / (1 + np.exp(-1.702 * 2.0)) * 3.0)                            # both at the limit
    low = plain.clamped_expert(np.array([[-10.0]]), w, "e.", 2.0)[0, 0]
    assert np.isclose(low, -10.0 / (1 + np.exp(17.02)) * (-2.0 + 1.0))                        # the gate has no lower limit, the other side has


def test_the_norm_stands_behind_the_weighted_sum():
    """One layer whose mixer gives nothing (a zero output projection): x <- LN(alpha x), which alpha leaves unchanged but for eps."""
    config = {"architecture": "Dupidra", "vocab": 11, "width": 8, "postln_alpha": 3.0, "norm": {"eps": 1e-12},
              "layers": [dm.mlstm(1, 2, 2, 4.0, mlp=None)]}
    weights = dm.random_weights(config, 0)
    weights["l0.mix.o"][:] = 0.0
    after = plain.residual_after_layers(config, weights, [1, 5, 7])[0]
    x = weights["embed"][[1, 5, 7]].astype(np.float64)
    centred = x - x.mean(-1, keepdims=True)
    want = centred / np.sqrt((centred ** 2).mean(-1, keepdims=True)) * weights["l0.norm1"] + weights["l0.norm1.b"]
    assert np.allclose(after, want, atol=1e-6)


# ---- the engine's logic on the torch double -------------------------------------------------------------------

LENGTHS = {"mixed": [5, 11, 1, 70, 33, 130], "plain": [1, 7, 23, 64, 90], "edges": [3, 65, 130, 2, 31], "deep": [2, 50, 129], "odd": [1, 40, 100]}


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


def test_the_residual_after_every_layer(folders):
    folder, config, weights = folders("mixed")
    tokens = schedules.random_requests(config["vocab"], [40], seed=2)[0]
    want = plain.residual_after_layers(config, weights, tokens)
    engine = make_engine(folder)
    seen = []
    for block in engine.model.own_blocks():
        def wrapped(ctx, hidden, *args, _inner=block.forward, **kw):
            result = _inner(ctx, hidden, *args, **kw)
            seen.append(hidden.clone().numpy())
            return result
        block.forward = wrapped
    slot = engine.alloc_slot()
    engine.step([StepEntry(slot, tokens, [0])])
    assert len(seen) == len(config["layers"])
    for run, (got, expected) in enumerate(zip(seen, want)):
        assert np.abs(got - expected).max() < 1e-4, run


def test_a_slot_that_is_used_again_starts_from_nothing(folders):
    """The memory's state (its running maximum too) is zero when a slot starts again, and windows' pages were given back."""
    folder, config, weights = folders("mixed")
    engine = make_engine(folder, max_slots=1)
    first, second = schedules.random_requests(config["vocab"], [90, 9], seed=3)
    for tokens in (first, second, first):
        slot = engine.alloc_slot()
        assert slot == 0
        got = engine.step([StepEntry(slot, tokens, list(range(len(tokens))))]).numpy()
        assert schedules.relative_error(got, plain.forward(config, weights, tokens)) < 1e-4
        engine.free_slot(slot)
    assert engine.cache.free_page_count() == engine.cache.n_pages


def test_a_failed_step_puts_the_memory_back(folders):
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


def test_pages_behind_a_chunk_or_a_window_are_given_back(folders):
    """Every attention of this model sees a bounded span, so a long sequence holds a bounded number of pages."""
    folder, config, weights = folders("mixed")
    engine = make_engine(folder, max_tokens=4096)
    tokens = schedules.random_requests(config["vocab"], [400], seed=4)[0]
    slot = engine.alloc_slot()
    engine.step([StepEntry(slot, tokens[:200], [])])
    held_early = engine.cache.n_pages - engine.cache.free_page_count()
    engine.step([StepEntry(slot, tokens[200:399], [])])
    held_late = engine.cache.n_pages - engine.cache.free_page_count()
    assert held_late <= held_early
    got = engine.step([StepEntry(slot, tokens[399:], [0])]).numpy()
    assert schedules.relative_error(got, plain.forward(config, weights, tokens)[-1:]) < 1e-4
    engine.free_slot(slot)


def test_greedy_generation_through_the_entry_point(tmp_path):
    config = dm.GENERATING
    weights = dm.random_weights(config, 5, gain=dm.GENERATING_GAIN)
    folder = dm.write_model(tmp_path / "generating", config, weights)
    prompts = schedules.random_requests(config["vocab"], [1, 9, 30], seed=6)
    engine = make_engine(folder)
    results = engine.generate(prompts, max_new_tokens=[6, 5, 6])
    assert len({token for r in results for token in r.token_ids}) >= 6      # the continuations vary
    for prompt, result, n in zip(prompts, results, [6, 5, 6]):
        assert result.token_ids == plain.greedy(config, weights, prompt, n)
    engine.cache.check_invariants()


@pytest.mark.parametrize("seed", range(6))
def test_drawn_configurations(seed, tmp_path):
    config = dm.drawn_config(200 + seed)
    weights = dm.random_weights(config, seed, gain=0.6)
    folder = dm.write_model(tmp_path / "drawn", config, weights)
    assert {s.name: tuple(s.shape) for s in beholdd.registry.resolve_architecture(config).build(DupidraConfig.from_dict(config)).tensor_specs()} \
        == dm.tensor_shapes(config)
    requests = schedules.random_requests(config["vocab"], [1, 19, 70], seed=seed)
    want = [plain.forward(config, weights, r) for r in requests]
    engine = make_engine(folder)
    for label, got in (("whole", schedules.whole(engine, requests)), ("batches", schedules.batches(engine, requests, batch_size=3)),
                       ("portions", schedules.portions(engine, requests, sizes=(2, 5, 1, 30, 3)))):
        for index, (g, e) in enumerate(zip(got, want)):
            assert schedules.relative_error(g, e) < 1e-4, (label, index, config)
