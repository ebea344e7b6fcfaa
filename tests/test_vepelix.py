"""Vepelix on the CPU: the configuration and its manifest, the plain implementation's mechanisms against closed forms, and
the engine's own logic (schedule with a loop entered with the embedding's output, pages beside a state in one layer run,
slots used again, portions, batches, generation) with the kernel library replaced by the torch double, against the plain
implementation."""

import copy
import math

import numpy as np
import pytest
import torch

import beholdd
import plain_vepelix as plain
import schedules
import vepelix_models as vm
from beholdd.config import ConfigError, VepelixConfig
from beholdd.engine import Engine, StepEntry
from beholdd.registry import configuration_of
from kernel_emulation import TorchKernels


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}

    def get(name, seed=5):
        if (name, seed) not in made:
            config = vm.CONFIGS[name]
            made[(name, seed)] = (vm.write_model(tmp_path_factory.mktemp(f"vepelix_{name}_{seed}"), config,
                                                 vm.random_weights(config, seed, vm.GAIN.get(name, 1.0))), config)
        return made[(name, seed)]

    return get


def make_engine(folder, dtype="float32", max_tokens=1024, **kw):
    return Engine(folder, dtype=dtype, max_tokens=max_tokens, device="cpu", kernels=TorchKernels(), **kw)


# ---- configuration -----------------------------------------------------------------------------------------

def test_the_loop_repeats_a_stretch_and_names_the_runs_that_are_entered_again():
    config = VepelixConfig.from_dict(vm.MIXED)
    assert config.run_order() == [0, 1, 2, 1, 2, 3] and config.pass_starts() == [3]
    assert config.schedule() == [(layer, run) for run, layer in enumerate([0, 1, 2, 1, 2, 3])]
    odd = VepelixConfig.from_dict(vm.ODD)
    assert odd.run_order() == [0, 1, 0, 1, 0, 1, 2] and odd.pass_starts() == [2, 4]
    assert VepelixConfig.from_dict(vm.PLAIN).run_order() == [0, 1, 2] and VepelixConfig.from_dict(vm.PLAIN).pass_starts() == []
    assert VepelixConfig.from_dict(vm.WIDE).pass_starts() == []                          # a loop that runs once
    empty = dict(vm.MIXED, loop={"start": 2, "stop": 2, "times": 5})
    assert VepelixConfig.from_dict(empty).run_order() == [0, 1, 2, 3] and VepelixConfig.from_dict(empty).pass_starts() == []


def test_every_constant_comes_from_the_file_or_a_tensors_shape():
    config = VepelixConfig.from_dict(vm.MIXED)
    assert (config.vocab, config.hidden, config.rms_eps, config.max_position) == (97, 64, 1e-5, None)
    first, second = config.layers[0].mixer, config.layers[1].mixer
    assert (first.heads, first.dim, first.rot_dim, first.vdim, first.kv_rank, first.q_rank, first.scale) == (3, 16, 16, 24, 48, 40, 0.3)
    assert (first.rot_dims, first.rot_base, first.rot_stretch) == (16, 500.0, (4.0, 64.0, 16.0, 1.0))
    assert (second.left.heads, second.left.kv_heads, second.left.dim, second.left.vdim, second.left.window) == (4, 2, 96, 40, 70)
    assert (second.left.rot_dims, second.left_scale, second.right_scale) == (48, 1.3, 0.8)
    assert (second.right.heads, second.right.dim, second.right.vdim, second.right.tau, second.right.decay_rank) == (2, 16, 24, 8.0, 8)
    assert config.layers[3].mixer.left.window == 0 and config.layers[3].mlp is None
    assert (config.layers[1].mlp.experts, config.layers[1].mlp.top, config.layers[1].mlp.shared_ff) == (6, 3, 0)
    # the decays' rank is the first size of a tensor; a checkpoint's header outranks the file's own word
    shaped = VepelixConfig.from_dict(vm.MIXED, shapes={"l1.mix.right.a1": (5, 64)})
    assert shaped.layers[1].mixer.right.decay_rank == 5
    bare = copy.deepcopy(vm.MIXED)
    bare["layers"][1]["mixer"]["right"].pop("decay_rank")
    with pytest.raises(ConfigError, match="rank"):
        VepelixConfig.from_dict(bare)


@pytest.mark.parametrize("change,message", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][0].update(type="convolution"), "not implemented"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "not implemented"),
    (lambda c: c["layers"][0]["mixer"].pop("q_rank"), "q_rank"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=32), "dims"),
    (lambda c: c["layers"][1]["mixer"]["left"].update(kv_heads=3), "group"),
    (lambda c: c["layers"][1]["mixer"]["right"].update(tau=0.0), "tau"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=7), "top"),
    (lambda c: c["layers"][1]["mixer"].pop("left_scale"), "left_scale"),
    (lambda c: c["loop"].update(stop=7), "stop"),
    (lambda c: c.update(layers=[]), "layers"),
])
def test_a_configuration_that_lacks_or_overreaches_is_refused(change, message):
    config = copy.deepcopy(vm.MIXED)
    change(config)
    with pytest.raises(ConfigError, match=message):
        VepelixConfig.from_dict(config)


@pytest.mark.parametrize("name", sorted(vm.CONFIGS))
def test_the_manifest_is_what_the_configuration_implies(name):
    config = vm.CONFIGS[name]
    entry = beholdd.resolve_architecture(config)
    model = entry.build(configuration_of(entry, config))
    assert {spec.name: tuple(spec.shape) for spec in model.tensor_specs()} == vm.tensor_shapes(config)


def test_the_decays_rank_is_read_from_the_checkpoint_where_the_file_does_not_say_it(tmp_path):
    config = vm.CONFIGS["mixed"]
    weights = vm.random_weights(config, 2)
    silent = copy.deepcopy(config)
    for layer in silent["layers"]:
        if layer["type"] == "parallel":
            layer["mixer"]["right"].pop("decay_rank")
    folder = vm.write_model(tmp_path / "silent", silent, weights)
    engine = make_engine(folder)
    assert engine.model.config.layers[1].mixer.right.decay_rank == 8 and engine.model.config.layers[3].mixer.right.decay_rank == 4
    tokens = schedules.random_requests(config["vocab"], [33], seed=1)[0]
    slot = engine.alloc_slot()
    got = engine.step([StepEntry(slot, tokens, list(range(len(tokens))))]).numpy()
    assert schedules.relative_error(got, plain.forward(config, weights, tokens)) < 1e-4
    import io
    from beholdd import cli
    out = io.StringIO()
    assert cli.main(["generate", "--model", folder, "--prompt-ids", "1,2,3", "--max-new-tokens", "4", "--dtype", "bfloat16", "--plan-only"], out=out) == 0


def test_a_checkpoint_with_other_tensors_is_refused(tmp_path):
    config = vm.CONFIGS["odd"]
    weights = vm.random_weights(config, 1)
    weights["l1.mix.sinks"] = weights.pop("l1.mix.sink")
    folder = vm.write_model(tmp_path / "odd", config, weights)
    with pytest.raises(beholdd.WeightError) as caught:
        make_engine(folder)
    assert caught.value.missing == ["l1.mix.sink"] and caught.value.unexpected == ["l1.mix.sinks"]


# ---- the plain implementation's mechanisms against closed forms --------------------------------------------

def test_plain_rotation_turns_neighbours_and_stretches_slow_pairs():
    x = np.zeros((1, 8))
    x[0, 2], x[0, 7] = 1.0, 5.0
    out = plain.turn_neighbours(x, [3], {"dims": 6, "base": 100.0})
    angle = 3 * 100.0 ** (-2.0 / 6)
    want = np.zeros(8)
    want[2], want[3], want[7] = np.cos(angle), np.sin(angle), 5.0       # dimension 2 pairs with 3; 6 and 7 pass
    assert np.abs(out[0] - want).max() < 1e-12
    # 16 dimensions, base 10000, a stretch by 4 of what turns less than once in 64 positions and none of what turns 8 times
    rot = {"dims": 16, "base": 10000.0, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}}
    got, magnitude = plain.stretched_frequencies(rot)
    assert abs(magnitude - (0.1 * math.log(4.0) + 1.0)) < 1e-15
    bare = np.array([10000.0 ** (-i / 8) for i in range(8)])
    turns = 64 * bare / (2 * math.pi)                                   # 10.2, 3.2, 1.0, 0.32, ...
    low, high = 0, 3                                                    # floor(0.21), ceil(2.02): by hand from the two formulas
    ramp = np.clip((np.arange(8) - low) / (high - low), 0, 1)
    assert np.abs(got - (bare / 4 * ramp + bare * (1 - ramp))).max() < 1e-15
    assert got[0] == bare[0] and abs(got[3] - bare[3] / 4) < 1e-18 and abs(got[7] - bare[7] / 4) < 1e-18 and turns[0] > 8 > turns[1]
    # scores depend on distances alone, with the stretch too
    rng = np.random.default_rng(0)
    q, k = rng.standard_normal((5, 16)), rng.standard_normal((5, 16))
    near = plain.turn_neighbours(q, range(5), rot) @ plain.turn_neighbours(k, range(5), rot).T
    far = plain.turn_neighbours(q, range(900, 905), rot) @ plain.turn_neighbours(k, range(900, 905), rot).T
    assert np.abs(near - far).max() < 1e-9


def test_plain_sink_is_a_key_without_a_value():
    rng = np.random.default_rng(1)
    scores = rng.standard_normal((4, 4))
    visible = np.tril(np.ones((4, 4), bool))
    got = plain.softmax_rows(scores, visible, sink=0.7)
    wider = np.concatenate([scores, np.full((4, 1), 0.7)], axis=1)
    want = plain.softmax_rows(wider, np.concatenate([visible, np.ones((4, 1), bool)], axis=1))[:, :4]
    assert np.abs(got - want).max() < 1e-15 and (got.sum(-1) < 1).all()
    assert np.abs(plain.softmax_rows(scores, visible, sink=-1e9) - plain.softmax_rows(scores, visible)).max() < 1e-15


def test_plain_latent_attention_first_token_and_distances():
    rng = np.random.default_rng(2)
    sizes = {"heads": 2, "dim": 4, "rot_dim": 6, "vdim": 3, "kv_rank": 5, "q_rank": 7, "scale": 0.7, "rot": {"dims": 6, "base": 50.0}}
    width = 8
    shapes = {"m.dq": (7, width), "m.dq.norm": (7,), "m.uq": (20, 7), "m.dkv": (11, width), "m.dkv.norm": (5,), "m.uk": (8, 5), "m.uv": (6, 5),
              "m.sink": (2,), "m.g": (2, width), "m.o": (width, 6)}
    w = {k: rng.standard_normal(s) for k, s in shapes.items()}
    h = rng.standard_normal((6, width))
    at_zero = plain.latent_attention(h, w, "m.", sizes, 1e-6)
    shifted = plain.latent_attention(h, w, "m.", sizes, 1e-6, first_position=37)
    assert np.abs(at_zero - shifted).max() < 1e-9 * np.abs(at_zero).max()
    # the first token sees itself and the sink: its head's output is gate * e^s / (e^s + e^sink) * Wuv c_0
    down = w["m.dkv"] @ h[0]
    c = down[:5] / np.sqrt((down[:5] ** 2).mean() + 1e-6) * w["m.dkv.norm"]
    dq = w["m.dq"] @ h[0]
    q = (w["m.uq"] @ (dq / np.sqrt((dq ** 2).mean() + 1e-6) * w["m.dq.norm"])).reshape(2, 10)
    heads = []
    for head in range(2):
        score = (q[head, :4] @ (w["m.uk"].reshape(2, 4, 5)[head] @ c) + q[head, 4:] @ down[5:]) * 0.7      # position 0: nothing turns
        share = 1.0 / (1.0 + np.exp(w["m.sink"][head] - score))
        heads.append(share / (1 + np.exp(-(w["m.g"][head] @ h[0]))) * (w["m.uv"].reshape(2, 3, 5)[head] @ c))
    want = w["m.o"] @ np.concatenate(heads)
    assert np.abs(at_zero[0] - want).max() < 1e-12 * np.abs(want).max()


def test_plain_gated_linear_attention_is_a_decayed_sum_that_can_be_continued():
    rng = np.random.default_rng(3)
    sizes = {"heads": 2, "dim": 5, "vdim": 3, "tau": 4.0}
    width, t_len = 7, 9
    shapes = {"m.q": (10, width), "m.k": (10, width), "m.v": (6, width), "m.g": (6, width), "m.norm": (3,), "m.a1": (2, width),
              "m.a2": (10, 2), "m.a2.b": (10,)}
    w = {k: rng.standard_normal(s) for k, s in shapes.items()}
    w["m.o"] = np.eye(width, 6)
    h = rng.standard_normal((t_len, width))
    got, state = plain.gated_linear_attention(h, w, "m.", sizes, 1e-6)
    q, k, v = (h @ w["m.q"].T).reshape(t_len, 2, 5) / np.sqrt(5), (h @ w["m.k"].T).reshape(t_len, 2, 5), (h @ w["m.v"].T).reshape(t_len, 2, 3)
    alpha = (1 / (1 + np.exp(-((h @ w["m.a1"].T) @ w["m.a2"].T + w["m.a2.b"])))) ** 0.25
    alpha = alpha.reshape(t_len, 2, 5)
    o = np.zeros((t_len, 2, 3))
    for t in range(t_len):
        for j in range(t + 1):
            kept = np.prod(alpha[j + 1:t + 1], axis=0)                      # a key channel's decays since the key came
            o[t] += np.einsum("hd,hd,hv->hv", q[t], kept * k[j], v[j])
    normed = o / np.sqrt((o * o).mean(-1, keepdims=True) + 1e-6) * w["m.norm"]
    gate = h @ w["m.g"].T
    want = normed.reshape(t_len, 6) * gate / (1 + np.exp(-gate))
    assert np.abs(got[:, :6] - want).max() < 1e-10 * np.abs(want).max()
    first, carried = plain.gated_linear_attention(h[:4], w, "m.", sizes, 1e-6)
    second, _ = plain.gated_linear_attention(h[4:], w, "m.", sizes, 1e-6, state=carried)
    assert np.abs(np.concatenate([first, second]) - got).max() < 1e-12 and state.shape == (2, 5, 3)


def test_plain_experts_weigh_their_inputs_by_unnormed_sigmoid_scores():
    rng = np.random.default_rng(4)
    width, ff = 6, 4
    w = {"m.router": rng.standard_normal((3, width))}
    for e in range(3):
        w.update({f"m.e{e}.gate": rng.standard_normal((ff, width)), f"m.e{e}.up": rng.standard_normal((ff, width)),
                  f"m.e{e}.down": rng.standard_normal((width, ff))})
    h = rng.standard_normal((5, width))
    chosen, scores = plain.route(h, w, "m.", 2)
    z = h @ w["m.router"].T
    assert np.array_equal(chosen, np.argsort(-z, axis=-1, kind="stable")[:, :2]) and np.abs(scores - 1 / (1 + np.exp(-np.sort(z)[:, :0:-1]))).max() < 1e-15
    tied = plain.route(np.zeros((1, width)), w, "m.", 2)[0]
    assert tied.tolist() == [[0, 1]]                                          # ties go to the lower index
    got = plain.experts(h, w, "m.", {"router": {"experts": 3, "top": 2}})
    want = np.zeros_like(h)
    for t in range(5):
        for e, s in zip(chosen[t], scores[t]):
            g, u = w[f"m.e{e}.gate"] @ (s * h[t]), w[f"m.e{e}.up"] @ (s * h[t])
            want[t] += w[f"m.e{e}.down"] @ (g / (1 + np.exp(-g)) * u)
    assert np.abs(got - want).max() < 1e-12
    # the weight is not a factor on the output: the activation stands between
    outside = sum(scores[0][j] * plain.silu_expert(h[:1], w, f"m.e{chosen[0][j]}.")[0] for j in range(2))
    assert np.abs(got[0] - outside).max() > 1e-3


def test_plain_clamped_activation_clamps_before_the_gate():
    w = {"m.gate": np.array([[1.0]]), "m.up": np.array([[1.0]]), "m.down": np.array([[1.0]])}
    big = plain.clamped_feed_forward(np.array([[10.0]]), w, "m.", 2.0)[0, 0]
    assert abs(big - 2.0 / (1 + np.exp(-1.702 * 2.0)) * 3.0) < 1e-12
    low = plain.clamped_feed_forward(np.array([[-10.0]]), w, "m.", 2.0)[0, 0]              # the gate is bounded above only
    assert abs(low - (-10.0) / (1 + np.exp(17.02)) * (-2.0 + 1.0)) < 1e-12


# ---- the engine's logic with the torch double ----------------------------------------------------------------

@pytest.mark.parametrize("name,lengths", [("mixed", [5, 70, 17, 131]), ("plain", [1, 23, 66]), ("odd", [3, 64, 65, 9]),
                                          ("wide", [40, 7, 90])])
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


def test_the_residual_after_every_layer_run(folders):
    """Layer by layer: the engine's float32 residual against the plain one after every run of the schedule, the entry of the
    loop's second pass among them."""
    folder, _ = folders("mixed")
    config, weights = plain.load(folder)
    tokens = schedules.random_requests(config["vocab"], [21], seed=12)[0]
    want = []
    plain.forward(config, weights, tokens, residuals=want)
    engine = make_engine(folder)
    seen = []
    for block in engine.model.own_blocks():
        real = block.forward

        def spy(ctx, hidden, cache, prepared=None, next_block=None, real=real):
            result = real(ctx, hidden, cache, prepared, next_block)
            seen.append(hidden.reshape(hidden.shape[0], -1).clone().numpy())
            return result

        block.forward = spy
    slot = engine.alloc_slot()
    engine.step([StepEntry(slot, tokens, [])])
    assert len(seen) == len(want) == 6
    for run, (g, e) in enumerate(zip(seen, want)):
        assert np.abs(g - e).max() < 1e-5 * np.abs(e).max(), run


def test_a_layer_run_keeps_pages_beside_a_state_and_every_run_its_own(folders):
    folder, _ = folders("mixed")
    engine = make_engine(folder)
    needs = engine.model.entry_needs
    assert len(needs) == 6
    assert [needs[run].kind for run in range(6)] == ["kv"] * 6
    side = needs[1]
    assert (side.kv_heads, side.head_dim, side.window, side.state_shape) == (2, 96, 70, (2, 16, 24))
    assert needs[3] == side and needs[5].window == 0 and needs[5].state_shape == (3, 8, 8)
    assert (needs[0].kv_heads, needs[0].head_dim, needs[0].state_shape) == (1, 64, ())          # the latent and the shared key part
    slot = engine.alloc_slot()
    engine.step([StepEntry(slot, [1, 2, 3, 4, 5], [])])
    states = [g.state for g in engine.cache.groups if g.need == side][0]
    assert states.shape[0] == 2                                 # the two passes of layer 1
    held = [states[run, slot].clone() for run in range(2)]
    assert all(float(h.abs().max()) > 0 for h in held) and not torch.equal(held[0], held[1])


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
    folder, _ = folders("odd")
    config, weights = plain.load(folder)
    tokens = schedules.random_requests(config["vocab"], [20], seed=4)[0]
    engine = make_engine(folder)
    slot = engine.alloc_slot()
    engine.step([StepEntry(slot, tokens[:10], [])])
    calls = {"n": 0}
    real = engine.kernels.gated_group_rmsnorm

    def failing(*args, **kw):
        calls["n"] += 1
        if calls["n"] == 2:                   # the second pass of the first layer: the first pass has advanced its state
            raise RuntimeError("injected")
        return real(*args, **kw)

    engine.kernels.gated_group_rmsnorm = failing
    with pytest.raises(RuntimeError, match="injected"):
        engine.step([StepEntry(slot, tokens[10:15], [])])
    engine.kernels.gated_group_rmsnorm = real
    assert engine.cache.length(slot) == 10
    got = engine.step([StepEntry(slot, tokens[10:], list(range(10)))]).numpy()
    assert schedules.relative_error(got, plain.forward(config, weights, tokens)[10:]) < 1e-4


def test_pages_behind_the_window_are_given_back(folders):
    folder, _ = folders("plain")
    config, weights = plain.load(folder)
    tokens = schedules.random_requests(config["vocab"], [300], seed=2)[0]
    engine = make_engine(folder, max_tokens=512)
    slot = engine.alloc_slot()
    engine.step([StepEntry(slot, tokens[:290], [])])
    windowed = [g for g in engine.cache.groups if g.need.kind == "kv" and g.need.window == 65][0]
    whole = [g for g in engine.cache.groups if g.need.kind == "kv" and g.need.window == 0][0]
    held = lambda group: sum(1 for page in group.tables[slot] if page >= 0) if hasattr(group, "tables") else None
    got = np.concatenate([engine.step([StepEntry(slot, [t], [0])]).numpy() for t in tokens[290:]])
    assert schedules.relative_error(got, plain.forward(config, weights, tokens)[290:]) < 1e-4
    engine.cache.check_invariants()
    if held(windowed) is not None:
        assert held(windowed) <= 3 < held(whole)


def test_far_tokens_decide_the_logits_of_the_test_models(folders):
    for name in ("mixed", "wide"):
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
    folder, _ = folders("odd")
    config, weights = plain.load(folder)
    prompts = schedules.random_requests(config["vocab"], [50, 3, 21], seed=9)
    engine = make_engine(folder, max_rows_per_step=8)
    results = engine.generate(prompts, max_new_tokens=4)
    for prompt, result in zip(prompts, results):
        assert result.token_ids == plain.greedy(config, weights, prompt, 4)


@pytest.mark.parametrize("seed", range(8))
def test_drawn_configurations_on_the_torch_double(seed, tmp_path):
    """Sizes, counts, constants and layer orders that nobody picked: whole prompts, a tail token by token, a batch."""
    config = vm.drawn_config(seed)
    folder = vm.write_model(tmp_path / "drawn", config, vm.random_weights(config, seed, gain=0.7))
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
    folder, _ = folders("mixed")
    out = io.StringIO()
    code = cli.main(["generate", "--model", folder, "--prompt-ids", "1,2,3", "--max-new-tokens", "70", "--dtype", "bfloat16",
                     "--plan-only"], out=out)
    text = out.getvalue()
    assert code == 0, text
    # three runs of latent layers (the first one's cached head is as large as the looped one's), the looped pair of mixers
    # side by side twice, with the state beside the pages
    assert "keys/values of 3 layers (1 heads x 64)" in text
    assert "keys/values of 2 layers (2 heads x 96, window 70)" in text and "and a state (2, 16, 24)" in text
    assert "not counted" not in text          # every part says what a step of its allocates
