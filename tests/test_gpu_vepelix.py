"""Vepelix on the GPU: every new kernel, and every new turn of an older one, alone against the plain implementation's
function of the same mechanism; the engine over every cut of the work (whole prompts, token by token, portions down to two
tokens, batches of unequal requests, slots and pages used again) in float32 and bfloat16 on configurations that differ in
every size; models in which ONE key decides the logits, far back, at page borders, at the first positions and just inside
and just outside the window, in a prompt and decoded, with a sink that outweighs it; a decaying memory that holds one token
for hundreds of steps; long decoding through the captured steps; greedy generation through the entry point and the trace
replay program."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_vepelix as plain
import schedules
import vepelix_models as vm
from test_gpu_pudorax import STRAY, TOLERANCE, check, check_each, dev, engine_for, ragged, rel, rounded, tol, tolerances_for

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = [torch.float32, torch.bfloat16]
PAGE = 64


@pytest.fixture(scope="module")
def K():
    from beholdd.kernels import HipKernels
    return HipKernels("cuda:0")


def selector(first, count, width):
    """The matrix that takes columns first .. first + count - 1 of a row of `width` numbers."""
    m = np.zeros((count, width))
    m[np.arange(count), first + np.arange(count)] = 1.0
    return m


# ---- kernels alone ------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,vdim,tau,rank,lengths", [(2, 5, 7, 3.0, 3, [5, 1, 31]), (1, 16, 24, 20.0, 4, [70]), (3, 48, 64, 8.0, 16, [3, 17, 2]),
                                                             (2, 128, 128, 1.0, 8, [40, 9]), (4, 33, 100, 4.0, 5, [1, 1, 1, 1, 1]),
                                                             (6, 64, 256, 2.0, 2, [130]), (2, 16, 24, 8.0, 4, [700, 64, 1, 333]), (3, 64, 128, 12.0, 8, [1030]),
                                                             (1, 40, 72, 4.0, 3, [129, 128, 127, 300])])
def test_gated_linear_attention_scan_norm_and_gate(K, dtype, heads, dim, vdim, tau, rank, lengths):
    """The recurrence over ragged rows of several sequences, into slots in another order than the batch's, then a second step
    that continues from the states the first one left; behind it the heads' norm with the gate after it.  The long sequences
    are walked in chunks side by side (beside short ones that are not), and must come out as if walked in one."""
    rng = np.random.default_rng(heads * dim + vdim)
    kw, vw = heads * dim, heads * vdim
    width = 3 + 2 * kw + 2 * vw + rank
    q_off, k_off, v_off, g_off, low_off = 3, 3 + kw, 3 + 2 * kw, 3 + 2 * kw + vw, 3 + 2 * kw + 2 * vw
    w = {"m.q": selector(q_off, kw, width), "m.k": selector(k_off, kw, width), "m.v": selector(v_off, vw, width), "m.g": selector(g_off, vw, width),
         "m.a1": selector(low_off, rank, width), "m.a2": rng.standard_normal((kw, rank)), "m.a2.b": rng.uniform(-1, 5, kw),
         "m.norm": 1 + 0.3 * rng.standard_normal(vdim), "m.o": np.eye(vw)}
    sizes = {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}
    slots = list(rng.permutation(len(lengths) + 2)[:len(lengths)])
    seq_start, seq_slot, _, starts = ragged(lengths, slots)
    state = torch.zeros(len(lengths) + 2, heads, dim, vdim, device="cuda:0")
    held = [None] * len(lengths)
    total, eps = sum(lengths), 1e-5
    norm_weight = dev(np.tile(w["m.norm"], heads).astype(np.float32))
    for step in range(2):
        rows_t, rows = rounded(rng.standard_normal((total, width)), dtype)
        z = (rows[:, low_off:low_off + rank].astype(np.float64) @ w["m.a2"].T).astype(np.float32)
        mixed = torch.empty(total, vw, device="cuda:0")
        K.gla_scan(dev(rows_t), q_off, k_off, v_off, dev(z), dev(w["m.a2.b"].astype(np.float32)), tau, dim ** -0.5, state, seq_start, seq_slot,
                   mixed, heads, dim, vdim, max_rows_per_seq=max(lengths))
        out = torch.empty(total, vw, dtype=dtype, device="cuda:0")
        K.gated_group_rmsnorm(mixed, dev(rows_t), g_off, norm_weight, eps, out, heads, gate_after=True)
        for s in range(len(lengths)):
            want, held[s] = plain.gated_linear_attention(rows[starts[s]:starts[s + 1]], w, "m.", sizes, eps, state=held[s])
            assert rel(out[starts[s]:starts[s + 1]], want) < tol(dtype, f32=5e-5, bf16=1e-2), (step, s)
            assert rel(state[slots[s]], held[s]) < 2e-5, (step, s)
    untouched = [s for s in range(len(lengths) + 2) if s not in slots]
    assert float(state[untouched].abs().max()) == 0.0


def attend_plain(q, k, v, scale, window, sinks, first_position):
    """q [T, H, d] at positions first_position .., k, v [first_position + T, G, d]: softmax with a window and sinks."""
    t_len, heads, _ = q.shape
    group = heads // k.shape[1]
    positions = first_position + np.arange(t_len)
    distance = positions[:, None] - np.arange(k.shape[0])[None, :]
    visible = (distance >= 0) & ((distance < window) if window else True)
    out = np.zeros((t_len, heads, v.shape[2]))
    for head in range(heads):
        scores = q[:, head].astype(np.float64) @ k[:, head // group].astype(np.float64).T * scale
        out[:, head] = plain.softmax_rows(scores, visible, sink=None if sinks is None else float(sinks[head])) @ v[:, head // group]
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,hd,past,rows,window", [(8, 2, 64, 0, 2100, 0), (8, 2, 64, 0, 2100, 150), (4, 1, 128, 700, 1, 0), (6, 2, 96, 130, 3, 70),
                                                                (2, 1, 256, 5000, 1, 0), (3, 3, 40, 200, 9, 0), (16, 1, 160, 64, 40, 0)])
def test_a_sink_in_every_attention_kernel(K, dtype, heads, kv_heads, hd, past, rows, window):
    """Prompts of many columns, decode rows, one long context in key splits and head sizes that the matrix cores do not take:
    exp(sink) joins the sum of every (row, head), sinks larger and smaller than the scores among them."""
    rng = np.random.default_rng(hd + rows)
    total, scale = past + rows, 1.0 / np.sqrt(hd)
    k_t, k = rounded(rng.standard_normal((total, kv_heads, hd)), dtype)
    v_t, v = rounded(rng.standard_normal((total, kv_heads, hd)), dtype)
    q_t, q = rounded(rng.standard_normal((rows, heads, hd)) * 2, dtype)
    sinks = rng.uniform(-3, 3, heads).astype(np.float32)
    sinks[0] = 9.0                                                                 # above every score: most of the weight
    n_pages = -(-total // PAGE)
    k_pages = torch.zeros(n_pages, kv_heads, PAGE, hd, dtype=dtype, device="cuda:0")
    v_pages = torch.zeros(n_pages, kv_heads, hd, PAGE, dtype=dtype, device="cuda:0")
    table = dev(rng.permutation(n_pages).astype(np.int32).reshape(1, n_pages))
    proj = torch.cat([torch.zeros(total, heads * hd, dtype=dtype), k_t.reshape(total, -1), v_t.reshape(total, -1)], dim=1)
    scrap = torch.empty(total, heads * hd, dtype=dtype, device="cuda:0")
    K.head_norm_rope_write(dev(proj), 0, None, None, None, 0.0, None, 0, dev(np.arange(total, dtype=np.int32)), dev(np.zeros(total, np.int32)),
                           scrap, k_pages, v_pages, table, heads, kv_heads, hd, hd, hd, True)

    class Layout:
        n_seqs, max_rows_per_seq, max_position = 1, rows, total - 1
        seq_start = dev(np.array([0, rows], np.int32))

    positions = dev(np.arange(past, total, dtype=np.int32))
    for use in (sinks, None):
        out = torch.empty(rows, heads * hd, dtype=dtype, device="cuda:0")
        K.attention(dev(q_t.reshape(rows, -1)), out, k_pages, v_pages, table, dev(np.zeros(rows, np.int32)), positions, heads, kv_heads, hd,
                    scale, window, layout=Layout, sinks=None if use is None else dev(use))
        want = attend_plain(q, k, v, scale, window, use, past)
        assert rel(out.float().reshape(rows, heads, hd), want) < tol(dtype, f32=3e-5, bf16=1.6e-2), use is None


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,pad,turned,stretch", [(4, 2, 32, 16, 32, 8, None), (2, 1, 80, 160, 160, 80, (4.0, 512, 16.0, 1.0)),
                                                                        (3, 3, 20, 12, 32, 20, (4.0, 64, 16.0, 1.0)), (1, 1, 64, 64, 64, 0, None)])
def test_head_norms_and_rotation_in_neighbouring_pairs(K, dtype, heads, kv_heads, dim, vdim, pad, turned, stretch):
    """Queries as the kernel leaves them, and keys and values through the attention that reads them: per-head norms with one
    weight, neighbours turned by stretched frequencies with the factor on cosine and sine, within a window."""
    from beholdd.parts.rope import RotaryFrequencies
    rng = np.random.default_rng(dim + vdim)
    t_len, eps, scale, window = 150, 1e-5, 0.2, 70
    q_width, k_width, v_width = heads * dim, kv_heads * dim, kv_heads * vdim
    proj_t, proj = rounded(rng.standard_normal((t_len, 5 + q_width + k_width + v_width)), dtype)
    wq, wk = 1 + 0.3 * rng.standard_normal(dim), 1 + 0.3 * rng.standard_normal(dim)
    rot = {"dims": turned, "base": 1000.0}
    if stretch:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), stretch))
    positions = np.arange(t_len)
    q = plain.weight_norm(proj[:, 5:5 + q_width].reshape(t_len, heads, dim), wq, eps)
    k = plain.weight_norm(proj[:, 5 + q_width:5 + q_width + k_width].reshape(t_len, kv_heads, dim), wk, eps)
    v = proj[:, 5 + q_width + k_width:].reshape(t_len, kv_heads, vdim)
    if turned:
        q, k = plain.turn_neighbours(q, positions, rot), plain.turn_neighbours(k, positions, rot)
    rotation = RotaryFrequencies(turned, 1000.0, stretch) if turned else None
    turning = dict(neighbours=True, magnitude=rotation.magnitude) if turned else {}
    k_pages = torch.zeros(3, kv_heads, PAGE, pad, dtype=dtype, device="cuda:0")
    v_pages = torch.zeros(3, kv_heads, pad, PAGE, dtype=dtype, device="cuda:0")
    table = dev(np.array([[2, 0, 1]], np.int32))
    q_out = torch.empty(t_len, heads * pad, dtype=dtype, device="cuda:0")
    K.head_norm_rope_write(dev(proj_t), 5, None, dev(wq.astype(np.float32)), dev(wk.astype(np.float32)), eps,
                           rotation.frequencies("cuda:0") if turned else None, turned, dev(positions.astype(np.int32)), dev(np.zeros(t_len, np.int32)),
                           q_out, k_pages, v_pages, table, heads, kv_heads, dim, vdim, pad, True, **turning)
    assert rel(q_out.float().reshape(t_len, heads, pad)[..., :dim], q) < tol(dtype, f32=2e-5, bf16=8e-3)
    assert float(q_out.float().reshape(t_len, heads, pad)[..., dim:].abs().max()) == 0.0 if pad > dim else True

    class Layout:
        n_seqs, max_rows_per_seq, max_position = 1, t_len, t_len - 1
        seq_start = dev(np.array([0, t_len], np.int32))

    attended = torch.empty(t_len, heads * pad, dtype=dtype, device="cuda:0")
    K.attention(q_out, attended, k_pages, v_pages, table, dev(np.zeros(t_len, np.int32)), dev(positions.astype(np.int32)), heads, kv_heads, pad,
                scale, window, layout=Layout)
    want = attend_plain(q, k, v, scale, window, None, 0)
    got = torch.empty(t_len, heads * vdim, dtype=dtype, device="cuda:0")
    K.gate_heads(attended, pad, None, 0, got, heads, vdim)                             # no gate: the heads' values side by side
    assert rel(got.float().reshape(t_len, heads, vdim), want) < tol(dtype, f32=3e-5, bf16=1.6e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rotated_query_parts_from_a_matrix_of_their_own_and_gates_a_head(K, dtype):
    from beholdd.parts.rope import RotaryFrequencies
    rng = np.random.default_rng(5)
    n, heads, dim, rot_dim, rank, vdim = 37, 3, 12, 8, 20, 10
    stretch = (8.0, 32, 16.0, 1.0)
    rotation = RotaryFrequencies(rot_dim, 100.0, stretch)
    rot = {"dims": rot_dim, "base": 100.0, "scaling": dict(zip(("factor", "original", "fast", "slow"), stretch))}
    down_t, down = rounded(rng.standard_normal((n, 4 + rank + rot_dim + heads)), dtype)
    heads_t, heads_rows = rounded(rng.standard_normal((n, heads * (dim + rot_dim))), dtype)
    positions = rng.integers(0, 128, n).astype(np.int32)
    query = torch.zeros(n, heads * (rank + rot_dim), dtype=dtype, device="cuda:0")
    k_pages = torch.zeros(2, 1, PAGE, rank + rot_dim, dtype=dtype, device="cuda:0")
    v_pages = torch.zeros(2, 1, rank + rot_dim, PAGE, dtype=dtype, device="cuda:0")
    K.latent_write(dev(down_t), 4, None, 1e-5, rotation.frequencies("cuda:0"), rot_dim, dev(positions), dev(np.zeros(n, np.int32)), k_pages, v_pages,
                   dev(np.array([[0, 1]], np.int32)), rank, rot_dim, write=False, query=query, query_head=rank + rot_dim, query_first=rank,
                   source_head=dim + rot_dim, source_first=dim, n_heads=heads, query_source=dev(heads_t), neighbours=True, magnitude=rotation.magnitude)
    want = plain.turn_neighbours(heads_rows.reshape(n, heads, dim + rot_dim)[..., dim:], positions, rot)
    got = query.float().reshape(n, heads, rank + rot_dim)
    assert rel(got[..., rank:], want) < tol(dtype, f32=2e-5, bf16=8e-3) and float(got[..., :rank].abs().max()) == 0.0
    # one gate a head, and the norm of a slice
    values_t, values = rounded(rng.standard_normal((n, heads * vdim)), dtype)
    out = torch.empty(n, heads * vdim, dtype=dtype, device="cuda:0")
    K.gate_heads(dev(values_t), vdim, dev(down_t), 4 + rank + rot_dim, out, heads, vdim, per_head=True)
    gate = plain.sigmoid(down[:, 4 + rank + rot_dim:])
    assert rel(out.float().reshape(n, heads, vdim), values.reshape(n, heads, vdim) * gate[:, :, None]) < tol(dtype, f32=2e-6, bf16=8e-3)
    weight = 1 + 0.3 * rng.standard_normal(rank)
    normed = torch.empty(n, rank, dtype=dtype, device="cuda:0")
    K.slice_rmsnorm(dev(down_t), 4, dev(weight.astype(np.float32)), 1e-5, normed)
    assert rel(normed, plain.weight_norm(down[:, 4:4 + rank], weight, 1e-5)) < tol(dtype, f32=2e-6, bf16=8e-3)
    a, b = rng.standard_normal((9, 70)).astype(np.float32), rng.standard_normal((9, 70)).astype(np.float32)
    total = dev(a)
    K.weighted_sum(total, total, 1.25, dev(b), -0.5)
    assert rel(total, 1.25 * a.astype(np.float64) - 0.5 * b) < 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,width,experts,top,ff", [(1, 64, 4, 1, 40), (37, 192, 8, 3, 96), (5, 130, 5, 5, 33), (700, 256, 16, 2, 64), (300, 128, 4, 1, 128)])
def test_experts_scored_by_sigmoids_and_weighed_on_their_inputs(K, dtype, rows, width, experts, top, ff):
    """The part with its three forms (pair by pair for odd sizes, an expert's rows at once, products over gathered rows) against the
    plain experts: routing by the largest scores, each expert's own sigmoid as its weight, the weight ahead of the activation."""
    from beholdd.parts.base import StepContext
    from beholdd.parts.experts import RoutedExperts
    from beholdd.parts.mlp import SwiGLU
    rng = np.random.default_rng(rows + experts)
    h_t, h = rounded(rng.standard_normal((rows, width)), dtype)
    names = {"m.router": rng.standard_normal((experts, width)) * 4 / np.sqrt(width)}
    for e in [f"e{e}" for e in range(experts)] + ["shared"]:
        names.update({f"m.{e}.gate": rng.standard_normal((ff, width)) / np.sqrt(width) * 2, f"m.{e}.up": rng.standard_normal((ff, width)) / np.sqrt(width) * 2,
                      f"m.{e}.down": rng.standard_normal((width, ff)) / np.sqrt(ff)})
    names = {k: rounded(v, dtype)[1] for k, v in names.items()}
    part = RoutedExperts(width, experts, top, ff, float("inf"), "m.", shared=SwiGLU(width, ff, "m.shared.", names=("gate", "up", "down")),
                         alpha=1.0, router_bias=False, scoring="sigmoid", weigh_input=True, shift=0.0)
    part.load(lambda name: dev(names[name], dtype))
    part.prepare(K)
    want = plain.experts(h, names, "m.", {"router": {"experts": experts, "top": top}, "shared": {"ff": ff}})
    chosen, scores = plain.route(h, names, "m.", top)
    for is_decode in (True, False):
        ctx = StepContext(kernels=K, act_dtype=dtype, device=torch.device("cuda:0"), n_rows=rows, n_seqs=rows if is_decode else 1, tokens=None,
                          positions=None, row_seq=None, seq_start=None, seq_slot=None, seq_past=None, host_seq_start=[], host_seq_slot=[],
                          host_seq_past=[], is_decode=is_decode, max_position=0)
        hidden = torch.zeros(rows, width, device="cuda:0")
        part.forward(ctx, dev(h_t), hidden)
        got_chosen, got_scores = ctx.extras["routing"]
        close = np.sort(plain.linear(h, names["m.router"]), axis=-1)
        sure = (close[:, -top] - close[:, -top - 1] > 1e-3) if top < experts else np.ones(rows, bool)     # no close call at the edge
        assert np.array_equal(got_chosen.cpu().numpy()[sure], chosen[sure]) and rel(got_scores[torch.from_numpy(sure)], scores[sure]) < 1e-5
        assert rel(hidden[torch.from_numpy(sure)], want[sure]) < tol(dtype, f32=5e-5, bf16=2e-2), is_decode


# ---- the engine over every cut --------------------------------------------------------------------------------------------

@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}

    def get(name, seed=5):
        if (name, seed) not in made:
            config = vm.CONFIGS[name]
            weights = vm.random_weights(config, seed, vm.GAIN.get(name, 1.0))
            made[(name, seed)] = (vm.write_model(tmp_path_factory.mktemp(f"vepelix_{name}_{seed}"), config, weights), config, weights)
        return made[(name, seed)]

    return get


LENGTHS = {"mixed": [5, 11, 1, 70, 33, 128, 300], "plain": [1, 7, 23, 64, 90, 200], "odd": [3, 65, 130, 2, 31], "wide": [2, 50, 129, 260]}


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
    tail = schedules.tail_one_by_one(engine, requests, tail=80)      # past every window's edge one token at a time
    check_each("last 80 one by one", tail, want, tolerances, stray)
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


# Without experts no choice magnifies a rounding: both mixers and the dense feed-forward are held at every position.
NO_EXPERTS = {
    "architecture": "Vepelix", "vocab": 83, "width": 64, "norm": {"eps": 1e-5}, "loop": {"start": 0, "stop": 2, "times": 2},
    "layers": [vm.parallel(4, 2, 32, 48, 0.2, 48, 4, 16, 24, 6.0, 8, 1.1, 0.9, dims=16, base=1000.0, stretch=(4.0, 64, 8.0, 1.0), mlp=vm.dense(96, 1.5)),
               vm.latent(4, 16, 16, 32, 48, 24, 0.25, stretch=(8.0, 32, 16.0, 1.0), mlp=vm.dense(40, 3.0)),
               vm.latent(2, 32, 32, 16, 64, 32, 0.2, base=300000.0)],
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_cut_without_experts_holds_at_every_position(tmp_path, dtype):
    config = NO_EXPERTS
    weights = vm.random_weights(config, 7)
    folder = vm.write_model(tmp_path / "bare", config, weights)
    requests = schedules.random_requests(config["vocab"], [1, 9, 66, 130, 200], seed=21)
    want = [plain.forward(config, weights, r) for r in requests]
    engine = engine_for(folder, dtype)
    tolerances = tolerances_for(folder, dtype, requests, want, least=1e-4 if dtype == "float32" else 3e-2)
    for label, got in (("whole", schedules.whole(engine, requests)), ("tail", schedules.tail_one_by_one(engine, requests, tail=80)),
                       ("batches", schedules.batches(engine, requests, batch_size=3)), ("portions", schedules.portions(engine, requests)),
                       ("small portions", schedules.portions(engine, requests, sizes=(2, 2, 3, 2, 1, 2), rest_every=3))):
        check_each(label, got, want, tolerances, 0.0 if dtype == "float32" else 0.03)
    engine.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_batch_changes_nothing_for_its_members(expected, dtype):
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


# ---- one key decides --------------------------------------------------------------------------------------------------

NEEDLE, ASKER = 7, 9


def one_key_model(tmp_path, kind, span, sink=0.0, seed=3):
    """One layer whose last query finds ONE key among hundreds: the token NEEDLE alone projects onto a key direction that the
    token ASKER alone asks for (the score stands out by far more than the others' spread), and the value behind that key is
    large, so the asker's logits hang on whether that one position is read.  kind: "latent" (every key seen; `sink` is what
    the heads' sums hold beside the keys), "window" (span = the window of the attention beside a silenced recurrence),
    "memory" (the recurrence beside a silenced attention: it forgets slowly and the asker reads the needle's key channel)."""
    if kind == "latent":
        layer = vm.latent(2, 16, 16, 16, 32, 16, 0.5)
    elif kind == "window":
        layer = vm.parallel(2, 1, 32, 16, 1.0, span, 1, 8, 8, 4.0, 2, 1.0, 0.0, dims=8)
    else:
        layer = vm.parallel(1, 1, 8, 8, 0.3, 0, 2, 16, 16, 1.0, 2, 0.0, 1.0)
    config = {"architecture": "Vepelix", "vocab": 40, "width": 32, "norm": {"eps": 1e-5}, "layers": [layer]}
    weights = vm.random_weights(config, seed)
    embed = weights["embed"]
    embed[:, :2] = 0.0                        # the other tokens have nothing in the two dimensions that needle and asker use
    embed[NEEDLE] = 0.0
    embed[NEEDLE, 0] = 8.0
    embed[ASKER] = 0.0
    embed[ASKER, 1] = 8.0
    weights["l0.norm1"][:] = 0.0
    weights["final.norm"][:] = 0.0
    weights["l0.ls1"][:] = 1.0
    m = "l0.mix."
    if kind == "latent":
        weights[m + "dq.norm"][:] = 1.0
        weights[m + "dkv.norm"][:] = 1.0
        weights[m + "dq"][:] *= 0.02
        weights[m + "dq"][3, 1] = 1.0                                     # the asker's query latent: its dimension 3
        weights[m + "uq"][:] *= 0.02
        weights[m + "uq"][3, 3] = weights[m + "uq"][32 + 3, 3] = 1.0      # which both heads' queries carry into their dimension 3
        weights[m + "dkv"][5, 0] = 3.0                                    # the needle's latent: its dimension 5
        weights[m + "uk"][:] *= 0.1
        weights[m + "uk"][3, 5] = weights[m + "uk"][16 + 3, 5] = 1.0      # which the heads' keys carry into dimension 3
        weights[m + "uv"][:, 5] = 2.0
        weights[m + "sink"][:] = sink
        weights[m + "g"][:] = 0.0
    elif kind == "window":
        a = m + "left."
        weights[a + "q.norm"][:] = 1.0
        weights[a + "k.norm"][:] = 1.0
        weights[a + "q"][:] *= 0.05
        weights[a + "q"][20, 1] = weights[a + "q"][32 + 20, 1] = 3.0      # the asker's query: dimension 20 of both heads (beyond the turned ones)
        weights[a + "k"][20, 0] = 3.0                                     # the needle's key: the same dimension; every key is normed to one length
        weights[a + "v"][:, 0] = 2.0                                      # and a value that stands out
    else:
        b = m + "right."
        weights[b + "a1"][:] = 0.0
        weights[b + "a2.b"][:] = 6.0                                      # a step keeps all but a four-hundredth
        weights[b + "k"][:] *= 0.05
        weights[b + "k"][2, 0] = weights[b + "k"][16 + 2, 0] = 1.0
        weights[b + "q"][:] *= 0.05
        weights[b + "q"][2, 1] = weights[b + "q"][16 + 2, 1] = 1.0
        weights[b + "v"][:, 0] = 1.0
        weights[b + "v"][::2, 0] = -1.0
        weights[b + "o"][:] *= 4.0                                        # the read-out has unit size: let it weigh beside the residual
        weights[b + "norm"][:] = 1.0
    weights = {k: torch.from_numpy(v).to(torch.bfloat16).to(torch.float32).numpy() for k, v in weights.items()}
    return vm.write_model(tmp_path / f"{kind}_{span}_{sink}", config, weights), config, weights


def needle_case(tmp_path, dtype, kind, span, needle_at, moves, length=420, sink=0.0):
    """The needle at `needle_at`, the asker last; `moves`: whether the needle may change the asker's logits at all (a number: by at
    least that share of the largest logit instead of a fifth)."""
    folder, config, weights = one_key_model(tmp_path, kind, span, sink)
    rng = np.random.default_rng(needle_at)
    others = [t for t in range(config["vocab"]) if t not in (NEEDLE, ASKER)]
    tokens = [int(rng.choice(others)) for _ in range(length)]
    without = list(tokens) + [ASKER]
    tokens[needle_at] = NEEDLE
    tokens.append(ASKER)
    want, blind = plain.forward(config, weights, tokens)[-1], plain.forward(config, weights, without)[-1]
    if moves:
        assert np.abs(want - blind).max() > (0.2 if moves is True else moves) * np.abs(want).max()             # the one key moves the logits
    else:
        assert np.abs(want - blind).max() < 1e-6 * np.abs(want).max()            # it lies outside what the asker sees
    engine = engine_for(folder, dtype, max_tokens=1024)
    from beholdd.engine import StepEntry
    slot = engine.alloc_slot()
    in_prompt = engine.step([StepEntry(slot, tokens, [len(tokens) - 1])]).float().cpu().numpy()[0]
    engine.free_slot(slot)
    slot = engine.alloc_slot()
    engine.step([StepEntry(slot, tokens[:200], [])])
    engine.step([StepEntry(slot, tokens[200:-3], [])])
    for token in tokens[-3:-1]:
        engine.step([StepEntry(slot, [token], [])])
    decoded = engine.step([StepEntry(slot, tokens[-1:], [0])]).float().cpu().numpy()[0]
    engine.free_slot(slot)
    for got in (in_prompt, decoded):          # sharp scores and large values: bfloat16 rounds them to a few parts in a hundred
        assert np.abs(got - want).max() < (1e-4 if dtype == "float32" else 6e-2) * np.abs(want).max()
    return want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("needle_at", [0, 1, 63, 64, 65, 127, 128, 300, 419])
def test_one_far_key_decides_where_every_key_is_seen(tmp_path, dtype, needle_at):
    needle_case(tmp_path, dtype, "latent", 0, needle_at, True)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_sink_that_outweighs_the_one_key(tmp_path, dtype):
    """With a sink above the needle's score the heads' outputs shrink to a fraction: the logits are others than with a small
    sink, and the engine's are the plain ones either way."""
    small = needle_case(tmp_path, dtype, "latent", 0, 300, True, sink=0.0)
    large = needle_case(tmp_path, dtype, "latent", 0, 300, 0.05, sink=14.0)
    assert np.abs(small - large).max() > 0.2 * np.abs(small).max()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("window", [64, 96, 130, 2, 65, 141])
def test_a_key_just_inside_and_just_outside_the_window(tmp_path, dtype, window):
    last = 420
    needle_case(tmp_path, dtype, "window", window, last - window + 1, True)   # the oldest position the window keeps
    needle_case(tmp_path, dtype, "window", window, last - window, False)      # the one that has just left it


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("needle_at", [0, 1, 100, 300])
def test_the_decaying_memory_keeps_one_token_for_hundreds_of_steps(tmp_path, dtype, needle_at):
    needle_case(tmp_path, dtype, "memory", 0, needle_at, True)


# ---- long runs, generation, programs ----------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompts_in_portions_and_long_decoding(folders, dtype):
    """A request of 700 tokens: the prompt in portions that end at, before and after page borders, then 150 tokens one by one
    through the captured steps, in a cache whose pages and slots were used before by other requests."""
    folder, config, weights = folders("wide")
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
    tolerance = tolerances_for(folder, dtype, [long_one], [want])[0]
    check("long", [np.concatenate(rows)], [want], tolerance, STRAY[dtype])
    if engine.graphs is not None:
        assert len(engine.graphs.graphs) >= 1          # the one-token steps were captured and replayed
    assert engine.cache.free_page_count() == engine.cache.n_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(tmp_path, dtype):
    import beholdd
    config = NO_EXPERTS
    weights = vm.random_weights(config, 5, gain=1.5)
    folder = vm.write_model(tmp_path / "generating", config, weights)
    prompts = schedules.random_requests(config["vocab"], [1, 9, 30, 70], seed=6)
    max_new = [12, 9, 12, 40]
    engine = beholdd.Engine(folder, dtype=dtype, max_tokens=1024)
    results = engine.generate(prompts, max_new_tokens=max_new)
    assert len({token for r in results for token in r.token_ids}) >= 6
    for prompt, result, n in zip(prompts, results, max_new):
        assert len(result.token_ids) == n
        if dtype == "float32":
            assert result.token_ids == plain.greedy(config, weights, prompt, n)
            continue
        fed = list(prompt)
        near = 0
        for token in result.token_ids:          # every choice is the plain one's, or lies within rounding of it
            row = plain.forward(config, weights, fed)[-1]
            near += int(row[token] >= row.max() - 0.04 * np.abs(row).max())
            fed.append(token)
        assert near >= 0.9 * n, (near, n)
    sampled = engine.generate(prompts, max_new_tokens=8, temperature=0.9, top_k=20, top_p=0.9, seed=4)
    again = engine.generate(prompts, max_new_tokens=8, temperature=0.9, top_k=20, top_p=0.9, seed=4)
    assert [r.token_ids for r in sampled] == [r.token_ids for r in again]
    engine.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_and_generate_programs(folders, tmp_path, dtype):
    folder, config, weights = folders("odd")
    requests = schedules.random_requests(config["vocab"], [40, 7, 66], seed=9)
    want = [plain.forward(config, weights, r) for r in requests]
    tolerances = tolerances_for(folder, dtype, requests, want)
    steps = schedules.trace_of(schedules.batches, requests, batch_size=3)
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                          "--out", str(tmp_path / "out"), "--max-tokens", "256"],
                         input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    got = [[] for _ in requests]      # every request's rows in the order of its positions, whatever step made them
    for record in steps:
        rows = np.fromfile(tmp_path / "out" / f"{record['step']}.f32", dtype="<f4").reshape(-1, config["vocab"])
        at = 0
        for entry in record["entries"]:
            assert entry["want"] == list(range(len(entry["tokens"])))
            got[int(entry["id"][1:])].append(rows[at:at + len(entry["want"])])
            at += len(entry["want"])
        assert at == len(rows)
    check_each("replayed", [np.concatenate(rows) for rows in got], want, tolerances, STRAY[dtype])
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "beholdd"), "generate", "--model", folder, "--dtype", dtype,
                          "--prompt-ids", ",".join(str(t) for t in requests[1]), "--max-new-tokens", "5"], capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    if dtype == "float32":
        expected_tokens = plain.greedy(config, weights, requests[1], 5)
        assert all(str(token) in run.stdout for token in expected_tokens), (run.stdout, expected_tokens)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(10))
def test_drawn_configurations(seed, dtype, tmp_path):
    """Sizes, counts, constants and layer orders that nobody picked, on the real kernels."""
    config = vm.drawn_config(100 + seed)
    weights = vm.random_weights(config, seed, gain=0.7)
    folder = vm.write_model(tmp_path / "drawn", config, weights)
    requests = schedules.random_requests(config["vocab"], [1, 19, 70, 150], seed=seed)
    want = [plain.forward(config, weights, r) for r in requests]
    engine = engine_for(folder, dtype)
    tolerances, stray = tolerances_for(folder, dtype, requests, want), STRAY[dtype]
    for label, got in (("whole", schedules.whole(engine, requests)), ("tail", schedules.tail_one_by_one(engine, requests, tail=70)),
                       ("batches", schedules.batches(engine, requests, batch_size=3)),
                       ("small portions", schedules.portions(engine, requests, sizes=(2, 2, 3, 2, 1, 2), rest_every=3))):
        check_each(f"{config} {label}", got, want, tolerances, stray)
    engine.cache.check_invariants()
