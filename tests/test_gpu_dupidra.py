"""Dupidra on the GPU: every new kernel alone against the plain implementation's function of the same mechanism, and the
engine over every cut of the work (whole prompts, token by token, portions down to two tokens, batches of unequal
requests, slots and pages used again) in float32 and bfloat16 on configurations that differ in every size; models in which
ONE key decides the logits, far back, at page borders, at the first positions and just inside and just outside a chunk and
a window, in a prompt and decoded; a memory that holds one token for hundreds of steps; long decoding through the captured
steps; greedy generation through the entry point and the trace replay program."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import dupidra_models as dm
import plain_dupidra as plain
import schedules
from test_gpu_pudorax import STRAY, TOLERANCE, check, check_each, dev, engine_for, ragged, rel, rounded, tol, tolerances_for

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = [torch.float32, torch.bfloat16]
PAGE = 64


@pytest.fixture(scope="module")
def K():
    from beholdd.kernels import HipKernels
    return HipKernels("cuda:0")


# ---- kernels alone ------------------------------------------------------------------------------------------

@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("rows,width,eps,alpha", [(1, 48, 1e-6, 1.0), (33, 1000, 1e-5, 2.5), (4, 5120, 1e-6, 0.3), (70, 260, 1e-2, 7.0), (3, 9001, 1e-6, 2.0), (5, 4096, 1e-5, 1.5)])
def test_norm_behind_the_weighted_sum(K, out_dtype, rows, width, eps, alpha):
    rng = np.random.default_rng(width)
    hidden = (rng.standard_normal((rows, width)) * 3 + 40).astype(np.float32)            # a mean far larger than the spread
    y = rng.standard_normal((rows, width)).astype(np.float32) * 5
    w = {"n": (1 + 0.3 * rng.standard_normal(width)).astype(np.float32), "n.b": rng.standard_normal(width).astype(np.float32)}
    want = plain.layer_norm(alpha * hidden.astype(np.float64) + y, w, "n", eps)
    on_device = dev(hidden)
    rounded_out = torch.empty(rows, width, dtype=out_dtype, device="cuda:0")
    K.sum_layernorm(on_device, dev(y), alpha, dev(w["n"]), dev(w["n.b"]), eps, rounded_out)
    assert rel(on_device, want) < 1e-4 and rel(rounded_out, want) < tol(out_dtype, f32=1e-4, bf16=8e-3)
    again = dev(hidden)
    K.sum_layernorm(again, dev(y), alpha, dev(w["n"]), dev(w["n.b"]), eps, None)             # nobody reads a rounded copy
    assert torch.equal(again, on_device)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gelu(K, dtype):
    x_t, x = rounded(np.random.default_rng(0).standard_normal((9, 130)) * 3, dtype)
    out = torch.empty(9, 130, dtype=dtype, device="cuda:0")
    K.gelu_tanh(dev(x_t), out)
    assert rel(out, plain.gelu_tanh(x)) < tol(dtype, bf16=8e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,pad,turned,base,chunk", [
    (6, 2, 24, 40, 64, 8, 1e4, 20), (4, 4, 64, 64, 64, 64, 500.0, 64), (8, 1, 12, 20, 32, 0, 1.0, 1), (2, 2, 272, 16, 272, 64, 1e6, 100),
    (3, 1, 128, 128, 128, 32, 1e6, 0), (16, 1, 64, 48, 64, 64, 2e4, 65), (17, 1, 32, 32, 32, 16, 1e4, 130)])
def test_bias_head_norms_rotation_cache_write_and_chunked_attention(K, dtype, heads, kv_heads, dim, vdim, pad, turned, base, chunk):
    """From the projected rows to the attended heads: biases, every head normed with the one weight, rotation in halves, keys
    and values of different sizes through one padded head, chunks counted from position 0; a prompt in two portions that end
    inside pages, then decode rows."""
    rng = np.random.default_rng(dim + vdim + chunk)
    t_len, eps, scale, first = 150, 1e-5, 0.2, 7
    q_width, k_width, v_width = heads * dim, kv_heads * dim, kv_heads * vdim
    proj_t, proj = rounded(rng.standard_normal((t_len, first + q_width + k_width + v_width + 3)), dtype)
    bias = (0.5 * rng.standard_normal(q_width + k_width + v_width)).astype(np.float32)
    wq, wk = (1 + 0.3 * rng.standard_normal(dim)).astype(np.float32), (1 + 0.3 * rng.standard_normal(dim)).astype(np.float32)
    x = proj[:, first:first + q_width + k_width + v_width].astype(np.float64) + bias
    positions = np.arange(t_len)
    q = plain.rotate_halves(plain.rms(x[:, :q_width].reshape(t_len, heads, dim), eps) * wq, positions, turned, base)
    k = plain.rotate_halves(plain.rms(x[:, q_width:q_width + k_width].reshape(t_len, kv_heads, dim), eps) * wk, positions, turned, base)
    v = x[:, q_width + k_width:].reshape(t_len, kv_heads, vdim)
    seen = plain.visible(t_len, "chunk", chunk) if chunk else plain.visible(t_len)
    want = plain.softmax_attention(q, k, v, scale, seen)
    freq = dev(np.array([base ** (-2.0 * i / turned) for i in range(turned // 2)], np.float32)) if turned else None
    k_pages = torch.full((5, kv_heads, PAGE, pad), 7.0, dtype=dtype, device="cuda:0")      # whatever a page held before
    v_pages = torch.full((5, kv_heads, pad, PAGE), 7.0, dtype=dtype, device="cuda:0")
    table = dev(np.array([[3, 0, 4, 1]], np.int32))

    class Layout:
        n_seqs, seq_start = 1, None
    got = []
    for lo, hi in [(0, 63), (63, 140)] + [(t, t + 1) for t in range(140, t_len)]:
        n = hi - lo
        pos = dev(np.arange(lo, hi, dtype=np.int32))
        q_out = torch.empty(n, heads * pad, dtype=dtype, device="cuda:0")
        K.head_norm_rope_write(dev(proj_t[lo:hi].contiguous()), first, dev(bias), dev(wq), dev(wk), eps, freq, turned, pos,
                               dev(np.zeros(n, np.int32)), q_out, k_pages, v_pages, table, heads, kv_heads, dim, vdim, pad, True)
        layout = Layout()
        layout.seq_start, layout.max_rows_per_seq, layout.max_position = dev(np.array([0, n], np.int32)), n, hi - 1
        attended = torch.empty(n, heads * pad, dtype=dtype, device="cuda:0")
        K.attention(q_out, attended, k_pages, v_pages, table, dev(np.zeros(n, np.int32)), pos, heads, kv_heads, pad, scale, 0, layout=layout,
                    chunk=chunk)
        got.append(attended.float().reshape(n, heads, pad)[..., :vdim].cpu().numpy())
        if pad > vdim:
            assert float(attended.float().reshape(n, heads, pad)[..., vdim:].abs().max()) == 0
    assert rel(np.concatenate(got), want) < tol(dtype, f32=3e-5, bf16=2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_heads_without_norm_bias_or_rotation_pass_as_they_are(K, dtype):
    rng = np.random.default_rng(4)
    heads, kv_heads, dim, vdim, pad, n = 3, 1, 20, 12, 32, 5
    proj_t, proj = rounded(rng.standard_normal((n, (heads + kv_heads) * dim + kv_heads * vdim)), dtype)
    k_pages = torch.zeros(1, kv_heads, PAGE, pad, dtype=dtype, device="cuda:0")
    v_pages = torch.zeros(1, kv_heads, pad, PAGE, dtype=dtype, device="cuda:0")
    q_out = torch.empty(n, heads * pad, dtype=dtype, device="cuda:0")
    pos = dev(np.arange(n, dtype=np.int32))
    K.head_norm_rope_write(dev(proj_t), 0, None, None, None, 0.0, None, 0, pos, dev(np.zeros(n, np.int32)), q_out, k_pages, v_pages,
                           dev(np.zeros((1, 1), np.int32)), heads, kv_heads, dim, vdim, pad, True)
    assert rel(q_out.float().reshape(n, heads, pad)[..., :dim], proj[:, :heads * dim].reshape(n, heads, dim)) == 0
    if K.kv_order(dtype, pad) == 0:
        assert rel(k_pages[0, 0, :n, :dim], proj[:, heads * dim:(heads + 1) * dim]) == 0
        assert rel(v_pages[0, 0, :vdim, :n].t(), proj[:, (heads + 1) * dim:]) == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,vdim,rank,window", [(3, 16, 12, 32, 27), (6, 32, 40, 96, 64), (2, 8, 8, 20, 1), (5, 16, 16, 64, 65), (1, 32, 32, 32, 0)])
def test_windowed_attention_over_a_latent_without_a_rotated_part(K, dtype, heads, dim, vdim, rank, window):
    rng = np.random.default_rng(rank + window)
    t_len, eps, scale = 150, 1e-5, 0.25
    down_t, down = rounded(rng.standard_normal((t_len, 4 + rank)), dtype)
    weight = (1 + 0.3 * rng.standard_normal(rank)).astype(np.float32)
    q_t, q = rounded(rng.standard_normal((t_len, heads * dim)), dtype)
    uk_t, uk = rounded(rng.standard_normal((heads * dim, rank)) / np.sqrt(rank), dtype)
    uv_t, uv = rounded(rng.standard_normal((heads * vdim, rank)) / np.sqrt(rank), dtype)
    latent = plain.rms(down[:, 4:], eps) * weight
    seen = plain.visible(t_len, "window", window) if window else plain.visible(t_len)
    want = plain.softmax_attention(q.reshape(t_len, heads, dim), (latent @ uk.T.astype(np.float64)).reshape(t_len, heads, dim),
                                   (latent @ uv.T.astype(np.float64)).reshape(t_len, heads, vdim), scale, seen)
    k_pages = torch.zeros(4, 1, PAGE, rank, dtype=dtype, device="cuda:0")
    v_pages = torch.zeros(4, 1, rank, PAGE, dtype=dtype, device="cuda:0")
    table = dev(np.array([[2, 0, 3]], np.int32))
    key_up = dev(uk_t).view(heads, dim, rank).contiguous()
    value_up = dev(uv_t).view(heads, vdim, rank).transpose(1, 2).contiguous()

    class Layout:
        n_seqs, seq_start = 1, None
    got = []
    for lo, hi in [(0, 100)] + [(t, t + 1) for t in range(100, t_len)]:
        n = hi - lo
        pos, row_seq = dev(np.arange(lo, hi, dtype=np.int32)), dev(np.zeros(n, np.int32))
        K.latent_write(dev(down_t[lo:hi].contiguous()), 4, dev(weight), eps, None, 0, pos, row_seq, k_pages, v_pages, table, rank, 0)
        query = torch.empty(n, heads * rank, dtype=dtype, device="cuda:0")
        K.heads_linear(dev(q_t[lo:hi].contiguous()), dim, 0, key_up, query, rank, 0, heads)
        layout = Layout()
        layout.seq_start, layout.max_rows_per_seq, layout.max_position = dev(np.array([0, n], np.int32)), n, hi - 1
        attended = torch.empty(n, heads * rank, dtype=dtype, device="cuda:0")
        K.attention(query, attended, k_pages, v_pages, table, row_seq, pos, heads, 1, rank, scale, window, layout=layout)
        values = torch.empty(n, heads * vdim, dtype=dtype, device="cuda:0")
        K.heads_linear(attended, rank, 0, value_up, values, vdim, 0, heads)
        got.append(values.float().reshape(n, heads, vdim).cpu().numpy())
    assert rel(np.concatenate(got), want) < tol(dtype, f32=3e-5, bf16=2.5e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,vdim,cap,lengths", [(3, 8, 20, 9.0, [5, 1, 31]), (1, 16, 16, 1.0, [70]), (4, 32, 40, 11.0, [3, 17, 2]),
                                                        (2, 80, 70, 15.0, [40]), (5, 4, 15, 8.0, [1, 1, 1, 1]), (2, 128, 128, 12.0, [9, 33]),
                                                        (1, 260, 16, 12.0, [18]), (3, 12, 33, 6.0, [200, 64, 65])])
def test_matrix_memory(K, dtype, heads, dim, vdim, cap, lengths):
    """Gates, recurrence and read-out over ragged rows of several sequences, into slots in another order than the batch's, and
    then a second step that continues from the states the first one left (the running maximum among them)."""
    rng = np.random.default_rng(heads * vdim + dim)
    key, value, eps = heads * dim, heads * vdim, 1e-5
    slots = list(rng.permutation(len(lengths) + 1)[:len(lengths)])
    seq_start, seq_slot, _, starts = ragged(lengths, slots)
    floats = K.mlstm_state_floats(heads, dim, vdim)
    assert floats == heads * ((vdim + 1) * dim + 1)
    state = torch.zeros(len(lengths) + 1, floats, device="cuda:0")
    total = sum(lengths)
    bias = np.concatenate([rng.standard_normal(heads), rng.uniform(0.5, 4, heads)]).astype(np.float32)
    norm_weight = (1 + 0.3 * rng.standard_normal(value)).astype(np.float32)
    steps = []
    for _ in range(2):
        proj_t, proj = rounded(rng.standard_normal((total, 3 + 2 * key + 2 * value)), dtype)
        pre = (rng.standard_normal((total, 2 * heads)) * 3).astype(np.float32)
        read = torch.empty(total, value, device="cuda:0")
        beside = torch.empty(total, 4 * heads, device="cuda:0")
        K.mlstm_gates(dev(pre), dev(bias), cap, state, seq_start, seq_slot, beside, heads, dim, vdim)
        K.mlstm_scan(dev(proj_t), 3, 3 + key, 3 + 2 * key, beside, state, seq_start, seq_slot, read, heads, dim, vdim)
        out = torch.empty(total, value, dtype=dtype, device="cuda:0")
        K.mlstm_finish(read, beside, dev(proj_t), 3 + 2 * key + value, dev(norm_weight), eps, out, heads, vdim)
        steps.append((proj, pre, out.float().cpu().numpy()))
    eye = np.eye(total)
    for i, n in enumerate(lengths):
        lo = starts[i]
        kept = None
        for proj, pre, got in steps:
            # the plain mechanism reads its q, k, v, g and gates through matrices: here they pick the given rows out of one-hot inputs
            w = {"m.q": proj[lo:lo + n, 3:3 + key].T, "m.k": proj[lo:lo + n, 3 + key:3 + 2 * key].T,
                 "m.v": proj[lo:lo + n, 3 + 2 * key:3 + 2 * key + value].T, "m.g": proj[lo:lo + n, 3 + 2 * key + value:].T,
                 "m.i": pre[lo:lo + n, :heads].T, "m.f": pre[lo:lo + n, heads:].T, "m.i.b": bias[:heads], "m.f.b": bias[heads:],
                 "m.norm": norm_weight, "m.o": np.eye(value)}
            want, kept = plain.matrix_memory(np.eye(n), w, "m.", {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}, eps, state=kept)
            assert rel(got[lo:lo + n], want) < tol(dtype, f32=1e-4, bf16=1.2e-2), (i, n)
        held = state[slots[i]].reshape(heads, (vdim + 1) * dim + 1).cpu().numpy()
        columns = held[:, :-1].reshape(heads, vdim + 1, dim)
        assert rel(columns[:, :vdim].transpose(0, 2, 1), kept[0]) < 1e-4 and rel(columns[:, vdim], kept[1]) < 1e-4
        assert rel(held[:, -1], kept[2]) < 1e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,vdim,cap,seqs", [(3, 8, 20, 9.0, 4), (1, 16, 16, 1.0, 1), (4, 32, 40, 11.0, 9), (2, 80, 70, 15.0, 2),
                                                     (5, 4, 15, 8.0, 3), (2, 128, 128, 12.0, 8), (1, 260, 16, 12.0, 2), (3, 12, 33, 6.0, 5)])
def test_matrix_memory_decode_step_in_one_launch(K, dtype, heads, dim, vdim, cap, seqs):
    """A step of one row a sequence through the one launch against the same step through the three kernels, from the states
    that a ragged prompt left, into slots in another order than the batch's; three steps in a row."""
    rng = np.random.default_rng(heads * vdim + dim + seqs)
    key, value, eps = heads * dim, heads * vdim, 1e-5
    lengths = [int(n) for n in rng.integers(1, 40, seqs)]
    slots = list(rng.permutation(seqs + 1)[:seqs])
    seq_start, seq_slot, _, _ = ragged(lengths, slots)
    state = torch.zeros(seqs + 1, K.mlstm_state_floats(heads, dim, vdim) + 3, device="cuda:0")      # (a slot's row may be longer)
    bias = dev(np.concatenate([rng.standard_normal(heads), rng.uniform(0.5, 4, heads)]).astype(np.float32))
    norm_weight = dev((1 + 0.3 * rng.standard_normal(value)).astype(np.float32))

    def three(proj, pre, state, seq_start):
        n = proj.shape[0]
        read, beside = torch.empty(n, value, device="cuda:0"), torch.empty(n, 4 * heads, device="cuda:0")
        K.mlstm_gates(pre, bias, cap, state, seq_start, seq_slot, beside, heads, dim, vdim)
        K.mlstm_scan(proj, 3, 3 + key, 3 + 2 * key, beside, state, seq_start, seq_slot, read, heads, dim, vdim)
        out = torch.empty(n, value, dtype=dtype, device="cuda:0")
        K.mlstm_finish(read, beside, proj, 3 + 2 * key + value, norm_weight, eps, out, heads, vdim)
        return out
    total = sum(lengths)
    three(dev(rounded(rng.standard_normal((total, 3 + 2 * key + 2 * value)), dtype)[0]), dev((rng.standard_normal((total, 2 * heads)) * 3).astype(np.float32)),
          state, seq_start)
    other = state.clone()
    one_each = dev(np.arange(seqs + 1, dtype=np.int32))
    for _ in range(3):
        proj = dev(rounded(rng.standard_normal((seqs, 3 + 2 * key + 2 * value)), dtype)[0])
        pre = dev((rng.standard_normal((seqs, 2 * heads)) * 3).astype(np.float32))
        want = three(proj, pre, state, one_each)
        got = torch.empty(seqs, value, dtype=dtype, device="cuda:0")
        K.mlstm_step(proj, 3, 3 + key, 3 + 2 * key, 3 + 2 * key + value, pre, bias, cap, other, seq_slot, norm_weight, eps, got, heads, dim, vdim)
        assert rel(got, want.double().cpu().numpy()) < tol(dtype, f32=2e-5, bf16=8e-3)
        assert rel(other, state.double().cpu().numpy()) < 1e-5
    assert float(other[:, -3:].abs().max()) == 0


# ---- the engine over every cut ------------------------------------------------------------------------------------

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


LENGTHS = {"mixed": [5, 11, 1, 70, 33, 128, 300], "plain": [1, 7, 23, 64, 90, 200], "edges": [3, 65, 130, 2, 31, 330], "deep": [2, 50, 129, 260], "odd": [1, 40, 100, 210]}


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
    tail = schedules.tail_one_by_one(engine, requests, tail=70)      # past every chunk's and window's edge one token at a time
    check_each("last 70 one by one", tail, want, tolerances, stray)
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


# Without experts no choice magnifies a rounding: the three mixers, the dense feed-forward and borrowed layers are held at
# every position in float32, and in bfloat16 at all but three in a hundred (the memory's read-out is divided by its own size
# head by head, which at a sequence's first positions can be small beside the rounding of q and k).
NO_EXPERTS = {
    "architecture": "Dupidra", "vocab": 83, "width": 64, "postln_alpha": 2.0, "norm": {"eps": 1e-5},
    "layers": [dm.attention(4, 2, 32, 48, 0.2, chunk=48, rot_dims=16, base=1000.0, mlp=dm.dense(96)),
               dm.mlstm(4, 16, 24, 10.0, mlp=None),
               dm.latent(4, 16, 16, 32, 0.25, window=70, mlp=dm.dense(40))],
}
NO_EXPERTS["layers"].append(dm.borrowed(NO_EXPERTS["layers"], 3, 1))
NO_EXPERTS["layers"].append(dm.borrowed(NO_EXPERTS["layers"], 4, 0))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_cut_without_experts_holds_at_every_position(tmp_path, dtype):
    config = NO_EXPERTS
    weights = dm.random_weights(config, 7)
    folder = dm.write_model(tmp_path / "bare", config, weights)
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


def one_key_model(tmp_path, kind, span, seed=3):
    """One layer whose last query finds ONE key among hundreds: the token NEEDLE alone projects onto a key direction that the
    token ASKER alone asks for (the score stands out by far more than the others' spread), and the value behind that key is
    large, so the asker's logits hang on whether that one position is read.  kind: "attention" (span = chunk), "latent"
    (span = window), "memory" (the needle opens the input gate wide and the memory forgets slowly)."""
    if kind == "attention":
        layer = dm.attention(2, 1, 32, 16, 1.0, chunk=span, rot_dims=8, mlp=None)
    elif kind == "latent":
        layer = dm.latent(2, 16, 16, 32, 0.5, window=span, mlp=None)
    else:
        layer = dm.mlstm(2, 16, 16, 12.0, mlp=None)
    config = {"architecture": "Dupidra", "vocab": 40, "width": 32, "postln_alpha": 1.0, "norm": {"eps": 1e-5}, "layers": [layer]}
    weights = dm.random_weights(config, seed)
    embed = weights["embed"]
    embed[:, :2] = 0.0                        # the other tokens have nothing in the two dimensions that needle and asker use
    embed[NEEDLE] = 0.0
    embed[NEEDLE, 0] = 8.0
    embed[ASKER] = 0.0
    embed[ASKER, 1] = 8.0
    for name in ("l0.norm1", "final.norm"):
        weights[name][:] = 1.0
        weights[name + ".b"][:] = 0.0
    m = "l0.mix."
    if kind == "attention":
        for name in ("q.b", "k.b", "v.b"):
            weights[m + name][:] = 0.0
        weights[m + "q.norm"][:] = 1.0
        weights[m + "k.norm"][:] = 1.0
        weights[m + "q"][:] *= 0.05
        weights[m + "q"][20, 1] = weights[m + "q"][32 + 20, 1] = 3.0      # the asker's query: dimension 20 of both heads (beyond the turned ones)
        weights[m + "k"][20, 0] = 3.0                                     # the needle's key: the same dimension; every key is normed to one length
        weights[m + "v"][:, 0] = 2.0                                      # and a value that stands out
    elif kind == "latent":
        weights[m + "dkv.norm"][:] = 1.0
        weights[m + "q"][:] *= 0.02
        weights[m + "q"][3, 1] = weights[m + "q"][16 + 3, 1] = 1.0        # the asker's query: dimension 3 of both heads
        weights[m + "dkv"][5, 0] = 3.0                                    # the needle's latent: its dimension 5
        weights[m + "uk"][:] *= 0.1
        weights[m + "uk"][3, 5] = weights[m + "uk"][16 + 3, 5] = 1.0      # which the heads' keys carry into dimension 3
        weights[m + "uv"][:, 5] = 2.0
    else:
        weights[m + "i"][:] = 0.0
        weights[m + "i"][:, 0] = 2.0                                      # the needle opens the input gate; for the others it is nearly shut
        weights[m + "i.b"][:] = -2.0
        weights[m + "f"][:] = 0.0
        weights[m + "f.b"][:] = 6.0                                       # a step keeps all but a four-hundredth
        weights[m + "k"][:] *= 0.05
        weights[m + "k"][2, 0] = weights[m + "k"][16 + 2, 0] = 1.0
        weights[m + "q"][:] *= 0.05
        weights[m + "q"][2, 1] = weights[m + "q"][16 + 2, 1] = 1.0
        weights[m + "v"][:, 0] = 1.0
        weights[m + "v"][::2, 0] = -1.0
        weights[m + "o"][:] *= 4.0                                        # the read-out has unit size: let it weigh beside the residual
        weights[m + "norm"][:] = 1.0
    weights = {k: torch.from_numpy(v).to(torch.bfloat16).to(torch.float32).numpy() for k, v in weights.items()}
    return dm.write_model(tmp_path / f"{kind}_{span}", config, weights), config, weights


def needle_case(tmp_path, dtype, kind, span, needle_at, moves, length=420):
    """The needle at `needle_at`, the asker last; `moves`: whether the needle may change the asker's logits at all."""
    folder, config, weights = one_key_model(tmp_path, kind, span)
    rng = np.random.default_rng(needle_at)
    others = [t for t in range(config["vocab"]) if t not in (NEEDLE, ASKER)]
    tokens = [int(rng.choice(others)) for _ in range(length)]
    without = list(tokens) + [ASKER]
    tokens[needle_at] = NEEDLE
    tokens.append(ASKER)
    want, blind = plain.forward(config, weights, tokens)[-1], plain.forward(config, weights, without)[-1]
    if moves:
        assert np.abs(want - blind).max() > 0.2 * np.abs(want).max()             # the one key moves the logits
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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("needle_at", [0, 1, 63, 64, 65, 127, 128, 300, 419])
def test_one_far_key_decides_where_every_key_is_seen(tmp_path, dtype, needle_at):
    needle_case(tmp_path, dtype, "attention", 0, needle_at, True)
    needle_case(tmp_path, dtype, "latent", 0, needle_at, True)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("chunk", [64, 100, 9, 200])
def test_a_key_just_inside_and_just_outside_the_chunk(tmp_path, dtype, chunk):
    last = 420
    start = last - last % chunk
    needle_case(tmp_path, dtype, "attention", chunk, start, True)             # the chunk's first position
    needle_case(tmp_path, dtype, "attention", chunk, start - 1, False)        # the last of the chunk before
    if start + 1 < last:
        needle_case(tmp_path, dtype, "attention", chunk, last - 1, True)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("window", [64, 96, 130, 2, 65])
def test_a_key_just_inside_and_just_outside_the_window(tmp_path, dtype, window):
    last = 420
    needle_case(tmp_path, dtype, "latent", window, last - window + 1, True)   # the oldest position the window keeps
    needle_case(tmp_path, dtype, "latent", window, last - window, False)      # the one that has just left it


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("needle_at", [0, 1, 100, 300])
def test_the_memory_keeps_one_token_for_hundreds_of_steps(tmp_path, dtype, needle_at):
    needle_case(tmp_path, dtype, "memory", 0, needle_at, True)


# ---- long runs, generation, programs ----------------------------------------------------------------------------------

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
    tolerance = tolerances_for(folder, dtype, [long_one], [want])[0]
    check("long", [np.concatenate(rows)], [want], tolerance, STRAY[dtype])
    if engine.graphs is not None:
        assert len(engine.graphs.graphs) >= 1          # the one-token steps were captured and replayed
    assert engine.cache.free_page_count() == engine.cache.n_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(tmp_path, dtype):
    import beholdd
    from beholdd.engine import StepEntry
    config = dm.GENERATING
    weights = dm.random_weights(config, 5, gain=dm.GENERATING_GAIN)
    folder = dm.write_model(tmp_path / "generating", config, weights)
    prompts = schedules.random_requests(config["vocab"], [1, 9, 30, 70], seed=6)
    max_new = [12, 9, 12, 40]
    engine = beholdd.Engine(folder, dtype=dtype, max_tokens=1024)
    results = engine.generate(prompts, max_new_tokens=max_new)
    assert len({token for r in results for token in r.token_ids}) >= 6
    # what bfloat16's rounding alone does to this model's logits (its sublayers outweigh the residual and magnify it)
    margin = 2 * max(tolerances_for(folder, dtype, prompts[1:], [plain.forward(config, weights, p) for p in prompts[1:]]))
    for prompt, result, n in zip(prompts, results, max_new):
        if dtype == "float32":
            assert result.token_ids == plain.greedy(config, weights, prompt, n)
            continue
        fed = list(prompt)
        near = 0
        for token in result.token_ids:          # as good as the choice from the whole sequence in one step, within rounding
            slot = engine.alloc_slot()
            row = engine.step([StepEntry(slot, fed, [len(fed) - 1])]).float().cpu().numpy()[0]
            engine.free_slot(slot)
            near += int(row[token] >= row.max() - margin * np.abs(row).max())
            fed.append(token)
        # (where a router's two candidates lie closer than bfloat16's rounding, a step of one row and a step of many choose
        # differently, and this model's sublayers outweigh its residual: such a token is counted, not excused.  How far
        # bfloat16 logits lie from the plain ones is the other tests' business: in this model the plain choice is mostly
        # another token within that distance.)
        assert near >= 0.8 * len(result.token_ids), (near, len(result.token_ids))
    sampled = engine.generate(prompts, max_new_tokens=8, temperature=0.9, top_k=20, top_p=0.9, seed=4)
    again = engine.generate(prompts, max_new_tokens=8, temperature=0.9, top_k=20, top_p=0.9, seed=4)
    assert [r.token_ids for r in sampled] == [r.token_ids for r in again]
    engine.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_and_generate_programs(folders, tmp_path, dtype):
    folder, config, weights = folders("edges")
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
    config = dm.drawn_config(100 + seed)
    weights = dm.random_weights(config, seed, gain=0.6)
    folder = dm.write_model(tmp_path / "drawn", config, weights)
    requests = schedules.random_requests(config["vocab"], [1, 19, 70, 150], seed=seed)
    want = [plain.forward(config, weights, r) for r in requests]
    engine = engine_for(folder, dtype, max_tokens=1024)
    tolerances = tolerances_for(folder, dtype, requests, want, least=1e-4 if dtype == "float32" else 3e-2)
    for label, got in (("whole", schedules.whole(engine, requests)), ("tail", schedules.tail_one_by_one(engine, requests, tail=20)),
                       ("batches", schedules.batches(engine, requests, batch_size=4)), ("portions", schedules.portions(engine, requests))):
        check_each(f"{label} {config}", got, want, tolerances, STRAY[dtype])
    engine.cache.check_invariants()
