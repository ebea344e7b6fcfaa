"""Decode and prefill throughput of the Qwen3-8B shape with random bfloat16 weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--context C] [--shape 8b|14b|32b]

A step is one decode step of the batch: every live sequence's next token through the whole
model, logits of each and a greedy choice.  The sequences' caches are filled with random keys
and values to just under the context length, so the timed steps read a full-length cache and
end exactly at the context length.  Prints one JSON line.
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0            # MI355X HBM3E
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

QWEN3_8B = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "num_hidden_layers": 36, "hidden_size": 4096,
    "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 12288,
    "vocab_size": 151936, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "max_position_embeddings": 40960,
    "tie_word_embeddings": False,
}


# The other shapes of the family, for measurements beside the default one (--shape).
QWEN3_14B = dict(QWEN3_8B, num_hidden_layers=40, hidden_size=5120, num_attention_heads=40, intermediate_size=17408)
QWEN3_32B = dict(QWEN3_8B, num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, intermediate_size=25600)
SHAPES = {"8b": ("Qwen3-8B shape", QWEN3_8B), "14b": ("Qwen3-14B shape", QWEN3_14B), "32b": ("Qwen3-32B shape", QWEN3_32B)}


def parse():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=32)
    parser.add_argument("--warmup", type=int, default=4)
    parser.add_argument("--shape", default="8b", choices=sorted(SHAPES), help="layer sizes; the default is the benchmark's")
    parser.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has")
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--context", type=int, default=8192)
    parser.add_argument("--prefill-tokens", type=int, default=2048)
    parser.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    parser.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 decode points")
    parser.add_argument("--workload", action="store_true",
                        help="instead of the step timings, generate through the engine's own loop for the batch the shape's "
                             "benchmark configuration names (8b: 8 prompts of 256 to 1,024 tokens up to the context; 14b: 16 "
                             "prompts of 64 to 4,096 tokens, 256 greedy tokens each; 32b: 32 prompts of 128 to 8,192 tokens, "
                             "128 tokens each at temperature 1) and print its tokens per second")
    parser.add_argument("--hbm-ceiling", action="store_true",
                        help="measure what a plain streaming read and a copy of 8 GB reach on this GPU, print it and exit")
    parser.add_argument("--gokazen", action="store_true",
                        help="the Gokazen design (linear attention with a decay, attention over a cached latent, residual "
                             "streams) at layer sizes of real models beside Qwen3 at equal width and depth: prefill and decode "
                             "tokens per second of both, and every kernel of the new design beside its like with the fraction "
                             "of its roofline; prints one JSON line and exits")
    parser.add_argument("--pudorax", action="store_true",
                        help="the Pudorax design (attention behind short convolutions with a gate, a state-space mixer, routed "
                             "experts, a per-layer token input, a looped stretch) at layer sizes of real models beside Qwen3 at "
                             "equal width and as many layer runs: prefill and decode tokens per second of both, and every kernel "
                             "of the new design beside its like with the fraction of its roofline; prints one JSON line and exits")
    parser.add_argument("--dupidra", action="store_true",
                        help="the Dupidra design (gated attention within chunks, windowed attention over a cached latent, a matrix "
                             "memory with exponential gates, routed experts and dense GELU feed-forwards behind post-norm sums, "
                             "layers that run another layer's tensors) at layer sizes of real models beside Pudorax and Qwen3 at "
                             "equal width and as many layer runs: prefill and decode tokens per second, and every kernel of the "
                             "new design beside its like with the fraction of its roofline; prints one JSON line and exits")
    parser.add_argument("--vepelix", action="store_true",
                        help="the Vepelix design (attention over a cached latent with a query latent, sinks and a gate a head; "
                             "windowed attention beside gated linear attention; experts weighed by sigmoid scores on their inputs; "
                             "a looped stretch entered with the embedding's output) at layer sizes of real models beside Gokazen, "
                             "Dupidra and Qwen3 at equal width and as many layer runs: prefill and decode tokens per second, and "
                             "every kernel of the new design beside its like with the fraction of its roofline; prints one JSON "
                             "line and exits")
    parser.add_argument("--alone", action="store_true",
                        help="with --dupidra or --vepelix: the new design's two models only, without the models beside them and without the "
                             "kernels timed alone (what a profiler should see of it)")
    parser.add_argument("--sampling", action="store_true",
                        help="time the selection kernel on 1, 8 and 64 rows of 151,936 logits (greedy, at a temperature, with "
                             "top-k, with top-p on rows of three spreads, with both), print the microseconds and exit")
    return parser.parse_args()


def fill_cache(engine, slots, length, torch):
    """Give each slot `length` tokens of random keys and values without running the model."""
    requests = [(slot, length) for slot in slots]
    engine.cache.reserve(requests)
    engine.cache.commit(requests)


def randomise_cache(engine, torch):
    generator = torch.Generator(device=engine.device).manual_seed(1)
    for group in engine.cache.groups:
        if group.k is not None:
            for tensor in (group.k, group.v):
                for layer in range(tensor.shape[0]):
                    tensor[layer].normal_(0.0, 1.0, generator=generator)


def decode_run(engine, batch, context, steps, warmup, torch):
    """Time `steps` decode steps of `batch` sequences that end at `context` tokens."""
    from beholdd.engine import StepEntry, decode_ahead
    from beholdd.sampling import SamplingParams

    start = context - steps - warmup - 1
    slots = [engine.alloc_slot() for _ in range(batch)]
    fill_cache(engine, slots, start, torch)
    greedy = [SamplingParams()] * batch
    tokens = [(7 * i + 3) % engine.model.vocab for i in range(batch)]

    # The generation loop's own way of stepping (engine/generation.py: decode_ahead): the next step is started
    # with the tokens still on the device, then the host reads the tokens chosen before it.
    requests = list(range(batch))
    logits = engine.step([StepEntry(slot, [token], [0]) for slot, token in zip(slots, tokens)])
    chosen = engine.select_async(logits, greedy, requests, [0] * batch)

    def one(step):
        nonlocal chosen
        ahead = decode_ahead(engine, slots, chosen, greedy, requests, [step + 1] * batch)
        chosen.result()
        chosen = ahead

    for step in range(warmup):
        one(step)
    chosen.result()
    torch.cuda.synchronize()
    begin = time.perf_counter()
    for step in range(steps):
        one(warmup + step)
    chosen.result()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - begin
    lengths = [engine.cache.length(slot) for slot in slots]
    for slot in slots:
        engine.free_slot(slot)
    mean_length = sum(lengths) / batch - steps / 2.0
    return elapsed / steps, mean_length


def prefill_run(engine, n_tokens, torch, repeats=3, prompts=1, host=False):
    """Seconds of one step that brings `prompts` prompts of `n_tokens` tokens each (the best of `repeats`); with
    `host` also the seconds until the step function returns, the device still busy."""
    from beholdd.engine import StepEntry
    tokens = [(31 * i + 5) % engine.model.vocab for i in range(n_tokens)]
    times, returned = [], []
    for _ in range(repeats + 1):          # the first run warms up and is dropped
        slots = [engine.alloc_slot() for _ in range(prompts)]
        torch.cuda.synchronize()
        begin = time.perf_counter()
        engine.step([StepEntry(slot, tokens, [n_tokens - 1]) for slot in slots])
        returned.append(time.perf_counter() - begin)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - begin)
        for slot in slots:
            engine.free_slot(slot)
    return (min(times[1:]), min(returned[1:])) if host else min(times[1:])


# Batches of the benchmark configurations: (prompts, shortest, longest, new tokens, temperature, context).
WORKLOADS = {"8b": (8, 256, 1024, 256, 0.0, 8192), "14b": (16, 64, 4096, 256, 0.0, 8192),
             "32b": (32, 128, 8192, 128, 1.0, 16384)}


def workload_run(engine, shape, torch):
    """Unequal prompts through `Engine.generate` (prompts in one step, then a token each, sequences that end
    give their slots back): what a user of the library gets, host loop and sampling included."""
    import random
    count, shortest, longest, new_tokens, temperature, _ = WORKLOADS[shape]
    rng = random.Random(0)
    lengths = [rng.randint(shortest, longest) for _ in range(count)]
    prompts = [[rng.randrange(engine.model.vocab) for _ in range(n)] for n in lengths]
    engine.generate(prompts, max_new_tokens=4)          # warms up: the graph of this batch size and page-table width is captured
    torch.cuda.synchronize()
    begin = time.perf_counter()
    results = engine.generate(prompts, max_new_tokens=new_tokens, temperature=temperature, seed=1)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - begin
    generated = sum(len(r.token_ids) for r in results)
    return {"prompts": count, "prompt_tokens": sum(lengths), "generated_tokens": generated,
            "seconds": round(elapsed, 3), "generated_tok_per_s": round(generated / elapsed, 1),
            "all_tok_per_s": round((generated + sum(lengths)) / elapsed, 1), "temperature": temperature}


def hbm_ceiling(torch):
    """What kernels that only stream memory reach here: torch's sum over 8 GB (read) and copy of 8 GB (read +
    write), and the library's own yardstick kernel, which reads 8 GB the way its weight and cache streams do
    (256 and 512 workgroups, with and without the streaming hint).  Not part of the product path; a yardstick
    for the roofline fractions."""
    from beholdd.kernels import HipKernels

    x = torch.empty(2 << 30, dtype=torch.float32, device="cuda:0").normal_()
    y = torch.empty_like(x)
    kernels = HipKernels("cuda:0")
    out = {}
    runs = [("hbm_read_GBs", lambda: x.sum(), x.numel() * 4), ("hbm_copy_GBs", lambda: y.copy_(x), 2 * x.numel() * 4)]
    for workgroups in (256, 512):
        for hint in (True, False):
            name = f"stream_read_{workgroups}wg_{'streaming' if hint else 'plain'}_GBs"
            runs.append((name, lambda w=workgroups, h=hint: kernels.stream_read(x, w, h), x.numel() * 4))
    for name, run, moved in runs:
        run()
        torch.cuda.synchronize()
        begin = time.perf_counter()
        for _ in range(10):
            run()
        torch.cuda.synchronize()
        out[name] = round(moved * 10 / (time.perf_counter() - begin) / 1e9, 1)
    return out


def sampling_times(torch):
    """Microseconds of one selection over rows of the benchmark's vocabulary, each mode replayed ten times from a
    captured graph so that the launches' host cost stays out."""
    from beholdd.kernels import HipKernels

    kernels, vocab, out = HipKernels("cuda:0"), QWEN3_8B["vocab_size"], {}
    for rows in (1, 8, 64):
        logits = torch.randn(rows, vocab, device="cuda:0") * 3
        tokens = torch.empty(rows, dtype=torch.int32, device="cuda:0")
        bad = torch.empty_like(tokens)
        temperature, uniform = torch.full((rows,), 0.8, device="cuda:0"), torch.rand(rows, device="cuda:0")
        top_k = torch.full((rows,), 50, dtype=torch.int32, device="cuda:0")
        top_p = torch.full((rows,), 0.9, device="cuda:0")
        # (top-p's share of these rows is a thousand tokens or so; of the "peaked" rows, three times the spread, under a
        # hundred, as of a trained model's mostly; of the "wide" rows, a sixth of the spread, most of the vocabulary)
        usual, peaked, wide = logits, logits * 3, logits / 6
        modes = {"greedy": {}, "temperature": dict(temperature=temperature, uniform=uniform),
                 "top_k": dict(temperature=temperature, uniform=uniform, top_k=top_k),
                 "top_p": dict(temperature=temperature, uniform=uniform, top_p=top_p),
                 "top_p_peaked": dict(temperature=temperature, uniform=uniform, top_p=top_p),
                 "top_p_wide": dict(temperature=temperature, uniform=uniform, top_p=top_p),
                 "top_k_top_p": dict(temperature=temperature, uniform=uniform, top_k=top_k, top_p=top_p)}
        for name, arguments in modes.items():
            logits = peaked if name.endswith("peaked") else wide if name.endswith("wide") else usual
            kernels.sample(logits, tokens, bad, **arguments)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for _ in range(10):
                    kernels.sample(logits, tokens, bad, **arguments)
            graph.replay()
            torch.cuda.synchronize()
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            begin.record()
            graph.replay()
            end.record()
            torch.cuda.synchronize()
            out[f"rows_{rows}_{name}_us"] = round(begin.elapsed_time(end) * 100, 1)
    return out


# ---- the Gokazen design beside Qwen3 at equal width and depth ---------------------------------------------

def gokazen_config(width, heads, layers, ff, vocab, rank=192, rot=64):
    """`layers` layers, three with linear attention to every one with attention over a cached latent (heads of 128, a
    latent of `rank` and a shared rotated key part of `rot`), two residual streams, a dense feed-forward in every layer."""
    decay = [1.0 - 2.0 ** (-5.0 - 3.0 * h / max(heads - 1, 1)) for h in range(heads)]
    lightning = {"type": "lightning", "mixer": {"heads": heads, "dim": 128, "vdim": 128, "decay": decay},
                 "mlp": {"kind": "dense", "ff": ff}}
    latent = {"type": "latent_attention", "mlp": {"kind": "dense", "ff": ff},
              "mixer": {"heads": heads, "dim": 128, "rot_dim": rot, "vdim": 128, "kv_rank": rank, "scale": (128 + rot) ** -0.5,
                        "rot": {"base": 10000.0, "dims": rot}}}
    return {"architecture": "Gokazen", "vocab": vocab, "width": width, "streams": 2, "logit_scale": 1.0, "norm": {"eps": 1e-6},
            "layers": [latent if i % 4 == 3 else lightning for i in range(layers)]}


def timed(call, torch, repeats=20):
    """Median microseconds of `call()` on the device (two calls first, untimed)."""
    call(), call()
    torch.cuda.synchronize()
    times = []
    for _ in range(repeats):
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record()
        call()
        end.record()
        end.synchronize()
        times.append(begin.elapsed_time(end) * 1e3)
    return sorted(times)[len(times) // 2]


def gokazen_kernels(K, torch, width, heads, rank, rot, context, streams=2):
    """Every kernel of the new design and its like among Qwen3's, alone, at a prompt of 2,048 rows and at a decode step of 8
    rows over `context` cached tokens: microseconds and the fraction of the roofline (the slower of its bytes at the HBM
    peak and its operations at the peak of the units it runs on: FMA for the recurrence, matrix cores for what is a
    matrix product)."""
    from types import SimpleNamespace
    bf16, f32, dev = torch.bfloat16, torch.float32, "cuda:0"
    dim = vdim = 128
    page = K.page_size
    out = {}

    def note(name, us, n_bytes, flops=0.0, peak=PEAK_FLOPS["fp32"]):
        floor = max(n_bytes / (PEAK_HBM_GBS * 1e9), flops / peak) * 1e6
        out[name] = {"us": round(us, 1), "roofline_us": round(floor, 2), "fraction": round(floor / us, 3)}

    def pages_for(n_seqs, length, kv_heads, head):
        per = -(-length // page)
        k_pages = torch.randn(n_seqs * per, kv_heads, page, head, device=dev).to(bf16)
        v_pages = torch.randn(n_seqs * per, kv_heads, head, page, device=dev).to(bf16)
        table = torch.arange(n_seqs * per, dtype=torch.int32, device=dev).view(n_seqs, per).contiguous()
        return k_pages, v_pages, table

    for rows, seqs, past, tag in ((2048, 1, 0, "prompt of 2,048"), (8, 8, context - 1, f"decode of 8 at {context}")):
        each = rows // seqs
        starts = torch.arange(0, rows + 1, each, dtype=torch.int32, device=dev)
        slots = torch.arange(seqs, dtype=torch.int32, device=dev)
        positions = (torch.arange(rows, dtype=torch.int32, device=dev) % each + past).contiguous()
        row_seq = (torch.arange(rows, dtype=torch.int32, device=dev) // each).contiguous()
        layout = SimpleNamespace(seq_start=starts, n_seqs=seqs, max_rows_per_seq=each, max_position=past + each - 1)
        # -- the new design
        proj = torch.randn(rows, 4 * heads * dim, device=dev).to(bf16)
        state = torch.zeros(seqs, heads, dim, vdim, device=dev)
        decay = torch.full((heads,), 0.99, device=dev)
        mixed = torch.empty(rows, heads * vdim, device=dev)
        us = timed(lambda: K.lightning_scan(proj, 0, heads * dim, 2 * heads * dim, state, decay, starts, slots, mixed, heads, dim, vdim), torch)
        note(f"lightning_scan, {tag}", us, 2 * state.numel() * 4 + rows * 3 * heads * dim * 2 + mixed.numel() * 4, 4.0 * rows * heads * dim * vdim)
        gated = torch.empty(rows, heads * vdim, device=dev, dtype=bf16)
        weight = torch.ones(heads * vdim, device=dev)
        us = timed(lambda: K.gated_rmsnorm(mixed, proj, 3 * heads * dim, weight, 1e-6, gated), torch)
        note(f"gated_rmsnorm, {tag}", us, mixed.numel() * 4 + 2 * gated.numel() * 2)
        x = torch.randn(rows, streams, width, device=dev)
        normed = torch.empty(rows, width, device=dev, dtype=bf16)
        take, ones = torch.ones(streams, device=dev), torch.ones(width, device=dev)
        us = timed(lambda: K.streams_rmsnorm(x, take, ones, 1e-6, normed), torch)
        note(f"streams_rmsnorm, {tag}", us, x.numel() * 4 + normed.numel() * 2)
        y, mix = torch.randn(rows, width, device=dev), torch.eye(streams, device=dev)
        us = timed(lambda: K.streams_update(x, y, mix, take, ones), torch)
        note(f"streams_update, {tag}", us, 2 * x.numel() * 4 + y.numel() * 4)
        q_head, kv_head = dim + rot, rank + rot
        qd = torch.randn(rows, heads * q_head + kv_head, device=dev).to(bf16)
        k_pages, v_pages, table = pages_for(seqs, past + each, 1, kv_head)
        freq, latent_weight = torch.ones(rot // 2, device=dev), torch.ones(rank, device=dev)
        query = torch.empty(rows, heads * kv_head, device=dev, dtype=bf16)
        us = timed(lambda: K.latent_write(qd, heads * q_head, latent_weight, 1e-6, freq, rot, positions, row_seq, k_pages, v_pages,
                                          table, rank, rot, query=query, query_head=kv_head, query_first=rank, source_head=q_head,
                                          source_first=dim, n_heads=heads), torch)
        note(f"latent_write with the queries' rotation, {tag}", us, rows * kv_head * 2 * 3 + 2 * rows * heads * rot * 2)
        key_up = torch.randn(heads, dim, rank, device=dev).to(bf16)
        us = timed(lambda: K.heads_linear(qd, q_head, 0, key_up, query, kv_head, 0, heads), torch)
        note(f"heads_linear (queries into the latent), {tag}", us, key_up.numel() * 2 + rows * heads * (dim + rank) * 2,
             2.0 * rows * heads * dim * rank, PEAK_FLOPS["bf16"])
        attended = torch.empty_like(query)
        scale = (dim + rot) ** -0.5
        us = timed(lambda: K.attention(query, attended, k_pages, v_pages, table, row_seq, positions, heads, 1, kv_head, scale, 0, layout=layout), torch)
        keys_seen = seqs * (past + each) if each == 1 else each * (each + 1) // 2
        note(f"attention over the latent ({heads} heads on one of {kv_head}), {tag}", us,
             2 * seqs * (past + each) * kv_head * 2 + 2 * query.numel() * 2, 4.0 * keys_seen * heads * kv_head, PEAK_FLOPS["bf16"])
        value_up = torch.randn(heads, rank, vdim, device=dev).to(bf16)
        values = torch.empty(rows, heads * vdim, device=dev, dtype=bf16)
        us = timed(lambda: K.heads_linear(attended, kv_head, 0, value_up, values, vdim, 0, heads), torch)
        note(f"heads_linear (latents into values), {tag}", us, value_up.numel() * 2 + rows * heads * (rank + vdim) * 2,
             2.0 * rows * heads * rank * vdim, PEAK_FLOPS["bf16"])
        inner = torch.randn(rows, 3 * width, device=dev).to(bf16)
        activated_sq = torch.empty_like(inner)
        us = timed(lambda: K.relu_squared(inner, activated_sq), torch)
        note(f"relu_squared, {tag}", us, 2 * inner.numel() * 2)
        # -- their like in Qwen3 at the same width: 4 query heads of 128 to a kv head
        kv_heads = max(heads // 4, 1)
        hidden = torch.randn(rows, width, device=dev)
        us = timed(lambda: K.rmsnorm(hidden, ones, 1e-6, normed), torch)
        note(f"qwen3 rmsnorm, {tag}", us, hidden.numel() * 4 + normed.numel() * 2)
        qkv = torch.randn(rows, (heads + 2 * kv_heads) * dim, device=dev).to(bf16)
        gk, gv, gtable = pages_for(seqs, past + each, kv_heads, dim)
        q_out = torch.empty(rows, heads * dim, device=dev, dtype=bf16)
        head_weight = torch.ones(dim, device=dev)
        cos = torch.ones(past + each, dim // 2, device=dev)
        us = timed(lambda: K.qk_norm_rope_cache(qkv, q_out, head_weight, head_weight, 1e-6, cos, cos, positions, row_seq, gk, gv,
                                                gtable, heads, kv_heads, dim, True, past + each - 1), torch)
        note(f"qwen3 qk_norm_rope_cache, {tag}", us, 2 * qkv.numel() * 2)
        g_out = torch.empty_like(q_out)
        us = timed(lambda: K.attention(q_out, g_out, gk, gv, gtable, row_seq, positions, heads, kv_heads, dim, dim ** -0.5, 0, layout=layout), torch)
        note(f"qwen3 attention ({heads} heads on {kv_heads} of {dim}), {tag}", us,
             2 * seqs * (past + each) * kv_heads * dim * 2 + 2 * q_out.numel() * 2, 4.0 * keys_seen * heads * dim, PEAK_FLOPS["bf16"])
        gate_up = torch.randn(rows, 6 * width, device=dev).to(bf16)
        activated = torch.empty(rows, 3 * width, device=dev, dtype=bf16)
        us = timed(lambda: K.swiglu(gate_up, activated), torch)
        note(f"qwen3 swiglu, {tag}", us, 3 * activated.numel() * 2)
    return out


def gokazen_bench(args, torch):
    from beholdd.engine import Engine, random_model_on_device

    device, points = "cuda:0", []
    t = min(args.prefill_tokens, args.context)
    layers = args.layers or 8
    for width, heads in ((2048, 16), (4096, 32)):
        pair = {"gokazen": gokazen_config(width, heads, layers, 3 * width, 32768),
                "qwen3": dict(QWEN3_8B, num_hidden_layers=layers, hidden_size=width, num_attention_heads=heads,
                              num_key_value_heads=heads // 4, intermediate_size=3 * width, vocab_size=32768)}
        point = {"width": width, "heads": heads, "layers": layers}
        for name, config in pair.items():
            model = random_model_on_device(config, seed=0, dtype="bfloat16", device=device)
            engine = Engine(model=model, dtype="bfloat16", max_tokens=args.batch * (-(-args.context // 64) * 64),
                            max_slots=args.batch, device=device)
            parameters = sum(int(np_prod(spec.shape)) for spec in model.tensor_specs())
            seconds, _ = decode_run(engine, args.batch, args.context, args.steps, args.warmup, torch)
            prefill = prefill_run(engine, t, torch)
            point[name] = {"parameters": parameters, "decode_ms_per_step": round(seconds * 1e3, 4),
                           "decode_tok_per_s": round(args.batch / seconds, 1), "prefill_ms": round(prefill * 1e3, 3),
                           "prefill_tok_per_s": round(t / prefill, 1)}
            kernels = engine.kernels
            del engine, model
            torch.cuda.empty_cache()
        points.append(point)
    line = {"metric": f"Gokazen beside Qwen3 at equal width and depth: decode tok/s @ batch {args.batch}, context {args.context}; prefill of {t} tokens",
            "unit": "tok/s", "value": points[-1]["gokazen"]["decode_tok_per_s"], "dtype": "bf16", "data": "synthetic", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "points": points,
            "kernels": gokazen_kernels(kernels, torch, 4096, 32, 192, 64, args.context)}
    print(json.dumps(line))
    return 0


def pudorax_config(width, heads, vocab, experts=32, top=4, expert_ff=None, shared_ff=None, side=256):
    """Six layers of which two run twice (eight layer runs): attention with heads of 128, four query heads to a key/value
    head, convolutions of four taps and a rotation over half a head; state-space layers of twice the width in heads of 64
    with a state of 128 rows; `experts` experts of which `top` are used, and a shared one; a token side input of `side`."""
    expert_ff, shared_ff = expert_ff or 3 * width // 8, shared_ff or 3 * width // 2
    mlp = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": expert_ff, "limit": 7.0},
           "shared": {"ff": shared_ff, "limit": 7.0}}
    attention = {"type": "attention", "mlp": mlp,
                 "mixer": {"heads": heads, "kv_heads": max(heads // 4, 1), "dim": 128, "vdim": 128, "conv": 4, "scale": 128 ** -0.5,
                           "rot": {"base": 1000000.0, "dims": 64}}}
    mamba = {"type": "mamba2", "mlp": mlp,
             "mixer": {"heads": 2 * width // 64, "vdim": 64, "state": 128, "groups": 8, "norm_groups": 8, "conv": 4}}
    return {"architecture": "Pudorax", "vocab": vocab, "width": width, "embedding": {"scale": 1.0}, "logit_softcap": 30.0,
            "norm": {"eps": 1e-6}, "token_side": {"dim": side}, "loop": {"start": 1, "stop": 3, "times": 2},
            "layers": [attention, mamba, attention, attention, mamba, attention]}


def pudorax_kernels(K, torch, width, heads, context, experts=32, top=4):
    """Every kernel of the design and its like among the other models', alone, at a prompt of 2,048 rows and at a decode step
    of 8 rows over `context` cached tokens: microseconds and the fraction of the roofline (the slower of its bytes at the HBM
    peak and its operations at the peak of the units it runs on)."""
    from types import SimpleNamespace
    bf16, f32, dev = torch.bfloat16, torch.float32, "cuda:0"
    dim = vdim = 128
    page = K.page_size
    out = {}

    def note(name, us, n_bytes, flops=0.0, peak=PEAK_FLOPS["fp32"]):
        floor = max(n_bytes / (PEAK_HBM_GBS * 1e9), flops / peak) * 1e6
        out[name] = {"us": round(us, 1), "roofline_us": round(floor, 2), "fraction": round(floor / us, 3)}

    def pages_for(n_seqs, length, kv_heads, head):
        per = -(-length // page)
        k_pages = torch.randn(n_seqs * per, kv_heads, page, head, device=dev).to(bf16)
        v_pages = torch.randn(n_seqs * per, kv_heads, head, page, device=dev).to(bf16)
        table = torch.arange(n_seqs * per, dtype=torch.int32, device=dev).view(n_seqs, per).contiguous()
        return k_pages, v_pages, table

    kv_heads = max(heads // 4, 1)
    ones = torch.ones(width, device=dev)
    for rows, seqs, past, tag in ((2048, 1, 0, "prompt of 2,048"), (8, 8, context - 1, f"decode of 8 at {context}")):
        each = rows // seqs
        starts = torch.arange(0, rows + 1, each, dtype=torch.int32, device=dev)
        slots = torch.arange(seqs, dtype=torch.int32, device=dev)
        positions = (torch.arange(rows, dtype=torch.int32, device=dev) % each + past).contiguous()
        row_seq = (torch.arange(rows, dtype=torch.int32, device=dev) // each).contiguous()
        layout = SimpleNamespace(seq_start=starts, n_seqs=seqs, max_rows_per_seq=each, max_position=past + each - 1)
        hidden = torch.randn(rows, width, device=dev)
        normed = torch.empty(rows, width, device=dev, dtype=bf16)
        # -- norms
        us = timed(lambda: K.layernorm(hidden, ones, ones, 1e-6, normed), torch)
        note(f"layernorm, {tag}", us, hidden.numel() * 4 + normed.numel() * 2)
        us = timed(lambda: K.rmsnorm(hidden, ones, 1e-6, normed), torch)
        note(f"qwen3 rmsnorm, {tag}", us, hidden.numel() * 4 + normed.numel() * 2)
        # -- attention: convolution, norm over the projection, rotation and cache write; the gate
        q_w, k_w = heads * dim, kv_heads * dim
        conv_w = q_w + 2 * k_w
        proj = torch.randn(rows, conv_w + q_w, device=dev).to(bf16)
        taps = 4
        conv_weight = torch.randn(conv_w, taps, device=dev)
        conv_state = torch.zeros(seqs, (taps - 1) * conv_w, device=dev)
        conv = torch.empty(rows, conv_w, device=dev)
        k_pages, v_pages, table = pages_for(seqs, past + each, kv_heads, dim)
        q_out = torch.empty(rows, heads * dim, device=dev, dtype=bf16)
        freq = torch.ones(32, device=dev)
        wq, wk = torch.ones(q_w, device=dev), torch.ones(k_w, device=dev)

        def convolved_write():
            K.conv_norm_rope_write(proj, 0, conv_weight, conv_state, 0, starts, slots, wq, wk, 1e-6, freq, 64, positions, row_seq, q_out,
                                   k_pages, v_pages, table, heads, kv_heads, dim, vdim, dim, True)
            K.short_conv_state(proj, 0, conv_w, taps, conv_state, 0, starts, slots)
        us = timed(convolved_write, torch)
        note(f"conv_norm_rope_write + short_conv_state, {tag}", us, 2 * rows * conv_w * 2)
        head_weight = torch.ones(dim, device=dev)
        cos = torch.ones(past + each, dim // 2, device=dev)
        qkv = torch.randn(rows, conv_w, device=dev).to(bf16)
        us = timed(lambda: K.qk_norm_rope_cache(qkv, q_out, head_weight, head_weight, 1e-6, cos, cos, positions, row_seq, k_pages, v_pages,
                                                table, heads, kv_heads, dim, True, past + each - 1), torch)
        note(f"qwen3 qk_norm_rope_cache, {tag}", us, 2 * qkv.numel() * 2)
        attended = torch.empty_like(q_out)
        us = timed(lambda: K.attention(q_out, attended, k_pages, v_pages, table, row_seq, positions, heads, kv_heads, dim, dim ** -0.5, 0, layout=layout), torch)
        keys_seen = seqs * (past + each) if each == 1 else each * (each + 1) // 2
        note(f"attention ({heads} heads on {kv_heads} of {dim}; the framework's own), {tag}", us,
             2 * seqs * (past + each) * kv_heads * dim * 2 + 2 * q_out.numel() * 2, 4.0 * keys_seen * heads * dim, PEAK_FLOPS["bf16"])
        gated = torch.empty(rows, q_w, device=dev, dtype=bf16)
        us = timed(lambda: K.gate_heads(attended, dim, proj, conv_w, gated, heads, vdim), torch)
        note(f"gate_heads, {tag}", us, 3 * gated.numel() * 2)
        # -- the state-space mixer
        s_heads, s_vdim, n_state, groups = 2 * width // 64, 64, 128, 8
        inner, bc = s_heads * s_vdim, 2 * groups * n_state
        s_proj = torch.randn(rows, 2 * inner + bc + s_heads, device=dev).to(bf16)
        s_state = torch.zeros(seqs, s_heads * n_state * s_vdim + (taps - 1) * (inner + bc), device=dev)
        xbc = torch.empty(rows, inner + bc, device=dev)
        s_conv_w, s_conv_b = torch.randn(inner + bc, taps, device=dev), torch.zeros(inner + bc, device=dev)

        def s_convolved():
            K.short_conv(s_proj, inner, s_conv_w, s_conv_b, s_state, s_heads * n_state * s_vdim, row_seq, starts, slots, xbc, silu=True)
            K.short_conv_state(s_proj, inner, inner + bc, taps, s_state, s_heads * n_state * s_vdim, starts, slots)
        us = timed(s_convolved, torch)
        note(f"short_conv with silu + state, {tag}", us, rows * (inner + bc) * (2 + 4))
        per_head = torch.zeros(s_heads, device=dev)
        y = torch.empty(rows, inner, device=dev)
        us = timed(lambda: K.ssm_scan(xbc, s_proj, 2 * inner + bc, per_head, per_head, per_head, s_state, 0, starts, slots, y, s_heads,
                                      s_vdim, n_state, groups), torch)
        note(f"ssm_scan, {tag}", us, 2 * seqs * s_heads * n_state * s_vdim * 4 + xbc.numel() * 4 + y.numel() * 4, 6.0 * rows * s_heads * n_state * s_vdim)
        l_heads = width // 128
        l_proj = torch.randn(rows, 4 * l_heads * 128, device=dev).to(bf16)
        l_state = torch.zeros(seqs, l_heads, 128, 128, device=dev)
        decay = torch.full((l_heads,), 0.99, device=dev)
        mixed = torch.empty(rows, l_heads * 128, device=dev)
        us = timed(lambda: K.lightning_scan(l_proj, 0, l_heads * 128, 2 * l_heads * 128, l_state, decay, starts, slots, mixed, l_heads, 128, 128), torch)
        note(f"gokazen lightning_scan, {tag}", us, 2 * l_state.numel() * 4 + rows * 3 * l_heads * 128 * 2 + mixed.numel() * 4, 4.0 * rows * l_heads * 128 * 128)
        s_normed = torch.empty(rows, inner, device=dev, dtype=bf16)
        s_weight = torch.ones(inner, device=dev)
        us = timed(lambda: K.gated_group_rmsnorm(y, s_proj, 0, s_weight, 1e-6, s_normed, groups), torch)
        note(f"gated_group_rmsnorm, {tag}", us, y.numel() * 4 + 2 * s_normed.numel() * 2)
        l_gated = torch.empty(rows, l_heads * 128, device=dev, dtype=bf16)
        l_weight = torch.ones(l_heads * 128, device=dev)
        us = timed(lambda: K.gated_rmsnorm(mixed, l_proj, 3 * l_heads * 128, l_weight, 1e-6, l_gated), torch)
        note(f"gokazen gated_rmsnorm, {tag}", us, mixed.numel() * 4 + 2 * l_gated.numel() * 2)
        # -- routed experts
        ff = 3 * width // 8
        logits = torch.randn(rows, experts, device=dev)
        chosen = torch.empty(rows, top, dtype=torch.int32, device=dev)
        shares = torch.empty(rows, top, device=dev)
        bias = torch.zeros(experts, device=dev)
        us = timed(lambda: K.route_top_k(logits, bias, chosen, shares), torch)
        note(f"route_top_k, {tag}", us, logits.numel() * 4 + 2 * chosen.numel() * 4)
        x = torch.randn(rows, width, device=dev).to(bf16)
        w_gu = (torch.randn(experts, 2 * ff, width, device=dev) * 0.02).to(bf16)
        w_d = (torch.randn(experts, width, ff, device=dev) * 0.02).to(bf16)
        active = int(torch.unique(chosen).numel())
        for name, call, n_bytes, flops in pudorax_expert_calls(K, torch, x, chosen, shares, w_gu, w_d, hidden, active, top, ff, width):
            us = timed(call, torch, repeats=5 if rows > 64 else 20)
            note(f"{name}, {tag}", us, n_bytes, flops, PEAK_FLOPS["bf16"])
        both = torch.randn(rows, 2 * ff * 4, device=dev).to(bf16)
        activated = torch.empty(rows, ff * 4, device=dev, dtype=bf16)
        us = timed(lambda: K.clamped_glu(both, activated, 7.0, 1.702), torch)
        note(f"clamped_glu, {tag}", us, 3 * activated.numel() * 2)
        us = timed(lambda: K.swiglu(both, activated), torch)
        note(f"qwen3 swiglu, {tag}", us, 3 * activated.numel() * 2)
        # -- the token's side input and the loop's entry
        side = 256
        table_w = torch.randn(4096, 6 * side, device=dev).to(bf16)
        gate = torch.randn(rows, side, device=dev).to(bf16)
        g_out = torch.empty_like(gate)
        tokens = torch.randint(0, 4096, (rows,), dtype=torch.int32, device=dev)
        us = timed(lambda: K.gelu_gate_table(gate, tokens, table_w, 2 * side, g_out), torch)
        note(f"gelu_gate_table, {tag}", us, 3 * gate.numel() * 2)
        yy = torch.randn(rows, width, device=dev)
        us = timed(lambda: K.rms_scale_add(hidden, yy, ones, 1e-6), torch)
        note(f"rms_scale_add, {tag}", us, 3 * hidden.numel() * 4)
        wide = torch.empty(rows, 2 * width, device=dev, dtype=bf16)
        us = timed(lambda: K.cast_concat(hidden, yy, wide), torch)
        note(f"cast_concat, {tag}", us, 2 * hidden.numel() * 4 + wide.numel() * 2)
    return out


def pudorax_expert_calls(K, torch, x, chosen, shares, w_gu, w_d, hidden, active, top, ff, width):
    """(name, call, bytes, operations) of the routed experts' work as a step of these rows runs it: grouped by expert, then for
    few rows a workgroup per expert and block of outputs, for many rows the framework's products on every expert's stretch."""
    from types import SimpleNamespace
    from beholdd.parts.experts import RoutedExperts
    rows, experts = x.shape[0], w_gu.shape[0]
    pairs = rows * top
    lists = torch.empty(experts, rows, dtype=torch.int32, device=x.device)
    counts = torch.empty(experts, dtype=torch.int32, device=x.device)
    K.experts_group(chosen, lists, counts)
    weights_read = active * 3 * ff * width * 2
    yield ("experts_group", lambda: K.experts_group(chosen, lists, counts), pairs * 4 * 2, 0.0)
    if pairs < RoutedExperts.PRODUCT_PAIRS * experts:
        inner = torch.empty(pairs, ff, device=x.device, dtype=x.dtype)
        y = torch.empty(pairs, width, device=x.device)
        yield ("experts_rows (gate and up)", lambda: K.experts_rows(x, top, lists, counts, w_gu, inner, gated=True, limit=7.0, alpha=1.702),
               weights_read * 2 // 3 + x.numel() * 2 + inner.numel() * 2, 4.0 * pairs * ff * width)
        yield ("experts_rows (down)", lambda: K.experts_rows(inner, 1, lists, counts, w_d, y), weights_read // 3 + inner.numel() * 2 + y.numel() * 4,
               2.0 * pairs * ff * width)
        yield ("experts_combine", lambda: K.experts_combine(y, None, shares, hidden), y.numel() * 4 + 2 * hidden.numel() * 4, 0.0)
        return
    part = RoutedExperts(width, experts, top, ff, 7.0, "m.")
    part.w_gate_up, part.w_down = w_gu, w_d
    part.prepare(K)
    ctx = SimpleNamespace(kernels=K, device=x.device, new_f32=lambda *shape: torch.empty(shape, device=x.device),
                          new_activations=lambda *shape, reader=None: torch.empty(shape, device=x.device, dtype=x.dtype))
    one = part.in_one_launch and 6.0 * pairs * ff * width <= part.ONE_LAUNCH_WORK
    form = "two launches over all experts" if one else f"{2 * experts} products, clamped_glu"
    yield (f"experts of a prompt (gather, {form}, combine)", lambda: part._as_products(ctx, x, lists, counts, shares, hidden),
           weights_read + pairs * (2 * width + 3 * ff) * 2 + pairs * width * 8, 6.0 * pairs * ff * width)


def pudorax_bench(args, torch):
    from beholdd.engine import Engine, random_model_on_device

    device, points = "cuda:0", []
    t = min(args.prefill_tokens, args.context)
    for width, heads in ((2048, 16), (4096, 32)):
        pair = {"pudorax": pudorax_config(width, heads, 32768),
                "qwen3": dict(QWEN3_8B, num_hidden_layers=8, hidden_size=width, num_attention_heads=heads,
                              num_key_value_heads=heads // 4, intermediate_size=3 * width, vocab_size=32768)}
        point = {"width": width, "heads": heads, "layer_runs": 8}
        for name, config in pair.items():
            model = random_model_on_device(config, seed=0, dtype="bfloat16", device=device)
            engine = Engine(model=model, dtype="bfloat16", max_tokens=args.batch * (-(-args.context // 64) * 64),
                            max_slots=args.batch, device=device)
            parameters = sum(int(np_prod(spec.shape)) for spec in model.tensor_specs())
            seconds, _ = decode_run(engine, args.batch, args.context, args.steps, args.warmup, torch)
            prefill = prefill_run(engine, t, torch)
            point[name] = {"parameters": parameters, "decode_ms_per_step": round(seconds * 1e3, 4),
                           "decode_tok_per_s": round(args.batch / seconds, 1), "prefill_ms": round(prefill * 1e3, 3),
                           "prefill_tok_per_s": round(t / prefill, 1)}
            kernels = engine.kernels
            del engine, model
            torch.cuda.empty_cache()
        points.append(point)
    line = {"metric": f"Pudorax beside Qwen3 at equal width and as many layer runs: decode tok/s @ batch {args.batch}, context {args.context}; prefill of {t} tokens",
            "unit": "tok/s", "value": points[-1]["pudorax"]["decode_tok_per_s"], "dtype": "bf16", "data": "synthetic", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "points": points,
            "kernels": pudorax_kernels(kernels, torch, 4096, 32, args.context)}
    print(json.dumps(line))
    return 0


# ---- the Dupidra design beside Pudorax and Qwen3 at equal width and as many layer runs ---------------------------

def dupidra_config(width, heads, vocab, experts=32, top=4, chunk=8192, window=4096, rank=256):
    """Eight layer runs of which two run an earlier layer's tensors: attention with heads of 128, four query heads to a
    key/value head, a rotation over half a head and chunks of `chunk` positions; attention over a latent of `rank` within a
    window; matrix memories with keys of 64 and values of 128 a head; `experts` experts of 3/8 of the width of which `top`
    are used in all layers but one, whose feed-forward is dense and three times the width."""
    mlp = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": 3 * width // 8, "limit": 7.0}}
    attention = {"type": "attention", "mlp": mlp,
                 "mixer": {"heads": heads, "kv_heads": max(heads // 4, 1), "dim": 128, "vdim": 128, "scale": 128 ** -0.5,
                           "mask": {"size": chunk}, "rot": {"base": 1000000.0, "dims": 64}}}
    latent = {"type": "latent_attention", "mlp": mlp,
              "mixer": {"heads": heads, "dim": 128, "vdim": 128, "kv_rank": rank, "scale": 128 ** -0.5, "mask": {"size": window}}}
    memory = {"type": "mlstm", "mlp": mlp, "mixer": {"heads": heads, "dim": 64, "vdim": 128, "gate_cap": 15.0}}
    first_memory = dict(memory, mlp={"kind": "dense", "ff": 3 * width})
    return {"architecture": "Dupidra", "vocab": vocab, "width": width, "postln_alpha": 2.0, "norm": {"eps": 1e-6},
            "layers": [attention, first_memory, latent, dict(attention, weights_of=0), memory, latent, dict(memory, weights_of=4),
                       attention]}


def dupidra_kernels(K, torch, width, heads, context, rank=256):
    """Every kernel that the design brought and its like among the other models', alone, at a prompt of 2,048 rows and at a
    decode step of 8 rows over `context` cached tokens: microseconds and the fraction of the roofline (the slower of its bytes
    at the HBM peak and its operations at the peak of the units it runs on)."""
    from types import SimpleNamespace
    bf16, dev = torch.bfloat16, "cuda:0"
    dim = vdim = 128
    page = K.page_size
    out = {}

    def note(name, us, n_bytes, flops=0.0, peak=PEAK_FLOPS["fp32"]):
        floor = max(n_bytes / (PEAK_HBM_GBS * 1e9), flops / peak) * 1e6
        out[name] = {"us": round(us, 1), "roofline_us": round(floor, 2), "fraction": round(floor / us, 3)}

    def pages_for(n_seqs, length, kv_heads, head):
        per = -(-length // page)
        k_pages = torch.randn(n_seqs * per, kv_heads, page, head, device=dev).to(bf16)
        v_pages = torch.randn(n_seqs * per, kv_heads, head, page, device=dev).to(bf16)
        table = torch.arange(n_seqs * per, dtype=torch.int32, device=dev).view(n_seqs, per).contiguous()
        return k_pages, v_pages, table

    kv_heads = max(heads // 4, 1)
    ones = torch.ones(width, device=dev)
    for rows, seqs, past, tag in ((2048, 1, 0, "prompt of 2,048"), (8, 8, context - 1, f"decode of 8 at {context}")):
        each = rows // seqs
        starts = torch.arange(0, rows + 1, each, dtype=torch.int32, device=dev)
        slots = torch.arange(seqs, dtype=torch.int32, device=dev)
        positions = (torch.arange(rows, dtype=torch.int32, device=dev) % each + past).contiguous()
        row_seq = (torch.arange(rows, dtype=torch.int32, device=dev) // each).contiguous()
        layout = SimpleNamespace(seq_start=starts, n_seqs=seqs, max_rows_per_seq=each, max_position=past + each - 1)
        keys_seen = seqs * (past + each) if each == 1 else each * (each + 1) // 2
        # -- the norm behind the sum, beside the norms that stand ahead
        hidden, result = torch.randn(rows, width, device=dev), torch.randn(rows, width, device=dev)
        normed = torch.empty(rows, width, device=dev, dtype=bf16)
        us = timed(lambda: K.sum_layernorm(hidden, result, 2.0, ones, ones, 1e-6, normed), torch)
        note(f"sum_layernorm, {tag}", us, 3 * hidden.numel() * 4 + normed.numel() * 2)
        us = timed(lambda: K.layernorm(hidden, ones, ones, 1e-6, normed), torch)
        note(f"pudorax layernorm, {tag}", us, hidden.numel() * 4 + normed.numel() * 2)
        us = timed(lambda: K.rmsnorm(hidden, ones, 1e-6, normed), torch)
        note(f"qwen3 rmsnorm, {tag}", us, hidden.numel() * 4 + normed.numel() * 2)
        # -- attention: biases, head norms, rotation and cache write; the attention within chunks; the gate
        q_w, k_w = heads * dim, kv_heads * dim
        proj = torch.randn(rows, 2 * q_w + 2 * k_w, device=dev).to(bf16)
        bias = torch.randn(q_w + 2 * k_w, device=dev)
        head_weight, freq = torch.ones(dim, device=dev), torch.ones(32, device=dev)
        k_pages, v_pages, table = pages_for(seqs, past + each, kv_heads, dim)
        q_out = torch.empty(rows, heads * dim, device=dev, dtype=bf16)
        us = timed(lambda: K.head_norm_rope_write(proj, 0, bias, head_weight, head_weight, 1e-6, freq, 64, positions, row_seq, q_out, k_pages,
                                                  v_pages, table, heads, kv_heads, dim, vdim, dim, True), torch)
        note(f"head_norm_rope_write, {tag}", us, 2 * rows * (q_w + 2 * k_w) * 2)
        qkv = torch.randn(rows, q_w + 2 * k_w, device=dev).to(bf16)
        cos = torch.ones(past + each, dim // 2, device=dev)
        us = timed(lambda: K.qk_norm_rope_cache(qkv, q_out, head_weight, head_weight, 1e-6, cos, cos, positions, row_seq, k_pages, v_pages,
                                                table, heads, kv_heads, dim, True, past + each - 1), torch)
        note(f"qwen3 qk_norm_rope_cache, {tag}", us, 2 * qkv.numel() * 2)
        attended = torch.empty_like(q_out)
        chunk = -(-(past + each) // page) * page      # the whole context is one chunk: as many keys as Qwen3's attention reads
        us = timed(lambda: K.attention(q_out, attended, k_pages, v_pages, table, row_seq, positions, heads, kv_heads, dim, dim ** -0.5, 0,
                                       layout=layout, chunk=chunk), torch)
        attention_bytes = 2 * seqs * (past + each) * kv_heads * dim * 2 + 2 * q_out.numel() * 2
        note(f"attention within a chunk ({heads} heads on {kv_heads} of {dim}), {tag}", us, attention_bytes, 4.0 * keys_seen * heads * dim,
             PEAK_FLOPS["bf16"])
        us = timed(lambda: K.attention(q_out, attended, k_pages, v_pages, table, row_seq, positions, heads, kv_heads, dim, dim ** -0.5, 0,
                                       layout=layout), torch)
        note(f"qwen3 attention ({heads} heads on {kv_heads} of {dim}), {tag}", us, attention_bytes, 4.0 * keys_seen * heads * dim,
             PEAK_FLOPS["bf16"])
        gated = torch.empty(rows, heads * vdim, device=dev, dtype=bf16)
        us = timed(lambda: K.gate_heads(attended, dim, proj, q_w + 2 * k_w, gated, heads, vdim), torch)
        note(f"gate_heads, {tag}", us, 3 * gated.numel() * 2)
        # -- attention over the latent, without a rotated part, within a window
        qd = torch.randn(rows, heads * dim + rank + heads * vdim, device=dev).to(bf16)
        lk, lv, ltable = pages_for(seqs, past + each, 1, rank)
        latent_weight = torch.ones(rank, device=dev)
        us = timed(lambda: K.latent_write(qd, heads * dim, latent_weight, 1e-6, None, 0, positions, row_seq, lk, lv, ltable, rank, 0), torch)
        note(f"latent_write without a rotated part, {tag}", us, rows * rank * 2 * 3)
        key_up = torch.randn(heads, dim, rank, device=dev).to(bf16)
        query = torch.empty(rows, heads * rank, device=dev, dtype=bf16)
        us = timed(lambda: K.heads_linear(qd, dim, 0, key_up, query, rank, 0, heads), torch)
        note(f"heads_linear (queries into the latent), {tag}", us, key_up.numel() * 2 + rows * heads * (dim + rank) * 2,
             2.0 * rows * heads * dim * rank, PEAK_FLOPS["bf16"])
        seen_window = min(4096, past + each)
        lat_out = torch.empty_like(query)
        us = timed(lambda: K.attention(query, lat_out, lk, lv, ltable, row_seq, positions, heads, 1, rank, dim ** -0.5, 4096, layout=layout), torch)
        note(f"attention over the latent within a window of 4,096 ({heads} heads on one of {rank}), {tag}", us,
             2 * seqs * seen_window * rank * 2 + 2 * query.numel() * 2, 4.0 * (seqs * seen_window if each == 1 else keys_seen) * heads * rank,
             PEAK_FLOPS["bf16"])
        value_up = torch.randn(heads, rank, vdim, device=dev).to(bf16)
        values = torch.empty(rows, heads * vdim, device=dev, dtype=bf16)
        us = timed(lambda: K.heads_linear(lat_out, rank, 0, value_up, values, vdim, 0, heads), torch)
        note(f"heads_linear (latents into values), {tag}", us, value_up.numel() * 2 + rows * heads * (rank + vdim) * 2,
             2.0 * rows * heads * rank * vdim, PEAK_FLOPS["bf16"])
        # -- the matrix memory beside the recurrences of the other designs
        m_dim = 64
        m_proj = torch.randn(rows, 2 * heads * m_dim + 2 * heads * vdim, device=dev).to(bf16)
        pre = torch.randn(rows, 2 * heads, device=dev)
        gate_bias = torch.ones(2 * heads, device=dev)
        m_state = torch.zeros(seqs, K.mlstm_state_floats(heads, m_dim, vdim), device=dev)
        beside = torch.empty(rows, 4 * heads, device=dev)
        read = torch.empty(rows, heads * vdim, device=dev)
        us = timed(lambda: K.mlstm_gates(pre, gate_bias, 15.0, m_state, starts, slots, beside, heads, m_dim, vdim), torch)
        note(f"mlstm_gates, {tag}", us, pre.numel() * 4 + beside.numel() * 4)
        us = timed(lambda: K.mlstm_scan(m_proj, 0, heads * m_dim, 2 * heads * m_dim, beside, m_state, starts, slots, read, heads, m_dim, vdim), torch)
        note(f"mlstm_scan, {tag}", us, 2 * m_state.numel() * 4 + rows * heads * (2 * m_dim + vdim) * 2 + read.numel() * 4,
             3.0 * rows * heads * m_dim * (vdim + 1))
        m_out = torch.empty(rows, heads * vdim, device=dev, dtype=bf16)
        m_weight = torch.ones(heads * vdim, device=dev)
        us = timed(lambda: K.mlstm_finish(read, beside, m_proj, 2 * heads * m_dim + heads * vdim, m_weight, 1e-6, m_out, heads, vdim), torch)
        note(f"mlstm_finish, {tag}", us, read.numel() * 4 + 2 * m_out.numel() * 2)
        if each == 1:      # the three in one launch, as a decode step runs them
            us = timed(lambda: K.mlstm_step(m_proj, 0, heads * m_dim, 2 * heads * m_dim, 2 * heads * m_dim + heads * vdim, pre, gate_bias, 15.0,
                                            m_state, slots, m_weight, 1e-6, m_out, heads, m_dim, vdim), torch)
            note(f"mlstm_step (gates, scan and finish in one launch), {tag}", us, 2 * m_state.numel() * 4 + m_proj.numel() * 2 + m_out.numel() * 2)
        l_proj = torch.randn(rows, 4 * heads * dim, device=dev).to(bf16)
        l_state = torch.zeros(seqs, heads, dim, vdim, device=dev)
        decay = torch.full((heads,), 0.99, device=dev)
        mixed = torch.empty(rows, heads * vdim, device=dev)
        us = timed(lambda: K.lightning_scan(l_proj, 0, heads * dim, 2 * heads * dim, l_state, decay, starts, slots, mixed, heads, dim, vdim), torch)
        note(f"gokazen lightning_scan, {tag}", us, 2 * l_state.numel() * 4 + rows * 3 * heads * dim * 2 + mixed.numel() * 4,
             4.0 * rows * heads * dim * vdim)
        l_gated = torch.empty(rows, heads * vdim, device=dev, dtype=bf16)
        us = timed(lambda: K.gated_rmsnorm(mixed, l_proj, 3 * heads * dim, m_weight, 1e-6, l_gated), torch)
        note(f"gokazen gated_rmsnorm, {tag}", us, mixed.numel() * 4 + 2 * l_gated.numel() * 2)
        # -- the dense feed-forward's activation beside the others'
        inner = torch.randn(rows, 3 * width, device=dev).to(bf16)
        activated = torch.empty_like(inner)
        us = timed(lambda: K.gelu_tanh(inner, activated), torch)
        note(f"gelu_tanh, {tag}", us, 2 * inner.numel() * 2)
        us = timed(lambda: K.relu_squared(inner, activated), torch)
        note(f"gokazen relu_squared, {tag}", us, 2 * inner.numel() * 2)
    return out


def dupidra_bench(args, torch):
    from beholdd.engine import Engine, random_model_on_device

    device, points = "cuda:0", []
    t = min(args.prefill_tokens, args.context)
    for width, heads in ((2048, 16), (4096, 32)):
        trio = {"dupidra": dupidra_config(width, heads, 32768),
                "pudorax": pudorax_config(width, heads, 32768),
                "qwen3": dict(QWEN3_8B, num_hidden_layers=8, hidden_size=width, num_attention_heads=heads,
                              num_key_value_heads=heads // 4, intermediate_size=3 * width, vocab_size=32768)}
        point = {"width": width, "heads": heads, "layer_runs": 8}
        if args.alone:
            trio = {"dupidra": trio["dupidra"]}
        for name, config in trio.items():
            model = random_model_on_device(config, seed=0, dtype="bfloat16", device=device)
            engine = Engine(model=model, dtype="bfloat16", max_tokens=args.batch * (-(-args.context // 64) * 64),
                            max_slots=args.batch, device=device)
            parameters = sum(int(np_prod(spec.shape)) for spec in model.tensor_specs())
            seconds, _ = decode_run(engine, args.batch, args.context, args.steps, args.warmup, torch)
            prefill = prefill_run(engine, t, torch)
            point[name] = {"parameters": parameters, "decode_ms_per_step": round(seconds * 1e3, 4),
                           "decode_tok_per_s": round(args.batch / seconds, 1), "prefill_ms": round(prefill * 1e3, 3),
                           "prefill_tok_per_s": round(t / prefill, 1)}
            kernels = engine.kernels
            del engine, model
            torch.cuda.empty_cache()
        points.append(point)
    line = {"metric": f"Dupidra beside Pudorax and Qwen3 at equal width and as many layer runs: decode tok/s @ batch {args.batch}, context {args.context}; prefill of {t} tokens",
            "unit": "tok/s", "value": points[-1]["dupidra"]["decode_tok_per_s"], "dtype": "bf16", "data": "synthetic", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "points": points,
            "kernels": {} if args.alone else dupidra_kernels(kernels, torch, 4096, 32, args.context)}
    print(json.dumps(line))
    return 0


def vepelix_config(width, heads, vocab, experts=32, top=4, window=4096, rank=192, rot=64):
    """Six layers of which two run twice (eight layer runs): attention over a latent of `rank` with a shared rotated key part of
    `rot`, heads of 128 and queries through a latent of 3/8 of the width; windowed attention (heads of 128, four query heads to a
    key/value head, a rotation over half a head) beside gated linear attention (keys of 64 and values of 128 a head, decays through
    a rank of 16); `experts` experts of 3/8 of the width of which `top` are used and a shared one of 3/2 of the width in all layers
    but the first, whose feed-forward is dense and three times the width."""
    stretch = {"factor": 4.0, "original": 4096, "fast": 16.0, "slow": 1.0}
    mlp = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": 3 * width // 8}, "shared": {"ff": 3 * width // 2}}
    latent = {"type": "latent_attention", "mlp": mlp,
              "mixer": {"heads": heads, "dim": 128, "rot_dim": rot, "vdim": 128, "kv_rank": rank, "q_rank": 3 * width // 8,
                        "scale": (128 + rot) ** -0.5, "rot": {"base": 10000.0, "dims": rot, "scaling": stretch}}}
    side = {"type": "parallel", "mlp": mlp,
            "mixer": {"left": {"heads": heads, "kv_heads": max(heads // 4, 1), "dim": 128, "vdim": 128, "scale": 128 ** -0.5,
                               "mask": {"size": window}, "rot": {"base": 100000.0, "dims": 64, "scaling": stretch}},
                      "right": {"heads": heads, "dim": 64, "vdim": 128, "tau": 8.0, "decay_rank": 16}, "left_scale": 1.0, "right_scale": 1.0}}
    first = dict(latent, mlp={"kind": "dense", "ff": 3 * width, "limit": 7.0})
    return {"architecture": "Vepelix", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "loop": {"start": 1, "stop": 3, "times": 2},
            "layers": [first, latent, side, latent, side, latent]}


def vepelix_kernels(K, torch, width, heads, context, rank=192, rot=64, window=4096):
    """Every kernel that the design brought, and every older kernel in the turn the design gives it, beside its like among the
    other models', alone, at a prompt of 2,048 rows and at a decode step of 8 rows over `context` cached tokens: microseconds and
    the fraction of the roofline (the slower of its bytes at the HBM peak and its operations at the peak of the units it runs on)."""
    from types import SimpleNamespace
    bf16, dev = torch.bfloat16, "cuda:0"
    dim = vdim = 128
    page = K.page_size
    out = {}

    def note(name, us, n_bytes, flops=0.0, peak=PEAK_FLOPS["fp32"]):
        floor = max(n_bytes / (PEAK_HBM_GBS * 1e9), flops / peak) * 1e6
        out[name] = {"us": round(us, 1), "roofline_us": round(floor, 2), "fraction": round(floor / us, 3)}

    def pages_for(n_seqs, length, kv_heads, head):
        per = -(-length // page)
        k_pages = torch.randn(n_seqs * per, kv_heads, page, head, device=dev).to(bf16)
        v_pages = torch.randn(n_seqs * per, kv_heads, head, page, device=dev).to(bf16)
        table = torch.arange(n_seqs * per, dtype=torch.int32, device=dev).view(n_seqs, per).contiguous()
        return k_pages, v_pages, table

    kv_heads = max(heads // 4, 1)
    for rows, seqs, past, tag in ((2048, 1, 0, "prompt of 2,048"), (8, 8, context - 1, f"decode of 8 at {context}")):
        each = rows // seqs
        starts = torch.arange(0, rows + 1, each, dtype=torch.int32, device=dev)
        slots = torch.arange(seqs, dtype=torch.int32, device=dev)
        positions = (torch.arange(rows, dtype=torch.int32, device=dev) % each + past).contiguous()
        row_seq = (torch.arange(rows, dtype=torch.int32, device=dev) // each).contiguous()
        layout = SimpleNamespace(seq_start=starts, n_seqs=seqs, max_rows_per_seq=each, max_position=past + each - 1)
        keys_seen = seqs * (past + each) if each == 1 else each * (each + 1) // 2
        # -- gated linear attention (keys of 64, values of 128 a head) beside the linear attention with one decay a head
        g_dim = 64
        proj = torch.randn(rows, 2 * heads * g_dim + 2 * heads * vdim, device=dev).to(bf16)
        decays = torch.randn(rows, heads * g_dim, device=dev)
        bias = torch.full((heads * g_dim,), 4.0, device=dev)
        state = torch.zeros(seqs, heads, g_dim, vdim, device=dev)
        mixed = torch.empty(rows, heads * vdim, device=dev)
        us = timed(lambda: K.gla_scan(proj, 0, heads * g_dim, 2 * heads * g_dim, decays, bias, 16.0, g_dim ** -0.5, state, starts, slots, mixed,
                                      heads, g_dim, vdim), torch)
        note(f"gla_scan, {tag}", us, 2 * state.numel() * 4 + rows * heads * (2 * g_dim + vdim) * 2 + decays.numel() * 4 + mixed.numel() * 4,
             4.0 * rows * heads * g_dim * vdim)
        l_proj = torch.randn(rows, 4 * heads * dim, device=dev).to(bf16)
        l_state = torch.zeros(seqs, heads, dim, vdim, device=dev)
        decay = torch.full((heads,), 0.99, device=dev)
        us = timed(lambda: K.lightning_scan(l_proj, 0, heads * dim, 2 * heads * dim, l_state, decay, starts, slots, mixed, heads, dim, vdim), torch)
        note(f"gokazen lightning_scan, {tag}", us, 2 * l_state.numel() * 4 + rows * 3 * heads * dim * 2 + mixed.numel() * 4, 4.0 * rows * heads * dim * vdim)
        gated = torch.empty(rows, heads * vdim, device=dev, dtype=bf16)
        weight = torch.ones(heads * vdim, device=dev)
        us = timed(lambda: K.gated_group_rmsnorm(mixed, proj, 2 * heads * g_dim + heads * vdim, weight, 1e-6, gated, heads, gate_after=True), torch)
        note(f"gated_group_rmsnorm with the gate behind the norm, {tag}", us, mixed.numel() * 4 + 2 * gated.numel() * 2)
        us = timed(lambda: K.gated_rmsnorm(mixed, l_proj, 3 * heads * dim, weight, 1e-6, gated), torch)
        note(f"gokazen gated_rmsnorm, {tag}", us, mixed.numel() * 4 + 2 * gated.numel() * 2)
        # -- the weighted sum of the two mixers' results, beside the residual's update
        a, b = torch.randn(rows, width, device=dev), torch.randn(rows, width, device=dev)
        us = timed(lambda: K.weighted_sum(a, a, 1.2, b, 1.1), torch)
        note(f"weighted_sum, {tag}", us, 3 * a.numel() * 4)
        x, ones = torch.randn(rows, 1, width, device=dev), torch.ones(width, device=dev)
        us = timed(lambda: K.streams_update(x, a, None, None, ones), torch)
        note(f"gokazen streams_update (one stream), {tag}", us, 3 * a.numel() * 4)
        # -- the latent layer: the query latent's norm, the cache write with stretched neighbour pairs, attention with sinks, the gate
        q_rank, q_head, kv_head = 3 * width // 8, dim + rot, rank + rot
        down = torch.randn(rows, q_rank + kv_head + heads, device=dev).to(bf16)
        latent_q = torch.empty(rows, q_rank, device=dev, dtype=bf16)
        rank_weight = torch.ones(q_rank, device=dev)
        us = timed(lambda: K.slice_rmsnorm(down, 0, rank_weight, 1e-6, latent_q), torch)
        note(f"slice_rmsnorm, {tag}", us, 2 * latent_q.numel() * 2)
        hidden = torch.randn(rows, width, device=dev)
        normed = torch.empty(rows, width, device=dev, dtype=bf16)
        us = timed(lambda: K.rmsnorm(hidden, ones, 1e-6, normed), torch)
        note(f"qwen3 rmsnorm, {tag}", us, hidden.numel() * 4 + normed.numel() * 2)
        heads_rows = torch.randn(rows, heads * q_head, device=dev).to(bf16)
        k_pages, v_pages, table = pages_for(seqs, past + each, 1, kv_head)
        freq, latent_weight = torch.ones(rot // 2, device=dev), torch.ones(rank, device=dev)
        query = torch.empty(rows, heads * kv_head, device=dev, dtype=bf16)
        us = timed(lambda: K.latent_write(down, q_rank, latent_weight, 1e-6, freq, rot, positions, row_seq, k_pages, v_pages, table, rank, rot,
                                          query=query, query_head=kv_head, query_first=rank, source_head=q_head, source_first=dim,
                                          n_heads=heads, query_source=heads_rows, neighbours=True, magnitude=1.2), torch)
        note(f"latent_write, neighbour pairs, queries from their own matrix, {tag}", us, rows * kv_head * 2 * 3 + 2 * rows * heads * rot * 2)
        attended = torch.empty_like(query)
        scale = (dim + rot) ** -0.5
        sinks = torch.randn(heads, device=dev)
        for name, kw in (("with sinks", dict(sinks=sinks)), ("gokazen, without", {})):
            us = timed(lambda: K.attention(query, attended, k_pages, v_pages, table, row_seq, positions, heads, 1, kv_head, scale, 0,
                                           layout=layout, **kw), torch)
            note(f"attention over the latent ({heads} heads on one of {kv_head}) {name}, {tag}", us,
                 2 * seqs * (past + each) * kv_head * 2 + 2 * query.numel() * 2, 4.0 * keys_seen * heads * kv_head, PEAK_FLOPS["bf16"])
        values = torch.randn(rows, heads * vdim, device=dev).to(bf16)
        gated_values = torch.empty_like(values)
        us = timed(lambda: K.gate_heads(values, vdim, down, q_rank + kv_head, gated_values, heads, vdim, per_head=True), torch)
        note(f"gate_heads, one gate a head, {tag}", us, 2 * values.numel() * 2)
        wide_gate = torch.randn(rows, heads * vdim, device=dev).to(bf16)
        us = timed(lambda: K.gate_heads(values, vdim, wide_gate, 0, gated_values, heads, vdim), torch)
        note(f"pudorax gate_heads, one gate a value, {tag}", us, 3 * values.numel() * 2)
        # -- the windowed attention: head norms, stretched neighbour pairs and the cache write; the attention within the window
        q_w, k_w = heads * dim, kv_heads * dim
        qkv = torch.randn(rows, q_w + 2 * k_w, device=dev).to(bf16)
        head_weight, half_freq = torch.ones(dim, device=dev), torch.ones(32, device=dev)
        wk, wv, wtable = pages_for(seqs, past + each, kv_heads, dim)
        q_out = torch.empty(rows, heads * dim, device=dev, dtype=bf16)
        for name, kw in (("neighbour pairs", dict(neighbours=True, magnitude=1.2)), ("dupidra, pairs half apart", {})):
            us = timed(lambda: K.head_norm_rope_write(qkv, 0, None, head_weight, head_weight, 1e-6, half_freq, 64, positions, row_seq, q_out, wk, wv,
                                                      wtable, heads, kv_heads, dim, dim, dim, True, **kw), torch)
            note(f"head_norm_rope_write, {name}, {tag}", us, 2 * qkv.numel() * 2)
        w_out = torch.empty_like(q_out)
        seen = min(window, past + each)
        us = timed(lambda: K.attention(q_out, w_out, wk, wv, wtable, row_seq, positions, heads, kv_heads, dim, dim ** -0.5, window, layout=layout), torch)
        note(f"attention within a window of {window} ({heads} heads on {kv_heads} of {dim}), {tag}", us,
             2 * seqs * seen * kv_heads * dim * 2 + 2 * q_out.numel() * 2, 4.0 * min(keys_seen, rows * seen) * heads * dim, PEAK_FLOPS["bf16"])
        # -- routing by sigmoids, and the experts of a decode step with the weights on their inputs
        experts, top, ff = 32, 4, 3 * width // 8
        logits = torch.randn(rows, experts, device=dev)
        chosen = torch.empty(rows, top, dtype=torch.int32, device=dev)
        shares = torch.empty(rows, top, device=dev)
        for name, kw in (("sigmoid scores", dict(scoring="sigmoid")), ("pudorax, softmax over the chosen", {})):
            us = timed(lambda: K.route_top_k(logits, None, chosen, shares, **kw), torch)
            note(f"route_top_k, {name}, {tag}", us, logits.numel() * 4 + 2 * chosen.numel() * 4)
        if each == 1:
            w_gu = torch.randn(experts, 2 * ff, width, device=dev).to(bf16) * 0.02
            lists = torch.empty(experts, rows, dtype=torch.int32, device=dev)
            counts = torch.empty(experts, dtype=torch.int32, device=dev)
            K.experts_group(chosen, lists, counts)
            active = int((counts > 0).sum())
            x_rows = torch.randn(rows, width, device=dev).to(bf16)
            inner = torch.empty(rows * top, ff, device=dev, dtype=bf16)
            for name, kw in (("silu, weights on the inputs", dict(limit=float("inf"), alpha=1.0, shift=0.0, in_weights=shares)),
                             ("pudorax, clamped, weights on the outputs", dict(limit=7.0, alpha=1.702))):
                us = timed(lambda: K.experts_rows(x_rows, top, lists, counts, w_gu, inner, gated=True, **kw), torch)
                note(f"experts_rows gate and up, {name}, {tag}", us, active * 2 * ff * width * 2)
    return out


def vepelix_bench(args, torch):
    from beholdd.engine import Engine, random_model_on_device

    device, points = "cuda:0", []
    t = min(args.prefill_tokens, args.context)
    for width, heads in ((2048, 16), (4096, 32)):
        models = {"vepelix": vepelix_config(width, heads, 32768),
                  "gokazen": gokazen_config(width, heads, 8, 3 * width, 32768),
                  "dupidra": dupidra_config(width, heads, 32768),
                  "qwen3": dict(QWEN3_8B, num_hidden_layers=8, hidden_size=width, num_attention_heads=heads,
                                num_key_value_heads=heads // 4, intermediate_size=3 * width, vocab_size=32768)}
        point = {"width": width, "heads": heads, "layer_runs": 8}
        if args.alone:
            models = {"vepelix": models["vepelix"]}
        for name, config in models.items():
            model = random_model_on_device(config, seed=0, dtype="bfloat16", device=device)
            engine = Engine(model=model, dtype="bfloat16", max_tokens=args.batch * (-(-args.context // 64) * 64),
                            max_slots=args.batch, device=device)
            parameters = sum(int(np_prod(spec.shape)) for spec in model.tensor_specs())
            seconds, _ = decode_run(engine, args.batch, args.context, args.steps, args.warmup, torch)
            prefill = prefill_run(engine, t, torch)
            point[name] = {"parameters": parameters, "decode_ms_per_step": round(seconds * 1e3, 4),
                           "decode_tok_per_s": round(args.batch / seconds, 1), "prefill_ms": round(prefill * 1e3, 3),
                           "prefill_tok_per_s": round(t / prefill, 1)}
            kernels = engine.kernels
            del engine, model
            torch.cuda.empty_cache()
        points.append(point)
    line = {"metric": f"Vepelix beside Gokazen, Dupidra and Qwen3 at equal width and as many layer runs: decode tok/s @ batch {args.batch}, context {args.context}; prefill of {t} tokens",
            "unit": "tok/s", "value": points[-1]["vepelix"]["decode_tok_per_s"], "dtype": "bf16", "data": "synthetic", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "points": points,
            "kernels": {} if args.alone else vepelix_kernels(kernels, torch, 4096, 32, args.context)}
    print(json.dumps(line))
    return 0


def np_prod(shape):
    total = 1
    for axis in shape:
        total *= int(axis)
    return total


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this single-GPU library")
        return 2
    import torch
    if args.hbm_ceiling:
        print(json.dumps(hbm_ceiling(torch)))
        return 0
    if args.sampling:
        print(json.dumps(sampling_times(torch)))
        return 0
    if args.gokazen:
        return gokazen_bench(args, torch)
    if args.pudorax:
        return pudorax_bench(args, torch)
    if args.dupidra:
        return dupidra_bench(args, torch)
    if args.vepelix:
        return vepelix_bench(args, torch)

    from beholdd.engine import Engine, random_model_on_device

    shape_name, shape = SHAPES[args.shape]
    config = dict(shape, num_hidden_layers=args.layers or shape["num_hidden_layers"])
    device = "cuda:0"
    dtype_tag = "bf16" if args.dtype == "bfloat16" else "fp32"
    element = 2 if args.dtype == "bfloat16" else 4
    model = random_model_on_device(config, seed=0, dtype=args.dtype, device=device)
    biggest = 1 if args.no_points else 64
    if args.workload:
        count, _, longest, new_tokens, _, context = WORKLOADS[args.shape]
        engine = Engine(model=model, dtype=args.dtype, max_tokens=count * (-(-(longest + new_tokens) // 64) * 64),
                        max_slots=count, device=device)
        line = {"metric": f"generation of the {shape_name} batch", "unit": "tok/s", "dtype": dtype_tag,
                "layers": config["num_hidden_layers"], "layers_of_full_model": shape["num_hidden_layers"], "context": context}
        line.update(workload_run(engine, args.shape, torch))
        line["value"] = line["generated_tok_per_s"]
        print(json.dumps(line))
        return 0
    max_tokens = max(args.batch, biggest) * (-(-args.context // 64) * 64)
    engine = Engine(model=model, dtype=args.dtype, max_tokens=max_tokens, max_slots=max(args.batch, biggest, 64),
                    device=device)
    randomise_cache(engine, torch)
    cfg = engine.config

    layer_params = (cfg.hidden * (cfg.q_width + 2 * cfg.kv_width) + cfg.q_width * cfg.hidden
                    + 3 * cfg.hidden * cfg.intermediate)
    weight_bytes = (cfg.n_layers * layer_params + cfg.vocab * cfg.hidden) * element
    kv_bytes_per_token = cfg.n_layers * 2 * cfg.kv_width * element

    seconds, mean_length = decode_run(engine, args.batch, args.context, args.steps, args.warmup, torch)
    step_bytes = weight_bytes + args.batch * mean_length * kv_bytes_per_token
    achieved = step_bytes / seconds / 1e9
    value = args.batch / seconds

    t = min(args.prefill_tokens, args.context)      # (a context shorter than the prompt: a prompt of the context's length)
    prefill_seconds = prefill_run(engine, t, torch)
    prefill_flops = (2.0 * cfg.n_layers * layer_params * t + cfg.n_layers * cfg.n_heads * 2.0 * t * t * cfg.head_dim
                     + 2.0 * cfg.vocab * cfg.hidden)
    # Other batch sizes and contexts: tokens a second, and beside each the fraction of the HBM peak that the
    # bytes of its step (all weights once, the live requests' caches) amount to.
    points, fractions = {}, {}
    if not args.no_points:
        for batch, context, name in ((1, args.context, "decode_b1"), (64, args.context, "decode_b64"),
                                     (1, 512, "decode_b1_ctx512"), (1, 2048, "decode_b1_ctx2048"),
                                     (8, 640, "decode_b8_ctx640"), (64, 640, "decode_b64_ctx640")):
            steps = max(4, args.steps // 2)
            s, length = decode_run(engine, batch, context, steps, 2, torch)
            points[name] = round(batch / s, 2)
            fractions[name] = round((weight_bytes + batch * length * kv_bytes_per_token) / s / 1e9 / PEAK_HBM_GBS, 4)
    # Prompts of other lengths: tokens a second and the fraction of the matrix-core peak; for the short ones, which
    # the host's launches bound, also the milliseconds until the step function returns.
    prefill_points = {}
    if not args.no_points:
        def flops(tokens, prompts=1):
            return prompts * (2.0 * cfg.n_layers * layer_params * tokens + cfg.n_layers * cfg.n_heads * 2.0 * tokens * tokens * cfg.head_dim
                              + 2.0 * cfg.vocab * cfg.hidden)
        for tokens in (16, 64, 128):
            seconds_all, seconds_host = prefill_run(engine, tokens, torch, host=True)
            prefill_points[f"tokens_{tokens}"] = {"ms": round(seconds_all * 1e3, 3), "host_ms": round(seconds_host * 1e3, 3),
                                                  "tok_per_s": round(tokens / seconds_all, 1)}
        for tokens, prompts in ((512, 1), (1024, 1), (4096, 1), (8192, 1), (2048, 4)):
            if tokens > args.context:
                continue
            seconds_all = prefill_run(engine, tokens, torch, repeats=2, prompts=prompts)
            name = f"tokens_{tokens}" if prompts == 1 else f"prompts_{prompts}x{tokens}"
            prefill_points[name] = {"ms": round(seconds_all * 1e3, 3), "tok_per_s": round(prompts * tokens / seconds_all, 1),
                                    "frac": round(flops(tokens, prompts) / seconds_all / PEAK_FLOPS[dtype_tag], 4)}
    generated = None
    if not args.no_points and args.shape == "8b":
        generated = workload_run(engine, args.shape, torch)     # the same batch through Engine.generate

    # what a kernel that does nothing but read reaches on this GPU (the library's yardstick kernel over 4 GB of the cache)
    cache_tensor = engine.cache.groups[0].k
    span = cache_tensor.view(-1)[: min(cache_tensor.numel(), 2 << 30)]
    yardstick = None
    if span.numel() * span.element_size() >= 256 << 20:      # (a cache of a few MB says nothing about streaming)
        engine.kernels.stream_read(span)
        torch.cuda.synchronize()
        begin = time.perf_counter()
        read = sum(engine.kernels.stream_read(span) for _ in range(4))
        torch.cuda.synchronize()
        yardstick = read / (time.perf_counter() - begin) / 1e9

    line = {
        "metric": f"decode tok/s @ batch {args.batch} ({shape_name}, context {args.context})", "value": round(value, 2), "unit": "tok/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(seconds * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype_tag,
        "data": "synthetic: seeded random weights, random token ids, caches filled with random keys and values",
        "config": {
            "model": shape_name, "layers": cfg.n_layers, "layers_of_full_model": shape["num_hidden_layers"],
            "hidden_size": cfg.hidden, "num_attention_heads": cfg.n_heads, "num_key_value_heads": cfg.n_kv_heads,
            "head_dim": cfg.head_dim, "intermediate_size": cfg.intermediate, "vocab_size": cfg.vocab,
            "rope_theta": cfg.rope_theta, "rms_norm_eps": cfg.rms_eps, "tie_word_embeddings": cfg.tie_word_embeddings,
            "global_batch": args.batch, "seq_len": args.context, "prefill_tokens": t, "parallelism": "single GPU",
        },
        "prefill": {"value": round(t / prefill_seconds, 1), "tokens": t, "ms": round(prefill_seconds * 1e3, 3),
                    "frac": round(prefill_flops / prefill_seconds / PEAK_FLOPS[dtype_tag], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4), "plain_read_GBs": round(yardstick, 1) if yardstick is not None else None},
        "points": points,
        "points_hbm_frac": fractions,
    }
    if prefill_points:
        line["prefill_points"] = prefill_points
    if generated is not None:
        line["generate"] = generated
    if not args.no_points and args.shape == "8b" and args.layers is None and args.dtype == "bfloat16":
        # the other two shapes of the family, full depth: decode at batch 8 and the prompt of 2,048 tokens
        del engine, model, cache_tensor, span
        line["shapes"] = {name: other_shape(name, args, torch) for name in ("14b", "32b")}
    print(json.dumps(line))
    return 0


def other_shape(name, args, torch):
    import gc

    from beholdd.engine import Engine, random_model_on_device
    gc.collect()
    torch.cuda.empty_cache()
    config = SHAPES[name][1]
    model = random_model_on_device(dict(config), seed=0, dtype="bfloat16", device="cuda:0")
    engine = Engine(model=model, dtype="bfloat16", max_tokens=8 * (-(-args.context // 64) * 64), max_slots=8, device="cuda:0")
    randomise_cache(engine, torch)
    cfg = engine.config
    layer_params = (cfg.hidden * (cfg.q_width + 2 * cfg.kv_width) + cfg.q_width * cfg.hidden + 3 * cfg.hidden * cfg.intermediate)
    weight_bytes = (cfg.n_layers * layer_params + cfg.vocab * cfg.hidden) * 2
    kv_bytes_per_token = cfg.n_layers * 2 * cfg.kv_width * 2
    steps = max(4, args.steps // 2)
    seconds, mean_length = decode_run(engine, 8, args.context, steps, 2, torch)
    t = min(args.prefill_tokens, args.context)
    prefill_seconds = prefill_run(engine, t, torch, repeats=2)
    prefill_flops = (2.0 * cfg.n_layers * layer_params * t + cfg.n_layers * cfg.n_heads * 2.0 * t * t * cfg.head_dim
                     + 2.0 * cfg.vocab * cfg.hidden)
    out = {"layers": cfg.n_layers, "decode_b8_tok_per_s": round(8 / seconds, 2), "decode_b8_ms": round(seconds * 1e3, 4),
           "decode_b8_hbm_frac": round((weight_bytes + 8 * mean_length * kv_bytes_per_token) / seconds / 1e9 / PEAK_HBM_GBS, 4),
           "prefill_tok_per_s": round(t / prefill_seconds, 1), "prefill_ms": round(prefill_seconds * 1e3, 3),
           "prefill_frac": round(prefill_flops / prefill_seconds / PEAK_FLOPS["bf16"], 4)}
    del engine, model
    gc.collect()
    torch.cuda.empty_cache()
    return out


if __name__ == "__main__":
    sys.exit(main())
