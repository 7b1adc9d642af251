"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--dtype bf16|fp32]
    python bench.py --shape llama8b --serve 64     (requests through the scheduler instead)

Default run: the layer sizes of the CWM-32B shape with random weights, a batch of 8
requests at a context of 32,768 tokens each; a step is one decode step of the whole
batch through the engine's step function and sampler, each step fed on the device by the
tokens that the one before sampled, with a host round trip every ten steps (the engine's
`sync_freq`, the reference's way of decoding).  It prints one JSON line:
`value` is decoded tokens a second; `prefill` is a 2,048-token prompt in one step;
`roofline` compares the bytes a decode step has to read (every weight once, and the
cache of the live requests) with the HBM peak.  The cache of the timed requests is filled
with random numbers instead of being computed (the weights are random too).

`points` holds the workload that the baseline names: batches of 1, 8 and 64 requests with
prompts of 1,024 random tokens and 256 new tokens each, through `Engine.step` (scheduler,
step function and sampler; decode steps run in bursts of `sync_freq` = 10 with one host round
trip a burst, as the reference's do); `decode_b<N>` is N times the number of steps in which all
N requests decode, over the time of those steps; `decode_b<N>_ms` is the median of their times
(a burst's time divided by its steps) and `decode_b<N>_frac` the bytes such a step has to read over that
median and the HBM peak.  `decode_b8_ctx<C>` are decode steps of 8 requests at other context
lengths through the step function, as the headline.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

CWM_32B = {
    "architecture": "llama3_dense",
    "dim": 6144,
    "n_layers": 64,
    "n_heads": 48,
    "n_kv_heads": 8,
    "head_dim": 128,
    "vocab_size": 128256,
    "ffn_dim_multiplier": 1.3125,
    "multiple_of": 256,
    "norm_eps": 1e-5,
    "pos_embed_impl": "scaled_rope",
    "rope_theta": 1000000.0,
    "scaled_rope": {"scale_factor": 16, "old_context_len": 8192, "low_freq_factor": 1, "high_freq_factor": 4},
    "window_attn": {"window_pattern": 4, "local_window": 8192, "global_last_layer": True},
    "max_seq_len": 131072,
}
LLAMA3_8B = {
    "architecture": "llama3_dense",
    "dim": 4096,
    "n_layers": 32,
    "n_heads": 32,
    "n_kv_heads": 8,
    "head_dim": 128,
    "vocab_size": 128256,
    "ffn_dim_multiplier": 1.3,
    "multiple_of": 1024,
    "norm_eps": 1e-5,
    "pos_embed_impl": "rope",
    "rope_theta": 500000.0,
    "max_seq_len": 8192,
}
LLAMA3_70B = dict(LLAMA3_8B, dim=8192, n_layers=80, n_heads=64, multiple_of=4096)
# a small model of the same family (heads of 64): launching its kernels takes the host longer than running them takes the GPU
SMALL_1B = dict(LLAMA3_8B, dim=2048, n_layers=16, n_heads=32, head_dim=64, ffn_dim_multiplier=1.5, multiple_of=256, max_seq_len=131072)
SHAPES = {
    "cwm32b": ("CWM-32B shape (Llama-3 dense, 3 local : 1 global)", CWM_32B),
    "llama8b": ("Llama-3 8B shape (all layers global)", LLAMA3_8B),
    "llama70b": ("Llama-3 70B shape (all layers global)", LLAMA3_70B),
    "small1b": ("16 layers of width 2,048 (32 heads of 64, all layers global)", SMALL_1B),
}


def layer_kinds(n_layers):
    """3 sliding-window layers, then 1 global one, repeated."""
    return ["global" if i % 4 == 3 else "local" for i in range(n_layers)]


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--shape", default="cwm32b", choices=sorted(SHAPES), help="layer sizes; the default is the headline configuration")
    ap.add_argument("--config", default=None, metavar="FILE", help="a config.json of the architecture whose layer sizes are measured instead of --shape's")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (both numbers are reported)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=32768)
    ap.add_argument("--page", type=int, default=256)
    ap.add_argument("--no-points", action="store_true")
    ap.add_argument("--graphs", type=int, default=16, help="decode steps kept as HIP graphs where the host is the limit, as the engine's default (0: none)")
    ap.add_argument(
        "--serve",
        type=int,
        default=0,
        metavar="N",
        help="instead of the step benchmark: N requests with prompts of 128 to 4,096 random tokens and --new tokens each, "
        "through the engine's scheduler (continuous batching, temperature 0.7, top-p 0.95)",
    )
    ap.add_argument("--new", type=int, default=512, help="tokens generated per request with --serve")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch

    from cwm_amd.cache import CacheManager, CacheStorage
    from cwm_amd.engine import ModelRunner, Portion, random_model
    from cwm_amd.parts import PagedKVSpec
    from cwm_amd.sampling import Sampler

    device = torch.device("cuda:0")
    shape_name, shape = SHAPES[args.shape]
    if args.config:
        with open(args.config) as f:
            shape_name, shape = f"the sizes of {os.path.basename(args.config)}", json.load(f)
    config = dict(shape)
    full_layers = shape["n_layers"]
    if args.layers is None:
        args.layers = full_layers
    config["n_layers"] = args.layers
    if "window_attn" in shape:
        config["layer_types"] = layer_kinds(args.layers)
    t0 = time.time()
    model, typed = random_model(config, seed=0, dtype=args.dtype, device=device)
    torch.cuda.synchronize()
    print(f"[bench] {args.layers}-layer model ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    if args.serve:
        return serve_run(args, model, typed, shape_name)
    esize = 2 if args.dtype == "bf16" else 4
    # what a step reads of the weights, from the model's own list of tensors: everything but the embedding
    # table (of which a step reads one row a token); `matrix_params` are the entries of the matrices, which
    # every token is multiplied with
    weight_bytes = 0
    matrix_params = 0
    head_params = 0
    head_names = model.tensor_names("head")
    embedding_only = model.tensor_names("embedding") - head_names  # tables of which a step reads one row a token
    for name, spec in model.tensor_specs().items():
        count = 1
        for n in spec.shape:
            count *= n
        if name in embedding_only:
            continue
        weight_bytes += count * esize
        if len(spec.shape) == 2:
            if name in head_names:
                head_params += count
            else:
                matrix_params += count
    windows = sorted({spec.window for spec in model.cache_specs if isinstance(spec, PagedKVSpec) and spec.window is not None})
    window = windows[0] if windows else None
    page = args.page
    sampler = Sampler(device)
    vocab = typed.vocab_size

    def cache_bytes(batch, ctx):
        total = 0
        for spec in model.cache_specs:
            if isinstance(spec, PagedKVSpec):
                keys = ctx if spec.window is None else min(ctx, spec.window)
                total += batch * keys * spec.bytes_per_token(esize)
        return total

    def make_runner(batch, ctx, extra):
        pages = {None: batch * ((ctx + extra + page - 1) // page + 1)}
        for w in windows:
            pages[w] = batch * ((min(ctx, w) + extra + 2 * page - 1) // page + 2)
        manager = CacheManager(model.cache_specs, page, pages, batch)
        storage = CacheStorage(manager, device, model.runtime.act_dtype)
        for t in storage.paged.values():
            t.normal_(0.0, 1.0)
        return ModelRunner(model, manager, storage, num_graphs=args.graphs, graphs_where_host_bound=True), manager

    def decode_run(batch, ctx, steps, warmup):
        """tokens/s and ms per step of `steps` decode steps of `batch` requests that
        already hold `ctx` tokens each."""
        runner, manager = make_runner(batch, ctx, steps + warmup + 2)
        for b in range(batch):
            runner.admit(b)
            held = 0
            while held < ctx:  # in pieces, so that window groups give pages back as they would have
                n = min(page, ctx - held)
                assert manager.extend(b, n)
                manager.advance(b, n)
                held += n
        # as the engine decodes (sync_freq, cwm/fastgen/generate.py:729-809): every step's tokens are sampled on the
        # device and feed the next step from there; they come to the host once in ten steps
        tokens = torch.tensor([(17 * b + 3) % vocab for b in range(batch)], dtype=torch.int32, device=device)
        params = torch.zeros((3, batch), dtype=torch.float32, device=device)
        params[1] = 1.0  # temperature 0 (greedy), top-p 1, uniform numbers 0
        placeholder = [Portion(b, [0], [0]) for b in range(batch)]  # the token ids come from the device

        def run(n_steps, tokens):
            for i in range(n_steps):
                for b in range(batch):
                    assert manager.extend(b, 1)
                logits = runner.step(placeholder, tokens_device=tokens)
                packed = sampler.sample_packed(logits, params[0], params[1], params[2])
                tokens = packed[0]
                if i % 10 == 9:
                    packed.cpu()
            return tokens

        tokens = run(warmup, tokens)
        torch.cuda.synchronize()
        start = time.perf_counter()
        tokens = run(steps, tokens)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - start
        del runner, manager
        torch.cuda.empty_cache()
        return batch * steps / elapsed, 1000.0 * elapsed / steps

    def prefill_run(n_tokens):
        runner, manager = make_runner(1, n_tokens, 8)
        best = None
        for rep in range(3):
            runner.admit(rep)
            assert manager.extend(rep, n_tokens)
            toks = [(31 * i + 7) % vocab for i in range(n_tokens)]
            torch.cuda.synchronize()
            start = time.perf_counter()
            runner.step([Portion(rep, toks, [n_tokens - 1])])
            torch.cuda.synchronize()
            elapsed = time.perf_counter() - start
            runner.release(rep)
            best = elapsed if best is None else min(best, elapsed)
        del runner, manager
        torch.cuda.empty_cache()
        return best

    # ---- the timed run ---------------------------------------------------------- #
    tok_s, ms_step = decode_run(args.batch, args.context, args.steps, args.warmup)
    read_bytes = weight_bytes + cache_bytes(args.batch, args.context)
    achieved = read_bytes / (ms_step * 1e-3) / 1e9

    n_prefill = 2048
    prefill_s = prefill_run(n_prefill)
    attn_flops = 0
    for call, slot in zip(model.run_order, model.cache_slot):
        spec = model.cache_specs[slot]
        if isinstance(spec, PagedKVSpec):
            # causal: token p reads min(p + 1, window) keys; 2 products (QK^T and PV) of 2 flops, for every query head
            keys = sum(min(p + 1, spec.window or (p + 1)) for p in range(n_prefill))
            query_heads = getattr(model.blocks[call.layer].mixer, "n_heads", spec.n_kv_heads)
            attn_flops += 4 * keys * query_heads * spec.head_dim
    prefill_flops = 2 * n_prefill * matrix_params + attn_flops + 2 * head_params
    prefill = {
        "value": round(n_prefill / prefill_s, 1),
        "tokens": n_prefill,
        "ms": round(prefill_s * 1e3, 2),
        "frac": round(prefill_flops / prefill_s / PEAK_FLOPS[args.dtype], 4),
    }

    points = {}
    if not args.no_points:
        for ctx in (8192, 131072):
            if ctx == args.context:
                continue
            free_bytes, _ = torch.cuda.mem_get_info(device)
            if cache_bytes(args.batch, ctx) > 0.9 * free_bytes:  # an all-global shape at 131,072 tokens does not fit beside its weights
                print(f"[bench] no point at context {ctx}: its cache does not fit", file=sys.stderr, flush=True)
                continue
            points[f"decode_b{args.batch}_ctx{ctx}"] = round(decode_run(args.batch, ctx, 10, 6)[0], 1)  # (a capture, if any, falls into the warm-up)
        for b in (1, 8, 64):
            tok_s_b, median_ms, n_steps = engine_point(model, b, 1024, 256, page, typed.vocab_size)
            bytes_b = weight_bytes + cache_bytes(b, 1024 + 128)  # the context grows from 1,024 to 1,280 over the run
            points[f"decode_b{b}"] = round(tok_s_b, 1)
            points[f"decode_b{b}_ms"] = round(median_ms, 3)
            points[f"decode_b{b}_frac"] = round(bytes_b / (median_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
            points[f"decode_b{b}_steps"] = n_steps

    line = {
        "metric": f"decode tok/s ({shape_name.split(' (')[0]}, batch {args.batch}, context {args.context})",
        "value": round(tok_s, 2),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_step, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic: random weights N(0, 0.02), random cache contents, fixed token ids",
        "config": {
            "model": shape_name,
            "global_batch": args.batch,
            "seq_len": args.context,
            "parallelism": "1 GPU",
            "n_layers": args.layers,
            "n_layers_full": full_layers,
            "dim": typed.dim,
            "n_heads": typed.n_heads,
            "n_kv_heads": typed.kv_heads,
            "head_dim": typed.head_size,
            "hidden_dim": typed.ffn_width,
            "vocab_size": typed.vocab_size,
            "local_window": window or 0,
            "page_size": page,
            "points_prompt_tokens": 1024,
            "points_new_tokens": 256,
            "prefill_tokens": n_prefill,
            "graphs": args.graphs,
        },
        "prefill": prefill,
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
        },
        "points": points,
    }
    print(json.dumps(line), flush=True)
    return 0


def engine_point(model, batch, prompt_tokens, new_tokens, page, vocab):
    """`batch` requests with prompts of `prompt_tokens` random tokens and `new_tokens` new tokens each
    through the engine (scheduler, step function, sampler).  Returns (decoded tokens a second over the
    steps in which all `batch` requests decode, the median time of such a step in ms, their number)."""
    import random
    import statistics

    import torch

    from cwm_amd.engine import Engine, GenArgs, Packet

    rng = random.Random(batch)
    gen_args = GenArgs(
        use_sampling=True, temperature=0.7, top_p=1.0, max_batch=batch, cache_block=page, max_prefill=4096,
        max_seq=batch * (prompt_tokens + new_tokens + 2 * page),
    )
    engine = Engine(gen_args, model)
    for i in range(batch):
        engine.submit(Packet(thread_id=i, tokens=[rng.randrange(vocab) for _ in range(prompt_tokens)], max_gen=new_tokens))
    times = []
    finished = 0
    torch.cuda.synchronize()
    while engine.scheduler.has_work():
        start = time.perf_counter()
        finished += len(engine.step())
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - start
        if engine.last_step_sequences == batch and engine.last_step_tokens == batch:
            # a call runs `last_step_burst` decode steps back to back (sync_freq) and syncs with the host once
            times.extend([elapsed / engine.last_step_burst] * engine.last_step_burst)
    assert finished == batch
    del engine
    torch.cuda.empty_cache()
    times = times[2:] if len(times) > 8 else times  # the first such steps still build their plans and buffers
    return batch * len(times) / sum(times), 1e3 * statistics.median(times), len(times)


def serve_run(args, model, typed, shape_name) -> int:
    """Requests of mixed prompt lengths through `Engine.generate`; one JSON line with the
    generated and the total tokens a second."""
    import queue
    import random

    import torch

    from cwm_amd.engine import Engine, GenArgs, Packet

    rng = random.Random(0)
    lengths = [rng.randint(128, 4096) for _ in range(args.serve)]
    gen_args = GenArgs(
        use_sampling=True,
        temperature=0.7,
        top_p=0.95,
        max_batch=min(args.serve, 64),
        max_seq=-1,  # the pools take what is free on the device
        expected_seq=4096 + args.new,
        cache_block=args.page,
        max_prefill=4096,
    )
    engine = Engine(gen_args, model)
    requests = queue.Queue()
    for i, n in enumerate(lengths):
        requests.put(Packet(thread_id=i, tokens=[rng.randrange(typed.vocab_size) for _ in range(n)], max_gen=args.new))
    requests.put(None)
    torch.cuda.synchronize()
    start = time.perf_counter()
    generated = 0
    for packet in engine.generate(requests):
        if packet is not None:
            generated += len(packet.tokens)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - start
    line = {
        "metric": f"generated tok/s ({shape_name.split(' (')[0]}, {args.serve} requests, continuous batching)",
        "value": round(generated / elapsed, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": engine.n_steps,
        "seconds": round(elapsed, 2),
        "total_tok_s": round((generated + sum(lengths)) / elapsed, 1),
        "higher_is_better": True,
        "dtype": args.dtype,
        "data": "synthetic: random weights N(0, 0.02), random token ids, prompt lengths uniform in [128, 4096]",
        "config": {
            "model": shape_name,
            "requests": args.serve,
            "prompt_tokens": sum(lengths),
            "new_tokens_each": args.new,
            "max_batch": gen_args.max_batch,
            "max_prefill": gen_args.max_prefill,
            "page_size": args.page,
            "n_layers": len(model.blocks),
        },
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
