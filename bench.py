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
lengths through the step function, as the headline.  `prefill_ctx32768` is a portion of 4,096 tokens of a
long prompt after 28,672 cached ones (tokens a second, and `_frac` of the matrix peak).  The default run then
makes the baseline's other two shapes: `llama8b_serve64` is 64 requests with prompts of 128 to 4,096 tokens
and 512 new tokens each through the engine's continuous batching (generated tokens a second; `_total` counts
the prompts' tokens too), `llama70b_decode_b8` a decode step of 8 requests at 8,192 tokens of context and
`llama70b_prefill` a 2,048-token prompt, with their fractions of the HBM and of the matrix peak.

Before anything else it measures what the GPU at hand reaches (`cwm_amd/csrc/ceilings.hip`): the rate of
a kernel that only reads, and the rate of the bfloat16 matrix instruction issued from registers.
`roofline.peak_measured` (GB/s, over a 4 GiB buffer; `_100mb` and `_500mb`: windows of that size launch after
launch, as a layer's matrices are read) and `prefill.peak_measured` (TFLOP/s) stand beside the published peaks,
with `frac_measured` the same rates over them.
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


def measure_ceilings(device):
    """What this GPU reaches: the rate of a kernel that only reads (windows of 100 MB and of 500 MB of a 4 GiB
    buffer, launch after launch, and the whole buffer), in GB/s, and of the bfloat16 matrix instruction issued
    from registers, in TFLOP/s.  Each is the best of a few launch shapes."""
    import torch

    from cwm_amd import ops

    out = {}
    buffer = torch.zeros(4 << 30, dtype=torch.uint8, device=device)
    for name, size, launches in (("read_100mb", 100 << 20, 40), ("read_500mb", 500 << 20, 16), ("read_4gb", 4 << 30, 4)):
        out[name] = round(max(ops.measure_read_rate(buffer, size, launches, blocks) for blocks in (512, 4096, 16384) for _ in range(2)), 1)
    del buffer
    torch.cuda.empty_cache()
    out["mfma_bf16"] = round(1e3 * max(ops.measure_mfma_rate(device, blocks, 20000) for blocks in (2048, 4096) for _ in range(2)), 1)
    return out


class ShapeBench:
    """A model of one shape with random weights and the measurements on it."""

    def __init__(self, shape_name, shape, layers, dtype, page, graphs, device):
        import torch

        from cwm_amd.engine import random_model
        from cwm_amd.parts import PagedKVSpec
        from cwm_amd.sampling import Sampler

        self.torch = torch
        self.device = device
        self.shape_name = shape_name
        self.dtype = dtype
        self.page = page
        self.graphs = graphs
        config = dict(shape)
        self.full_layers = shape["n_layers"]
        self.layers = self.full_layers if layers is None else layers
        config["n_layers"] = self.layers
        if "window_attn" in shape:
            config["layer_types"] = layer_kinds(self.layers)
        t0 = time.time()
        self.model, self.typed = random_model(config, seed=0, dtype=dtype, device=device)
        torch.cuda.synchronize()
        print(f"[bench] {shape_name.split(' (')[0]}: {self.layers}-layer model ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
        model = self.model
        self.esize = 2 if dtype == "bf16" else 4
        # what a step reads of the weights, from the model's own list of tensors: everything but the embedding
        # table (of which a step reads one row a token); `matrix_params` are the entries of the matrices, which
        # every token is multiplied with
        self.weight_bytes = 0
        self.matrix_params = 0
        self.head_params = 0
        head_names = model.tensor_names("head")
        embedding_only = model.tensor_names("embedding") - head_names  # tables of which a step reads one row a token
        for name, spec in model.tensor_specs().items():
            count = 1
            for n in spec.shape:
                count *= n
            if name in embedding_only:
                continue
            self.weight_bytes += count * self.esize
            if len(spec.shape) == 2:
                if name in head_names:
                    self.head_params += count
                else:
                    self.matrix_params += count
        self.paged = [spec for spec in model.cache_specs if isinstance(spec, PagedKVSpec)]
        self.windows = sorted({spec.window for spec in self.paged if spec.window is not None})
        self.sampler = Sampler(device)
        self.vocab = self.typed.vocab_size

    def close(self):
        import gc

        del self.model, self.sampler
        gc.collect()
        self.torch.cuda.empty_cache()

    def cache_bytes(self, batch, ctx):
        total = 0
        for spec in self.paged:
            keys = ctx if spec.window is None else min(ctx, spec.window)
            total += batch * keys * spec.bytes_per_token(self.esize)
        return total

    def step_bytes(self, batch, ctx):
        """What a decode step of `batch` requests at `ctx` tokens has to read: every weight once, and their cache."""
        return self.weight_bytes + self.cache_bytes(batch, ctx)

    def prefill_flops(self, n_tokens, offset=0):
        """Flops of a portion of `n_tokens` after `offset` cached tokens whose last token's logits are wanted:
        2 for every matrix entry and token, the causal attention's two products, and the head for one row."""
        attn = 0
        for call, slot in zip(self.model.run_order, self.model.cache_slot):
            spec = self.model.cache_specs[slot] if slot is not None else None
            if spec in self.paged:
                # token p reads min(p + 1, window) keys; 2 products (QK^T and PV) of 2 flops, for every query head
                keys = sum(min(p + 1, spec.window or (p + 1)) for p in range(offset, offset + n_tokens))
                query_heads = getattr(self.model.blocks[call.layer].mixers()[0], "n_heads", spec.n_kv_heads)
                attn += 4 * keys * query_heads * spec.head_dim
        return 2 * n_tokens * self.matrix_params + attn + 2 * self.head_params

    def make_runner(self, batch, ctx, extra, step_tokens=1):
        """A runner whose pools hold `batch` requests of `ctx` + `extra` tokens that grow by at most `step_tokens` a step."""
        from cwm_amd.cache import CacheManager, CacheStorage
        from cwm_amd.engine import ModelRunner

        page = self.page
        pages = {None: batch * ((ctx + extra + page - 1) // page + 1)}
        for w in self.windows:
            pages[w] = batch * ((min(ctx, w - 1 + step_tokens) + extra + 2 * page - 1) // page + 2)
        manager = CacheManager(self.model.cache_specs, page, pages, batch)
        storage = CacheStorage(manager, self.device, self.model.runtime.act_dtype)
        for t in storage.paged.values():
            t.normal_(0.0, 1.0)
        return ModelRunner(self.model, manager, storage, num_graphs=self.graphs, graphs_where_host_bound=True), manager

    def _hold(self, manager, rid, ctx):
        held = 0
        while held < ctx:  # in pieces, so that window groups give pages back as they would have
            n = min(self.page, ctx - held)
            assert manager.extend(rid, n)
            manager.advance(rid, n)
            held += n

    def decode_run(self, batch, ctx, steps, warmup):
        """tokens/s and ms per step of `steps` decode steps of `batch` requests that
        already hold `ctx` tokens each."""
        from cwm_amd.engine import Portion

        torch = self.torch
        runner, manager = self.make_runner(batch, ctx, steps + warmup + 2)
        for b in range(batch):
            runner.admit(b)
            self._hold(manager, b, ctx)
        # as the engine decodes (sync_freq, cwm/fastgen/generate.py:729-809): every step's tokens are sampled on the
        # device and feed the next step from there; they come to the host once in ten steps
        tokens = torch.tensor([(17 * b + 3) % self.vocab for b in range(batch)], dtype=torch.int32, device=self.device)
        params = torch.zeros((3, batch), dtype=torch.float32, device=self.device)
        params[1] = 1.0  # temperature 0 (greedy), top-p 1, uniform numbers 0
        placeholder = [Portion(b, [0], [0]) for b in range(batch)]  # the token ids come from the device

        def run(n_steps, tokens):
            for i in range(n_steps):
                for b in range(batch):
                    assert manager.extend(b, 1)
                logits = runner.step(placeholder, tokens_device=tokens)
                packed = self.sampler.sample_packed(logits, params[0], params[1], params[2])
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

    def prefill_run(self, n_tokens, offset=0):
        """Seconds (the best of three) of one step that brings `n_tokens` of a prompt after `offset` cached tokens."""
        from cwm_amd.engine import Portion

        torch = self.torch
        runner, manager = self.make_runner(1, offset + n_tokens, 8, step_tokens=n_tokens)
        best = None
        for rep in range(3):
            runner.admit(rep)
            self._hold(manager, rep, offset)
            assert manager.extend(rep, n_tokens)
            toks = [(31 * i + 7) % self.vocab for i in range(n_tokens)]
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
    ap.add_argument("--prefill-tokens", type=int, default=2048, help="tokens of the prompt portion that `prefill` times")
    ap.add_argument("--prefill-offset", type=int, default=0, help="tokens already cached before that portion (0: a fresh prompt)")
    ap.add_argument("--no-ceilings", action="store_true", help="do not measure what the GPU reaches (the read rate and the matrix instruction's rate)")
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

    device = torch.device("cuda:0")
    shape_name, shape = SHAPES[args.shape]
    if args.config:
        with open(args.config) as f:
            shape_name, shape = f"the sizes of {os.path.basename(args.config)}", json.load(f)
    ceilings = {} if args.no_ceilings or args.serve else measure_ceilings(device)
    if ceilings:
        print(f"[bench] this GPU reaches: {ceilings}", file=sys.stderr, flush=True)
    bench = ShapeBench(shape_name, shape, args.layers, args.dtype, args.page, args.graphs, device)
    if args.serve:
        print(json.dumps(serve_run(bench, args.serve, args.new)), flush=True)
        return 0
    typed = bench.typed

    def hbm_fractions(read_bytes, ms):
        achieved = read_bytes / (ms * 1e-3) / 1e9
        return achieved, round(achieved / HBM_PEAK_GBS, 4)

    # ---- the timed run ---------------------------------------------------------- #
    tok_s, ms_step = bench.decode_run(args.batch, args.context, args.steps, args.warmup)
    achieved, frac = hbm_fractions(bench.step_bytes(args.batch, args.context), ms_step)
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": frac}
    if ceilings:
        # the rate a kernel that only reads reaches on this GPU over a buffer far larger than its caches
        roofline["peak_measured"] = ceilings["read_4gb"]
        roofline["frac_measured"] = round(achieved / ceilings["read_4gb"], 4)
        roofline["peak_measured_100mb"] = ceilings["read_100mb"]
        roofline["peak_measured_500mb"] = ceilings["read_500mb"]

    n_prefill = args.prefill_tokens
    prefill_s = bench.prefill_run(n_prefill, offset=args.prefill_offset)
    prefill_rate = bench.prefill_flops(n_prefill, offset=args.prefill_offset) / prefill_s
    prefill = {
        "value": round(n_prefill / prefill_s, 1),
        "tokens": n_prefill,
        "ms": round(prefill_s * 1e3, 2),
        "frac": round(prefill_rate / PEAK_FLOPS[args.dtype], 4),
    }
    if args.prefill_offset:
        prefill["offset"] = args.prefill_offset
    if ceilings and args.dtype == "bf16":
        prefill["peak_measured"] = ceilings["mfma_bf16"]  # TFLOP/s of the matrix instruction issued from registers
        prefill["frac_measured"] = round(prefill_rate / (ceilings["mfma_bf16"] * 1e12), 4)

    points = {}
    if not args.no_points:
        for ctx in (8192, 131072):
            if ctx == args.context:
                continue
            free_bytes, _ = torch.cuda.mem_get_info(device)
            if bench.cache_bytes(args.batch, ctx) > 0.9 * free_bytes:  # an all-global shape at 131,072 tokens does not fit beside its weights
                print(f"[bench] no point at context {ctx}: its cache does not fit", file=sys.stderr, flush=True)
                continue
            points[f"decode_b{args.batch}_ctx{ctx}"] = round(bench.decode_run(args.batch, ctx, 10, 6)[0], 1)  # (a capture, if any, falls into the warm-up)
        if (typed.max_seq_len or 0) >= 32768:
            # a portion of 4,096 tokens of a long prompt, after 28,672 cached ones
            seconds = bench.prefill_run(4096, offset=28672)
            points["prefill_ctx32768"] = round(4096 / seconds, 1)
            points["prefill_ctx32768_frac"] = round(bench.prefill_flops(4096, offset=28672) / seconds / PEAK_FLOPS[args.dtype], 4)
        for b in (1, 8, 64):
            tok_s_b, median_ms, n_steps = engine_point(bench.model, b, 1024, 256, args.page, typed.vocab_size)
            points[f"decode_b{b}"] = round(tok_s_b, 1)
            points[f"decode_b{b}_ms"] = round(median_ms, 3)
            points[f"decode_b{b}_frac"] = hbm_fractions(bench.step_bytes(b, 1024 + 128), median_ms)[1]  # the context grows from 1,024 to 1,280 over the run
            points[f"decode_b{b}_steps"] = n_steps
    layers = bench.layers
    full_layers = bench.full_layers
    window = bench.windows[0] if bench.windows else None
    if not args.no_points and args.shape == "cwm32b" and not args.config and args.dtype == "bf16" and args.layers is None:
        # the other two workloads that the baseline names, each on a model of its own shape
        bench.close()
        other = ShapeBench(*SHAPES["llama8b"], None, args.dtype, args.page, args.graphs, device)
        served = serve_run(other, 64, 512)
        points["llama8b_serve64"] = served["value"]  # generated tokens a second, 64 requests, continuous batching
        points["llama8b_serve64_total"] = served["total_tok_s"]
        other.close()
        other = ShapeBench(*SHAPES["llama70b"], None, args.dtype, args.page, args.graphs, device)
        tok_s_70, ms_70 = other.decode_run(8, 8192, 20, 4)
        points["llama70b_decode_b8"] = round(tok_s_70, 1)
        points["llama70b_decode_b8_frac"] = hbm_fractions(other.step_bytes(8, 8192), ms_70)[1]
        seconds = other.prefill_run(2048)
        points["llama70b_prefill"] = round(2048 / seconds, 1)
        points["llama70b_prefill_frac"] = round(other.prefill_flops(2048) / seconds / PEAK_FLOPS[args.dtype], 4)
        other.close()

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
            "n_layers": layers,
            "n_layers_full": full_layers,
            "dim": typed.dim,
            "n_heads": typed.n_heads,
            "n_kv_heads": typed.kv_heads,
            "head_dim": typed.head_size,
            "hidden_dim": typed.ffn_width,
            "vocab_size": typed.vocab_size,
            "local_window": window or 0,
            "page_size": args.page,
            "points_prompt_tokens": 1024,
            "points_new_tokens": 256,
            "prefill_tokens": n_prefill,
            "graphs": args.graphs,
        },
        "prefill": prefill,
        "roofline": roofline,
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


def serve_run(bench, n_requests, new_tokens):
    """`n_requests` requests of mixed prompt lengths (128 to 4,096 random tokens, `new_tokens` new tokens each)
    through `Engine.generate` (continuous batching, temperature 0.7, top-p 0.95); the record of the run with the
    generated and the total tokens a second."""
    import queue
    import random

    import torch

    from cwm_amd.engine import Engine, GenArgs, Packet

    rng = random.Random(0)
    lengths = [rng.randint(128, 4096) for _ in range(n_requests)]
    gen_args = GenArgs(
        use_sampling=True,
        temperature=0.7,
        top_p=0.95,
        max_batch=min(n_requests, 64),
        max_seq=-1,  # the pools take what is free on the device
        expected_seq=4096 + new_tokens,
        cache_block=bench.page,
        max_prefill=4096,
    )
    engine = Engine(gen_args, bench.model)
    requests = queue.Queue()
    for i, n in enumerate(lengths):
        requests.put(Packet(thread_id=i, tokens=[rng.randrange(bench.vocab) for _ in range(n)], max_gen=new_tokens))
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
        "metric": f"generated tok/s ({bench.shape_name.split(' (')[0]}, {n_requests} requests, continuous batching)",
        "value": round(generated / elapsed, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": engine.n_steps,
        "seconds": round(elapsed, 2),
        "total_tok_s": round((generated + sum(lengths)) / elapsed, 1),
        "higher_is_better": True,
        "dtype": bench.dtype,
        "data": "synthetic: random weights N(0, 0.02), random token ids, prompt lengths uniform in [128, 4096]",
        "config": {
            "model": bench.shape_name,
            "requests": n_requests,
            "prompt_tokens": sum(lengths),
            "new_tokens_each": new_tokens,
            "max_batch": gen_args.max_batch,
            "max_prefill": gen_args.max_prefill,
            "page_size": bench.page,
            "n_layers": len(bench.model.blocks),
        },
    }
    del engine
    torch.cuda.empty_cache()
    return line


if __name__ == "__main__":
    sys.exit(main())
