"""The generation engine end to end without a GPU (kernels replaced by torch
stand-ins): greedy generation against the plain implementation, a cache so small
that requests are preempted, per-request random streams, the command line."""

import json
import queue

import pytest

from helpers import configs, cpu_ops, generation, models, traces


def _engine(folder, monkeypatch, **kw):
    from cwm_amd.engine import Engine, GenArgs

    cpu_ops.install(monkeypatch)
    args = GenArgs(**{"use_sampling": False, "max_batch": 4, "max_seq": 512, "cache_block": 4, "max_prefill": 16, **kw})
    return Engine.from_folder(folder, args, dtype="float32", device="cpu")


def test_greedy_generation_matches_plain(tmp_path, monkeypatch):
    folder = models.make_folder(tmp_path, "tiny_b", seed=2, dtype="float32")
    vocab = configs.get("tiny_b")["vocab_size"]
    prompts = [traces.random_tokens(i, n, vocab) for i, n in enumerate([9, 40, 23])]
    engine = _engine(folder, monkeypatch)
    got = engine.generate_tokens(prompts, max_gen=10)
    import torch
    for p, g in zip(prompts, got):
        assert g == generation.plain_greedy(folder, p, 10, dtype=torch.float32)
    engine.manager.check()
    assert engine.manager.live_requests() == []


def test_tiny_cache_gives_the_same_tokens(tmp_path, monkeypatch):
    folder = models.make_folder(tmp_path, "tiny_a", seed=2, dtype="float32")
    vocab = configs.get("tiny_a")["vocab_size"]
    prompts = [traces.random_tokens(10 + i, n, vocab) for i, n in enumerate([12, 25, 7, 18])]
    big = _engine(folder, monkeypatch).generate_tokens(prompts, max_gen=12)
    small_engine = _engine(folder, monkeypatch, max_seq=64)
    small = small_engine.generate_tokens(prompts, max_gen=12)
    assert any(e.startswith("preempt") for e in small_engine.scheduler.events)
    assert small == big


def test_sampled_tokens_do_not_depend_on_the_batch(tmp_path, monkeypatch):
    from cwm_amd.engine import Packet

    folder = models.make_folder(tmp_path, "tiny_a", seed=2, dtype="float32")
    vocab = configs.get("tiny_a")["vocab_size"]
    prompts = {f"p{i}": traces.random_tokens(20 + i, n, vocab) for i, n in enumerate([6, 14, 9])}

    def run(ids):
        engine = _engine(folder, monkeypatch, use_sampling=True, temperature=0.8, top_p=0.9)
        q = queue.Queue()
        for rid in ids:
            q.put(Packet(thread_id=rid, tokens=prompts[rid], max_gen=8))
        q.put(None)
        return {p.thread_id: p.tokens for p in engine.generate(q) if p is not None}

    together = run(["p0", "p1", "p2"])
    alone = run(["p1"])
    assert together["p1"] == alone["p1"]
    assert len(set(map(tuple, together.values()))) == 3


def test_stop_tokens_and_packets(tmp_path, monkeypatch):
    from cwm_amd.engine import Engine, GenArgs, Packet

    folder = models.make_folder(tmp_path, "tiny_a", seed=2, dtype="float32")
    vocab = configs.get("tiny_a")["vocab_size"]
    prompt = traces.random_tokens(5, 11, vocab)
    free = _engine(folder, monkeypatch).generate_tokens([prompt], max_gen=10)[0]
    cpu_ops.install(monkeypatch)
    engine = Engine.from_folder(folder, GenArgs(use_sampling=False, max_batch=2, max_seq=256, cache_block=8, logprobs=True),
                                dtype="float32", device="cpu", stop_tokens=[free[3]])
    q = queue.Queue()
    q.put(Packet(thread_id="x", tokens=prompt, max_gen=10))
    q.put(None)
    out = [p for p in engine.generate(q) if p is not None]
    assert len(out) == 1 and out[0].thread_id == "x"
    cut = free.index(free[3])
    assert out[0].tokens == free[: cut + 1] and out[0].finish_reason == "stop"
    assert len(out[0].logprobs) == len(out[0].tokens) and all(lp <= 0 for lp in out[0].logprobs)
    with pytest.raises(ValueError, match="tokenizer"):
        engine.submit(Packet(thread_id="y", tokens=[1], stop_str="END"))
    with pytest.raises(ValueError, match="vocabulary"):
        engine.submit(Packet(thread_id="z", tokens=[vocab]))


def test_command_line(tmp_path, monkeypatch, capsys):
    from cwm_amd import generate

    cpu_ops.install(monkeypatch)
    folder = models.make_folder(tmp_path, "tiny_a", seed=2, dtype="float32")
    vocab = configs.get("tiny_a")["vocab_size"]
    prompts = [traces.random_tokens(30 + i, n, vocab) for i, n in enumerate([5, 9])]
    path = tmp_path / "prompts.jsonl"
    path.write_text("".join(json.dumps({"id": f"q{i}", "tokens": p, "max_gen": 6}) + "\n" for i, p in enumerate(prompts)))
    rc = generate.main([f"checkpoint_dir={folder}", f"prompts={path}", "dtype=float32", "device=cpu", "gen_args.use_sampling=false",
                        "gen_args.max_seq=256", "gen_args.cache_block=8", "gen_args.max_batch=2"])
    assert rc == 0
    lines = [json.loads(l) for l in capsys.readouterr().out.strip().splitlines()]
    got = {rec["id"]: rec["tokens"] for rec in lines}
    import torch
    for i, p in enumerate(prompts):
        assert got[f"q{i}"] == generation.plain_greedy(folder, p, 6, dtype=torch.float32)


def test_prompt_logprobs(tmp_path, monkeypatch):
    """With prompt_logprobs the packet's logprobs start with log P(prompt[p+1] | prompt[:p+1])
    for every prompt position, also when the prompt is cut into portions and when the
    request is preempted and recomputed."""
    import torch
    from cwm_amd.engine import Packet
    from plain import llama3_plain

    folder = models.make_folder(tmp_path, "tiny_b", seed=2, dtype="float32")
    config, weights = models.read_folder(folder)
    vocab = configs.get("tiny_b")["vocab_size"]
    prompts = {f"p{i}": traces.random_tokens(50 + i, n, vocab) for i, n in enumerate([21, 9, 30])}
    for max_seq in (512, 48):
        engine = _engine(folder, monkeypatch, prompt_logprobs=True, max_prefill=8, max_seq=max_seq, max_batch=3)
        engine.scheduler.headroom = 0  # requests join as soon as their prompts fit, and outgrow the small cache together
        q = queue.Queue()
        for rid, toks in prompts.items():
            q.put(Packet(thread_id=rid, tokens=toks, max_gen=12))
        q.put(None)
        out = {p.thread_id: p for p in engine.generate(q) if p is not None}
        if max_seq == 48:
            assert any(e.startswith("preempt") for e in engine.scheduler.events)
        for rid, toks in prompts.items():
            pkt = out[rid]
            full = toks + pkt.tokens
            logp = torch.log_softmax(llama3_plain.forward_from_config(weights, config, full, dtype=torch.float64), -1)
            want = [float(logp[p, full[p + 1]]) for p in range(len(full) - 1)]
            assert len(pkt.logprobs) == len(toks) - 1 + len(pkt.tokens)
            assert max(abs(a - b) for a, b in zip(pkt.logprobs, want)) < 1e-3


def test_pool_sizes(tmp_path, monkeypatch):
    """Pages per layer group: from max_seq, or from free memory when max_seq is negative;
    a window group never gets more than its requests can use."""
    import torch
    from cwm_amd.engine import GenArgs, load_model, pool_sizes

    cpu_ops.install(monkeypatch)
    folder = models.make_folder(tmp_path, "tiny_b", seed=2, dtype="bfloat16")
    model, _ = load_model(folder, "bfloat16", "cpu")
    sizes = pool_sizes(model, GenArgs(max_seq=4096, cache_block=16, max_batch=2, max_prefill=64), torch.device("cpu"))
    assert sizes[None] == 256
    assert sizes[8] == 2 * ((8 - 1 + 64 + 15) // 16 + 2)  # window 8: far fewer pages than the keep-all group
    small = pool_sizes(model, GenArgs(max_seq=64, cache_block=16, max_batch=2, max_prefill=64), torch.device("cpu"))
    assert small == {None: 4, 8: 4}
    # from free memory: 1 GB free, 0.5 GB reserve
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda device=None: (10 ** 9, 2 * 10 ** 9))
    auto = pool_sizes(model, GenArgs(max_seq=-1, cache_block=16, max_batch=2, max_prefill=64, prefill_gb=0.5), torch.device("cuda:0"))
    per_page_global = 1 * 2 * 1 * 32 * 16 * 2  # one global layer: k and v, 1 head of 32, 16 tokens, 2 bytes
    per_page_local = 3 * per_page_global
    assert auto[8] == sizes[8]
    assert auto[None] == (int(0.9 * 0.5e9) - auto[8] * per_page_local) // per_page_global
    with pytest.raises(ValueError):
        pool_sizes(model, GenArgs(max_seq=-1), torch.device("cpu"))


def _model_without_weights(config):
    import torch
    from cwm_amd.config import parse_config
    from cwm_amd.models import Model
    from cwm_amd.parts import Runtime

    arch, typed = parse_config(config)
    model = Model(arch.build_plan(typed))
    model.runtime = Runtime(torch.device("cpu"), torch.bfloat16)
    return model


CWM_32B_SHAPE = {
    "architecture": "llama3_dense", "dim": 6144, "n_layers": 64, "n_heads": 48, "n_kv_heads": 8, "head_dim": 128,
    "vocab_size": 128256, "ffn_dim_multiplier": 1.3125, "multiple_of": 256, "norm_eps": 1e-5, "pos_embed_impl": "scaled_rope",
    "rope_theta": 1000000.0, "scaled_rope": {"scale_factor": 16, "old_context_len": 8192, "low_freq_factor": 1, "high_freq_factor": 4},
    "window_attn": {"window_pattern": 4, "local_window": 8192, "global_last_layer": True}, "max_seq_len": 131072,
}


@pytest.mark.parametrize("max_batch", [128, 256])
def test_default_options_size_the_pools_of_the_32b_shape(max_batch):
    """max_seq = -1 with the reference's default options at the CWM-32B shape on a 288 GB
    device: both pools fit into what is free beside 65 GB of weights, neither is reserved for the
    worst case of max_batch requests, and the split follows the expected request."""
    import torch
    from cwm_amd.engine import GenArgs, pool_sizes

    model = _model_without_weights(CWM_32B_SHAPE)
    free = int(288e9 - 65.2e9)
    budget = 0.9 * (free - 2e9)
    page_bytes = 2 * 8 * 128 * 256 * 2  # keys and values of one layer's page of 256 tokens
    n_global = sum(1 for spec in model.cache_specs if spec.window is None)
    n_local = len(model.cache_specs) - n_global
    assert (n_global, n_local) == (17, 47)  # cwm/model/transformer.py:79-85 with pattern 4 and a global last layer

    def bytes_of(sizes):
        return sizes[None] * n_global * page_bytes + sizes[8192] * n_local * page_bytes

    # the context the configuration names (131,072): a request needs 513 pages of the keep-all
    # group and 49 of the window group (8,191 + 4,096 tokens)
    sizes = pool_sizes(model, GenArgs(max_batch=max_batch), torch.device("cuda:0"), free_bytes=free)
    assert 0.97 * budget <= bytes_of(sizes) <= budget
    assert abs(sizes[None] / sizes[8192] - 513 / 49) < 0.1
    assert sizes[None] * 256 >= 8 * 131072  # several requests of full length fit
    # short requests expected: as many tokens in either group
    short = pool_sizes(model, GenArgs(max_batch=max_batch, expected_seq=2048), torch.device("cuda:0"), free_bytes=free)
    assert 0.97 * budget <= bytes_of(short) <= budget
    assert abs(short[None] - short[8192]) <= 1
    assert short[8192] < max_batch * 50  # not the worst case of every request
    # a window group is never larger than max_batch requests can fill; the keep-all group gets the rest
    few = pool_sizes(model, GenArgs(max_batch=4, expected_seq=2048), torch.device("cuda:0"), free_bytes=free)
    assert few[8192] == 4 * ((8191 + 4096 + 255) // 256 + 2)
    assert 0.97 * budget <= bytes_of(few) <= budget
    # too little memory is an error that says so
    with pytest.raises(MemoryError, match="no room"):
        pool_sizes(model, GenArgs(), torch.device("cuda:0"), free_bytes=int(2.1e9))


def test_metrics_log_and_profile_window(tmp_path, monkeypatch):
    """FG_METRICS names a file that receives the scheduler's events as JSON lines (the
    reference's kinds `nactive`, `yield`, `unpark`, and `preempt`); request_profile() traces
    the next FG_PROFILE_ITERS steps and leaves a Chrome trace in FG_PROFILE_DIR."""
    import gzip

    path = tmp_path / "metrics.jsonl"
    monkeypatch.setenv("FG_METRICS", str(path))
    monkeypatch.setenv("FG_PROFILE_ITERS", "2")
    monkeypatch.setenv("FG_PROFILE_DIR", str(tmp_path))
    folder = models.make_folder(tmp_path, "tiny_a", seed=2, dtype="float32")
    vocab = configs.get("tiny_a")["vocab_size"]
    prompts = [traces.random_tokens(10 + i, n, vocab) for i, n in enumerate([12, 25, 7, 18])]
    engine = _engine(folder, monkeypatch, max_seq=64)
    engine.scheduler.headroom = 0
    engine.request_profile()
    got = engine.generate_tokens(prompts, max_gen=12)
    engine.metrics.close()
    records = [json.loads(line) for line in path.read_text().splitlines()]
    kinds = [r["kind"] for r in records]
    assert kinds.count("yield") == len(prompts)
    assert sorted(r["tokens"] for r in records if r["kind"] == "yield") == sorted(len(g) for g in got)
    assert "nactive" in kinds and all("timestamp" in r for r in records)
    first = next(r for r in records if r["kind"] == "nactive")
    assert first["lanes"] >= 1 and len(first["free_pages"]) == len(engine.manager.groups)
    assert kinds.count("preempt") == engine.scheduler.n_preemptions >= 1
    assert kinds.count("unpark") >= 1
    # the trace of two steps
    assert engine.last_profile_path is not None and engine.last_profile_path.startswith(str(tmp_path))
    with gzip.open(engine.last_profile_path, "rt") as fh:
        trace = json.load(fh)
    assert trace["traceEvents"]
    # without the variable nothing is written
    monkeypatch.delenv("FG_METRICS")
    other = _engine(folder, monkeypatch)
    other.generate_tokens(prompts[:1], max_gen=2)
    assert len(path.read_text().splitlines()) == len(records)


def test_decode_bursts_give_the_same_tokens_as_single_steps(tmp_path, monkeypatch):
    """sync_freq decode steps run back to back, each fed by the tokens the one before sampled on
    the device; the host sees tokens once a burst.  Same tokens as one step at a time, greedy and
    sampled; a stop token inside a burst ends its request there and is kept; no request outgrows
    its max_gen; a burst is not started when its pages are not free."""
    from cwm_amd.engine import Engine, GenArgs, Packet

    folder = models.make_folder(tmp_path, "tiny_b", seed=2, dtype="float32")
    vocab = configs.get("tiny_b")["vocab_size"]
    prompts = {f"p{i}": traces.random_tokens(70 + i, n, vocab) for i, n in enumerate([9, 30, 17])}

    def run(sync_freq, stop=(), max_seq=1024, **kw):
        cpu_ops.install(monkeypatch)
        args = GenArgs(**{"use_sampling": True, "temperature": 0.8, "top_p": 0.9, "max_batch": 4, "max_seq": max_seq,
                          "cache_block": 4, "max_prefill": 16, "sync_freq": sync_freq, "logprobs": True, **kw})
        engine = Engine.from_folder(folder, args, dtype="float32", device="cpu", stop_tokens=stop, seed=5)
        q = queue.Queue()
        for i, (rid, toks) in enumerate(prompts.items()):
            q.put(Packet(thread_id=rid, tokens=toks, max_gen=[23, 7, 12][i], temperature=0.0 if i == 2 else None))
        q.put(None)
        bursts = []
        out = {}
        for pkt in engine.generate(q):
            bursts.append(engine.last_step_burst)
            if pkt is not None:
                out[pkt.thread_id] = pkt
        engine.manager.check()
        assert engine.manager.live_requests() == []
        return out, bursts, engine

    single, bursts1, _ = run(1)
    assert set(bursts1) == {1}
    many, bursts10, engine = run(10)
    assert max(bursts10) > 1 and engine.n_steps > engine.n_iterations
    for rid in prompts:
        assert many[rid].tokens == single[rid].tokens
        assert len(many[rid].tokens) == {"p0": 23, "p1": 7, "p2": 12}[rid]
        assert max(abs(a - b) for a, b in zip(many[rid].logprobs, single[rid].logprobs)) < 1e-5
        assert many[rid].sample_logprobs == pytest.approx(single[rid].sample_logprobs, abs=1e-5)
    # a stop token in the middle of p0's tokens: the burst that contains it ends p0 there
    stop = single["p0"].tokens[11]
    cut = single["p0"].tokens.index(stop)
    stopped, _, _ = run(10, stop=[stop])
    assert stopped["p0"].tokens == single["p0"].tokens[: cut + 1] and stopped["p0"].finish_reason == "stop"
    for rid in ("p1", "p2"):
        want = single[rid].tokens
        if stop in want:
            want = want[: want.index(stop) + 1]
        assert stopped[rid].tokens == want
    # a cache with hardly a page to spare: bursts that do not fit are not started, tokens stay the same
    tight, bursts_tight, _ = run(10, max_seq=96)
    for rid in prompts:
        assert tight[rid].tokens == single[rid].tokens


def test_a_dropped_engine_is_freed_at_once(tmp_path, monkeypatch):
    """An engine registers callbacks with its own scheduler; they must not keep it in a cycle of references,
    or its cache (and its graphs) would stay on the device until the collector finds them, and a graph must
    not be destroyed while another is captured."""
    import gc
    import weakref

    folder = models.make_folder(tmp_path, "tiny_a", seed=2, dtype="float32")
    gc.collect()
    gc.disable()
    try:
        engine = _engine(folder, monkeypatch)
        engine.generate_tokens([[1, 2, 3]], max_gen=3)
        assert any(e.startswith("finish") for e in engine.scheduler.events)  # the callback is alive while the engine is
        gone = weakref.ref(engine)
        cache = weakref.ref(next(iter(engine.storage.paged.values())))
        del engine
        assert gone() is None and cache() is None
    finally:
        gc.enable()


def test_profile_window_by_signal(tmp_path, monkeypatch):
    """SIGUSR2 asks for a profile window from outside the process, as the reference's handler does
    (cwm/fastgen/generate.py:159-169,405-406); a handler that someone else has set is left alone."""
    import os
    import signal

    monkeypatch.setenv("FG_PROFILE_ITERS", "1")
    monkeypatch.setenv("FG_PROFILE_DIR", str(tmp_path))
    folder = models.make_folder(tmp_path, "tiny_a", seed=2, dtype="float32")
    vocab = configs.get("tiny_a")["vocab_size"]
    engine = _engine(folder, monkeypatch)
    saved = signal.getsignal(signal.SIGUSR2)
    try:
        signal.signal(signal.SIGUSR2, signal.SIG_DFL)
        assert engine.install_profile_signal() is True
        assert engine._profile_state == "inactive"
        os.kill(os.getpid(), signal.SIGUSR2)
        for _ in range(100):  # the handler runs between bytecodes of the main thread
            if engine._profile_state == "requested":
                break
        assert engine._profile_state == "requested"
        engine.generate_tokens([traces.random_tokens(1, 9, vocab)], max_gen=3)
        assert engine.last_profile_path is not None and os.path.exists(engine.last_profile_path)
        # a second engine finds the first one's handler set and leaves it
        assert _engine(folder, monkeypatch).install_profile_signal() is False
        # the handler does not keep its engine alive, and outlives it harmlessly
        del engine
        os.kill(os.getpid(), signal.SIGUSR2)
    finally:
        signal.signal(signal.SIGUSR2, saved)
