"""Generation through the entry points on the GPU: greedy tokens against the plain
implementation (float32), a cache so small that requests are preempted, the command
line as a child process, and a toy mixer with state of its own that is registered,
built and stepped without touching the framework's files."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from helpers import compare as cmp, configs, generation, models, traces

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("name", ["tiny_a", "tiny_b", "tiny_c", "tiny_d"])
def test_greedy_generation_float32(tmp_path, name):
    from cwm_amd.engine import Engine, GenArgs

    folder = models.make_folder(tmp_path, name, seed=8, dtype="float32")
    vocab = configs.get(name)["vocab_size"]
    prompts = [traces.random_tokens(i, n, vocab) for i, n in enumerate([5, 17, 33, 64])]
    args = GenArgs(use_sampling=False, max_batch=4, max_seq=2048, cache_block=16, max_prefill=48)
    engine = Engine.from_folder(folder, args, dtype="float32")
    got = engine.generate_tokens(prompts, max_gen=16)
    for p, g in zip(prompts, got):
        assert g == generation.plain_greedy(folder, p, 16)
    # a cache that holds barely more than the longest sequence: preemption and recomputation
    small = Engine.from_folder(folder, GenArgs(use_sampling=False, max_batch=4, max_seq=96, cache_block=4, max_prefill=48), dtype="float32")
    again = small.generate_tokens(prompts, max_gen=16)
    assert any(e.startswith("preempt") for e in small.scheduler.events)
    assert again == got


def _plain_sampled(folder, prompt, n_new, temperature, top_p, stream):
    """Generation with the plain implementation: softmax(logits / T), the nucleus, and the draw
    by inverse CDF with the request's own uniform numbers."""
    from plain import llama3_plain

    config, weights = models.read_folder(folder)
    toks, out = list(prompt), []
    for _ in range(n_new):
        logits = llama3_plain.forward_from_config(weights, config, toks, dtype=torch.float64)[-1]
        if temperature > 0:
            probs = llama3_plain.sampling_probabilities(logits, temperature, top_p)
            nxt = llama3_plain.sample_inverse_cdf(probs, stream.next_uniform())
        else:
            nxt = llama3_plain.greedy(logits)
        toks.append(nxt)
        out.append(nxt)
    return out


def test_sampled_generation_equals_the_plain_draw(tmp_path):
    """Prompts of 9, 40 and 100 tokens in portions of 16 beside 24 decode steps at temperature
    0.7 and top-p 0.9, in float32: every token equals the plain implementation's draw from the
    plain logits with the request's own stream of uniform numbers, for each request alone and
    for all in one batch; one request overrides temperature, top-p and seed in its packet,
    another is greedy by its packet's temperature 0."""
    import queue

    from cwm_amd.engine import Engine, GenArgs, Packet
    from cwm_amd.sampling.sampler import RequestStream

    folder = models.make_folder(tmp_path, "tiny_b", seed=8, dtype="float32")
    vocab = configs.get("tiny_b")["vocab_size"]
    prompts = {f"p{i}": traces.random_tokens(40 + i, n, vocab) for i, n in enumerate([9, 40, 100, 23])}
    args = GenArgs(use_sampling=True, temperature=0.7, top_p=0.9, max_batch=4, max_seq=2048, cache_block=16, max_prefill=16,
                   handover_frequency=3)
    overrides = {"p1": dict(temperature=1.3, top_p=0.6, seed=777), "p3": dict(temperature=0.0)}
    engine_seed = 3

    def packet(rid):
        return Packet(thread_id=rid, tokens=prompts[rid], max_gen=24, **overrides.get(rid, {}))

    want = {}
    for rid, prompt in prompts.items():
        o = overrides.get(rid, {})
        stream = RequestStream(engine_seed, o.get("seed", rid))
        want[rid] = _plain_sampled(folder, prompt, 24, o.get("temperature", 0.7), o.get("top_p", 0.9), stream)
    assert want["p0"] != _plain_sampled(folder, prompts["p0"], 24, 0.7, 0.9, RequestStream(engine_seed + 1, "p0"))

    def run(rids):
        engine = Engine.from_folder(folder, args, dtype="float32", seed=engine_seed)
        q = queue.Queue()
        for rid in rids:
            q.put(packet(rid))
        q.put(None)
        out, handovers = {}, 0
        for pkt in engine.generate(q):
            if pkt is None:
                handovers += 1
            else:
                out[pkt.thread_id] = pkt.tokens
        assert handovers == engine.n_iterations // 3  # control is handed back every third iteration
        assert engine.n_steps > engine.n_iterations  # decode steps ran in bursts without a host sync between them
        return out

    together = run(list(prompts))
    for rid in prompts:
        assert together[rid] == want[rid], f"{rid} in a batch: engine {together[rid]} != plain draw {want[rid]}"
        assert run([rid])[rid] == want[rid], f"{rid} alone"


@pytest.mark.parametrize("name", ["tiny_b", "tiny_d"])
@pytest.mark.parametrize("sampling", [False, True])
def test_bfloat16_generation_through_the_engine_against_the_plain_logits(tmp_path, name, sampling):
    """bfloat16 through the whole engine (scheduler, portions of 24 tokens, bursts of decode steps fed on the
    device, decode steps replayed from graphs, six requests over four places so that they come and go): the
    log-probabilities that the engine returns for the prompt's and for its own generated tokens are those of
    the plain implementation on prompt + generated tokens, within what bfloat16 rounding costs there (a logit
    error of e moves a log-probability by at most 2e), and every greedy token lies that near the top."""
    import queue

    from cwm_amd.engine import Engine, GenArgs, Packet

    folder = models.make_folder(tmp_path, name, seed=8, dtype="bfloat16")
    vocab = configs.get(name)["vocab_size"]
    prompts = {i: traces.random_tokens(300 + i, n, vocab) for i, n in enumerate([5, 33, 64, 90, 12, 41])}
    args = GenArgs(use_sampling=sampling, temperature=0.8, top_p=0.9, max_batch=4, max_seq=4096, cache_block=8, max_prefill=24,
                   logprobs=True, prompt_logprobs=True, num_cuda_graphs=16, sync_freq=5)
    engine = Engine.from_folder(folder, args, dtype="bfloat16")
    q = queue.Queue()
    for rid, prompt in prompts.items():
        q.put(Packet(thread_id=rid, tokens=list(prompt), max_gen=40))
    q.put(None)
    packets = {pkt.thread_id: pkt for pkt in engine.generate(q) if pkt is not None}
    assert engine.runner.n_replays > 0 and engine.n_steps > engine.n_iterations  # graphs and bursts were in it
    for rid, prompt in prompts.items():
        pkt = packets[rid]
        toks = list(prompt) + list(pkt.tokens)
        assert len(pkt.tokens) == 40 and len(pkt.logprobs) == len(toks) - 1
        want = cmp.expected(folder, {"x": toks}, "bfloat16")["x"]
        exact = torch.log_softmax(torch.from_numpy(want.exact).double(), -1)
        limit = 2 * cmp.BF16_MAX_RATIO * want.max
        for place in range(len(toks) - 1):  # the logits after token `place` score token `place + 1`
            plain_lp = float(exact[place, toks[place + 1]])
            assert abs(pkt.logprobs[place] - plain_lp) <= limit, (
                f"{name} request {rid}: log-probability of token {place + 1} is {pkt.logprobs[place]:.5f}, plain {plain_lp:.5f}, limit {limit:.2e}")
            if not sampling and place >= len(prompt) - 1:
                row = want.exact[place]
                assert row[toks[place + 1]] >= row.max() - limit, f"{name} request {rid}: generated token {place + 1 - len(prompt)} is not near the top"


def test_a_request_without_max_gen_runs_until_the_cache_is_full(tmp_path):
    """max_gen None in the options and in the packet: the request's longest length is the cache's
    (cwm/fastgen/generate.py:91-96), and it ends with reason "length" there."""
    from cwm_amd.engine import Engine, GenArgs

    folder = models.make_folder(tmp_path, "tiny_a", seed=8, dtype="float32")
    vocab = configs.get("tiny_a")["vocab_size"]
    prompt = traces.random_tokens(5, 10, vocab)
    engine = Engine.from_folder(folder, GenArgs(use_sampling=False, max_batch=2, max_seq=64, cache_block=16, max_gen=None), dtype="float32")
    got = engine.generate_tokens([prompt])[0]
    assert len(prompt) + len(got) == 64
    assert got == generation.plain_greedy(folder, prompt, 54)


def test_command_line_child_process(tmp_path):
    folder = models.make_folder(tmp_path, "tiny_a", seed=8, dtype="float32")
    vocab = configs.get("tiny_a")["vocab_size"]
    prompts = [traces.random_tokens(60 + i, n, vocab) for i, n in enumerate([6, 21])]
    path = tmp_path / "prompts.jsonl"
    path.write_text("".join(json.dumps({"id": i, "tokens": p}) + "\n" for i, p in enumerate(prompts)))
    cmd = [sys.executable, "-m", "cwm_amd.generate", f"checkpoint_dir={folder}", f"prompts={path}", "dtype=float32",
           "gen_args.use_sampling=false", "gen_args.max_gen=9", "gen_args.max_seq=512", "gen_args.cache_block=16", "gen_args.max_batch=4"]
    res = subprocess.run(cmd, cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr
    got = {rec["id"]: rec["tokens"] for rec in map(json.loads, res.stdout.strip().splitlines())}
    for i, p in enumerate(prompts):
        assert got[i] == generation.plain_greedy(folder, p, 9)


def test_trace_run_program(tmp_path):
    """bin/trace_run as a child process: steps on standard input, `done` lines on
    standard output, logits files in --out."""
    folder = models.make_folder(tmp_path, "tiny_b", seed=8, dtype="bfloat16")
    vocab = configs.get("tiny_b")["vocab_size"]
    requests = {f"r{i}": traces.random_tokens(70 + i, n, vocab) for i, n in enumerate([40, 75, 33])}
    steps = traces.mixed(requests)
    for dtype in ("float32", "bfloat16"):
        out = tmp_path / f"out_{dtype}"
        cmd = [os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", str(out),
               "--max-tokens", str(traces.max_live_tokens(steps))]
        res = subprocess.run(cmd, input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=300)
        assert res.returncode == 0, res.stderr
        assert [l for l in res.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
        outputs = {}
        for s in steps:
            n_want = sum(len(e["want"]) for e in s["entries"])
            f = out / f"{s['step']}.f32"
            if n_want:
                outputs[s["step"]] = np.fromfile(f, dtype="<f4").reshape(n_want, vocab)
            else:
                assert not f.exists()
        got = traces.gather(steps, outputs, {k: len(v) for k, v in requests.items()}, vocab)
        want = cmp.expected(folder, requests, dtype)
        for rid in requests:
            cmp.check(got[rid], want[rid], dtype, f"trace_run {dtype} {rid}")


# ---- a toy mixer with state of its own -------------------------------------------------- #
def test_toy_mixer_with_state_registers_builds_and_steps(tmp_path):
    """A mixer that keeps a running sum of its inputs per request (fixed-size state,
    no pages) is registered under a new name, a toy architecture uses it in one
    layer beside attention in another, and the model is stepped in portions: the
    result must not depend on the cut.  Nothing in the framework's files changes."""
    from dataclasses import dataclass

    from cwm_amd.cache import CacheManager, CacheStorage
    from cwm_amd.config import ARCHITECTURES, register_architecture
    from cwm_amd.engine import ModelRunner, Portion
    from cwm_amd.models import Model
    from cwm_amd.parts import (LayerCall, LayerPlan, Mixer, ModelPlan, PartChoice, Runtime, StateSpec, TensorSpec, register_part)
    from cwm_amd.parts.base import MIXERS
    from cwm_amd.weights import random_tensors

    class RunningSumMixer(Mixer):
        """y_t = scale * sum_{s <= t} x_s over the request's tokens so far."""

        def __init__(self, dim):
            self.dim = dim

        def cache_spec(self):
            return StateSpec((self.dim,), torch.float32)

        def tensor_specs(self):
            return {"scale": TensorSpec((self.dim,), init="norm")}

        def bind(self, tensors, runtime):
            super().bind(tensors, runtime)
            self.scale = tensors["scale"].float()

        def forward(self, x, batch, cache, write_cache=True):
            out = torch.empty_like(x)
            start = 0
            for b, n in enumerate(batch.q_lens):
                slot = int(batch.state_slots[b])
                run = cache.state[slot] + torch.cumsum(x[start : start + n].float(), 0)
                out[start : start + n] = (run * self.scale).to(x.dtype)
                cache.state[slot] = run[-1]
                start += n
            return out

    @dataclass(frozen=True)
    class ToyConfig:
        architecture: str
        dim: int
        vocab_size: int

    def toy_plan(cfg):
        norm = PartChoice("rmsnorm", {"dim": cfg.dim, "eps": 1e-5})
        ff = PartChoice("swiglu", {"dim": cfg.dim, "hidden_dim": 2 * cfg.dim})
        names = {"norm1": "n1.", "mixer": "mix.", "norm2": "n2.", "feed_forward": "ff."}
        attn = PartChoice("paged_attention", {"dim": cfg.dim, "n_heads": 2, "n_kv_heads": 1, "head_dim": 16, "scale": 0.25,
                                              "window": 5, "position_encoding": PartChoice("rotary", {"head_dim": 16, "theta": 100.0})})
        layers = [
            LayerPlan.standard("l0.", "pre_norm", norm, PartChoice("toy_running_sum", {"dim": cfg.dim}), ff, names),
            LayerPlan.standard("l1.", "pre_norm", norm, attn, ff, names),
        ]
        # the run order names layer 1 twice (shared weights, a cache each) and ends with the toy layer again
        order = [LayerCall(0), LayerCall(1), LayerCall(1), LayerCall(0)]
        return ModelPlan.standard(cfg.vocab_size, cfg.dim, "emb", layers, order, norm, "final", "head")

    register_part("mixer", "toy_running_sum", RunningSumMixer)
    register_architecture("toy_state_model", ToyConfig, toy_plan)
    try:
        from cwm_amd.config import parse_config

        arch, cfg = parse_config({"architecture": "toy_state_model", "dim": 48, "vocab_size": 61})
        model = Model(arch.build_plan(cfg))
        assert [type(s).__name__ for s in model.cache_specs] == ["StateSpec", "PagedKVSpec", "PagedKVSpec", "StateSpec"]
        runtime = Runtime(torch.device("cuda:0"), torch.float32)
        tensors = {k: v.to("cuda:0") for k, v in random_tensors(model.tensor_specs(), seed=1, std=0.2, norm_init="uniform", dtype=torch.float32).items()}
        model.bind(tensors, runtime)

        def run(cuts):
            manager = CacheManager(model.cache_specs, 4, 64, 4)
            storage = CacheStorage(manager, runtime.device, runtime.act_dtype)
            runner = ModelRunner(model, manager, storage)
            toks = {"a": traces.random_tokens(1, 23, 61), "b": traces.random_tokens(2, 17, 61)}
            got = {k: [] for k in toks}
            cur = {k: 0 for k in toks}
            for rid in toks:
                runner.admit(rid)
            for step in cuts:
                portions = []
                for rid, n in step.items():
                    n = min(n, len(toks[rid]) - cur[rid])
                    if n <= 0:
                        continue
                    assert manager.extend(rid, n)
                    portions.append(Portion(rid, toks[rid][cur[rid] : cur[rid] + n], list(range(n))))
                    cur[rid] += n
                if not portions:
                    continue
                logits = runner.step(portions).cpu()
                row = 0
                for p in portions:
                    got[p.rid].append(logits[row : row + len(p.tokens)])
                    row += len(p.tokens)
            assert all(cur[k] == len(toks[k]) for k in toks)
            return {k: torch.cat(v) for k, v in got.items()}

        whole = run([{"a": 23}, {"b": 17}])
        cut = run([{"a": 5, "b": 1}, {"a": 1, "b": 7}, {"a": 2}, {"a": 9, "b": 2}, {"b": 3, "a": 6}, {"b": 4}])
        for k in whole:
            assert torch.isfinite(whole[k]).all()
            torch.testing.assert_close(cut[k], whole[k], rtol=1e-4, atol=1e-5)
        # the state matters: another request's logits differ from a fresh run of the same tokens after other input
        assert not torch.allclose(whole["a"][5], whole["a"][4])

        # a state slot that is used again starts at zero: with one slot, "b" after "a" gives what "b" alone gives
        manager = CacheManager(model.cache_specs, 4, 64, 1)
        storage = CacheStorage(manager, runtime.device, runtime.act_dtype)
        runner = ModelRunner(model, manager, storage)
        toks_a, toks_b = traces.random_tokens(1, 23, 61), traces.random_tokens(2, 17, 61)
        slot_a = runner.admit("a")
        assert manager.extend("a", 23)
        runner.step([Portion("a", toks_a, [22])])
        assert all(float(t[slot_a].abs().max()) > 0 for t in storage.state.values())  # it has left its sums there
        runner.release("a")
        slot_b = runner.admit("b")
        assert slot_b == slot_a
        assert manager.extend("b", 17)
        after = runner.step([Portion("b", toks_b, list(range(17)))]).cpu()
        torch.testing.assert_close(after, whole["b"], rtol=1e-4, atol=1e-5)
    finally:
        del MIXERS["toy_running_sum"]
        del ARCHITECTURES["toy_state_model"]


def test_logprobs_of_prompt_and_generated_tokens(tmp_path):
    import queue

    from cwm_amd.engine import Engine, GenArgs, Packet
    from plain import llama3_plain

    folder = models.make_folder(tmp_path, "tiny_c", seed=8, dtype="float32")
    config, weights = models.read_folder(folder)
    vocab = configs.get("tiny_c")["vocab_size"]
    prompts = {f"p{i}": traces.random_tokens(80 + i, n, vocab) for i, n in enumerate([21, 9, 70])}
    args = GenArgs(use_sampling=False, prompt_logprobs=True, max_batch=3, max_seq=1024, cache_block=8, max_prefill=16)
    engine = Engine.from_folder(folder, args, dtype="float32")
    q = queue.Queue()
    for rid, toks in prompts.items():
        q.put(Packet(thread_id=rid, tokens=toks, max_gen=5))
    q.put(None)
    out = {p.thread_id: p for p in engine.generate(q) if p is not None}
    for rid, toks in prompts.items():
        pkt = out[rid]
        full = toks + pkt.tokens
        logp = torch.log_softmax(llama3_plain.forward_from_config(weights, config, full, dtype=torch.float64), -1)
        want = [float(logp[p, full[p + 1]]) for p in range(len(full) - 1)]
        assert len(pkt.logprobs) == len(want)
        assert max(abs(a - b) for a, b in zip(pkt.logprobs, want)) < 1e-3
        assert pkt.sample_logprobs == [0.0] * len(pkt.tokens)  # greedy
