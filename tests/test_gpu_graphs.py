"""Decode steps that are captured as HIP graphs and replayed, against the same steps launched kernel by
kernel and against the plain implementation: through the replay driver (tails decoded one by one, mixed
steps between them, pages given back and used again, sequences that outgrow a capture) and through the
engine (greedy and sampled generation)."""

import numpy as np
import pytest
import torch

from helpers import compare as cmp, configs, models, traces

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("models")
    return {(name, dtype): models.make_folder(root, name, seed=11, dtype=dtype) for name in ("tiny_a", "tiny_b", "tiny_d") for dtype in ("float32", "bfloat16")}


def decode_steps(requests, tail):
    """Everything but the last `tail` tokens of each request in one step, then one token of every request a
    step; the shortest request ends first, so the steps see a falling number of requests."""
    steps = [{"step": 0, "entries": [{"id": rid, "tokens": toks[:-tail], "want": list(range(len(toks) - tail))} for rid, toks in requests.items()], "end": []}]
    done = {rid: len(toks) - tail for rid, toks in requests.items()}
    live = list(requests)
    while live:
        entries = []
        for rid in live:
            entries.append({"id": rid, "tokens": [requests[rid][done[rid]]], "want": [0]})
            done[rid] += 1
        end = [rid for rid in live if done[rid] == len(requests[rid])]
        steps.append({"step": len(steps), "entries": entries, "end": end})
        live = [rid for rid in live if rid not in end]
    return steps


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["tiny_a", "tiny_b", "tiny_d"])
def test_replayed_steps_give_the_logits_of_launched_ones(folders, name, dtype):
    """150 and more single-token steps of up to four requests, across many pages, chunks of keys and (tiny_b,
    tiny_d) the window, with pages that go back to the pool and are poisoned: the logits of every step are
    those of the run without graphs, bit for bit, and those of the plain implementation within the limits;
    a capture serves many steps."""
    from cwm_amd.replay import Replayer

    vocab = configs.get(name)["vocab_size"]
    lengths = [260, 200, 171, 333]
    requests = {f"r{i}": traces.random_tokens(31 * i + 5, n, vocab) for i, n in enumerate(lengths)}
    steps = decode_steps(requests, tail=150)
    max_tokens = traces.max_live_tokens(steps)
    page_size = 32 if name == "tiny_d" else 8
    outputs = {}
    for graphs in (0, 4):
        rep = Replayer(folders[name, dtype], dtype, max_tokens, page_size=page_size, poison_freed_pages=True, num_graphs=graphs)
        outputs[graphs] = traces.run_in_process(rep, steps)
        if graphs:
            assert rep.runner.n_replays > 100 and rep.runner.n_captures <= 24, (rep.runner.n_replays, rep.runner.n_captures)
        assert rep.manager.live_requests() == []
    for step, want in outputs[0].items():
        assert np.array_equal(outputs[4][step], want), f"step {step} differs between the replayed and the launched run"
    got = traces.gather(steps, outputs[4], {k: len(v) for k, v in requests.items()}, vocab)
    want = cmp.expected(folders[name, dtype], requests, dtype)
    for rid in requests:
        cmp.check(got[rid], want[rid], dtype, f"{name} {dtype} graphs {rid}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_steps_between_replays(folders, dtype):
    """Up to four live requests, portions of prompts beside decoded tokens and steps of decoded tokens only
    (which are replayed) in turn, with so few pages that they are used again: the plain implementation's
    logits within the limits, and bit for bit those of the run without graphs."""
    from cwm_amd.replay import Replayer

    name = "tiny_b"
    vocab = configs.get(name)["vocab_size"]
    requests = {f"r{i}": traces.random_tokens(3 * i + 1, n, vocab) for i, n in enumerate([9, 40, 100, 57, 230, 77])}
    steps = traces.mixed(requests, decode_tail=40)
    max_tokens = traces.max_live_tokens(steps)
    outputs = {}
    for graphs in (0, 3):
        rep = Replayer(folders[name, dtype], dtype, max_tokens, page_size=4, poison_freed_pages=True, num_graphs=graphs)
        outputs[graphs] = traces.run_in_process(rep, steps)
        if graphs:
            assert rep.runner.n_replays > 5, (rep.runner.n_replays, rep.runner.n_captures)
    for step, out in outputs[0].items():
        assert np.array_equal(outputs[3][step], out), f"step {step} differs between the replayed and the launched run"
    got = traces.gather(steps, outputs[3], {k: len(v) for k, v in requests.items()}, vocab)
    want = cmp.expected(folders[name, dtype], requests, dtype)
    for rid in requests:
        cmp.check(got[rid], want[rid], dtype, f"{name} {dtype} mixed with graphs {rid}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_generation_with_and_without_graphs(folders, dtype, monkeypatch):
    """Greedy and sampled generation of requests that come and go (so the number of decoding requests changes,
    and bursts of decode steps feed each other on the device): the same tokens and log-probabilities with decode
    steps replayed from graphs (the default), with two graphs only, and with none."""
    from cwm_amd.engine import Engine, GenArgs

    name = "tiny_b"
    vocab = configs.get(name)["vocab_size"]
    prompts = [traces.random_tokens(70 + i, n, vocab) for i, n in enumerate([5, 33, 64, 90, 12, 41])]
    results = {}
    for label, graphs, env in (("default", 16, None), ("two", 2, None), ("none", 0, None), ("switch", 16, "1")):
        if env is None:
            monkeypatch.delenv("FG_NO_CUDA_GRAPHS", raising=False)
        else:
            monkeypatch.setenv("FG_NO_CUDA_GRAPHS", env)
        for sampling in (False, True):
            args = GenArgs(use_sampling=sampling, temperature=0.8, top_p=0.9, max_batch=4, max_seq=4096, cache_block=8, max_prefill=64,
                           logprobs=True, num_cuda_graphs=graphs, sync_freq=5)
            engine = Engine.from_folder(folders[name, dtype], args, dtype=dtype)
            results[label, sampling] = engine.generate_tokens(prompts, max_gen=60)
            replays = engine.runner.n_replays
            assert (replays > 0) == (label in ("default", "two")), (label, replays)
    for sampling in (False, True):
        for label in ("two", "none", "switch"):
            assert results[label, sampling] == results["default", sampling], f"{label}, sampling {sampling}"


def test_a_model_whose_steps_have_no_fixed_form_is_launched_step_by_step(capfd):
    """144 query heads on one key/value head: a decoded token's rows fill more than eight tiles, which go to
    the kernel for blocks of many rows, and that has no work list of a fixed length.  The runner says so once
    and launches every step; the logits are those of a run that never tried."""
    from cwm_amd.replay import Replayer

    config = {"architecture": "llama3_dense", "dim": 64, "n_layers": 2, "n_heads": 144, "n_kv_heads": 1, "head_dim": 16,
              "vocab_size": 300, "hidden_dim": 96, "norm_eps": 1e-5, "rope_theta": 10000.0, "max_seq_len": 512}
    requests = {"a": traces.random_tokens(1, 90, 300), "b": traces.random_tokens(2, 70, 300)}
    steps = decode_steps(requests, tail=30)
    outputs = {}
    for graphs in (0, 2):
        rep = Replayer(None, "bfloat16", traces.max_live_tokens(steps), page_size=16, random_config=config, seed=3, num_graphs=graphs)
        outputs[graphs] = traces.run_in_process(rep, steps)
        assert rep.runner.n_captures == 0 and rep.runner.n_replays == 0
    assert "not captured as graphs" in capfd.readouterr().err
    for step, want in outputs[0].items():
        assert np.array_equal(outputs[2][step], want)


def test_garbage_that_holds_a_graph_does_not_disturb_a_capture(folders):
    """An engine with captured steps that only the collector can free (it sits in a cycle), and a collector set
    to run at every opportunity: the next engine's capture collects first and keeps the collector off meanwhile
    (destroying a graph while a stream captures is refused by HIP), and generates what it should."""
    import gc

    from cwm_amd.engine import Engine, GenArgs

    vocab = configs.get("tiny_a")["vocab_size"]
    prompts = [traces.random_tokens(5 + i, n, vocab) for i, n in enumerate([7, 20])]
    args = GenArgs(use_sampling=False, max_batch=2, max_seq=1024, cache_block=8, max_prefill=64, sync_freq=4)
    first = Engine.from_folder(folders["tiny_a", "bfloat16"], args, dtype="bfloat16")
    want = first.generate_tokens(prompts, max_gen=30)
    assert first.runner.n_captures > 0
    cycle = [first]
    cycle.append(cycle)
    del first, cycle
    thresholds = gc.get_threshold()
    gc.set_threshold(1, 1, 1)
    try:
        second = Engine.from_folder(folders["tiny_a", "bfloat16"], args, dtype="bfloat16")
        assert second.generate_tokens(prompts, max_gen=30) == want
        assert second.runner.n_captures > 0
    finally:
        gc.set_threshold(*thresholds)


def test_replays_across_the_step_from_few_to_many_partial_results(folders):
    """A sequence that grows from 16,330 to 16,450 keys beside a short one: its chunks of 512 keys become more
    than 32, from where another launch of the merge kernel takes its partial results; the capture was made with
    room for that, and every replayed step gives the bits of the launched one."""
    from cwm_amd.replay import Replayer

    name, dtype = "tiny_a", "bfloat16"
    vocab = configs.get(name)["vocab_size"]
    requests = {"long": traces.random_tokens(3, 16450, vocab), "short": traces.random_tokens(4, 200, vocab)}
    steps = decode_steps(requests, tail=120)
    steps[0]["entries"] = [dict(e, want=[len(e["tokens"]) - 1]) for e in steps[0]["entries"]]
    outputs = {}
    for graphs in (0, 2):
        rep = Replayer(folders[name, dtype], dtype, traces.max_live_tokens(steps), page_size=64, num_graphs=graphs)
        outputs[graphs] = traces.run_in_process(rep, steps)
        if graphs:
            assert rep.runner.n_replays >= 110 and rep.runner.n_captures <= 4, (rep.runner.n_replays, rep.runner.n_captures)
    for step, want in outputs[0].items():
        assert np.isfinite(want).all()
        assert np.array_equal(outputs[2][step], want), f"step {step} differs between the replayed and the launched run"


@pytest.mark.parametrize("says_so", [True, False])
def test_a_part_from_outside_opts_into_captured_steps(says_so):
    """An attention defined here that normalises query and key heads between projection and rotation
    (`transform_qk`): decode steps of its model are captured only if it says that the hook keeps to the rule
    of captured steps (`transform_replayable`), and then give the bits of launched steps."""
    from dataclasses import dataclass

    from cwm_amd.cache import CacheManager, CacheStorage
    from cwm_amd.config import ARCHITECTURES, parse_config, register_architecture
    from cwm_amd.engine import ModelRunner, Portion
    from cwm_amd.models import Model
    from cwm_amd.parts import LayerCall, LayerPlan, ModelPlan, PartChoice, Runtime, register_part
    from cwm_amd.parts.attention import PagedAttention
    from cwm_amd.parts.base import MIXERS
    from cwm_amd.weights import random_tensors

    class UnitNormAttention(PagedAttention):
        transform_replayable = says_so

        def transform_qk(self, q, k, batch):
            for t in (q, k):
                if t is not None:
                    t.copy_(torch.nn.functional.normalize(t.float(), dim=-1).to(t.dtype))

    @dataclass(frozen=True)
    class ToyConfig:
        architecture: str
        dim: int
        vocab_size: int

    def toy_plan(cfg):
        rope = PartChoice("rotary", {"head_dim": 16, "theta": 100.0})
        attn = PartChoice("toy_unit_norm_attention_for_graphs", {"dim": cfg.dim, "n_heads": 4, "n_kv_heads": 2, "head_dim": 16, "scale": 3.0,
                                                                 "position_encoding": rope})
        names = {"norm1": "n1.", "mixer": "attn.", "norm2": "n2.", "feed_forward": "ff."}
        norm = PartChoice("rmsnorm", {"dim": cfg.dim, "eps": 1e-5})
        layer = LayerPlan.standard("l0.", "pre_norm", norm, attn, PartChoice("swiglu", {"dim": cfg.dim, "hidden_dim": 48}), names)
        return ModelPlan.standard(cfg.vocab_size, cfg.dim, "emb", [layer], [LayerCall(0)], norm, "final", "head")

    register_part("mixer", "toy_unit_norm_attention_for_graphs", UnitNormAttention)
    register_architecture("toy_graph_model", ToyConfig, toy_plan)
    try:
        arch, cfg = parse_config({"architecture": "toy_graph_model", "dim": 32, "vocab_size": 83})
        model = Model(arch.build_plan(cfg))
        runtime = Runtime(torch.device("cuda:0"), torch.bfloat16)
        host = random_tensors(model.tensor_specs(), seed=2, std=0.2, norm_init="uniform", dtype=torch.bfloat16)
        model.bind({k: v.to("cuda:0") for k, v in host.items()}, runtime)
        assert model.replayable == says_so
        toks = {"a": traces.random_tokens(1, 70, 83), "b": traces.random_tokens(2, 45, 83)}
        outputs = {}
        for graphs in (0, 2):
            manager = CacheManager(model.cache_specs, 8, 32, 2)
            storage = CacheStorage(manager, runtime.device, runtime.act_dtype)
            runner = ModelRunner(model, manager, storage, num_graphs=graphs)
            out = []
            for rid in toks:
                runner.admit(rid)
                assert manager.extend(rid, 5)
                runner.step([Portion(rid, toks[rid][:5], [])])
            for i in range(5, 45):
                for rid in toks:
                    assert manager.extend(rid, 1)
                out.append(runner.step([Portion(rid, [toks[rid][i]], [0]) for rid in toks]).cpu())
            outputs[graphs] = torch.stack(out)
            if graphs:
                assert (runner.n_replays > 30) == says_so and (runner.n_captures > 0) == says_so
        assert torch.isfinite(outputs[0]).all() and torch.equal(outputs[0], outputs[2])
    finally:
        del ARCHITECTURES["toy_graph_model"]
        del MIXERS["toy_unit_norm_attention_for_graphs"]
