"""The engine against the plain implementation through the replay driver, in float32
and in bfloat16: each request alone and whole; most of it in one step and the last
32 tokens one by one; in portions of changing size down to two tokens; and mixed,
up to four live requests with so few pages that they are used again (given-back
pages are overwritten with NaN first)."""

import numpy as np
import pytest
import torch

from helpers import compare as cmp, configs, models, traces

pytestmark = pytest.mark.gpu

LENGTHS = {"tiny_a": [5, 17, 33, 64, 128], "tiny_b": [9, 40, 100, 57, 230], "tiny_c": [70, 41, 190], "tiny_d": [150, 90, 260]}
# tokens in a page, by regime; tiny_d runs with pages of 32 and 64
PAGE_SIZES = {"whole": 16, "tail": 16, "portions": 8, "mixed": 4}
PAGE_SIZES_D = {"whole": 64, "tail": 32, "portions": 32, "mixed": 32}


def requests_for(name):
    vocab = configs.get(name)["vocab_size"]
    return {f"r{i}": traces.random_tokens(7 * i + len(name), n, vocab) for i, n in enumerate(LENGTHS[name])}


def compare(got, want, dtype, what):
    for rid in want:
        cmp.check(got[rid], want[rid], dtype, f"{what} {rid}")


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("models")
    out = {}
    for name in configs.ALL:
        for dtype in ("float32", "bfloat16"):
            out[name, dtype] = models.make_folder(root, name, seed=5, dtype=dtype)
    return out


@pytest.fixture(scope="module")
def plain_cache():
    return {}


def plain_for(folders, plain_cache, name, dtype):
    key = (name, dtype)
    if key not in plain_cache:
        plain_cache[key] = cmp.expected(folders[key], requests_for(name), dtype)
    return plain_cache[key]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(configs.ALL))
@pytest.mark.parametrize("regime", ["whole", "tail", "portions", "mixed"])
def test_replay_regimes(folders, plain_cache, name, dtype, regime):
    from cwm_amd.replay import Replayer

    requests = requests_for(name)
    vocab = configs.get(name)["vocab_size"]
    steps = {"whole": traces.whole, "tail": traces.tail_one_by_one, "portions": traces.portions, "mixed": traces.mixed}[regime](requests)
    max_tokens = traces.max_live_tokens(steps)
    page_size = (PAGE_SIZES_D if name == "tiny_d" else PAGE_SIZES)[regime]
    rep = Replayer(folders[name, dtype], dtype, max_tokens, page_size=page_size, poison_freed_pages=True)
    page_use = traces.PageUse(rep.manager)
    outputs = traces.run_in_process(rep, steps, page_use)
    got = traces.gather(steps, outputs, {k: len(v) for k, v in requests.items()}, vocab)
    compare(got, plain_for(folders, plain_cache, name, dtype), dtype, f"{name} {dtype} {regime}")
    assert rep.manager.live_requests() == []
    if regime == "mixed":
        # "so few pages that they are used again": in every layer group physical pages have served two requests
        for g in rep.manager.groups:
            assert page_use.pages_shared_between_requests(g.index) > 0, f"group {g.index} (window {g.window}): no page served two requests"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_and_long_decoding(folders, plain_cache, dtype):
    """The first tokens of a sequence one by one from an empty cache, then a long run
    of single-token steps across many pages and past the window."""
    from cwm_amd.replay import Replayer

    name = "tiny_b"
    vocab = configs.get(name)["vocab_size"]
    toks = traces.random_tokens(99, 300, vocab)
    steps = [{"step": i, "entries": [{"id": "x", "tokens": [t], "want": [0]}], "end": []} for i, t in enumerate(toks)]
    rep = Replayer(folders[name, dtype], dtype, 320, page_size=4, poison_freed_pages=True)
    outputs = traces.run_in_process(rep, steps)
    got = traces.gather(steps, outputs, {"x": len(toks)}, vocab)
    want = cmp.expected(folders[name, dtype], {"x": toks}, dtype)
    compare(got, want, dtype, f"{name} {dtype} one-by-one")
    # the window group never holds more than the window needs
    local = [g.index for g in rep.manager.groups if g.window is not None]
    for g in local:
        assert rep.manager.pages_held("x")[g] <= (8 - 1 + 1 + 3) // 4 + 1


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_many_requests_decode_together(folders, dtype):
    """Ninety requests in one batch: their prompts in one step of 270 rows, five steps of 90 single
    tokens, then, fifty of them ended, five steps of 40: the row counts at which the products change
    kernels (blocks of 128 rows, of 64, the library above 256)."""
    from cwm_amd.replay import Replayer

    name = "tiny_a"
    vocab = configs.get(name)["vocab_size"]
    requests = {f"q{i}": traces.random_tokens(1000 + i, 3 + 5 + (5 if i < 40 else 0), vocab) for i in range(90)}
    steps = [{"step": 0, "entries": [{"id": rid, "tokens": toks[:3], "want": [0, 1, 2]} for rid, toks in requests.items()], "end": []}]
    for k in range(5):
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [toks[3 + k]], "want": [0]} for rid, toks in requests.items()],
                      "end": [f"q{i}" for i in range(40, 90)] if k == 4 else []})
    for k in range(5):
        steps.append({"step": len(steps), "entries": [{"id": f"q{i}", "tokens": [requests[f"q{i}"][8 + k]], "want": [0]} for i in range(40)],
                      "end": [f"q{i}" for i in range(40)] if k == 4 else []})
    rep = Replayer(folders[name, dtype], dtype, 90 * 64, page_size=8, max_requests=90, poison_freed_pages=True)
    outputs = traces.run_in_process(rep, steps)
    got = traces.gather(steps, outputs, {k: len(v) for k, v in requests.items()}, vocab)
    compare(got, cmp.expected(folders[name, dtype], requests, dtype), dtype, f"{name} {dtype} ninety requests")
    assert rep.manager.live_requests() == []


@pytest.mark.parametrize("name", ["tiny_b", "tiny_d"])
def test_streaming_copies_change_no_bit(folders, name):
    """A model that keeps its matrices' streaming copies (the default where they fit) gives the logits of the same
    model without them bit for bit, under a trace that mixes portions and single tokens: the copies hold the same
    values, and the products add them in the same order."""
    from cwm_amd.cache import CacheManager, CacheStorage
    from cwm_amd.engine import ModelRunner, Portion, load_model

    requests = requests_for(name)
    steps = traces.mixed(requests)
    outputs = {}
    for copies in (False, True):
        model, _ = load_model(folders[name, "bfloat16"], "bfloat16", "cuda:0", stream_copies=copies)
        assert model.runtime.stream_copies == copies
        assert (model.head.weights.streamed is not None) == copies
        manager = CacheManager(model.cache_specs, 8, 2 * traces.max_live_tokens(steps) // 8, 8)
        storage = CacheStorage(manager, model.runtime.device, model.runtime.act_dtype)
        runner = ModelRunner(model, manager, storage)
        got = []
        for st in steps:
            portions = []
            for e in st["entries"]:
                if not e["tokens"]:
                    continue
                if e["id"] not in manager:
                    runner.admit(e["id"])
                assert manager.extend(e["id"], len(e["tokens"]))
                portions.append(Portion(e["id"], e["tokens"], e["want"]))
            logits = runner.step(portions) if portions else None
            if logits is not None:
                got.append(logits.cpu())
            for rid in st["end"]:
                runner.release(rid)
        outputs[copies] = torch.cat(got)
    assert outputs[True].shape[0] > 100 and torch.equal(outputs[True], outputs[False])
