"""Two layers of the CWM-32B width through the step function, against the plain
implementation in float64 on the device: width 6,144, 48 query and 8 key/value heads of 128,
feed-forward width 21,504, the 128,256-entry vocabulary, a window of 8,192 keys on the first
layer, pages of 256 tokens.  A request of about 9,000 tokens runs in portions of 4,096 and
then 40 single tokens, beside a short second request, in pools so small that the window
group's pages are given back and used again (they are overwritten with NaN in between).  Once with
every step launched kernel by kernel and once with the steps of a single token replayed from a graph."""

import numpy as np
import pytest
import torch

from helpers import compare as cmp, traces
from plain import llama3_plain

pytestmark = pytest.mark.gpu

CONFIG = {
    "architecture": "llama3_dense", "dim": 6144, "n_layers": 2, "n_heads": 48, "n_kv_heads": 8, "head_dim": 128,
    "vocab_size": 128256, "ffn_dim_multiplier": 1.3125, "multiple_of": 256, "norm_eps": 1e-5, "pos_embed_impl": "scaled_rope",
    "rope_theta": 1000000.0, "scaled_rope": {"scale_factor": 16, "old_context_len": 8192, "low_freq_factor": 1, "high_freq_factor": 4},
    "window_attn": {"window_pattern": 4, "local_window": 8192, "global_last_layer": True},
    "layer_types": ["local", "global"], "max_seq_len": 131072,
}
PAGE = 256


@pytest.mark.parametrize("graphs", [0, 2])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_two_layers_of_the_32b_width(dtype, graphs):
    from cwm_amd.cache import CacheManager, CacheStorage
    from cwm_amd.engine import ModelRunner, Portion, random_model
    from cwm_amd.weights.random_init import random_tensor

    device = torch.device("cuda:0")
    model, typed = random_model(CONFIG, seed=4, dtype=dtype, device=device, norm_init="uniform")
    assert typed.ffn_width == 21504 and typed.layer_windows() == [8192, None]
    vocab = CONFIG["vocab_size"]
    long_toks = traces.random_tokens(1, 9001, vocab)
    short_toks = traces.random_tokens(2, 300, vocab)
    # the long request: 4,096 + 4,096 + 769 tokens, then 40 single tokens; the short one joins beside the decoded tokens
    cuts = [4096, 4096, 769] + [1] * 40
    assert sum(cuts) == len(long_toks)
    every = 97  # logits are wanted at every 97th place of a portion, at its last place, and at every single token

    # pools: the window group holds (8,191 + 4,096) tokens of the long request and the short one, no more
    pages = {None: (len(long_toks) + PAGE - 1) // PAGE + 2, 8192: (8191 + 4096 + PAGE - 1) // PAGE + 1 + 2}
    manager = CacheManager(model.cache_specs, PAGE, pages, 2)
    storage = CacheStorage(manager, device, model.runtime.act_dtype)
    for t in storage.paged.values():
        t.fill_(float("nan"))  # nothing is read that was not written
    runner = ModelRunner(model, manager, storage, num_graphs=graphs)  # with graphs, the steps of one token alone are replayed
    freed_pages = []

    def poison(group, gone):
        freed_pages.extend((group, p) for p in gone)
        storage.fill_pages(group, gone, float("nan"))

    runner.on_pages_freed = poison
    page_use = traces.PageUse(manager)
    runner.admit("long")
    got = {"long": {}, "short": {}}
    cur = 0
    short_cur = 0
    for k, n in enumerate(cuts):
        portions = []
        want = sorted(set(range(0, n, every)) | {n - 1})
        assert manager.extend("long", n)
        portions.append(Portion("long", long_toks[cur : cur + n], want))
        wanted = [("long", cur + w) for w in want]
        if k == 5:
            runner.admit("short")
        if k >= 5 and short_cur < len(short_toks):
            # its prompt in portions beside the long request's decoded tokens: steps of 131, 101 and 71 rows, which
            # the products take in a block of 256 rows (or the library), of 128 and of 64
            m = min([130, 100, 70][min(k - 5, 2)], len(short_toks) - short_cur)
            assert manager.extend("short", m)
            swant = sorted({0, m // 2, m - 1})
            portions.append(Portion("short", short_toks[short_cur : short_cur + m], swant))
            wanted += [("short", short_cur + w) for w in swant]
            short_cur += m
        page_use.note()
        logits = runner.step(portions)
        manager.check()
        assert logits.shape == (len(wanted), vocab)
        for row, (rid, pos) in enumerate(wanted):
            got[rid][pos] = logits[row].clone()
        cur += n
    assert short_cur == len(short_toks)
    assert (runner.n_replays >= 30) == (graphs > 0), runner.n_replays
    # the window group gave pages back while the long request ran, and took them again
    window_group = next(g.index for g in manager.groups if g.window == 8192)
    assert any(g == window_group for g, _ in freed_pages)
    assert page_use.pages_used_again(window_group) > 0, "no page of the window group was taken again after it had been given back"
    assert manager.pages_held("long")[window_group] <= (8191 + 1 + PAGE - 1) // PAGE + 1

    # the plain implementation on whole sequences, float64 on the device, from the same random tensors
    specs = model.tensor_specs()
    store = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    weights = {name: random_tensor(name, spec, 4, 0.02, "uniform", store, device).double() for name, spec in specs.items()}
    del model, runner, storage
    torch.cuda.empty_cache()
    for rid, toks in (("long", long_toks), ("short", short_toks)):
        places = sorted(got[rid])
        mine = torch.stack([got[rid][p] for p in places]).cpu().numpy()
        with torch.no_grad():
            exact = llama3_plain.forward_from_config(weights, CONFIG, toks, dtype=torch.float64)[places].float().cpu().numpy()
            rounded = None
            if dtype == "bfloat16":
                rounded = (
                    llama3_plain.forward_from_config(weights, CONFIG, toks, dtype=torch.float64, rounding=llama3_plain.ROUND_AS_ENGINE)[places]
                    .float().cpu().numpy()
                )
        cmp.check(mine, cmp.Expected(exact, rounded), dtype, f"32B width, {dtype}, request {rid} (places {places[0]}..{places[-1]})")
