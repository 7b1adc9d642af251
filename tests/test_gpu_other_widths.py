"""One layer of the Llama-3 8B and of the 70B width, and of a small one with heads of 64, through the step
function, against the plain implementation in float64 on the device: widths 4,096, 8,192 (longer than the
products that keep a whole row of activations in registers take in one piece) and 2,048; 32, 64 and 32 query
heads on 8 key/value heads; feed-forward widths 14,336, 28,672 and 8,192; pages of 256 tokens.  Two requests: one
prompt in portions of 300, 129 and 71 tokens, the other whole; then 24 steps of single tokens for both."""

import pytest
import torch

from helpers import compare as cmp, traces
from plain import llama3_plain

pytestmark = pytest.mark.gpu

WIDTHS = {
    "8b": dict(dim=4096, n_heads=32, head_dim=128, ffn_dim_multiplier=1.3, multiple_of=1024, hidden=14336),
    "70b": dict(dim=8192, n_heads=64, head_dim=128, ffn_dim_multiplier=1.3, multiple_of=4096, hidden=28672),
    "small": dict(dim=2048, n_heads=32, head_dim=64, ffn_dim_multiplier=1.5, multiple_of=256, hidden=8192),
}
PAGE = 256


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("width", ["8b", "70b", "small"])
def test_one_layer_of_another_width(width, dtype):
    from cwm_amd.cache import CacheManager, CacheStorage
    from cwm_amd.engine import ModelRunner, Portion, random_model
    from cwm_amd.weights.random_init import random_tensor

    w = WIDTHS[width]
    config = {
        "architecture": "llama3_dense", "dim": w["dim"], "n_layers": 1, "n_heads": w["n_heads"], "n_kv_heads": 8, "head_dim": w["head_dim"],
        "vocab_size": 2048, "ffn_dim_multiplier": w["ffn_dim_multiplier"], "multiple_of": w["multiple_of"], "norm_eps": 1e-5,
        "pos_embed_impl": "rope", "rope_theta": 500000.0, "max_seq_len": 8192,
    }
    device = torch.device("cuda:0")
    model, typed = random_model(config, seed=9, dtype=dtype, device=device, norm_init="uniform")
    assert typed.ffn_width == w["hidden"]
    vocab = config["vocab_size"]
    requests = {"a": traces.random_tokens(1, 524, vocab), "b": traces.random_tokens(2, 90, vocab)}
    manager = CacheManager(model.cache_specs, PAGE, {None: 8}, 2)
    storage = CacheStorage(manager, device, model.runtime.act_dtype)
    for t in storage.paged.values():
        t.fill_(float("nan"))
    runner = ModelRunner(model, manager, storage)
    got = {rid: {} for rid in requests}
    done = {rid: 0 for rid in requests}
    runner.admit("a")
    runner.admit("b")
    steps = [{"a": 300, "b": 66}, {"a": 129}, {"a": 71}] + [{"a": 1, "b": 1}] * 24
    for step in steps:
        portions, wanted = [], []
        for rid, n in step.items():
            assert manager.extend(rid, n)
            want = sorted({0, n // 2, n - 1})
            portions.append(Portion(rid, requests[rid][done[rid] : done[rid] + n], want))
            wanted += [(rid, done[rid] + p) for p in want]
            done[rid] += n
        logits = runner.step(portions)
        manager.check()
        for row, (rid, pos) in enumerate(wanted):
            got[rid][pos] = logits[row].clone()
    assert done == {rid: len(toks) for rid, toks in requests.items()}

    specs = model.tensor_specs()
    store = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    weights = {name: random_tensor(name, spec, 9, 0.02, "uniform", store, device).double() for name, spec in specs.items()}
    del model, runner, storage
    torch.cuda.empty_cache()
    for rid, toks in requests.items():
        places = sorted(got[rid])
        mine = torch.stack([got[rid][p] for p in places]).cpu().numpy()
        with torch.no_grad():
            exact = llama3_plain.forward_from_config(weights, config, toks, dtype=torch.float64)[places].float().cpu().numpy()
            rounded = None
            if dtype == "bfloat16":
                rounded = (
                    llama3_plain.forward_from_config(weights, config, toks, dtype=torch.float64, rounding=llama3_plain.ROUND_AS_ENGINE)[places]
                    .float().cpu().numpy()
                )
        cmp.check(mine, cmp.Expected(exact, rounded), dtype, f"{width} width, {dtype}, request {rid}")
