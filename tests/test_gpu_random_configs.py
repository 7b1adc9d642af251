"""Seeded random configurations of the architecture (head sizes with and without a
matrix-core path, odd widths and vocabularies, windows of every pattern, biases, rope
scaling) with random traces (whole, decoded tail, portions, mixed) and random page
sizes, through the replay driver against the plain implementation."""

import random

import numpy as np
import pytest

from helpers import compare as cmp, traces

pytestmark = pytest.mark.gpu


def random_config(rng):
    n_kv = rng.choice([1, 2, 3, 4])
    cfg = {
        "architecture": "llama3_dense",
        "dim": rng.choice([64, 72, 96, 100, 120, 128, 160, 200, 256]),
        "n_layers": rng.choice([1, 2, 3, 5]),
        "n_heads": n_kv * rng.choice([1, 2, 3, 4, 6, 8]),
        "n_kv_heads": n_kv,
        "head_dim": rng.choice([8, 16, 24, 32, 40, 48, 64, 80, 96, 128]),
        "vocab_size": rng.choice([97, 256, 331, 1000]),
        "norm_eps": rng.choice([1e-5, 1e-6, 3e-4]),
        "rope_theta": rng.choice([1e4, 5e5, 1e6]),
        "max_seq_len": 1024,
    }
    if rng.random() < 0.5:
        cfg["hidden_dim"] = rng.choice([40, 64, 72, 100, 130, 296, 320])
    else:
        cfg["ffn_dim_multiplier"] = rng.choice([0.5, 1.0, 1.3])
        cfg["multiple_of"] = rng.choice([8, 20, 32, 64])
    if rng.random() < 0.5:
        cfg["pos_embed_impl"] = "scaled_rope"
        cfg["scaled_rope"] = {
            "scale_factor": rng.choice([2, 8, 16]), "old_context_len": rng.choice([16, 64, 8192]),
            "low_freq_factor": 1, "high_freq_factor": rng.choice([2, 4]),
        }
    if rng.random() < 0.6:
        cfg["window_attn"] = {
            "window_pattern": rng.choice([1, 2, 3, 4]), "local_window": rng.choice([3, 8, 17, 40, 64, 100]),
            "global_last_layer": rng.random() < 0.5,
        }
    if rng.random() < 0.3:
        cfg["qkv_biases"] = True
    return cfg


def random_trace(rng, vocab):
    lengths = [rng.choice([1, 2, 5, 17, 33, 64, 65, 100, 129, 200]) for _ in range(rng.randint(1, 5))]
    requests = {f"r{i}": traces.random_tokens(rng.randrange(10**6), n, vocab) for i, n in enumerate(lengths)}
    sizes = [rng.choice([1, 2, 3, 5, 8, 16, 31, 64, 130]) for _ in range(9)]
    kind = rng.choice(["whole", "tail", "portions", "mixed", "mixed"])
    if kind == "whole":
        steps = traces.whole(requests)
    elif kind == "tail":
        steps = traces.tail_one_by_one(requests, tail=rng.choice([1, 8, 32]))
    elif kind == "portions":
        steps = traces.portions(requests, sizes)
    else:
        steps = traces.mixed(requests, max_live=rng.choice([2, 3, 4]), decode_tail=rng.choice([0, 3, 12]), sizes=sizes)
    return requests, steps


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(12))
def test_random_configuration_and_trace(tmp_path, seed, dtype):
    from cwm_amd.replay import Replayer
    from cwm_amd.weights import write_random_model

    rng = random.Random(1000 * seed + (dtype == "bfloat16"))
    config = random_config(rng)
    folder = str(tmp_path / "model")
    write_random_model(folder, config, seed=seed, std=rng.choice([0.02, 0.05, 0.1]), norm_init="uniform", dtype=dtype)
    requests, steps = random_trace(rng, config["vocab_size"])
    page_size = rng.choice([1, 4, 8, 16, 32, 64])
    replayer = Replayer(folder, dtype, traces.max_live_tokens(steps, multiple=max(64, page_size)), page_size=page_size, poison_freed_pages=True)
    outputs = traces.run_in_process(replayer, steps)
    got = traces.gather(steps, outputs, {k: len(v) for k, v in requests.items()}, config["vocab_size"])
    want = cmp.expected(folder, requests, dtype)
    for rid in want:
        cmp.check(got[rid], want[rid], dtype, f"{rid} (config {config}, page {page_size})")
    assert replayer.manager.live_requests() == []


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_deep_narrow_model(tmp_path, dtype):
    """24 layers of width 72, interleaved windows, weights of std 0.1: rounding has many layers to
    grow through, and the limit (derived from the plain implementation's own bfloat16 run) grows
    with it; in portions, mixed with other requests, with pages used again."""
    from cwm_amd.replay import Replayer
    from cwm_amd.weights import write_random_model

    config = {
        "architecture": "llama3_dense", "dim": 72, "n_layers": 24, "n_heads": 6, "n_kv_heads": 2, "head_dim": 16,
        "vocab_size": 131, "hidden_dim": 104, "norm_eps": 1e-5, "rope_theta": 10000.0, "max_seq_len": 512,
        "window_attn": {"window_pattern": 3, "local_window": 24, "global_last_layer": True},
    }
    folder = str(tmp_path / "model")
    write_random_model(folder, config, seed=3, std=0.1, norm_init="uniform", dtype=dtype)
    requests = {f"r{i}": traces.random_tokens(500 + i, n, config["vocab_size"]) for i, n in enumerate([90, 33, 150])}
    steps = traces.mixed(requests, max_live=3)
    replayer = Replayer(folder, dtype, traces.max_live_tokens(steps), page_size=8, poison_freed_pages=True)
    outputs = traces.run_in_process(replayer, steps)
    got = traces.gather(steps, outputs, {k: len(v) for k, v in requests.items()}, config["vocab_size"])
    want = cmp.expected(folder, requests, dtype)
    for rid in want:
        cmp.check(got[rid], want[rid], dtype, f"deep-narrow {rid}")
