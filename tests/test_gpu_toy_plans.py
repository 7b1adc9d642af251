"""Shapes of model that the framework's own architecture does not have, put together from outside: a layer
with four norms, a mixer whose cached row is one compressed vector instead of a key and a value, and a head
that caps its logits.  Each is registered here, built from a plan, stepped through the engine's own runner in
portions and single tokens, and compared with a whole-sequence computation written in this file.  Nothing under
cwm_amd/ changes for them.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Tuple

import pytest
import torch

from helpers import traces
from plain import llama3_plain as plain

pytestmark = pytest.mark.gpu


@dataclass(frozen=True)
class ToyConfig:
    architecture: str
    dim: int
    vocab_size: int


def _step_through(model, runtime, toks, cuts, page_size=4, pages=64):
    """Feeds the requests of `toks` in the portions that `cuts` lists; returns the logits of every token, and the storage."""
    from cwm_amd.cache import CacheManager, CacheStorage
    from cwm_amd.engine import ModelRunner, Portion

    manager = CacheManager(model.cache_specs, page_size, pages, 4)
    storage = CacheStorage(manager, runtime.device, runtime.act_dtype)
    runner = ModelRunner(model, manager, storage)
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
        manager.check()
        row = 0
        for p in portions:
            got[p.rid].append(logits[row : row + len(p.tokens)])
            row += len(p.tokens)
    assert all(cur[k] == len(toks[k]) for k in toks)
    return {k: torch.cat(v) for k, v in got.items()}, storage


CUTS = [{"a": 5, "b": 2}, {"a": 1, "b": 1}, {"a": 1, "b": 6}, {"a": 2}, {"a": 14, "b": 3}]


def _attention(cfg_dim, n_heads, n_kv, hd, theta, window=None):
    from cwm_amd.parts import PartChoice

    return PartChoice("paged_attention", {"dim": cfg_dim, "n_heads": n_heads, "n_kv_heads": n_kv, "head_dim": hd, "scale": hd**-0.5, "window": window,
                                          "position_encoding": PartChoice("rotary", {"head_dim": hd, "theta": theta})})


def _plain_attention(x, w, prefix, n_heads, n_kv, hd, theta, window=None):
    n = x.shape[0]
    pos = torch.arange(n)
    freqs = plain.rope_frequencies(hd, theta)
    q = plain.rope_apply(plain.linear(x, w[prefix + "wq.weight"]).view(n, n_heads, hd), pos, freqs)
    k = plain.rope_apply(plain.linear(x, w[prefix + "wk.weight"]).view(n, n_kv, hd), pos, freqs)
    v = plain.linear(x, w[prefix + "wv.weight"]).view(n, n_kv, hd)
    out = plain.attention(q, k, v, window_left=-1 if window is None else window - 1, scale=hd**-0.5)
    return plain.linear(out.reshape(n, -1), w[prefix + "wo.weight"])


# ---- a layer with four norms ----------------------------------------------------------------------- #
def test_toy_block_with_four_norms():
    """h += post1(mixer(pre1(h))); h += post2(feed_forward(pre2(h))): a norm before and after each of the two
    (every one with weights and an eps of its own).  The layer's plan names six roles; the block is a subclass of
    `Block` that only writes `forward`."""
    from cwm_amd.config import ARCHITECTURES, parse_config, register_architecture
    from cwm_amd.models import Model
    from cwm_amd.parts import Block, LayerCall, LayerPlan, ModelPlan, PartChoice, PartSlot, Runtime, register_part
    from cwm_amd.parts.base import BLOCKS
    from cwm_amd.weights import random_tensors

    class SandwichBlock(Block):
        def __init__(self, names, pre_mixer, mixer, post_mixer, pre_ff, feed_forward, post_ff):
            super().__init__(names, pre_mixer=pre_mixer, mixer=mixer, post_mixer=post_mixer, pre_ff=pre_ff, feed_forward=feed_forward, post_ff=post_ff)

        def forward(self, h, delta, batch, cache, write_cache=True):
            p = self.parts
            x = p["pre_mixer"].forward(h, delta)
            mixed = p["mixer"].forward(x, batch, cache, write_cache)
            # a norm of something that is not the residual stream: it adds `mixed` into zeros and normalises that
            mixed = p["post_mixer"].forward(torch.zeros_like(h), mixed)
            x = p["pre_ff"].forward(h, mixed)
            out = p["feed_forward"].forward(x, batch)
            return p["post_ff"].forward(torch.zeros_like(h), out)

    n_heads, n_kv, hd, theta, hidden = 3, 1, 16, 150.0, 56
    eps = {"pre_mixer": 1e-5, "post_mixer": 1e-2, "pre_ff": 1e-4, "post_ff": 0.3}
    prefixes = {"pre_mixer": "n_a.", "post_mixer": "n_b.", "pre_ff": "n_c.", "post_ff": "n_d."}

    def toy_plan(cfg):
        def layer(i):
            parts = {role: PartSlot("norm", PartChoice("rmsnorm", {"dim": cfg.dim, "eps": e}), prefixes[role]) for role, e in eps.items()}
            parts["mixer"] = PartSlot("mixer", _attention(cfg.dim, n_heads, n_kv, hd, theta), "attn.")
            parts["feed_forward"] = PartSlot("feed_forward", PartChoice("swiglu", {"dim": cfg.dim, "hidden_dim": hidden}), "ff.")
            return LayerPlan(f"l{i}.", "toy_sandwich", parts)

        return ModelPlan.standard(cfg.vocab_size, cfg.dim, "emb", [layer(0), layer(1)], [LayerCall(0), LayerCall(1)],
                                  PartChoice("rmsnorm", {"dim": cfg.dim, "eps": 1e-5}), "final", "head")

    register_part("block", "toy_sandwich", SandwichBlock)
    register_architecture("toy_sandwich_model", ToyConfig, toy_plan)
    try:
        arch, cfg = parse_config({"architecture": "toy_sandwich_model", "dim": 40, "vocab_size": 67})
        model = Model(arch.build_plan(cfg))
        specs = model.tensor_specs()
        assert {n for n in specs if n.startswith("l1.n_")} == {"l1.n_a.weight", "l1.n_b.weight", "l1.n_c.weight", "l1.n_d.weight"}
        assert model.replayable  # every part of it is the framework's own and says so; the block asks its parts
        runtime = Runtime(torch.device("cuda:0"), torch.float32)
        host = random_tensors(specs, seed=3, std=0.3, norm_init="uniform", dtype=torch.float32)
        model.bind({k: v.to("cuda:0") for k, v in host.items()}, runtime)

        def whole_sequence(tokens, eps=eps):
            w = {k: v.double() for k, v in host.items()}
            h = w["emb.weight"][torch.tensor(tokens)]
            for i in range(2):
                p = f"l{i}."
                x = plain.rms_norm(h, w[p + "n_a.weight"], eps["pre_mixer"])
                a = _plain_attention(x, w, p + "attn.", n_heads, n_kv, hd, theta)
                h = h + plain.rms_norm(a, w[p + "n_b.weight"], eps["post_mixer"])
                x = plain.rms_norm(h, w[p + "n_c.weight"], eps["pre_ff"])
                f = plain.swiglu(x, w[p + "ff.w1.weight"], w[p + "ff.w2.weight"], w[p + "ff.w3.weight"])
                h = h + plain.rms_norm(f, w[p + "n_d.weight"], eps["post_ff"])
            return plain.linear(plain.rms_norm(h, w["final.weight"], 1e-5), w["head.weight"]).float()

        toks = {"a": traces.random_tokens(5, 23, 67), "b": traces.random_tokens(6, 12, 67)}
        cut, _ = _step_through(model, runtime, toks, CUTS)
        for k in toks:
            torch.testing.assert_close(cut[k], whole_sequence(toks[k]), rtol=2e-4, atol=2e-4)
        # each norm's own eps counts: with the last one's exchanged for the first one's the logits differ
        assert not torch.allclose(cut["a"], whole_sequence(toks["a"], {**eps, "post_ff": eps["pre_mixer"]}), rtol=1e-2, atol=1e-2)
    finally:
        del ARCHITECTURES["toy_sandwich_model"]
        del BLOCKS["toy_sandwich"]


# ---- a mixer that caches one compressed row a token ------------------------------------------------ #
def test_toy_mixer_with_a_cache_of_one_plane_of_another_width():
    """A mixer that caches, instead of keys and values, one compressed row c = x Wc of width 24 a token and
    attends over those rows (scores q . c, output softmax(scores) c, then a projection back).  Its cache need is
    a subclass of `PagedKVSpec` that answers `page_shape` and `bytes_per_token` differently; storage, pool
    sizes and block tables follow.  One such layer (with a window, so that its pages are given back) and one
    layer of the framework's own attention, whose group keeps everything."""
    from cwm_amd.config import ARCHITECTURES, parse_config, register_architecture
    from cwm_amd.engine import GenArgs
    from cwm_amd.engine.engine import pool_sizes
    from cwm_amd.models import Model
    from cwm_amd.parts import LayerCall, LayerPlan, Mixer, ModelPlan, PagedKVSpec, PartChoice, Runtime, TensorSpec, register_part
    from cwm_amd.parts.base import MIXERS
    from cwm_amd.weights import random_tensors

    @dataclass(frozen=True)
    class CompressedRowSpec(PagedKVSpec):
        width: int = 0

        def page_shape(self, page_size: int) -> Tuple[int, ...]:
            return (page_size, self.width)

    class CompressedRowMixer(Mixer):
        def __init__(self, dim, width, window, scale):
            self.dim, self.width, self.window, self.scale = dim, width, window, scale

        def cache_spec(self):
            return CompressedRowSpec(n_kv_heads=1, head_dim=self.width, window=self.window, width=self.width)

        def tensor_specs(self):
            return {"wc.weight": TensorSpec((self.width, self.dim)), "wq.weight": TensorSpec((self.width, self.dim)),
                    "wo.weight": TensorSpec((self.dim, self.width))}

        def bind(self, tensors, runtime):
            super().bind(tensors, runtime)
            self.wc, self.wq, self.wo = (tensors[n + ".weight"].float() for n in ("wc", "wq", "wo"))

        def forward(self, x, batch, cache, write_cache=True):
            assert cache.cache.shape[1:] == (cache.page_size, self.width)
            x = x.float()
            rows, queries = x @ self.wc.T, x @ self.wq.T
            out = torch.empty_like(rows)
            start = 0
            for b, (n, total) in enumerate(zip(batch.q_lens, batch.kv_lens)):
                table = cache.block_table[b].long()
                pos = torch.arange(total - n, total, device=x.device)
                if write_cache:
                    cache.cache[table[pos // cache.page_size], pos % cache.page_size] = rows[start : start + n].to(cache.cache.dtype)
                for i in range(n):
                    p = total - n + i
                    keys = torch.arange(max(0, p - (self.window - 1)), p + 1, device=x.device)
                    held = cache.cache[table[keys // cache.page_size], keys % cache.page_size].float()
                    out[start + i] = torch.softmax((held @ queries[start + i]) * self.scale, 0) @ held
                start += n
            return (out @ self.wo.T).to(x.dtype)

    width, window, n_heads, n_kv, hd, theta, hidden = 24, 6, 2, 2, 16, 90.0, 48

    def toy_plan(cfg):
        norm = PartChoice("rmsnorm", {"dim": cfg.dim, "eps": 1e-5})
        ff = PartChoice("swiglu", {"dim": cfg.dim, "hidden_dim": hidden})
        names = {"norm1": "n1.", "mixer": "mix.", "norm2": "n2.", "feed_forward": "ff."}
        layers = [
            LayerPlan.standard("l0.", "pre_norm", norm, PartChoice("toy_compressed_rows", {"dim": cfg.dim, "width": width, "window": window, "scale": 0.4}), ff, names),
            LayerPlan.standard("l1.", "pre_norm", norm, _attention(cfg.dim, n_heads, n_kv, hd, theta), ff, names),
        ]
        return ModelPlan.standard(cfg.vocab_size, cfg.dim, "emb", layers, [LayerCall(0), LayerCall(1)], norm, "final", "head", max_positions=64)

    register_part("mixer", "toy_compressed_rows", CompressedRowMixer)
    register_architecture("toy_compressed_model", ToyConfig, toy_plan)
    try:
        arch, cfg = parse_config({"architecture": "toy_compressed_model", "dim": 32, "vocab_size": 53})
        model = Model(arch.build_plan(cfg))
        runtime = Runtime(torch.device("cuda:0"), torch.float32)
        host = random_tensors(model.tensor_specs(), seed=9, std=0.3, norm_init="uniform", dtype=torch.float32)
        model.bind({k: v.to("cuda:0") for k, v in host.items()}, runtime)

        def whole_sequence(tokens):
            w = {k: v.double() for k, v in host.items()}
            n = len(tokens)
            h = w["emb.weight"][torch.tensor(tokens)]
            x = plain.rms_norm(h, w["l0.n1.weight"], 1e-5)
            rows, queries = x @ w["l0.mix.wc.weight"].T, x @ w["l0.mix.wq.weight"].T
            mixed = torch.stack([
                torch.softmax((rows[max(0, p - (window - 1)) : p + 1] @ queries[p]) * 0.4, 0) @ rows[max(0, p - (window - 1)) : p + 1] for p in range(n)
            ]) @ w["l0.mix.wo.weight"].T
            h = h + mixed
            h = h + plain.swiglu(plain.rms_norm(h, w["l0.n2.weight"], 1e-5), w["l0.ff.w1.weight"], w["l0.ff.w2.weight"], w["l0.ff.w3.weight"])
            h = h + _plain_attention(plain.rms_norm(h, w["l1.n1.weight"], 1e-5), w, "l1.mix.", n_heads, n_kv, hd, theta)
            h = h + plain.swiglu(plain.rms_norm(h, w["l1.n2.weight"], 1e-5), w["l1.ff.w1.weight"], w["l1.ff.w2.weight"], w["l1.ff.w3.weight"])
            return plain.linear(plain.rms_norm(h, w["final.weight"], 1e-5), w["head.weight"]).float()

        toks = {"a": traces.random_tokens(7, 23, 53), "b": traces.random_tokens(8, 12, 53)}
        cut, storage = _step_through(model, runtime, toks, CUTS, page_size=4, pages=16)
        for k in toks:
            torch.testing.assert_close(cut[k], whole_sequence(toks[k]), rtol=2e-4, atol=2e-4)
        # the storage laid the two caches out as their needs said
        assert storage.paged[0].shape == (16, 4, width) and storage.paged[1].shape == (16, 2, n_kv, 4 * hd)
        # and the pool sizes price a token of each group by its own need: 24 against 2 * 2 * 16 elements
        assert model.cache_specs[0].bytes_per_token(4) == 4 * width and model.cache_specs[1].bytes_per_token(4) == 4 * 2 * n_kv * hd
        sizes = pool_sizes(model, GenArgs(max_batch=64, cache_block=4, max_prefill=8, prefill_gb=0, expected_seq=1000), torch.device("cuda:0"),
                           free_bytes=10_000_000)
        spent = sizes[window] * 4 * 4 * width + sizes[None] * 4 * 4 * 2 * n_kv * hd
        assert 0.8 * 9_000_000 <= spent <= 9_000_000  # nine tenths of the memory, in these bytes
    finally:
        del ARCHITECTURES["toy_compressed_model"]
        del MIXERS["toy_compressed_rows"]


# ---- a head that caps its logits -------------------------------------------------------------------- #
def test_toy_head_with_a_cap_and_a_bias_and_an_embedding_with_positions():
    """What a model does at its two ends belongs to two parts: here an embedding that adds a learned row per
    position to the token's row, and a head with a bias whose logits are capped, cap * tanh(logits / cap).
    Both are registered from here and named in the plan."""
    from cwm_amd.config import ARCHITECTURES, parse_config, register_architecture
    from cwm_amd.models import Model
    from cwm_amd.parts import Embedding, Head, LayerCall, LayerPlan, ModelPlan, PartChoice, PartSlot, Runtime, TensorSpec, register_part
    from cwm_amd.parts.base import EMBEDDINGS, HEADS
    from cwm_amd.weights import random_tensors

    class PositionedEmbedding(Embedding):
        def __init__(self, vocab_size, dim, max_positions):
            self.vocab_size, self.dim, self.max_positions = vocab_size, dim, max_positions

        def tensor_specs(self):
            return {"tokens.weight": TensorSpec((self.vocab_size, self.dim)), "positions.weight": TensorSpec((self.max_positions, self.dim))}

        def bind(self, tensors, runtime):
            super().bind(tensors, runtime)
            self.tokens, self.positions = tensors["tokens.weight"].float(), tensors["positions.weight"].float()

        def forward(self, batch):
            return self.tokens[batch.tokens.long()] + self.positions[batch.positions.long()]

    class CappedHead(Head):
        def __init__(self, vocab_size, dim, cap):
            self.vocab_size, self.dim, self.cap = vocab_size, dim, cap

        def tensor_specs(self):
            return {"weight": TensorSpec((self.vocab_size, self.dim)), "bias": TensorSpec((self.vocab_size,), precision="stored")}

        def bind(self, tensors, runtime):
            super().bind(tensors, runtime)
            self.weight, self.bias = tensors["weight"], tensors["bias"].float()

        def forward(self, x):
            from cwm_amd import ops

            logits = ops.linear(x, self.weight, None, torch.float32) + self.bias
            return self.cap * torch.tanh(logits / self.cap)

    n_heads, n_kv, hd, theta, hidden, cap = 2, 1, 16, 120.0, 40, 1.5

    def toy_plan(cfg):
        norm = PartChoice("rmsnorm", {"dim": cfg.dim, "eps": 1e-5})
        names = {"norm1": "n1.", "mixer": "attn.", "norm2": "n2.", "feed_forward": "ff."}
        layer = LayerPlan.standard("l0.", "pre_norm", norm, _attention(cfg.dim, n_heads, n_kv, hd, theta),
                                   PartChoice("swiglu", {"dim": cfg.dim, "hidden_dim": hidden}), names)
        return ModelPlan(
            cfg.vocab_size, cfg.dim, [layer], [LayerCall(0)],
            embedding=PartSlot("embedding", PartChoice("toy_positioned", {"vocab_size": cfg.vocab_size, "dim": cfg.dim, "max_positions": 32}), "in."),
            final_norm=PartSlot("norm", norm, "final."),
            head=PartSlot("head", PartChoice("toy_capped", {"vocab_size": cfg.vocab_size, "dim": cfg.dim, "cap": cap}), "out."),
        )

    register_part("embedding", "toy_positioned", PositionedEmbedding)
    register_part("head", "toy_capped", CappedHead)
    register_architecture("toy_capped_model", ToyConfig, toy_plan)
    try:
        arch, cfg = parse_config({"architecture": "toy_capped_model", "dim": 32, "vocab_size": 59})
        model = Model(arch.build_plan(cfg))
        specs = model.tensor_specs()
        assert {"in.tokens.weight", "in.positions.weight", "out.weight", "out.bias", "final.weight"} <= set(specs)
        assert model.tensor_names("head") == {"out.weight", "out.bias"}
        assert not model.replayable  # the toy parts do not say that their steps may be captured
        runtime = Runtime(torch.device("cuda:0"), torch.float32)
        host = random_tensors(specs, seed=2, std=0.4, norm_init="uniform", dtype=torch.float32)
        model.bind({k: v.to("cuda:0") for k, v in host.items()}, runtime)

        def whole_sequence(tokens, capped=True):
            w = {k: v.double() for k, v in host.items()}
            n = len(tokens)
            h = w["in.tokens.weight"][torch.tensor(tokens)] + w["in.positions.weight"][:n]
            h = h + _plain_attention(plain.rms_norm(h, w["l0.n1.weight"], 1e-5), w, "l0.attn.", n_heads, n_kv, hd, theta)
            h = h + plain.swiglu(plain.rms_norm(h, w["l0.n2.weight"], 1e-5), w["l0.ff.w1.weight"], w["l0.ff.w2.weight"], w["l0.ff.w3.weight"])
            logits = plain.linear(plain.rms_norm(h, w["final.weight"], 1e-5), w["out.weight"]) + w["out.bias"]
            return (cap * torch.tanh(logits / cap) if capped else logits).float()

        toks = {"a": traces.random_tokens(3, 23, 59), "b": traces.random_tokens(4, 12, 59)}
        cut, _ = _step_through(model, runtime, toks, CUTS)
        for k in toks:
            torch.testing.assert_close(cut[k], whole_sequence(toks[k]), rtol=2e-4, atol=2e-4)
        assert float(cut["a"].abs().max()) <= cap and float(whole_sequence(toks["a"], capped=False).abs().max()) > 2 * cap  # the cap bites
    finally:
        del ARCHITECTURES["toy_capped_model"]
        del EMBEDDINGS["toy_positioned"]
        del HEADS["toy_capped"]
