"""Configuration, registry and the weight loader's errors."""

import json
import os

import pytest
import torch

from helpers import configs, models


def test_config_round_trip_and_derived_sizes():
    from cwm_amd.config import parse_config, to_dict

    arch, cfg = parse_config(configs.get("tiny_b"))
    assert arch.name == "llama3_dense"
    assert cfg.ffn_width == 320 and cfg.head_size == 32 and cfg.kv_heads == 1
    assert cfg.layer_windows() == [8, 8, 8, None]
    again = parse_config(to_dict(cfg))[1]
    assert again == cfg
    _, a = parse_config(configs.get("tiny_a"))
    assert a.ffn_width == 192 and a.layer_windows() == [None, None]
    _, c = parse_config(configs.get("tiny_c"))
    assert c.layer_windows() == [70, 20, 70] and c.ffn_width == 296


def test_reference_layer_rule_and_big_shapes():
    from cwm_amd.config import parse_config

    big = dict(architecture="llama3_dense", dim=6144, n_layers=64, n_heads=48, n_kv_heads=8, head_dim=128, vocab_size=128256,
               ffn_dim_multiplier=1.3125, multiple_of=256, window_attn={"window_pattern": 4, "local_window": 8192})
    _, cfg = parse_config(big)
    wins = cfg.layer_windows()
    assert cfg.ffn_width == 21504
    assert wins.count(None) == 17 and wins[0] is None and wins[63] is None and wins[1] == 8192
    for dim, mult, mo, want in ((4096, 1.3, 1024, 14336), (8192, 1.3, 4096, 28672)):
        _, c = parse_config(dict(architecture="llama3_dense", dim=dim, n_layers=2, n_heads=dim // 128, vocab_size=10, ffn_dim_multiplier=mult, multiple_of=mo))
        assert c.ffn_width == want


@pytest.mark.parametrize("change,fragment", [
    ({"architecture": "gpt9"}, "unknown architecture"),
    ({"bogus": 1}, "unknown key"),
    ({"dim": "64"}, "dim"),
    ({"n_heads": 5}, "multiple"),
    ({"weight_tying": True}, "weight_tying"),
    ({"kv_lora_rank": 16}, "latent"),
    ({"qk_norm": True}, "qk_norm"),
    ({"attn_impl": "sdpa"}, "attn_impl"),
    ({"pos_embed_impl": "alibi"}, "pos_embed_impl"),
    ({"scaled_rope": {"scale_factor": 1}}, "scale_factor"),
    ({"scaled_rope": {"low_freq_factor": 8, "high_freq_factor": 4}}, "wavelength"),
    ({"window_attn": {"window_pattern": 2}}, "local_window"),
    ({"layer_types": ["global"]}, "layer_types"),
    ({"layer_types": ["local", "global"]}, "local_window"),
    ({"norm_eps": 0}, "norm_eps"),
])
def test_config_errors(change, fragment):
    from cwm_amd.config import ConfigError, parse_config

    data = configs.get("tiny_a")
    data.update(change)
    with pytest.raises(ConfigError) as err:
        parse_config(data)
    assert fragment in str(err.value)


def test_missing_required_key_is_named():
    from cwm_amd.config import ConfigError, parse_config

    data = configs.get("tiny_a")
    del data["vocab_size"]
    with pytest.raises(ConfigError, match="vocab_size"):
        parse_config(data)
    with pytest.raises(ConfigError, match="architecture"):
        parse_config({"dim": 4})


def test_config_without_a_name_goes_to_the_architecture_it_fits():
    from cwm_amd.config import ARCHITECTURES, ConfigError, parse_config, register_architecture
    from cwm_amd.config.llama3 import Llama3DenseConfig
    from cwm_amd.models.llama3_dense import build_plan

    data = configs.get("tiny_b")
    del data["architecture"]
    arch, cfg = parse_config(data)
    assert arch.name == "llama3_dense" and cfg.dim == configs.get("tiny_b")["dim"]
    # two architectures that both take these keys: the name is needed
    register_architecture("llama3_dense_alias_for_test", Llama3DenseConfig, build_plan)
    try:
        with pytest.raises(ConfigError, match="several"):
            parse_config(data)
    finally:
        del ARCHITECTURES["llama3_dense_alias_for_test"]


def test_reference_params_json_is_read(tmp_path):
    """A folder with the reference's params.json (model keys under "model",
    cwm/fastgen/utils/loading.py:39-41) gives the same configuration."""
    import json

    from cwm_amd.config import load_config

    data = configs.get("tiny_b")
    del data["architecture"]
    (tmp_path / "params.json").write_text(json.dumps({"model": data, "tokenizer": {"name": "unused"}}))
    arch, cfg = load_config(str(tmp_path))
    assert arch.name == "llama3_dense"
    (tmp_path / "config.json").write_text(json.dumps(configs.get("tiny_b")))
    assert load_config(str(tmp_path))[1] == cfg


def test_load_config_errors(tmp_path):
    from cwm_amd.config import ConfigError, load_config

    with pytest.raises(ConfigError, match="does not exist"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text("{ not json")
    with pytest.raises(ConfigError, match="not valid JSON"):
        load_config(str(tmp_path))


def test_registry_takes_another_architecture():
    from cwm_amd.config import ARCHITECTURES, get_architecture, register_architecture
    from cwm_amd.config.llama3 import Llama3DenseConfig
    from cwm_amd.models.llama3_dense import build_plan

    register_architecture("llama3_dense_alias_for_test", Llama3DenseConfig, build_plan)
    try:
        assert get_architecture("llama3_dense_alias_for_test").build_plan is build_plan
    finally:
        del ARCHITECTURES["llama3_dense_alias_for_test"]


def _specs(name):
    from cwm_amd.config import parse_config
    from cwm_amd.models import Model

    arch, cfg = parse_config(configs.get(name))
    return Model(arch.build_plan(cfg)).tensor_specs()


def test_tensor_names_are_the_reference_module_names():
    specs = _specs("tiny_c")
    assert specs["tok_embeddings.weight"].shape == (263, 120)
    assert specs["layers.2.attention.wq.weight"].shape == (240, 120)
    assert specs["layers.0.attention.wk.bias"].shape == (240,)
    assert specs["layers.1.feed_forward.w2.weight"].shape == (120, 296)
    assert specs["layers.1.ffn_norm.weight"].shape == (120,) and specs["norm.weight"].shape == (120,)
    assert specs["output.weight"].shape == (263, 120)
    assert "layers.0.attention.wq.bias" not in _specs("tiny_a")


def test_random_folder_round_trip(tmp_path):
    from cwm_amd.weights import load_tensors

    folder = models.make_folder(tmp_path, "tiny_b", seed=4, dtype="bfloat16")
    again = models.make_folder(tmp_path / "again", "tiny_b", seed=4, dtype="bfloat16")
    config, stored = models.read_folder(folder)
    _, stored2 = models.read_folder(again)
    assert all(torch.equal(stored[k], stored2[k]) for k in stored)  # same seed, same weights
    other = models.read_folder(models.make_folder(tmp_path / "other", "tiny_b", seed=5, dtype="bfloat16"))[1]
    assert not torch.equal(stored["output.weight"], other["output.weight"])
    specs = _specs("tiny_b")
    bf = load_tensors(folder, specs, torch.bfloat16, torch.device("cpu"))
    assert set(bf) == set(specs) and all(t.dtype == torch.bfloat16 for t in bf.values())
    assert all(torch.equal(bf[k], stored[k]) for k in stored)
    f32 = load_tensors(folder, specs, torch.float32, torch.device("cpu"))
    assert all(t.dtype == torch.float32 for t in f32.values())
    assert abs(float(stored["layers.0.attention.wq.weight"].float().std()) - 0.05) < 0.01
    assert 0.5 <= float(stored["norm.weight"].float().min()) and float(stored["norm.weight"].float().max()) <= 1.5


def test_types_after_loading_in_bfloat16_mode(tmp_path):
    """Matrices stored in 32 bits are cast to bfloat16, as the reference casts every parameter
    (cwm/model/parallelize_transformer.py:50-59), so that every product runs on the bfloat16
    kernels; a tensor whose spec keeps its stored precision (norm weights) stays float32; with
    keep_float32 every tensor stored in 32 bits stays so; float16 becomes bfloat16."""
    from safetensors.torch import save_file
    from cwm_amd.engine import load_model
    from cwm_amd.weights import load_tensors

    folder = models.make_folder(tmp_path, "tiny_a", seed=1, dtype="float32")
    _, stored = models.read_folder(folder)
    assert all(t.dtype == torch.float32 for t in stored.values())
    stored["layers.0.attention.wk.weight"] = stored["layers.0.attention.wk.weight"].to(torch.float16)
    save_file(stored, os.path.join(folder, "model.safetensors"))
    specs = _specs("tiny_a")
    got = load_tensors(folder, specs, torch.bfloat16, torch.device("cpu"))
    for name, t in got.items():
        want = torch.float32 if specs[name].precision == "stored" else torch.bfloat16
        assert t.dtype == want, name
    assert got["norm.weight"].dtype == torch.float32 and got["layers.1.ffn_norm.weight"].dtype == torch.float32
    assert got["layers.0.attention.wq.weight"].dtype == torch.bfloat16 and got["tok_embeddings.weight"].dtype == torch.bfloat16
    assert torch.equal(got["output.weight"], stored["output.weight"].bfloat16())
    kept = load_tensors(folder, specs, torch.bfloat16, torch.device("cpu"), keep_float32=True)
    assert kept["layers.0.attention.wq.weight"].dtype == torch.float32
    assert kept["layers.0.attention.wk.weight"].dtype == torch.bfloat16  # stored in 16 bits
    # through the model: the joined projections are bfloat16
    model, _ = load_model(folder, "bfloat16", "cpu")
    assert model.blocks[0].mixer.qkv.weight.dtype == torch.bfloat16
    assert model.blocks[0].feed_forward.gate_up.weight.dtype == torch.bfloat16
    assert model.blocks[0].norm1.weight.dtype == torch.float32


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    from safetensors.torch import save_file
    from cwm_amd.weights import WeightError, load_tensors

    folder = models.make_folder(tmp_path, "tiny_a", seed=1, dtype="float32")
    _, stored = models.read_folder(folder)
    del stored["layers.1.ffn_norm.weight"]
    del stored["output.weight"]
    stored["extra.tensor"] = torch.zeros(3)
    stored["layers.0.attention.wk.weight"] = torch.zeros(16, 64)
    save_file(stored, os.path.join(folder, "model.safetensors"))
    with pytest.raises(WeightError) as err:
        load_tensors(folder, _specs("tiny_a"), torch.float32, torch.device("cpu"))
    text = str(err.value)
    assert "missing (2)" in text and "layers.1.ffn_norm.weight" in text and "output.weight" in text
    assert "unexpected (1)" in text and "extra.tensor" in text
    assert "wrong shape (1)" in text and "layers.0.attention.wk.weight: expected (32, 64), found (16, 64)" in text


def test_tensors_may_be_split_over_files(tmp_path):
    from safetensors.torch import save_file
    from cwm_amd.weights import WeightError, load_tensors

    folder = models.make_folder(tmp_path, "tiny_a", seed=1, dtype="float32")
    _, stored = models.read_folder(folder)
    names = sorted(stored)
    os.remove(os.path.join(folder, "model.safetensors"))
    save_file({k: stored[k] for k in names[::2]}, os.path.join(folder, "model-00001-of-00002.safetensors"))
    save_file({k: stored[k] for k in names[1::2]}, os.path.join(folder, "model-00002-of-00002.safetensors"))
    got = load_tensors(folder, _specs("tiny_a"), torch.float32, torch.device("cpu"))
    assert all(torch.equal(got[k], stored[k]) for k in stored)
    with pytest.raises(WeightError, match="no .safetensors"):
        load_tensors(str(tmp_path / "empty"), _specs("tiny_a"), torch.float32, torch.device("cpu"))


def test_kernels_refuse_the_cpu():
    from cwm_amd import ops

    with pytest.raises(ops.KernelError, match="no CPU path"):
        ops.embedding(torch.zeros(2, dtype=torch.int32), torch.zeros(4, 4))


def test_cli_dotlist(tmp_path):
    from cwm_amd.config import ConfigError
    from cwm_amd.config.cli import load_from_cli
    from cwm_amd.generate import GenerateArgs

    (tmp_path / "c.yaml").write_text("gen_args:\n  temperature: 0.3\n  max_batch: 4\nseed: 5\n")
    args = load_from_cli(GenerateArgs, [f"config={tmp_path / 'c.yaml'}", "gen_args.max_batch=8", "checkpoint_dir=/m", "stop_tokens=[1,2]", "prompt=[3,4,5]"])
    assert args.gen_args.temperature == 0.3 and args.gen_args.max_batch == 8 and args.seed == 5
    assert args.gen_args.top_p == 0.95 and args.gen_args.sync_freq == 1  # the reference's server defaults
    assert args.stop_tokens == [1, 2] and args.prompt == [3, 4, 5] and args.checkpoint_dir == "/m"
    with pytest.raises(ConfigError, match="unknown key"):
        load_from_cli(GenerateArgs, ["gen_args.tempreture=1"])
    with pytest.raises(ConfigError, match="key=value"):
        load_from_cli(GenerateArgs, ["--help-me"])


def test_a_head_size_no_kernel_takes_is_refused_when_the_model_is_built():
    """Before any weight is read: a head size above the attention kernels' limit fails as the plan's parts are made."""
    from cwm_amd.config import parse_config
    from cwm_amd.models import Model

    data = configs.get("tiny_a")
    data.update(head_dim=272, dim=64)
    arch, cfg = parse_config(data)
    with pytest.raises(ValueError, match="head_dim 272"):
        Model(arch.build_plan(cfg))


def test_streaming_copies_are_kept_where_the_matrices_fit_twice_into_half_the_memory(monkeypatch):
    """The rule of `wants_stream_copies`: bfloat16 on a GPU only; an explicit choice or CWM_AMD_STREAM_COPIES
    decides; else the matrices, twice, against half of the device's memory (32B shape: 127 GB of 288 fit,
    70B shape: 278 GB do not)."""
    import types

    import torch

    from cwm_amd.config import parse_config
    from cwm_amd.engine import loading
    from cwm_amd.models import Model

    def model_of(**sizes):
        config = {"architecture": "llama3_dense", "vocab_size": 128256, "ffn_dim_multiplier": 1.3, "multiple_of": 256, "head_dim": 128,
                  "n_kv_heads": 8, "norm_eps": 1e-5, "rope_theta": 500000.0, **sizes}
        arch, typed = parse_config(config)
        return Model(arch.build_plan(typed))

    small = model_of(dim=6144, n_layers=64, n_heads=48, ffn_dim_multiplier=1.3125)  # the 32B shape
    large = model_of(dim=8192, n_layers=80, n_heads=64, multiple_of=4096)  # the 70B shape
    gpu, cpu = torch.device("cuda:0"), torch.device("cpu")
    monkeypatch.setattr(torch.cuda, "get_device_properties", lambda device: types.SimpleNamespace(total_memory=288 * 2**30))
    monkeypatch.delenv("CWM_AMD_STREAM_COPIES", raising=False)
    assert loading.wants_stream_copies(small, torch.bfloat16, gpu) is True
    assert loading.wants_stream_copies(large, torch.bfloat16, gpu) is False
    assert loading.wants_stream_copies(small, torch.float32, gpu) is False
    assert loading.wants_stream_copies(small, torch.bfloat16, cpu) is False
    assert loading.wants_stream_copies(large, torch.bfloat16, gpu, choice=True) is True
    monkeypatch.setenv("CWM_AMD_STREAM_COPIES", "0")
    assert loading.wants_stream_copies(small, torch.bfloat16, gpu) is False
    assert loading.wants_stream_copies(small, torch.bfloat16, gpu, choice=True) is True  # the argument outranks the environment
    monkeypatch.setenv("CWM_AMD_STREAM_COPIES", "1")
    assert loading.wants_stream_copies(large, torch.bfloat16, gpu) is True
