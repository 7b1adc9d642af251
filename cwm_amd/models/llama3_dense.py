"""The Llama-3 dense decoder of cwm/model/transformer.py as a plan of parts."""

from __future__ import annotations

from ..config.llama3 import Llama3DenseConfig
from ..config.registry import register_architecture
from ..parts.base import LayerCall, LayerPlan, ModelPlan, PartChoice

ARCHITECTURE_NAME = "llama3_dense"


def build_plan(config: Llama3DenseConfig) -> ModelPlan:
    """Parts per layer from the configuration.

    Tensor names are the reference's module names (cwm/model/transformer.py:173-193,
    214-228,244-252,301-313).  Per layer: RMSNorm, grouped-query attention with
    rotary positions and the layer's window (:253-270), RMSNorm, SwiGLU, pre-norm
    order (cwm/fastgen/forward.py:563-786).  One eps for every norm (forward.py:493),
    softmax scale head_dim ** -0.5 (forward.py:651).
    """
    hd = config.head_size
    scaling = None
    if config.pos_embed_impl == "scaled_rope":
        sr = config.scaled_rope
        scaling = {
            "scale_factor": sr.scale_factor,
            "old_context_len": sr.old_context_len,
            "low_freq_factor": sr.low_freq_factor,
            "high_freq_factor": sr.high_freq_factor,
        }
    positions = PartChoice("rotary", {"head_dim": hd, "theta": config.rope_theta, "llama3_scaling": scaling})
    norm = PartChoice("rmsnorm", {"dim": config.dim, "eps": config.norm_eps})
    feed_forward = PartChoice("swiglu", {"dim": config.dim, "hidden_dim": config.ffn_width})
    names = {"norm1": "attention_norm.", "mixer": "attention.", "norm2": "ffn_norm.", "feed_forward": "feed_forward."}
    layers = []
    for i, window in enumerate(config.layer_windows()):
        mixer = PartChoice(
            "paged_attention",
            {
                "dim": config.dim,
                "n_heads": config.n_heads,
                "n_kv_heads": config.kv_heads,
                "head_dim": hd,
                "scale": hd ** -0.5,
                "window": window,
                "bias": config.qkv_biases,
                "position_encoding": positions,
            },
        )
        layers.append(
            LayerPlan.standard(prefix=f"layers.{i}.", block="pre_norm", norm=norm, mixer=mixer, feed_forward=feed_forward, names=names)
        )
    return ModelPlan.standard(
        vocab_size=config.vocab_size,
        dim=config.dim,
        embedding_name="tok_embeddings",
        layers=layers,
        run_order=[LayerCall(layer=i) for i in range(config.n_layers)],
        final_norm=norm,
        final_norm_name="norm",
        head_name="output",
        max_positions=config.max_seq_len,
    )


register_architecture(ARCHITECTURE_NAME, Llama3DenseConfig, build_plan)
