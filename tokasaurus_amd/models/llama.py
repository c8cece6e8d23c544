"""Llama as a choice of parts (the architecture of tokasaurus/model/llama.py:603):
pre-norm blocks of grouped-query attention with rotary positions and a SwiGLU
feed-forward, RMSNorm everywhere, checkpoint names as at llama.py:824-847."""

from __future__ import annotations

from tokasaurus_amd.config.model_config import LlamaConfig
from tokasaurus_amd.models.spec import ModelSpec, RunEntry
from tokasaurus_amd.parts.base import PartSpec


def llama_spec(cfg: LlamaConfig) -> ModelSpec:
    position = PartSpec(
        "rotary",
        {
            "head_dim": cfg.head_dim,
            "theta": cfg.rope_theta,
            "max_positions": cfg.max_position_embeddings,
            "scaling": cfg.rope_scaling.to_dict() if cfg.rope_scaling else None,
        },
    )
    layers = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}"
        layers.append(
            PartSpec(
                "pre_norm",
                {
                    "mixer_norm": PartSpec(
                        "rmsnorm",
                        {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps, "name": f"{p}.input_layernorm.weight"},
                    ),
                    "mixer": PartSpec(
                        "paged_attention",
                        {
                            "hidden_size": cfg.hidden_size,
                            "num_heads": cfg.num_attention_heads,
                            "num_kv_heads": cfg.num_key_value_heads,
                            "head_dim": cfg.head_dim,
                            "position": position,
                            "names": {
                                "q": f"{p}.self_attn.q_proj.weight",
                                "k": f"{p}.self_attn.k_proj.weight",
                                "v": f"{p}.self_attn.v_proj.weight",
                                "o": f"{p}.self_attn.o_proj.weight",
                            },
                        },
                    ),
                    "ff_norm": PartSpec(
                        "rmsnorm",
                        {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps, "name": f"{p}.post_attention_layernorm.weight"},
                    ),
                    "feed_forward": PartSpec(
                        "swiglu",
                        {
                            "hidden_size": cfg.hidden_size,
                            "intermediate_size": cfg.intermediate_size,
                            "names": {
                                "gate": f"{p}.mlp.gate_proj.weight",
                                "up": f"{p}.mlp.up_proj.weight",
                                "down": f"{p}.mlp.down_proj.weight",
                            },
                        },
                    ),
                },
            )
        )
    embedding = "model.embed_tokens.weight"
    final_norm = PartSpec("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps, "name": "model.norm.weight"})
    return ModelSpec(
        vocab_size=cfg.vocab_size,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size, "name": embedding}),
        # a tied checkpoint's head names the embedding's tensor: both parts then share one buffer
        head=PartSpec("norm_linear", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size, "norm": final_norm,
                                      "name": embedding if cfg.tie_word_embeddings else "lm_head.weight"}),
        ignorable_tensors=("lm_head.weight",) if cfg.tie_word_embeddings else (),
        layers=tuple(layers),
        run_order=tuple(RunEntry(i) for i in range(cfg.num_hidden_layers)),
        max_positions=cfg.max_position_embeddings,
        eos_token_ids=cfg.eos_token_ids,
    )
