"""``LlamaForCausalLM``: its configuration keys, its model as a list of parts, its tensor names.

Structure (src/model/llama.cpp:297-386): embedding, then per layer RMSNorm -> attention (rotary
positions, grouped kv heads) -> residual, RMSNorm -> SwiGLU -> residual, then RMSNorm and the
output head, which is the embedding matrix when ``tie_word_embeddings`` holds
(src/model/llama.cpp:651-661).  Tensor names are those of the checkpoint
(tools/export_llama3.py:568-592).
"""
from __future__ import annotations

from ..config.model_config import LlamaConfig
from ..config.spec import BlockSpec, LayerRun, ModelSpec, PartSpec
from ..registry import Architecture, register_architecture
from ..weights.random_init import InitRule


def build_spec(cfg: LlamaConfig) -> ModelSpec:
    d = cfg.hidden_size
    scaling = None if cfg.rope_scaling is None else {
        "kind": cfg.rope_scaling.rope_type,
        "factor": cfg.rope_scaling.factor,
        "low_freq_factor": cfg.rope_scaling.low_freq_factor,
        "high_freq_factor": cfg.rope_scaling.high_freq_factor,
        "original_max_position_embeddings": cfg.rope_scaling.original_max_position_embeddings,
    }
    position = PartSpec("rope", {"rotary_dim": cfg.head_dim, "theta": cfg.rope_theta, "scaling": scaling,
                                 "max_positions": cfg.max_position_embeddings})
    blocks = []
    for i in range(cfg.num_hidden_layers):
        pre = f"model.layers.{i}."
        blocks.append(BlockSpec(kind="prenorm", parts=dict(
            mixer_norm=PartSpec("rmsnorm", {"size": d, "eps": cfg.rms_norm_eps},
                                {"weight": pre + "input_layernorm.weight"}),
            mixer=PartSpec("attention",
                           {"hidden_size": d, "num_heads": cfg.num_attention_heads,
                            "num_kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                            "scale": None, "window": None, "position": position},
                           {"q": pre + "self_attn.q_proj.weight", "k": pre + "self_attn.k_proj.weight",
                            "v": pre + "self_attn.v_proj.weight", "o": pre + "self_attn.o_proj.weight"}),
            ffn_norm=PartSpec("rmsnorm", {"size": d, "eps": cfg.rms_norm_eps},
                              {"weight": pre + "post_attention_layernorm.weight"}),
            ffn=PartSpec("swiglu", {"hidden_size": d, "intermediate_size": cfg.intermediate_size},
                         {"gate": pre + "mlp.gate_proj.weight", "up": pre + "mlp.up_proj.weight",
                          "down": pre + "mlp.down_proj.weight"}),
        )))
    embed_name = "model.embed_tokens.weight"
    head_name = embed_name if cfg.tie_word_embeddings else "lm_head.weight"
    return ModelSpec(
        vocab_size=cfg.vocab_size,
        hidden_size=d,
        max_positions=cfg.max_position_embeddings,
        embedding=PartSpec("table", {"vocab_size": cfg.vocab_size, "hidden_size": d}, {"weight": embed_name}),
        blocks=blocks,
        order=[LayerRun(block=i, cache=i) for i in range(cfg.num_hidden_layers)],
        final_norm=PartSpec("rmsnorm", {"size": d, "eps": cfg.rms_norm_eps}, {"weight": "model.norm.weight"}),
        head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": d}, {"weight": head_name}),
        bos_token_id=cfg.bos_token_id,
        eos_token_ids=cfg.eos_token_ids,
        duplicates={"lm_head.weight": embed_name} if cfg.tie_word_embeddings else {},
        ignorable_suffixes=("rotary_emb.inv_freq",),
    )


LLAMA = register_architecture(Architecture(
    name="LlamaForCausalLM",
    config_from_dict=LlamaConfig.from_dict,
    build_spec=build_spec,
    init=InitRule(matrix_std=0.02, vector_mean=1.0, vector_std=0.05),
))
