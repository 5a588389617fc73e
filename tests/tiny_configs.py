"""Small configurations for the tests.  A and B differ in every size and option; C has sizes that
are neither powers of two nor multiples of a wavefront."""

TINY_A = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 64, "num_hidden_layers": 2, "num_attention_heads": 4, "num_key_value_heads": 2,
    "head_dim": 16, "intermediate_size": 160, "vocab_size": 256, "rms_norm_eps": 1e-5,
    "rope_theta": 10000.0, "rope_scaling": None, "max_position_embeddings": 256,
    "tie_word_embeddings": True, "hidden_act": "silu", "bos_token_id": 1, "eos_token_id": 2,
}

TINY_B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 192, "num_hidden_layers": 3, "num_attention_heads": 6, "num_key_value_heads": 1,
    "head_dim": 32, "intermediate_size": 512, "vocab_size": 1000, "rms_norm_eps": 1e-6,
    "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 4.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 64},
    "max_position_embeddings": 512, "tie_word_embeddings": False, "hidden_act": "silu",
    "bos_token_id": 0, "eos_token_id": [998, 999],
}

# hidden size that is not heads x head_dim, odd vocabulary, five query heads on five kv heads
TINY_C = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 100, "num_hidden_layers": 2, "num_attention_heads": 5, "num_key_value_heads": 5,
    "head_dim": 48, "intermediate_size": 136, "vocab_size": 777, "rms_norm_eps": 3e-6,
    "rope_theta": 25000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 2.0,
                     "original_max_position_embeddings": 32},
    "max_position_embeddings": 640, "tie_word_embeddings": True, "hidden_act": "silu",
}


# many heads on few kv heads and positions for long sequences: with 32 query heads a lone portion of
# 512 tokens far into its sequence, or a prompt of 4,096, reaches the attention's larger tiles and key runs
TINY_D = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 96, "num_hidden_layers": 1, "num_attention_heads": 32, "num_key_value_heads": 8,
    "head_dim": 32, "intermediate_size": 112, "vocab_size": 300, "rms_norm_eps": 2e-5,
    "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 16.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 1024},
    "max_position_embeddings": 8192, "tie_word_embeddings": True, "hidden_act": "silu",
}


# the head sizes and head counts of the family (64 with 32 heads on 8, 128 with 24 on 8) on one narrow layer,
# with positions for prompts of thousands of tokens: what the attention kernels do at the sizes they meet in
# use (tiles of two blocks, key runs), through the engine, at a cost the plain implementation can bear
TINY_E64 = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 128, "num_hidden_layers": 1, "num_attention_heads": 32, "num_key_value_heads": 8,
    "head_dim": 64, "intermediate_size": 144, "vocab_size": 211, "rms_norm_eps": 1e-5,
    "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 1024},
    "max_position_embeddings": 8192, "tie_word_embeddings": True, "hidden_act": "silu",
}
TINY_E128 = dict(TINY_E64, hidden_size=96, num_attention_heads=24, head_dim=128, intermediate_size=112, vocab_size=173)

# two heads on one, a narrow layer, and positions past 16,384: a sequence whose block table no longer fits
# one segment of the attention kernels' table in LDS (1,024 pages of 16 tokens)
TINY_F = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 64, "num_hidden_layers": 1, "num_attention_heads": 2, "num_key_value_heads": 1,
    "head_dim": 64, "intermediate_size": 80, "vocab_size": 61, "rms_norm_eps": 1e-5,
    "rope_theta": 500000.0, "rope_scaling": None,
    "max_position_embeddings": 17408, "tie_word_embeddings": True, "hidden_act": "silu",
}


def _family(hidden, heads, kv_heads, head_dim, inter, vocab, factor, tied):
    return {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama",
        "hidden_size": hidden, "num_hidden_layers": 2, "num_attention_heads": heads, "num_key_value_heads": kv_heads,
        "head_dim": head_dim, "intermediate_size": inter, "vocab_size": vocab, "rms_norm_eps": 1e-5,
        "rope_theta": 500000.0,
        "rope_scaling": {"rope_type": "llama3", "factor": factor, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                         "original_max_position_embeddings": 8192},
        "max_position_embeddings": 131072, "tie_word_embeddings": tied, "hidden_act": "silu",
        "bos_token_id": 128000, "eos_token_id": 128001,
    }


# The layer sizes of the Llama 3 family (3.2 1B, 3.2 3B, 3.1 8B), two layers each: the widths, head
# sizes and groups that the kernels meet in use.  1B keeps the family's vocabulary; the other two
# a smaller, odd one, to keep the files small.
FAMILY_1B = _family(2048, 32, 8, 64, 8192, 128256, 32.0, True)
FAMILY_3B = _family(3072, 24, 8, 128, 8192, 16033, 32.0, True)
FAMILY_8B = _family(4096, 32, 8, 128, 14336, 16033, 8.0, False)

TINY = {"A": TINY_A, "B": TINY_B, "C": TINY_C}
ALL = {**TINY, "D": TINY_D, "E64": TINY_E64, "E128": TINY_E128, "F": TINY_F, "1B": FAMILY_1B, "3B": FAMILY_3B, "8B": FAMILY_8B}
