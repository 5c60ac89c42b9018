"""Tiny Qwen2-MoE configurations that differ in every size and option."""

# MHA, head 16, theta 1e4, eps 1e-6, no window, 8 experts top-2 un-normalised, every layer sparse, norm weights 1
TINY_A = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe",
    "vocab_size": 256, "hidden_size": 64, "num_hidden_layers": 2, "num_attention_heads": 4,
    "num_key_value_heads": 4, "intermediate_size": 96, "moe_intermediate_size": 32,
    "shared_expert_intermediate_size": 64, "num_experts": 8, "num_experts_per_tok": 2, "norm_topk_prob": False,
    "decoder_sparse_step": 1, "mlp_only_layers": [], "rope_theta": 10000.0, "rms_norm_eps": 1e-6,
    "use_sliding_window": False, "sliding_window": 4096, "max_window_layers": 2, "max_position_embeddings": 512,
    "tie_word_embeddings": False, "torch_dtype": "float32",
}
TINY_A_INIT = dict(seed=0, std=0.02, norm_std=0.0)

# GQA 3:1, head 24, theta 1e6, eps 1e-5, window 24 from layer 1, 12 experts top-3 normalised, sparse step 2 with
# layer 0 dense (so layers 0 and 2 are dense, 1 sparse), sizes that are no power of two, norm weights N(1, .02)
TINY_B = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe",
    "vocab_size": 384, "hidden_size": 144, "num_hidden_layers": 3, "num_attention_heads": 6,
    "num_key_value_heads": 2, "head_dim": 24, "intermediate_size": 160, "moe_intermediate_size": 48,
    "shared_expert_intermediate_size": 96, "num_experts": 12, "num_experts_per_tok": 3, "norm_topk_prob": True,
    "decoder_sparse_step": 2, "mlp_only_layers": [0], "rope_theta": 1000000.0, "rms_norm_eps": 1e-5,
    "use_sliding_window": True, "sliding_window": 24, "max_window_layers": 1, "max_position_embeddings": 1024,
    "tie_word_embeddings": False, "torch_dtype": "float32", "eos_token_id": [7, 11],
}
TINY_B_INIT = dict(seed=1, std=0.02, norm_std=0.02)

# heads of 32 on 2 kv heads (the matrix-core attention takes them; hidden size is not heads x head size), a window of
# 40 from layer 1 (smaller than a page of the cache and no multiple of anything), one expert per token out of 5,
# normalised, no shared expert, layer 1 dense, tied embeddings, theta 5e4
TINY_C = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe",
    "vocab_size": 200, "hidden_size": 96, "num_hidden_layers": 3, "num_attention_heads": 6,
    "num_key_value_heads": 2, "head_dim": 32, "intermediate_size": 112, "moe_intermediate_size": 40,
    "shared_expert_intermediate_size": 0, "num_experts": 5, "num_experts_per_tok": 1, "norm_topk_prob": True,
    "decoder_sparse_step": 1, "mlp_only_layers": [1], "rope_theta": 50000.0, "rms_norm_eps": 1e-6,
    "use_sliding_window": True, "sliding_window": 40, "max_window_layers": 1, "max_position_embeddings": 2048,
    "tie_word_embeddings": True, "torch_dtype": "float32",
}
TINY_C_INIT = dict(seed=5, std=0.02, norm_std=0.02)

# a folder as newer tools write it: the layers' kinds listed one by one (sliding first, then full, then sliding: not what
# max_window_layers would give), the rotation's base inside rope_parameters, "dtype" for the stored type, q, k, v without
# bias; 4 layers, heads of 16 on one kv head, window 19, 6 experts top-4 un-normalised
TINY_D = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe",
    "vocab_size": 300, "hidden_size": 80, "num_hidden_layers": 4, "num_attention_heads": 5,
    "num_key_value_heads": 1, "head_dim": 16, "intermediate_size": 72, "moe_intermediate_size": 24,
    "shared_expert_intermediate_size": 40, "num_experts": 6, "num_experts_per_tok": 4, "norm_topk_prob": False,
    "decoder_sparse_step": 1, "mlp_only_layers": [2], "rope_parameters": {"rope_type": "default", "rope_theta": 250000.0},
    "rms_norm_eps": 2e-6, "use_sliding_window": True, "sliding_window": 19, "max_window_layers": 3,
    "layer_types": ["sliding_attention", "full_attention", "sliding_attention", "full_attention"],
    "qkv_bias": False, "max_position_embeddings": 1024, "tie_word_embeddings": False, "dtype": "float32",
}
TINY_D_INIT = dict(seed=9, std=0.02, norm_std=0.02)

TINY = {"D": (TINY_D, TINY_D_INIT), "A": (TINY_A, TINY_A_INIT), "B": (TINY_B, TINY_B_INIT), "C": (TINY_C, TINY_C_INIT)}
