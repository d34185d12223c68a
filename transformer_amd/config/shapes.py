"""config.json contents of the layer sizes that the measurements are quoted on: the shapes of
Llama-3.1-8B, Llama-2-7B and Llama-3-70B without their weights (random ones stand in)."""

LLAMA31_8B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 32, "hidden_size": 4096, "num_attention_heads": 32,
    "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 14336,
    "vocab_size": 128256, "rope_theta": 500000.0, "rms_norm_eps": 1e-5,
    "tie_word_embeddings": False, "max_position_embeddings": 4096, "rope_scaling": None,
}
LLAMA2_7B = {**LLAMA31_8B, "num_key_value_heads": 32, "intermediate_size": 11008,
             "vocab_size": 32000, "rope_theta": 10000.0}
LLAMA3_70B = {**LLAMA31_8B, "num_hidden_layers": 80, "hidden_size": 8192, "num_attention_heads": 64,
              "intermediate_size": 28672, "max_position_embeddings": 8192}
SHAPES = {"8b": ("Llama-3.1-8B", LLAMA31_8B), "7b": ("Llama-2-7B", LLAMA2_7B),
          "70b": ("Llama-3-70B", LLAMA3_70B)}
