"""Two tiny Qwen2-MoE configurations that differ in every size and option, and
helpers that make a model folder and read it back for the plain implementation."""
import json
import os

import torch

CONFIG_A = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16,
    "num_experts": 4, "num_experts_per_tok": 2, "moe_intermediate_size": 32, "shared_expert_intermediate_size": 64,
    "intermediate_size": 128, "decoder_sparse_step": 1, "mlp_only_layers": [], "norm_topk_prob": False,
    "vocab_size": 256, "rope_theta": 10000.0, "rms_norm_eps": 1e-6, "max_position_embeddings": 128,
    "use_sliding_window": False, "tie_word_embeddings": False,
}

CONFIG_B = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe",
    "num_hidden_layers": 4, "hidden_size": 96, "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 32,
    "num_experts": 8, "num_experts_per_tok": 3, "moe_intermediate_size": 48, "shared_expert_intermediate_size": 80,
    "intermediate_size": 160, "decoder_sparse_step": 2, "mlp_only_layers": [0], "norm_topk_prob": True,
    "vocab_size": 384, "rope_theta": 1000000.0, "rms_norm_eps": 1e-5, "max_position_embeddings": 256,
    "use_sliding_window": True, "sliding_window": 16, "max_window_layers": 2, "tie_word_embeddings": True,
}

# sizes that are no power of two and no multiple of 16 where the architecture allows it
CONFIG_C = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe",
    "num_hidden_layers": 3, "hidden_size": 72, "num_attention_heads": 6, "num_key_value_heads": 3, "head_dim": 48,
    "num_experts": 5, "num_experts_per_tok": 1, "moe_intermediate_size": 40, "shared_expert_intermediate_size": 0,
    "intermediate_size": 104, "decoder_sparse_step": 1, "mlp_only_layers": [1], "norm_topk_prob": False,
    "vocab_size": 301, "rope_theta": 50000.0, "rms_norm_eps": 1e-5, "max_position_embeddings": 512,
    "use_sliding_window": True, "sliding_window": 24, "max_window_layers": 1, "tie_word_embeddings": False,
    "qkv_bias": False,
}

# awkward sizes: nothing is a multiple of 8 where the architecture allows it; the kernels' general paths run
CONFIG_D = {
    "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe",
    "num_hidden_layers": 2, "hidden_size": 100, "num_attention_heads": 5, "num_key_value_heads": 5, "head_dim": 24,
    "num_experts": 3, "num_experts_per_tok": 2, "moe_intermediate_size": 36, "shared_expert_intermediate_size": 28,
    "intermediate_size": 52, "decoder_sparse_step": 1, "mlp_only_layers": [0], "norm_topk_prob": True,
    "vocab_size": 131, "rope_theta": 10000.0, "rms_norm_eps": 1e-6, "max_position_embeddings": 256,
    "use_sliding_window": False, "tie_word_embeddings": False,
}

CONFIGS = {"A": CONFIG_A, "B": CONFIG_B, "C": CONFIG_C, "D": CONFIG_D}


def make_folder(raw_config: dict, seed: int, out_dir: str, dtype: str = "bfloat16", std_scale: float = 1.0) -> str:
    from inferx_amd.config import config_from_dict
    from inferx_amd.weights import write_model_folder
    raw = dict(raw_config)
    if std_scale != 1.0:
        raw["initializer_range"] = 0.02 * std_scale
    write_model_folder(config_from_dict(raw), seed, out_dir, dtype)
    return out_dir


def read_folder(model_dir: str):
    """config dict and tensors, through the safetensors library (not the framework's reader)."""
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    return cfg, load_file(os.path.join(model_dir, "model.safetensors"))


def random_tokens(n: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def random_config(seed: int) -> dict:
    """A tiny configuration drawn from the sizes the architecture allows: any number of heads and groups, head sizes
    in steps of 16 up to 256 and a few that are no multiple of 16, widths and vocabularies that are no power of
    two, up to 130 experts, pages of 16 to 64 (returned under the key "_page_size", which is no config key)."""
    import random
    rnd = random.Random(seed)
    kv = rnd.choice([1, 2, 3, 4, 5])
    heads = kv * rnd.choice([1, 2, 3, 4])
    head_dim = 16 * rnd.randint(1, 16) if rnd.random() < 0.7 else rnd.choice([24, 40, 72])
    experts = rnd.choice([2, 3, 5, 8, 16, 60, 130])
    layers = rnd.randint(1, 4)
    cfg = {
        "architectures": ["Qwen2MoeForCausalLM"], "model_type": "qwen2_moe", "num_hidden_layers": layers,
        "hidden_size": rnd.choice([64, 72, 88, 96, 100, 136, 200, 264]), "num_attention_heads": heads,
        "num_key_value_heads": kv, "head_dim": head_dim, "num_experts": experts,
        "num_experts_per_tok": rnd.randint(1, min(experts, 8)),
        "moe_intermediate_size": rnd.choice([24, 32, 40, 56, 72, 136]),
        "shared_expert_intermediate_size": rnd.choice([0, 28, 64, 88]),
        "intermediate_size": rnd.choice([52, 96, 104, 160]), "decoder_sparse_step": rnd.choice([1, 1, 2]),
        "mlp_only_layers": [rnd.randrange(layers)] if (layers > 1 and rnd.random() < 0.4) else [],
        "norm_topk_prob": rnd.random() < 0.5, "vocab_size": rnd.choice([131, 256, 301, 1000]),
        "rope_theta": rnd.choice([1e4, 1e6]), "rms_norm_eps": rnd.choice([1e-5, 1e-6]),
        "max_position_embeddings": 512, "use_sliding_window": rnd.random() < 0.5,
        "sliding_window": rnd.choice([8, 16, 24, 40]), "max_window_layers": rnd.randrange(layers + 1),
        "tie_word_embeddings": rnd.random() < 0.3, "qkv_bias": rnd.random() < 0.7,
        "_page_size": rnd.choice([16, 16, 32, 64]),
    }
    if rnd.random() < 0.3:  # the windowed layers named outright
        cfg["layer_types"] = [rnd.choice(["full_attention", "sliding_attention"]) for _ in range(layers)]
    sparse = [l for l in range(layers)
              if (l + 1) % cfg["decoder_sparse_step"] == 0 and l not in cfg["mlp_only_layers"]]
    if not sparse:  # the architecture wants at least one layer of experts
        cfg["decoder_sparse_step"], cfg["mlp_only_layers"] = 1, []
    return cfg
