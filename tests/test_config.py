"""Configuration and registry (no GPU).  Fixtures follow the reference's
tests/unit/config_test.cc:93-201."""
import json

import pytest

from inferx_amd.config import (ConfigError, Qwen2MoeConfig, config_from_dict, config_from_json, known_architectures,
                               register_architecture)
import tiny

A27B = {
    "architectures": ["Qwen2MoeForCausalLM"], "hidden_size": 2048, "intermediate_size": 5632,
    "num_hidden_layers": 24, "num_attention_heads": 16, "num_key_value_heads": 16, "vocab_size": 151936,
    "num_experts": 60, "num_experts_per_tok": 4, "moe_intermediate_size": 1408, "norm_topk_prob": False,
    "shared_expert_intermediate_size": 5632,
}


def test_parses_the_a27b_shape():
    # reference: config_test.cc:152-177
    c = config_from_dict(A27B)
    assert isinstance(c, Qwen2MoeConfig)
    assert (c.num_experts, c.num_experts_per_tok, c.moe_intermediate_size) == (60, 4, 1408)
    assert c.shared_expert_intermediate_size == 5632
    assert c.norm_topk_prob is False
    assert c.intermediate_size == 5632  # the dense width is not overwritten by the expert width
    assert c.head_dim == 128 and c.q_dim == 2048 and c.kv_dim == 2048
    assert c.qkv_bias is True  # q/k/v are biased in this architecture unless the file says otherwise
    assert all(c.is_moe_layer(l) for l in range(24))
    assert all(c.window_of_layer(l) == 0 for l in range(24))


def test_defaults():
    c = config_from_dict({k: v for k, v in A27B.items() if k not in ("num_key_value_heads", "norm_topk_prob")})
    assert c.num_key_value_heads == 16 and c.norm_topk_prob is False
    assert c.rms_norm_eps == 1e-6 and c.rope_theta == 10000.0 and c.tie_word_embeddings is False
    assert c.decoder_sparse_step == 1 and c.mlp_only_layers == []


def test_which_layer_is_which():
    b = config_from_dict(tiny.CONFIG_B)
    assert [b.is_moe_layer(l) for l in range(4)] == [False, True, False, True]
    assert [b.window_of_layer(l) for l in range(4)] == [0, 0, 16, 16]
    a = config_from_dict(tiny.CONFIG_A)
    assert [a.is_moe_layer(l) for l in range(2)] == [True, True]
    spec = b.model_spec()
    assert [l.parts["feed_forward"].kind for l in spec.layers] == ["dense_mlp", "moe", "dense_mlp", "moe"]
    assert [l.parts["mixer"].params["window"] for l in spec.layers] == [0, 0, 16, 16]
    # B ties its head to the embedding: both parts name the same checkpoint tensor
    assert spec.head.tensor_name("weight") == spec.embedding.tensor_name("weight") == "model.embed_tokens.weight"
    assert a.model_spec().head.tensor_name("weight") == "lm_head.weight"
    assert spec.layers[1].parts["feed_forward"].params["renormalize"] is True
    assert spec.layers[0].parts["mixer_norm"].params["eps"] == 1e-5
    assert all(l.block == "prenorm" and sorted(l.parts) == ["feed_forward", "feed_forward_norm", "mixer",
                                                            "mixer_norm"] for l in spec.layers)


def test_layer_types_name_the_windowed_layers_outright():
    raw = dict(tiny.CONFIG_B, layer_types=["sliding_attention", "full_attention", "sliding_attention",
                                           "full_attention"])
    c = config_from_dict(raw)
    assert [c.window_of_layer(l) for l in range(4)] == [16, 0, 16, 0]
    assert [l.parts["mixer"].params["window"] for l in c.model_spec().layers] == [16, 0, 16, 0]
    assert config_from_dict(c.to_dict()).layer_types == raw["layer_types"]
    assert "layer_types" not in config_from_dict(tiny.CONFIG_B).to_dict()
    # the list decides alone, whatever use_sliding_window says
    off = config_from_dict(dict(raw, use_sliding_window=False))
    assert [off.window_of_layer(l) for l in range(4)] == [16, 0, 16, 0]
    for bad, needle in [(["full_attention"] * 3, "names 3 layers"), (["chunked"] * 4, "only full_attention"),
                        ("full_attention", "list of strings")]:
        with pytest.raises(ConfigError, match=needle):
            config_from_dict(dict(raw, layer_types=bad))
    with pytest.raises(ConfigError, match="sliding_window is not positive"):
        config_from_dict(dict(raw, sliding_window=0, use_sliding_window=False))


@pytest.mark.parametrize("change, needle", [
    ({"num_experts_per_tok": 8, "num_experts": 4}, "exceeds num_experts"),            # config_test.cc:179-189
    ({"num_experts_per_tok": None}, "nobody would route"),                            # config_test.cc:191-201
    ({"architectures": ["NoSuchModel"]}, "unknown architecture"),
    ({"architectures": ["A", "B"]}, "exactly one"),
    ({"num_key_value_heads": 5}, "not a multiple"),
    ({"head_dim": 7}, "even"),
    ({"hidden_size": None}, "required key 'hidden_size'"),
    ({"vocab_size": 0}, "must be positive"),
    ({"rms_norm_eps": 0.0}, "rms_norm_eps"),
    ({"rope_scaling": {"type": "yarn", "factor": 4}}, "rope_scaling"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"mlp_only_layers": list(range(24))}, "no layer is sparse"),
    ({"decoder_sparse_step": 0}, "decoder_sparse_step"),
    ({"use_sliding_window": True, "sliding_window": 0}, "sliding_window"),
    ({"eos_token_id": 151936}, "outside the vocabulary"),
    ({"eos_token_id": "2"}, "eos_token_id"),
    ({"hidden_size": "2048"}, "must be int"),
    ({"num_hidden_layers": True}, "must be an integer"),
])
def test_rejects(change, needle):
    raw = dict(A27B)
    for k, v in change.items():
        if v is None:
            raw.pop(k, None)
        else:
            raw[k] = v
    with pytest.raises(ConfigError) as e:
        config_from_dict(raw)
    assert needle in str(e.value)


def test_unknown_architecture_lists_known_ones():
    with pytest.raises(ConfigError) as e:
        config_from_json(json.dumps({**A27B, "architectures": ["LlamaForCausalLM"]}))
    assert "Qwen2MoeForCausalLM" in str(e.value)
    assert "Qwen2MoeForCausalLM" in known_architectures()


def test_not_json():
    with pytest.raises(ConfigError):
        config_from_json("{not json")


def test_round_trip_through_to_dict():
    for raw in list(tiny.CONFIGS.values()) + [{**tiny.CONFIG_A, "eos_token_id": 7}, {**tiny.CONFIG_B, "eos_token_id": [1, 2]}]:
        c = config_from_dict(raw)
        assert config_from_dict(c.to_dict()) == c


def test_end_of_sequence_ids():
    assert config_from_dict(A27B).eos_token_ids == []
    assert config_from_dict({**A27B, "eos_token_id": 151643}).eos_token_ids == [151643]
    assert config_from_dict({**A27B, "eos_token_id": [151645, 151643]}).eos_token_ids == [151645, 151643]


def test_registering_another_architecture():
    class ToyConfig:
        @classmethod
        def from_dict(cls, raw):
            return cls()

        def validate(self):
            pass

    register_architecture("ToyArchitectureForTest", ToyConfig)
    assert isinstance(config_from_dict({"architectures": ["ToyArchitectureForTest"]}), ToyConfig)
